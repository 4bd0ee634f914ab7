// WKV7 backward for gfx950: chunk-parallel prepare -> reverse dstate scan -> chunk-parallel gradients.
//
// Replaces backward_kernel of the reference (attn.cu:131-326), same mathematics
// (rwkv7_attn_triton.py:72-156).  The forward's intermediates are recomputed per chunk from the inputs,
// the chunk-start state checkpoint and U (both saved by the forward).  With dS the gradient arriving at
// the chunk's end state:
//   prepare:   D0 = Tinv^T (QB^T dY),  Bm = Tinv^T bf
//   scan:      dab_u = D0 + Bm dS^T ;  dS' = dS diag(fw) + dY^T wq + dab_u^T wa   (same kernel as forward)
//   gradients: everything else (see bwd_grads_kernel)
// The decay gradient uses the closed form
//   dlogw_k = sum_{t>=k} (wq*Bq - kwi*Bk - bwi*Bb)_t + sum_{t>k} (wa*Ba)_t + sum_i S'[i,:]*dS[i,:]
// where Bq,Bk,Bb,Ba are the un-scaled brackets of dq,dk,db,da; it equals the pair sums the reference
// evaluates with fast_dw (tile.cuh:394-503, attn.cu:299-308) because every pair (t,s) with both ends on
// the same side of k appears once with each sign.
#include <type_traits>

#include "ln_epilogue.hpp"
#include "device_info.hpp"
#include "wkv7_common.hpp"
#include "wkv7_kernels.hpp"

namespace wkv {

// ------------------------------------------------------------------------------------------------
// attn_ln runs the epilogue's backward first, as a kernel of its own (one wavefront per chunk, per token in
// registers): it leaves dg, the bonus part of dv, sum_c dx2*v per token, the per-chunk parameter gradient
// partials, and the gradient of the plain WKV7 output (dY), which the reverse scan and bwd_grads_kernel then
// take as their dy.
struct LnBwdArgs {
    const __bf16 *k, *v, *g, *y_wkv;   // [B,T,H,64]
    const float* centers;              // the centres y_wkv was kept with (ln_epilogue.hpp), or null
    const float* params;               // [3][H*64]
    __bf16 *dg, *dY, *dv;              // [B,T,H,64]
    float* ddot;                       // [nchunks][16]
    float* dparams_part;               // [nchunks][3][64]
};

__global__ __launch_bounds__(256) void ln_epilogue_bwd_kernel(int T, int H, int nchunks, const __bf16* __restrict__ q_,
                                                              const __bf16* __restrict__ dy_, LnBwdArgs ln) {
    const int wid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wid >= nchunks) return;
    const int cid = H >= 16 ? head_major_chunk(wid, nchunks, T) : wid;   // (long rows: see head_major_chunk)
    const Lane L;
    const ChunkAddr ca(cid, T, H);
    const TileB q = load_rows16(q_ + ca.row0, ca.ld, L);
    const TileB dy = load_rows16(dy_ + ca.row0, ca.ld, L);
    const TileB k = load_rows16(ln.k + ca.row0, ca.ld, L);
    const TileB v = load_rows16(ln.v + ca.row0, ca.ld, L);
    const TileB g = load_rows16(ln.g + ca.row0, ca.ld, L);
    const TileB y = load_rows16(ln.y_wkv + ca.row0, ca.ld, L);
    const LnParams p = load_ln_params(ln.params, ca.bh % H, H, L);
    const LnBackward r = ln_backward(uncentre(y, ln.centers, ca.row0 / HEAD + (long)L.n * H), q, k, v, g, dy, p);
    store_rows16(ln.dg + ca.row0, ca.ld, L, r.dg);
    store_rows16(ln.dY + ca.row0, ca.ld, L, r.dy);
    store_rows16(ln.dv + ca.row0, ca.ld, L, r.dv_bonus);
    if (L.g == 0) ln.ddot[(long)cid * CHUNK + L.n] = r.ddot;
    // parameter gradients: sum over the chunk's 16 tokens (lanes of a row); lane n = 15 holds the total
    float* part = ln.dparams_part + (long)cid * 3 * HEAD;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        f32x4 sw, sb, sbo;
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            sw[rr] = row_prefix_sum(r.dw.f[ib][rr]);
            sb[rr] = row_prefix_sum(r.db.f[ib][rr]);
            sbo[rr] = row_prefix_sum(r.dbonus.f[ib][rr]);
        }
        if (L.n == 15) {
            const int ch = chan16(ib, 4 * L.g);
            *reinterpret_cast<f32x4*>(part + 0 * HEAD + ch) = sw;
            *reinterpret_cast<f32x4*>(part + 1 * HEAD + ch) = sb;
            *reinterpret_cast<f32x4*>(part + 2 * HEAD + ch) = sbo;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// gradients: one wavefront per chunk.
//   in:  the seven sequence tiles, U^T (saved by forward), dab_u^T and dS (from the reverse scan),
//        S0 (forward checkpoint)
//   out: dw, dq, dk, dv, da, db for the chunk's 16 tokens
// ------------------------------------------------------------------------------------------------
// With LN the bonus term's gradients are added: dq += k*bonus*ddot, dk += q*bonus*ddot, dv += dot*dx2
// (the last one was left in the dv buffer by ln_epilogue_bwd_kernel).
// MODE 1: the scans left a state and U^T (dab_u^T) per chunk (Saved both; an odd number of chunks, or interval 16).
// MODE 3: the scans kept a state only per PAIR of chunks (32 tokens) in both directions (SavedPair both): the
// forward the state entering chunk 2p, the backward the dstate arriving at the end of chunk 2p+1, and U^T / dab_u^T per
// chunk.  A wavefront takes a pair.  It first advances the forward state across chunk 2p itself,
//     S(start of chunk 2p+1) = (S(start of chunk 2p) + V^T kwi + U^T bwi) diag(fw)        (operands of chunk 2p),
// then handles chunk 2p+1, which hands the dstate on,
//     dS(end of chunk 2p) = dS(end of chunk 2p+1) diag(fw) + dY^T wq + dab_u^T wa          (operands of chunk 2p+1),
// and then chunk 2p: sixteen matrix instructions each, on fragments the chunks' own gradients need anyway.
// What a pair needs from memory besides the tiles that go straight into arithmetic arrives by global -> LDS loads
// (no registers, so nothing is live across the chunk before): both states and, for either chunk, w, k, b, v and U^T,
// 36 KiB per wavefront; only q, a, dY and dab_u^T of the next chunk wait in registers.  Needs an even number of chunks.
namespace pairlds {   // byte offsets inside a wavefront's 36 KiB
constexpr int STASH = 0;              // the state entering the pair: [ib][half][lane] x 16 B (fragments jb = 2 half, 2 half + 1)
constexpr int CARRY = 8192;           // the dstate arriving at the end of the current chunk, same layout
constexpr int TILES = 16384;          // two sets, of chunk 2p and of chunk 2p+1
constexpr int SET = 10240;            // w, k, b, v: [tile][pr][lane] x 16 B (2 KiB each); then U^T: 4 fragments of [lane] x 8 B
constexpr int BYTES = TILES + 2 * SET;
// lane l's 16 bytes at (descriptor base + voff + soff) land at lds + 16 l.  The constant part of an address goes into
// the scalar offset: the instruction's immediate offset would move the LDS address as well, so constants added to the
// lane offset would each become a vector register of their own, kept across the loop.
__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t r, unsigned voff, int soff, unsigned char* lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, lds, 16, voff, soff, 0, 0);
}
__device__ __forceinline__ TileB tile(const unsigned char* set, int t, int lane) {
    TileB x;
#pragma unroll
    for (int pr = 0; pr < NBLK / 2; pr++) {
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(set + t * 2048 + pr * 1024 + lane * 16);
        x.f[2 * pr] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
        x.f[2 * pr + 1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
    }
    return x;
}
__device__ __forceinline__ TileB frags(const unsigned char* p, int lane) {   // four fragments, [ib][lane] x 8 B
    TileB x;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) x.f[ib] = *reinterpret_cast<const bf16x4*>(p + ib * 512 + lane * 8);
    return x;
}
__device__ __forceinline__ TileB state(const unsigned char* p, int ib, int lane) {   // fragments (ib, 0 .. 3)
    TileB x;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(p + (2 * ib + h) * 1024 + lane * 16);
        x.f[2 * h] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
        x.f[2 * h + 1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
    }
    return x;
}
// F(M^T) of the 16x16 block (ib, jb) of a state kept in the layout above, by the LDS read that transposes 16-bit elements
// (ds_read_b64_tr_b16): lane p of each group of 16 points at the 8 bytes of row 4g + p/4, columns 4(p%4) .. +3, and
// receives rows 4g .. 4g+3 of column p.  In the fragment layout those 8 bytes belong to lane 16 (p%4) + 4g + p/4.
typedef s16x4 __attribute__((address_space(3))) lds_s16x4;
typedef unsigned char __attribute__((address_space(3))) lds_u8;
__device__ __forceinline__ int tr_lane_offset(const Lane& L) { return (16 * (L.n & 3) + 4 * L.g + (L.n >> 2)) * 16; }
__device__ __forceinline__ bf16x4 state_t(const unsigned char* p, int ib, int jb, int tr_off) {
    return __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                          (lds_s16x4*)(lds_u8*)(p + (2 * ib + (jb >> 1)) * 1024 + (jb & 1) * 8 + tr_off)));
}
}   // namespace pairlds

template <bool LN, int MODE>
__global__ __launch_bounds__(256) void bwd_grads_kernel(int T, int H, int nchunks,
                                                        const __bf16* __restrict__ w_, const __bf16* __restrict__ q_,
                                                        const __bf16* __restrict__ k_, const __bf16* __restrict__ v_,
                                                        const __bf16* __restrict__ a_, const __bf16* __restrict__ b_,
                                                        const __bf16* __restrict__ dy_,
                                                        const __bf16* __restrict__ rec_fwd, const __bf16* __restrict__ rec_bwd,
                                                        __bf16* __restrict__ dw_, __bf16* __restrict__ dq_,
                                                        __bf16* __restrict__ dk_, __bf16* __restrict__ dv_,
                                                        __bf16* __restrict__ da_, __bf16* __restrict__ db_,
                                                        const float* __restrict__ ln_params,
                                                        const float* __restrict__ ln_ddot, int ds_run) {
    // Persistent wavefronts: each walks items id0, id0 + total, ... (an item is a pair of chunks, or one chunk) and
    // loads the next chunk's nine input tiles while it works on the current one.  With ~380 live registers only one
    // wavefront fits a SIMD, so without this the kernel alternates between waiting for memory and computing (measured:
    // 64 us of pure memory time + 34 us of arithmetic = 98 us); the prefetch lets the two overlap.
    static_assert(MODE == 1 || MODE == 3, "a state per chunk, or per pair of chunks");
    constexpr bool LDSP = MODE == 3;                  // states per pair in both directions, prefetched into LDS
    constexpr int AFTER_PREFETCH = 10;
    constexpr bool PAIRED = LDSP;                     // an item is a pair of chunks
    using RF = Saved;
    using RB = Saved;
    const int lane = threadIdx.x & 63;
    const int total = gridDim.x * 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // (uniform: chunk addresses then live in scalar registers)
    const int id0 = blockIdx.x * 4 + wave;
    const int NC = T / CHUNK, NP = SavedPair::pairs(NC);
    const int nitems = PAIRED ? (nchunks / NC) * NP : nchunks;
    // MODE 3: a wavefront takes RUNS of RUN consecutive pairs (runs id0, id0 + total, ...), each from its last pair down,
    // and carries the dstate from a pair to the one before it as it does from a pair's later chunk to its earlier
    // one; the reverse scan kept the dstate only where a run starts (SavedPair::ds_kept).  Everywhere else RUN = 1.
    // ds_run < 0: the runs are cut per (batch, head) (RH of them each) and handed out head-major - walking index i is
    // run i / BH of (batch, head) i % BH - so that wavefronts that run side by side read the same rows' neighbouring
    // 128-byte pieces instead of rows 128 H bytes apart (measured, gradient kernel alone: 32 heads x 16384 tokens
    // 303 -> 270 us, 2 x 24 heads x 8192 211 -> 196, 16 heads x 16384 184 -> 179, 12 heads: no difference).
    const int RUN = MODE == 3 ? (ds_run < 0 ? -ds_run : ds_run) : 1;
    const bool HM = MODE == 3 && ds_run < 0;
    const int BH = nchunks / NC, RH = (NP + RUN - 1) / RUN;
    const int nruns = HM ? BH * RH : (nitems + RUN - 1) / RUN;
    if (id0 >= nruns) return;
    // the pair a run starts with (its last one)
    auto run_first_item = [&](int i) {
        if (HM) {
            const int rr = i / BH, bh = i - rr * BH, e = (rr + 1) * RUN;
            return bh * NP + (e < NP ? e : NP) - 1;
        }
        const int e = (i + 1) * RUN;
        return (e < nitems ? e : nitems) - 1;
    };
    // the item after `it` in this wavefront's walk; nitems when there is none
    auto next_item = [&](int it) {
        const int key = HM ? it % NP : it;              // position within what the runs cut
        if (RUN > 1 && key % RUN != 0) return it - 1;
        const int i = (HM ? (key / RUN) * BH + it / NP : it / RUN) + total;
        return i < nruns ? run_first_item(i) : nitems;
    };
    const Lane L;
    const bf16x4 eye = identity_bf16(L);
    // pair_of: walking index -> index of the pair in the kept arrays (head * NP + pair)
    auto pair_of = [&](int item) { return item; };
    // the chunk an item starts with: the later chunk of the pair (or its only one)
    auto first_chunk = [&](int item) {
        if constexpr (!PAIRED) return item;
        const int pid = pair_of(item), bh = pid / NP, p = pid - bh * NP;
        return bh * NC + (2 * p + 1 < NC ? 2 * p + 1 : 2 * p);
    };

    // Every access is a buffer instruction: a descriptor in scalar registers made from a wave-uniform address (tensor +
    // chunk offset) and ONE 32-bit lane offset - no 64-bit address is formed or kept per lane.  (Written as pointer
    // arithmetic, the compiler hoists the 64-bit extensions of the loop-invariant lane offsets out of the loop, dozens
    // of register pairs that then spill.)  voff_n: the lane's row n of a tile (bytes); + 16 g: its 16-byte piece.
    const unsigned voff_n = (unsigned)(L.n * H * HEAD) * 2;
    auto rs = [](const void* p) { return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, 0x7fffffff, 0x00020000); };
    using Rsrc = decltype(rs(nullptr));
    auto ld16 = [](Rsrc r, unsigned voff) { return __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0)); };
    auto ld8 = [](Rsrc r, unsigned voff) { return __builtin_bit_cast(bf16x4, __builtin_amdgcn_raw_buffer_load_b64(r, voff, 0, 0)); };
    auto rows16 = [&](const __bf16* t, long row0, unsigned voff) {   // load_rows16: lane offset voff = row n, piece g
        TileB x;
        const Rsrc r = rs(t + row0);
#pragma unroll
        for (int pr = 0; pr < NBLK / 2; pr++) {
            const bf16x8 v = ld16(r, voff + 64 * pr);
            x.f[2 * pr] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
            x.f[2 * pr + 1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
        }
        return x;
    };
    auto put16 = [&](__bf16* t, long row0, const TileB& x) {          // store_rows16
        const Rsrc r = rs(t + row0);
#pragma unroll
        for (int pr = 0; pr < NBLK / 2; pr++)
            __builtin_amdgcn_raw_buffer_store_b128(
                __builtin_bit_cast(i32x4, __builtin_shufflevector(x.f[2 * pr], x.f[2 * pr + 1], 0, 1, 2, 3, 4, 5, 6, 7)), r,
                voff_n + 16 * L.g + 64 * pr, 0, 0);
    };
    auto frags4 = [&](const __bf16* p, int ln) {                      // load_frags: four fragments, [i][lane] x 8 B
        TileB x;
        const Rsrc r = rs(p);
#pragma unroll
        for (int i = 0; i < NBLK; i++) x.f[i] = ld8(r, ln * 8 + i * 512);
        return x;
    };
    auto lane16 = [&](const __bf16* p, int ln) {                      // load_lane16: 16 bf16 per lane
        TileB x;
        const Rsrc r = rs(p);
        const bf16x8 lo = ld16(r, ln * 32), hi = ld16(r, ln * 32 + 16);
        x.f[0] = __builtin_shufflevector(lo, lo, 0, 1, 2, 3);
        x.f[1] = __builtin_shufflevector(lo, lo, 4, 5, 6, 7);
        x.f[2] = __builtin_shufflevector(hi, hi, 0, 1, 2, 3);
        x.f[3] = __builtin_shufflevector(hi, hi, 4, 5, 6, 7);
        return x;
    };
    struct In {
        TileB w, q, k, v, a, b, dy, UT, DT;
        TileB s0[LDSP ? 1 : NBLK], ds[LDSP ? 1 : NBLK];   // chunk-start state and arriving dstate, [ib] x fragments jb
    };
    // `live` = false (the round after a wavefront's last chunk) keeps the same instruction stream - a branch
    // around the loads would make every wait conservative - but folds all lanes onto one row / one lane's
    // slot, so the whole fetch touches a few cache lines instead of 47 KiB.
    auto fetch = [&](int c, int item, bool live) {
        const ChunkAddr ca(c, T, H);
        const unsigned vo = (live ? voff_n : 0u) + 16 * L.g;
        const int ln = live ? lane : 0;
        In t;
        t.q = rows16(q_, ca.row0, vo);
        t.a = rows16(a_, ca.row0, vo);
        t.dy = rows16(dy_, ca.row0, vo);
        if constexpr (PAIRED) t.DT = frags4(rec_bwd + SavedPair::ut(pair_of(item), ca.c), ln);   // F(dab_u_ib^T)  lane = value ch
        else t.DT = frags4(rec_bwd + RB::ut(c), ln);
        if constexpr (LDSP) return t;                 // (everything else of a chunk comes through LDS)
        t.w = rows16(w_, ca.row0, vo);
        t.k = rows16(k_, ca.row0, vo);
        t.v = rows16(v_, ca.row0, vo);
        t.b = rows16(b_, ca.row0, vo);
        t.UT = frags4(rec_fwd + RF::ut(c), ln);                                      // F(U_ib^T)      lane = value ch
#pragma unroll
        for (int ib = 0; ib < (LDSP ? 1 : NBLK); ib++) {
            t.s0[ib] = lane16(rec_fwd + RF::ckpt(c, ib), ln);
            t.ds[ib] = lane16(rec_bwd + RB::ckpt(c, ib), ln);
        }
        return t;
    };
    // MODE 3: a wavefront's 36 KiB (see pairlds), private to it: no barrier.  (The dstate a pair's later chunk hands to
    // its earlier one waits there too, not in registers: it would be live through the whole key-channel loop, the
    // kernel's tightest spot.)
    __shared__ __attribute__((aligned(16))) unsigned char lds_all[LDSP ? 4 * pairlds::BYTES : 16];
    unsigned char* const mine = lds_all + wave * (LDSP ? pairlds::BYTES : 0);
    // MODE 3: everything pair `item` (chunks c0 = 2p and c0 + 1) needs through LDS; the wavefront's LDS reads of the
    // pair before are complete when this is called
    const unsigned voff_rows = voff_n + 16 * L.g;   // a lane's 16 bytes of a tile: row n, channels 8g ..
    using pairlds::dma16;
    // (the scheduling barriers make the compiler build one descriptor, issue its loads, and go on to the next: left
    // to itself it builds all twelve first, and with the scalar registers that takes it runs out of them)
    // Order: what the state advance at the head of the pair needs first (the entering state and the tiles of the earlier
    // chunk, 18 loads), then the dstate and the later chunk's tiles (18 loads).
    auto dma_pair = [&](int walk, bool carried) {   // carried: the dstate is already in place (handed on by the pair before)
        const int item = pair_of(walk);
        const int bh = item / NP, p = item - bh * NP;
        const long c0 = (long)bh * NC + 2 * p;
        auto state = [&](int d) {                     // d = 0: the state entering the pair, 1: the dstate arriving at its end
            // (chunk records: the forward state in the record of the pair's even chunk, the dstate in the odd chunk's)
            const Rsrc r = rs((d ? rec_bwd : rec_fwd) + SavedPair::ds(item, 0));
            unsigned char* dst = mine + (d ? pairlds::CARRY : pairlds::STASH);
#pragma unroll
            for (int i = 0; i < 2 * NBLK; i++)        // (ib, half): a state's 8 KiB are [ib][lane] x 32 B
                dma16(r, lane * 32, (i >> 1) * 2048 + (i & 1) * 16, dst + i * 1024);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto tiles = [&](int e) {                     // w, k, b, v and U^T of chunk 2p + e
            const ChunkAddr ca((int)c0 + e, T, H);
            unsigned char* set = mine + pairlds::TILES + e * pairlds::SET;
            const __bf16* const src[4] = {w_, k_, b_, v_};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const Rsrc r = rs(src[t] + ca.row0);
#pragma unroll
                for (int pr = 0; pr < NBLK / 2; pr++) dma16(r, voff_rows, 64 * pr, set + t * 2048 + pr * 1024);
                __builtin_amdgcn_sched_barrier(0);
            }
            const Rsrc ru = rs(rec_fwd + SavedPair::ut(item, 2 * p + e));
#pragma unroll
            for (int i = 0; i < 2; i++) dma16(ru, lane * 16, i * 1024, set + 8192 + i * 1024);
            __builtin_amdgcn_sched_barrier(0);
        };
        state(0);
        tiles(0);
        if (!carried) state(1);
        tiles(1);
    };
    constexpr int DMA_SECOND_HALF = 18;   // loads of a pair that the state advance does not wait for
    int item = run_first_item(id0), cid = first_chunk(item);
    bool first = true;   // MODE 3: the later chunk of a pair, which is handled first
    In nxt = fetch(cid, item, true);
    if constexpr (LDSP) dma_pair(item, false);
    bool started = false;   // MODE 3: whether the wavefront's first pair is in (its loads have nothing to hide behind)
    for (;;) {
    const ChunkAddr ca(cid, T, H);
    const In cur = nxt;
    TileB w, k, v, b, UT;
    const TileB &q = cur.q, &a = cur.a, &dy = cur.dy, &DT = cur.DT;
    TileB s0_[NBLK];   // MODE 3: the state entering this chunk
    if constexpr (LDSP) {
        // The compiler does not wait for global -> LDS loads before LDS reads (it tracks registers), so the wait is
        // explicit.  Memory instructions complete in issue order as far as the counter goes, and every iteration ends
        // with the ten stores of dq, da, dk, db and dw, all issued after its prefetch point: "at most ten outstanding"
        // therefore means that the loads into LDS (and into `cur`) of the iteration before are in, without waiting
        // for those stores.  The wavefront's very first pair has no stores behind it: there the state advance starts as
        // soon as its own half of the loads is in, and the rest is waited for after it.
        if (started) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AFTER_PREFETCH) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DMA_SECOND_HALF) : "memory");
        if (first) {
            // the state entering this chunk from the one entering the pair: (S + V^T kwi + U^T bwi) diag(fw), operands of
            // the pair's earlier chunk (the forward scan's update, there on the fp32 state)
            const unsigned char* set0 = mine + pairlds::TILES;
            const TileB w0 = pairlds::tile(set0, 0, lane), k0 = pairlds::tile(set0, 1, lane), b0 = pairlds::tile(set0, 2, lane);
            const TileB v0 = pairlds::tile(set0, 3, lane), UT0 = pairlds::frags(set0 + 8192, lane);
            TileB VT0;
#pragma unroll
            for (int ib = 0; ib < NBLK; ib++) VT0.f[ib] = transpose(v0.f[ib], eye);
#pragma unroll
            for (int jb = 0; jb < NBLK; jb++) {
                constexpr float LOG2E = 1.4426950408889634f, LOG2_LOG2E = 0.5287663729448977f;
                const f32x4 wf = to_f32(w0.f[jb]), kf0 = to_f32(k0.f[jb]), bf0 = to_f32(b0.f[jb]);
                f32x4 kw, bw, fwv;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float lc2 = row_prefix_sum(-__builtin_amdgcn_exp2f(fmaf(wf[r], LOG2E, LOG2_LOG2E)));
                    const float Pi = __builtin_amdgcn_exp2f(-lc2);
                    fwv[r] = row_bcast_last(__builtin_amdgcn_exp2f(lc2));
                    kw[r] = kf0[r] * Pi;
                    bw[r] = bf0[r] * Pi;
                }
                const bf16x4 kwiT = transpose(to_bf16(kw), eye), bwiT = transpose(to_bf16(bw), eye);
#pragma unroll
                for (int ib = 0; ib < NBLK; ib++) {
                    const bf16x4 old = *reinterpret_cast<const bf16x4*>(mine + pairlds::STASH + (2 * ib + (jb >> 1)) * 1024 + lane * 16 + (jb & 1) * 8);
                    s0_[ib].f[jb] = to_bf16(mma2(to_f32(old), kwiT, bwiT, VT0.f[ib], UT0.f[ib]) * fwv);
                }
            }
        } else {
#pragma unroll
            for (int ib = 0; ib < NBLK; ib++) s0_[ib] = pairlds::state(mine + pairlds::STASH, ib, lane);
        }
        __builtin_amdgcn_sched_barrier(0);   // (the advance has the registers to itself; nothing of the chunk proper starts before it is done)
        if (!started) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            started = true;
        }
        const unsigned char* set = mine + pairlds::TILES + (ca.c & 1) * pairlds::SET;
        w = pairlds::tile(set, 0, lane);
        k = pairlds::tile(set, 1, lane);
        b = pairlds::tile(set, 2, lane);
        v = pairlds::tile(set, 3, lane);
        UT = pairlds::frags(set + 8192, lane);
    } else {
        w = cur.w;
        k = cur.k;
        v = cur.v;
        b = cur.b;
        UT = cur.UT;
    }

    const Decay d = chunk_decay(w);
    const TileB wq = to_bf16(mul(q, d.P));
    const TileB wa = to_bf16(mul(a, d.Px));
    const TileF kwi_f = mul(k, d.Pi);
    const TileB kwi = to_bf16(kwi_f);
    const TileB bwi = to_bf16(mul(b, d.Pi));
    const TileB kf = to_bf16(mul(kwi_f, d.fw));

    // token-major ("row") copies of U and dab_u, value-major copy of dY
    TileB Ur, Dr, dYT;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        Ur.f[ib] = transpose(UT.f[ib], eye);    // F(U_ib)       lane = token
        Dr.f[ib] = transpose(DT.f[ib], eye);    // F(dab_u_ib)   lane = token
        dYT.f[ib] = transpose(dy.f[ib], eye);   // F(dY_ib^T)    lane = value ch
    }

    // 16x16 products over the value channels, each in both orientations
    const bf16x4 dab = to_bf16(mask_lower_strict(tile_xyT(Dr, Ur), L));   // [t][s] = dab_u_t . U_s,  s <  t
    const bf16x4 dabT = to_bf16(mask_upper_strict(tile_xyT(Ur, Dr), L));  // [s][t]
    const bf16x4 dak = to_bf16(mask_lower_strict(tile_xyT(Dr, v), L));    // [t][s] = dab_u_t . v_s
    const bf16x4 dakT = to_bf16(mask_upper_strict(tile_xyT(v, Dr), L));
    const bf16x4 dqb = to_bf16(mask_lower_incl(tile_xyT(dy, Ur), L));     // [t][s] = dY_t . U_s,     s <= t
    const bf16x4 dqbT = to_bf16(mask_upper_incl(tile_xyT(Ur, dy), L));
    const bf16x4 dqk = to_bf16(mask_lower_incl(tile_xyT(dy, v), L));      // [t][s] = dY_t . v_s
    const bf16x4 dqkT = to_bf16(mask_upper_incl(tile_xyT(v, dy), L));
    // 16x16 products over the key channels (transposed orientation, rows = the token being written)
    const bf16x4 QKT = to_bf16(mask_upper_incl(tile_xyT(kwi, wq), L));    // [t][s] = kwi_t . wq_s,   s >= t
    const bf16x4 AKT = to_bf16(mask_upper_strict(tile_xyT(kwi, wa), L));  // [t][s] = kwi_t . wa_s,   s >  t

    // dS in both orientations, S0 transposed; sum_i S0*dS on the fly
    bf16x4 dS[NBLK][NBLK], dST[NBLK][NBLK], S0T[NBLK][NBLK];   // [ib][jb], [jb][ib], [jb][ib]
    f32x4 sds[NBLK];                                           // per key block: partial sum over value rows
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) sds[jb] = zero4();
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        TileB s0, ds;
        if constexpr (LDSP) {
            s0 = s0_[ib];
            ds = pairlds::state(mine + pairlds::CARRY, ib, lane);
        } else {
            s0 = cur.s0[ib];
            ds = cur.ds[ib];
        }
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            if constexpr (!LDSP) dS[ib][jb] = ds.f[jb];
            sds[jb] += to_f32(s0.f[jb]) * to_f32(ds.f[jb]);
            if constexpr (!LDSP) {
                S0T[jb][ib] = transpose(s0.f[jb], eye);
                dST[jb][ib] = transpose(ds.f[jb], eye);
            }
        }
    }
    if constexpr (LDSP) {
        // The transposed fragments of a state that lies in LDS come out of it transposed (no matrix instruction, no
        // rounding step): always the dstate, and the forward state where it is the one that arrived from memory (the
        // pair's earlier chunk; the later chunk's state was advanced in registers above).
        const int tr_off = pairlds::tr_lane_offset(L);
#pragma unroll
        for (int ib = 0; ib < NBLK; ib++)
#pragma unroll
            for (int jb = 0; jb < NBLK; jb++) dST[jb][ib] = pairlds::state_t(mine + pairlds::CARRY, ib, jb, tr_off);
        if (first) {
#pragma unroll
            for (int ib = 0; ib < NBLK; ib++)
#pragma unroll
                for (int jb = 0; jb < NBLK; jb++) S0T[jb][ib] = transpose(s0_[ib].f[jb], eye);
        } else {
#pragma unroll
            for (int ib = 0; ib < NBLK; ib++)
#pragma unroll
                for (int jb = 0; jb < NBLK; jb++) S0T[jb][ib] = pairlds::state_t(mine + pairlds::STASH, ib, jb, tr_off);
        }
    }

    // next chunk's tiles and states: they have the rest of this chunk's arithmetic to arrive
    int nitem = item, ncid = cid - 1;
    bool nfirst = false;
    if (!PAIRED || !first) {   // (the earlier chunk of a pair follows its later one directly)
        nitem = next_item(item);
        nfirst = true;
        ncid = nitem < nitems ? first_chunk(nitem) : cid;
    }
    const bool more = nitem < nitems;
    // whether this chunk hands its dstate on: a pair's later chunk to its earlier one, and a pair's earlier chunk to the
    // pair before it in the run (same (batch, head))
    const bool hand_on = PAIRED && (first || (MODE == 3 && more && nitem == item - 1 && item % NP != 0));
    nxt = fetch(ncid, more ? nitem : item, more);

    // dv = QK^T dY + kf dS^T + AK^T dab_u          (rows = tokens)
    TileB out;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        f32x4 acc = mma2(zero4(), dYT.f[ib], DT.f[ib], QKT, AKT);
        // (MODE 3: the dstate is read where it is used, here and below, out of the wavefront's LDS instead of being held
        // in 32 registers from the top)
        TileB dsi;
        if constexpr (LDSP) dsi = pairlds::state(mine + pairlds::CARRY, ib, lane);
        else for (int jb = 0; jb < NBLK; jb++) dsi.f[jb] = dS[ib][jb];
        acc = mma2(acc, dsi.f[0], dsi.f[1], kf.f[0], kf.f[1]);
        acc = mma2(acc, dsi.f[2], dsi.f[3], kf.f[2], kf.f[3]);
        if constexpr (LN) acc += to_f32(ld8(rs(dv_ + ca.row0), voff_n + 2 * chan16(ib, 4 * L.g)));
        out.f[ib] = to_bf16(acc);
    }
    put16(dv_, ca.row0, out);
    if constexpr (LDSP) {
        // After a pair's second chunk the next pair sets out.  Not before this point: the loop above was the last reader
        // of this pair's dstate in LDS (all LDS reads so far are waited for here).
        if (nfirst && more) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            dma_pair(nitem, hand_on);
        }
    }
    if constexpr (PAIRED) {
        // the dstate for the pair's earlier chunk, dS diag(fw) + dY^T wq + dab_u^T wa, here rather than in the loop below
        // (which makes the same transposes again) so that dS is dead before that loop starts
        if (hand_on) {   // (else the next pair's dstate is on its way into this buffer)
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            const bf16x4 waT = transpose(wa.f[jb], eye), wqT = transpose(wq.f[jb], eye);
#pragma unroll
            for (int ib = 0; ib < NBLK; ib++) {
                bf16x4* slot = reinterpret_cast<bf16x4*>(mine + pairlds::CARRY + (2 * ib + (jb >> 1)) * 1024 + lane * 16 + (jb & 1) * 8);
                *slot = to_bf16(mma2(to_f32(*slot) * d.fw.f[jb], wqT, waT, dYT.f[ib], DT.f[ib]));   // (in place)
            }
        }
        }
    }

    float ddot = 0.f;
    if constexpr (LN) ddot = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs(ln_ddot + (long)cid * CHUNK), 4 * L.n, 0, 0));

    // key-channel gradients, one block of 16 key channels at a time
    TileB o_dq, o_da, o_dk, o_db, o_dw;
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) {
        // attn_ln: k and q of this key block re-read here, four channels per lane out of the cache (held from the top
        // they are sixteen more live registers through this loop, which then spills), with the head's bonus vector
        // ([2][H*64] of the parameters); requested first, used last
        bf16x4 k_re = {}, q_re = {};
        f32x4 bonus = zero4();
        if constexpr (LN) {
            const unsigned piece = voff_n + 2 * chan16(jb, 4 * L.g);
            k_re = ld8(rs(k_ + ca.row0), piece);
            q_re = ld8(rs(q_ + ca.row0), piece);
            bonus = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                rs(ln_params + 2L * H * HEAD + (long)(ca.bh % H) * HEAD), 4 * chan16(jb, 4 * L.g), 0, 0));
        }
        const bf16x4 bwiT = transpose(bwi.f[jb], eye), kwiT = transpose(kwi.f[jb], eye);
        const bf16x4 waT = transpose(wa.f[jb], eye), wqT = transpose(wq.f[jb], eye);
        // brackets (rows = tokens, columns = key channels of this block)
        f32x4 Bq = mma2(zero4(), bwiT, kwiT, dqb, dqk);
        f32x4 Ba = mma2(zero4(), bwiT, kwiT, dab, dak);
        f32x4 Bb = mma2(zero4(), waT, wqT, dabT, dqbT);
        f32x4 Bk = mma2(zero4(), waT, wqT, dakT, dqkT);
        f32x4 UdS = zero4(), VdS = zero4();
        Bq = mma2(Bq, S0T[jb][0], S0T[jb][1], dy.f[0], dy.f[1]);
        Bq = mma2(Bq, S0T[jb][2], S0T[jb][3], dy.f[2], dy.f[3]);
        Ba = mma2(Ba, S0T[jb][0], S0T[jb][1], Dr.f[0], Dr.f[1]);
        Ba = mma2(Ba, S0T[jb][2], S0T[jb][3], Dr.f[2], Dr.f[3]);
        UdS = mma2(UdS, dST[jb][0], dST[jb][1], Ur.f[0], Ur.f[1]);
        UdS = mma2(UdS, dST[jb][2], dST[jb][3], Ur.f[2], Ur.f[3]);
        VdS = mma2(VdS, dST[jb][0], dST[jb][1], v.f[0], v.f[1]);
        VdS = mma2(VdS, dST[jb][2], dST[jb][3], v.f[2], v.f[3]);

        const f32x4 wqf = to_f32(wq.f[jb]), waf = to_f32(wa.f[jb]), kwif = to_f32(kwi.f[jb]), bwif = to_f32(bwi.f[jb]);
        f32x4 dq, da, dk, db, dw;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float fw = d.fw.f[jb][r];
            const float fwU = fw * UdS[r], fwV = fw * VdS[r];
            const float bb = Bb[r] + fwU, bk = Bk[r] + fwV;
            dq[r] = d.P.f[jb][r] * Bq[r];
            da[r] = d.Px.f[jb][r] * Ba[r];
            const float pi = d.Pi.f[jb][r];
            db[r] = pi * bb;
            dk[r] = pi * bk;
            // decay gradient
            const float g_incl = wqf[r] * Bq[r] - kwif[r] * bk - bwif[r] * bb;
            const float g_strict = waf[r] * Ba[r];
            // (fw is the same in every lane of a row, so the two sums over the row are one; likewise the two suffix sums)
            const float tail = row_sum(kwif[r] * fwV + bwif[r] * fwU + fw * sds[jb][r]);
            const float dlogw = row_suffix_sum(g_incl + g_strict) - g_strict + tail;
            dw[r] = dlogw * d.lw.f[jb][r];
        }
        if constexpr (LN) {
            dq += to_f32(k_re) * bonus * ddot;
            dk += to_f32(q_re) * bonus * ddot;
        }
        o_dq.f[jb] = to_bf16(dq);
        o_da.f[jb] = to_bf16(da);
        o_dk.f[jb] = to_bf16(dk);
        o_db.f[jb] = to_bf16(db);
        o_dw.f[jb] = to_bf16(dw);
    }
    put16(dq_, ca.row0, o_dq);
    put16(da_, ca.row0, o_da);
    put16(dk_, ca.row0, o_dk);
    put16(db_, ca.row0, o_db);
    put16(dw_, ca.row0, o_dw);
    if (!more) break;
    item = nitem;
    cid = ncid;
    first = nfirst;
    }   // chunk loop
}

// ------------------------------------------------------------------------------------------------
// The reduction of attn_ln's parameter-gradient partials as a launch of its own (dparams_reduce_block): one block per
// (head, parameter).  Where the reverse scan leaves compute units idle, its launch carries these blocks instead.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void dparams_reduce_kernel(int B, int H, int NC, const float* __restrict__ part,
                                                              float* __restrict__ dparams) {
    __shared__ float red[16 * HEAD];
    dparams_reduce_block(B, H, NC, part, dparams, blockIdx.x, blockIdx.y, red, 16);
}

// ------------------------------------------------------------------------------------------------
// host launchers
// ------------------------------------------------------------------------------------------------
void launch_ln_epilogue_bwd(int B, int T, int H, const void* q, const void* dy, const LnBackwardBuffers& ln,
                            hipStream_t stream) {
    const int nchunks = B * H * (T / CHUNK);
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    auto m = [](void* p) { return static_cast<__bf16*>(p); };
    const LnBwdArgs args{c(ln.k), c(ln.v), c(ln.g), c(ln.y_wkv), ln.centers, static_cast<const float*>(ln.params),
                         m(ln.dg), m(ln.dY), m(ln.dv), ln.ddot, ln.dparams_part};
    hipLaunchKernelGGL(ln_epilogue_bwd_kernel, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(q), c(dy),
                       args);
}

void launch_bwd_grads(int B, int T, int H, const void* w, const void* q, const void* k, const void* v, const void* a,
                      const void* b, const void* dy, const void* rec_fwd, const void* rec_bwd,
                      void* dw, void* dq, void* dk, void* dv, void* da, void* db, int fused, hipStream_t stream,
                      const float* ln_params, const float* ln_ddot) {
    const int nchunks = B * H * (T / CHUNK);
    const int ds_run = fused == 3 ? dstate_run(B, T, H) : 1;
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    auto m = [](void* p) { return static_cast<__bf16*>(p); };
    // one block (four wavefronts, one per SIMD) per compute unit; fewer if there is less work
    const int num_cu = compute_units();
    const int NP = SavedPair::pairs(T / CHUNK), run = ds_run < 0 ? -ds_run : ds_run;
    // what a wavefront takes at a time: a run of pairs (cut per (batch, head) or from the flattened pairs), or a chunk
    const int items = fused != 3 ? nchunks : ds_run < 0 ? B * H * ((NP + run - 1) / run) : (B * H * NP + run - 1) / run;
    const int blocks = (items + 3) / 4 < num_cu ? (items + 3) / 4 : num_cu;
    auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, stream, T, H, nchunks, c(w), c(q), c(k), c(v), c(a), c(b),
                           c(dy), c(rec_fwd), c(rec_bwd), m(dw), m(dq), m(dk), m(dv), m(da), m(db), ln_params, ln_ddot, ds_run);
    };
    if (fused == 3) {
        if (ln_params) go(bwd_grads_kernel<true, 3>);
        else go(bwd_grads_kernel<false, 3>);
    } else {
        if (ln_params) go(bwd_grads_kernel<true, 1>);
        else go(bwd_grads_kernel<false, 1>);
    }
}

int dstate_run(int B, int T, int H) {
    const long NP = SavedPair::pairs(T / CHUNK), BH = (long)B * H, waves = 4L * compute_units();
    const bool head_major = H >= 16;
    // pairs the busiest wavefront handles with runs of r: the longest runs it gets, one after the other
    auto busiest = [&](long r) {
        const long nruns = head_major ? BH * ((NP + r - 1) / r) : (BH * NP + r - 1) / r;
        return (nruns + waves - 1) / waves * r;
    };
    // the longest run that costs the busiest wavefront at most 15 % over the best choice: longer runs keep fewer dstates,
    // and where the kernel is bound by its traffic the wavefronts that finish early leave the memory to the others
    const long best = busiest(1) < busiest(3) ? (busiest(1) < busiest(6) ? busiest(1) : busiest(6))
                                              : (busiest(3) < busiest(6) ? busiest(3) : busiest(6));
    int run = 1;
    for (int r : {3, 6})
        if (busiest(r) * 100 <= best * 115) run = r;
    return head_major ? -run : run;
}

void launch_dparams_reduce(int B, int T, int H, const float* part, float* dparams, hipStream_t stream) {
    hipLaunchKernelGGL(dparams_reduce_kernel, dim3(H, 3), dim3(1024), 0, stream, B, H, T / CHUNK, part, dparams);
}

}  // namespace wkv
