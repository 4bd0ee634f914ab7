// WKV7 for gfx950: chunk preparation and the sequential state scan in ONE kernel, handing the per-chunk operands
// from producer wavefronts to the chain wavefronts through LDS instead of through memory.
//
// Replaces forward_kernel / the first half of backward_kernel of the reference (attn.cu:11-106, 131-326;
// mathematics rwkv7_attn_triton.py:27-69, 72-156).  The reference runs one block of four warps per (batch, head),
// every warp taking part in every product of a chunk (~60 block barriers per chunk).  Here a block per (batch, head)
// has two kinds of wavefronts:
//   * FUSE_P producer wavefronts.  Each takes every FUSE_P-th chunk and does ALL the state-independent algebra of it
//     alone (decays, the 16x16 products, the triangular inverse, U0 = Tinv AK V, Wm = Tinv wa, transposes), reading
//     the caller's tensors and writing the chunk's operands into a slot of an LDS ring.
//   * four chain wavefronts, each owning 16 value rows of the 64x64 fp32 state in its accumulators.  Per chunk:
//         U^T = U0^T + S Wm^T ;   S <- (S + V^T kwi + U^T bwi) diag(fw) ;   forward also Y = QK V + QB U + wq S^T
//     (kwi = k / P_t, bwi = b / P_t, fw = P_K the chunk's whole decay: S diag(fw) + V^T kf + U^T bf with the
//     decay applied once to the sum)
//     They read their operands from the ring and leave the checkpoint (the state entering the chunk, bf16), U^T and
//     y in a second LDS ring; they touch memory neither way.
//   * one store wavefront that copies what the chain left two steps ago to memory.  A store issued behind a
//     producer's eleven tile loads waits in the compute unit's memory pipeline until they are through, and on a chain
//     wavefront that wait is on the critical path of the step (measured at B=8, H=12 with the chain's stores taken out:
//     T=4096 forward 194 -> 144 us; with inputs that the last-level cache does not hold, T=1024 56 -> 46 us); the
//     store wavefront has the whole step to get its handful of stores accepted.
// All wavefronts run in lock step, one block barrier per chunk: a producer's work on a chunk is cut into FUSE_P
// segments with a barrier after each, producer p starts p steps late, so exactly one chunk is completed per step and
// the chain consumes it two steps later.  No flags, no polling: every wavefront executes the same number of barriers.
// Nothing of the operands (13.25 KiB per chunk forward, 10.25 KiB backward) touches memory.
//
// The backward direction runs the same chain in reverse over dS with its own producers:
//   producers:  D0 = Tinv^T (QB^T dY),  Bm = Tinv^T bf        chain:  dab_u = D0 + Bm dS^T ;
//                                                                     dS' = dS diag(fw) + dY^T wq + dab_u^T wa
// and leaves the dstate arriving at each chunk's end plus dab_u^T for bwd_grads_kernel.
#include "device_info.hpp"
#include "ln_epilogue.hpp"
#include "wkv7_common.hpp"
#include "wkv7_kernels.hpp"

namespace wkv {

// A producer's work on a chunk has twelve possible cut points (see the SEG() marks in the kernel); bit k of CUTS says
// whether mark k carries a step barrier.  Their number is the number of producer wavefronts: a chunk takes a producer
// that many steps, and one chunk must be completed per step.  Twelve producers (0xfff), one segment each, are not the
// fastest: a block's wavefronts go to the four SIMDs round robin, and what counts is how many share a SIMD with a
// chain wavefront, whose round is the critical path of a step.
// Ten, for two blocks per head (2 chain wavefronts; 14 wavefronts would put a chain wavefront and three producers on
// two of the SIMDs): the triangular products with the start of the inverse, U0 with Wm.  Measured at B=8, T=1024, H=12
// against twelve: forward 49.4 -> 48.0 us, reverse scan 44.4 -> 42.8 us; nine and eight are no better than ten.
constexpr int CUTS_TEN = 0xeef;
// Eight, for one block per head (a chain wavefront and two producers per SIMD; with attn_ln's epilogue wavefronts
// there is room for no more anyway): the decay blocks one each, products + start of the inverse, the rest of the
// inverse, U0 + Wm + first stores, second stores.  Measured against twelve at H=12, T=1024: B=16 254 -> 251 us per
// step, B=64 851 -> 840 us; attn_ln at B=64 against eight cut as "decay blocks in pairs, the inverse in two parts"
// (0xeda): 1260 -> 1252 us.
constexpr int CUTS_EIGHT_EVEN = 0xcaf;
constexpr int fused_producers(int cuts) { return __builtin_popcount(cuts); }
// attn_ln adds three wavefronts that take turns applying the epilogue (GroupNorm, bonus, gate) to the chunk the chain
// finished a step ago: one step of work, two idle steps in which the tiles of the wavefront's next chunk arrive
// (measured: one such wavefront, with a step between request and use, 122 us at B8 T1024 H12 against 86 us; the work
// cut in two steps over four wavefronts 109 us - the statistics held across the barrier spill)
constexpr int LN_WAVES = 3;
// VS: blocks per (batch, head), each owning 4 / VS of the four value blocks (16 value rows each) of the state
// (MAP: two sets of chain wavefronts and nothing to store)
constexpr int fused_threads(int cuts, bool ln, int vs = 1, bool map = false) {
    return ((map ? 2 : 1) * (4 / vs) + fused_producers(cuts) + (ln ? LN_WAVES : 0) + (map ? 0 : 1)) * 64;
}
constexpr int FUSE_SLOTS = 4;                   // ring slots; a producer stores in its last two segments only
// slot layout (bytes): six fragment pairs of the chain, the chunk decay, the four private (U0^T, V^T) pairs, and
// forward only the three pairs of the output (wq as two pairs, then (QK, QB))
constexpr int SL_J = 0, SL_FW = 6 * 1024, SL_I = SL_FW + 256, SL_Y = SL_I + 4 * 1024;
constexpr int SLOT_FWD = SL_Y + 3 * 1024, SLOT_BWD = SL_Y;
// The chain's results on their way to memory: per chain wavefront the kept state (2 KiB), U^T (512 B), y (512 B) and
// the output's centres (64 B), each laid out as its place in memory so that the store wavefront copies 16 bytes per
// lane.  Chunk st sits in slot st % OUT_SLOTS; the store wavefront takes it two steps after the chain's round, which
// is when the chain's LDS writes are known to have landed without the chain ever waiting for them (its next round
// waits for operands it requested after them, and a wavefront's LDS accesses complete in order).
constexpr int OUT_SLOTS = 4;
constexpr int out_ck(int) { return 0; }
constexpr int out_ut(int nch) { return nch * 2048; }
constexpr int out_y(int nch) { return out_ut(nch) + nch * 512; }
constexpr int out_cen(int nch) { return out_y(nch) + nch * 512; }
constexpr int out_slot(int nch) { return out_cen(nch) + nch * 64; }

struct FusedArgs {
    int T, H, NC, BH;
    int s_in_f32, s_out_f32;
    const __bf16 *w, *q, *k, *v, *a, *b, *dy;   // forward: w q k v a b; backward: w q a b dy
    __bf16* saved;                              // forward: per chunk checkpoint + U^T (Saved); backward: SavedPair
    const void* s_in;
    void* s_out;
    __bf16* y;                                  // forward only
    // attn_ln forward: gate, parameters [3][H*64] and where the plain WKV7 output is kept for the backward pass
    const __bf16* g;
    const float* params;
    __bf16* y_wkv;
    // attn_ln: where the per-block centres of the kept WKV7 output go (see Centred in ln_epilogue.hpp).  Also set for the
    // plain forward when its y is that kept output (the epilogue then runs as a kernel of its own): y is written centred.
    float* centers;
    int paired;                                 // a state per pair of chunks (SavedPair) or per chunk (Saved)
    // attn_ln backward, optional: the last 3 H blocks of the grid reduce the parameter-gradient partials that the
    // backward epilogue left (dparams_reduce_block) on compute units the scan does not fill
    const float* dparams_part;
    float* dparams;
    int B;
    int ds_run;                                 // backward, paired: see SavedPair::ds_kept
    // Long sequences on few heads: a (batch, head)'s NC chunks as NSEG segments of LS, a block each.  The MAP form of
    // the kernel leaves every segment's affine map (S_out = S_in M + N) in `maps`, segment_carry_kernel composes them
    // into the state entering each segment, and the kernel proper starts each segment from its entry of s_in
    // ([B*H*NSEG][64][64] fp32 then).  NSEG = 1, LS = NC: the whole sequence in one block.
    int NSEG, LS;
    float* maps;                                // MAP: [B*H*NSEG][2][64][64], N in fragment order and M transposed
};

#define STEP_BARRIER() step_barrier()
#define SEG(k) do { if constexpr ((CUTS >> (k)) & 1) STEP_BARRIER(); } while (0)
// (the scheduling barriers keep each segment's arithmetic inside its step: the compiler would otherwise move it
// freely across the barrier, which only orders LDS traffic, and unbalance the steps)
__device__ __forceinline__ void step_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    __builtin_amdgcn_sched_barrier(0);
}

// The barrier of a wavefront that only READS the ring: it has nothing to publish, so it does not wait for its own
// outstanding LDS reads (the operands of its next round); they arrive during the barrier and the round's first
// instructions, and each is waited for where it is used.  (A fence would make the compiler wait for all of them
// here; the memory clobber keeps every access on its side of the barrier.)
__device__ __forceinline__ void reader_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void lds_pair(unsigned char* p, int lane, bf16x4 u, bf16x4 v) {
    *reinterpret_cast<bf16x8*>(p + lane * 16) = __builtin_shufflevector(u, v, 0, 1, 2, 3, 4, 5, 6, 7);
}

template <bool FWD, bool SAVE, bool LN, int CUTS, int VS = 1, bool MAP = false>
__global__ __launch_bounds__(fused_threads(CUTS, LN, VS, MAP)) void wkv7_fused_kernel(const FusedArgs A) {
    static_assert(!MAP || (!SAVE && !LN), "the map pass keeps and writes nothing but the maps");
    static_assert((CUTS >> 10 & 3) == 3, "the two storing segments are separate steps (ring slots are sized for that)");
    static_assert(!LN || FWD, "the epilogue belongs to the forward direction");
    static_assert(VS == 1 || (VS == 2 && !LN), "the epilogue needs the whole head in one block");
    constexpr int NCH = 4 / VS;                 // value blocks of this block = chain wavefronts of a set
    constexpr int NCW = (MAP ? 2 : 1) * NCH;    // chain wavefronts: MAP runs a second set on the homogeneous recurrence
    constexpr int SLOT = FWD ? SLOT_FWD : SLOT_BWD;
    constexpr int P = fused_producers(CUTS);
    constexpr int YRING = FUSE_SLOTS * SLOT;    // attn_ln: two slots of 4 KiB, the chain's fp32 output of one chunk each
    constexpr int ORING = YRING + (LN ? 2 * 4096 : 0), OSLOT = out_slot(NCH);
    __shared__ __attribute__((aligned(16))) unsigned char ring[ORING + OUT_SLOTS * OSLOT];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Two blocks per head: blocks i and i + 8 are the two halves of one head, so that (blocks going to the eight XCDs
    // round robin) both read the head's key-side tensors through the same L2; ids past the last head do nothing.
    if constexpr (!FWD) {
        const int extra = A.dparams != nullptr ? 3 * A.H : 0, scan_blocks = (int)gridDim.x - extra;
        if ((int)blockIdx.x >= scan_blocks) {   // (the whole block, before any step barrier)
            const int e = (int)blockIdx.x - scan_blocks;
            dparams_reduce_block(A.B, A.H, A.NC, A.dparams_part, A.dparams, e % A.H, e / A.H, reinterpret_cast<float*>(ring),
                                 (int)blockDim.x / 64);
            return;
        }
    }
    const int unit = VS == 1 ? (int)blockIdx.x : 8 * (int)(blockIdx.x >> 4) + (int)(blockIdx.x & 7);   // (batch, head, segment)
    const int vb0 = VS == 1 ? 0 : (int)((blockIdx.x >> 3) & 1) * NCH;    // first value block of this block
    if (VS == 2 && unit >= A.BH * A.NSEG) return;   // (the whole block, before any barrier)
    // (the attn_ln form is never segmented: its launches are for many heads)
    const int bh = LN ? unit : unit / A.NSEG, seg = LN ? 0 : unit - bh * A.NSEG;
    const int NC = A.NC;            // chunks of the sequence: what the kept arrays are indexed with
    const int LS = A.LS;            // chunks this block walks
    const int STEPS = LS + P + 2;   // barriers every wavefront executes
    const Lane L;
    // processing order: forward walks the chunks up, backward down; segments are numbered in that order too
    auto chunk_of = [&](int st) -> int { return FWD ? seg * LS + st : NC - 1 - (seg * LS + st); };

    // Buffer loads: a tile is addressed as (descriptor of the tensor's rows of this (batch, head), wave-uniform chunk
    // offset, one 32-bit byte offset per lane that never changes), so no 64-bit address lives in vector registers;
    // reads past the head's last row would return zero instead of faulting.
    const int voff = (L.n * A.H * HEAD + 8 * L.g) * 2;
    const long head0 = ((long)(bh / A.H) * A.T * A.H + (bh % A.H)) * HEAD;                // elements
    const unsigned extent = (unsigned)((((long)A.T - 1) * A.H * HEAD + HEAD) * 2);      // bytes from head0
    // (a descriptor of zero extent for the fetch after a producer's last chunk: same instructions, no memory access)
    auto rsrc = [&](const __bf16* base, unsigned bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<__bf16*>(base + head0), 0, bytes, 0x00020000);
    };
    using Rsrc = decltype(rsrc(A.w, 0u));
    auto tile = [&](Rsrc r, int soff) {
        TileB t;
#pragma unroll
        for (int pr = 0; pr < NBLK / 2; pr++) {
            const bf16x8 v = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(r, voff + 64 * pr, soff, 0));
            t.f[2 * pr] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
            t.f[2 * pr + 1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
        }
        return t;
    };

    // the value-side tile (v, backward dY): this block's NCH value blocks only, as blocks 0 .. NCH-1
    auto tile_v = [&](Rsrc r, int soff) {
        TileB t;
#pragma unroll
        for (int pr = 0; pr < NCH / 2; pr++) {
            const bf16x8 v = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(r, voff + 64 * (vb0 / 2 + pr), soff, 0));
            t.f[2 * pr] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
            t.f[2 * pr + 1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
        }
        return t;
    };

    if constexpr (LN) {
        if (wave >= NCW + P && wave < NCW + P + LN_WAVES) {
            // ------------------------------------------------------------------------------------------------
            // epilogue wavefront e (attn_ln, attn_ln.cu:11-37): chunks e, e + 3, ...; chunk st in step st + P + 2, one
            // step after the chain left its fp32 output in the y ring (the statistics are taken on the fp32 values).
            // The tiles of its next chunk are requested when a chunk is done and have two idle steps to arrive.
            // ------------------------------------------------------------------------------------------------
            const int e = wave - (NCW + P);
            struct Ep {
                TileB q, k, v, g;
            };
            auto fetch_ep = [&](int st) {
                const unsigned bytes = st < LS ? extent : 0u;
                const int soff = st < LS ? chunk_of(st) * (CHUNK * HEAD * 2) * A.H : 0;
                Ep t;
                t.q = tile(rsrc(A.q, bytes), soff);
                t.k = tile(rsrc(A.k, bytes), soff);
                t.v = tile(rsrc(A.v, bytes), soff);
                t.g = tile(rsrc(A.g, bytes), soff);
                return t;
            };
            const LnParams prm = load_ln_params(A.params, bh % A.H, A.H, L);
            const long ld = (long)A.H * HEAD;
            Ep cur = fetch_ep(e);
            int done = 0;
            for (; done < P + 2 + e && done < STEPS; done++) STEP_BARRIER();
            for (int st = e; st < LS; st += LN_WAVES) {
                const unsigned char* ys = ring + YRING + (st & 1) * 4096;
                TileF yf;
#pragma unroll
                for (int i = 0; i < NBLK; i++) yf.f[i] = *reinterpret_cast<const f32x4*>(ys + i * 1024 + lane * 16);
                const long row0 = head0 + (long)chunk_of(st) * CHUNK * ld;
                if constexpr (SAVE) {
                    Centred kept;
                    store_rows16(A.y + row0, ld, L, ln_forward(yf, cur.q, cur.k, cur.v, cur.g, prm, &kept));
                    store_rows16(A.y_wkv + row0, ld, L, kept.y);
                    if (L.g == 0) *reinterpret_cast<f32x4*>(A.centers + 4 * (((long)(bh / A.H) * A.T + chunk_of(st) * CHUNK + L.n) * A.H + bh % A.H)) = kept.c;
                } else {
                    store_rows16(A.y + row0, ld, L, ln_forward(yf, cur.q, cur.k, cur.v, cur.g, prm));
                }
                cur = fetch_ep(st + LN_WAVES);
#pragma unroll
                for (int i = 0; i < LN_WAVES; i++) {
                    if (done < STEPS) {
                        STEP_BARRIER();
                        done++;
                    }
                }
            }
            for (; done < STEPS; done++) STEP_BARRIER();
            return;
        }
    }
    if (wave >= NCW && wave < NCW + P) {
        // ------------------------------------------------------------------------------------------------
        // producer p: chunks p, p + P, ... in processing order; segment k of chunk st runs in step st + k
        // ------------------------------------------------------------------------------------------------
        const int p = wave - NCW;
        struct In {
            TileB w, q, k, v, a, b;   // backward: v holds dy, k unused
        };
        auto fetch = [&](int st) {
            const unsigned bytes = st < LS ? extent : 0u;
            const int soff = st < LS ? chunk_of(st) * (CHUNK * HEAD * 2) * A.H : 0;
            In t;
            t.w = tile(rsrc(A.w, bytes), soff);
            t.q = tile(rsrc(A.q, bytes), soff);
            t.a = tile(rsrc(A.a, bytes), soff);
            t.b = tile(rsrc(A.b, bytes), soff);
            t.v = tile_v(rsrc(FWD ? A.v : A.dy, bytes), soff);
            if constexpr (FWD) t.k = tile(rsrc(A.k, bytes), soff);
            else t.k = t.v;
            return t;
        };
        In nxt = fetch(p);
        int done = 0;
        for (; done < p; done++) STEP_BARRIER();
        for (int st = p; st < LS; st += P) {
            unsigned char* slot = ring + (st % FUSE_SLOTS) * SLOT;
            const In cur = nxt;
            const bf16x4 eye = identity_bf16(L);
            // ---- segments 0, 1: decay factors and the scaled operands, two blocks of 16 key channels each ----
            // (see chunk_decay in wkv7_common.hpp for the factors; kept per block here so that only the bf16 operands
            // live on across the step barriers)
            TileB wq, wa, bwi, bf, kwi;   // (bf backward only, kwi forward only)
            float fw1 = 0.f;   // the chunk decay is the same in all 16 token lanes: lane n keeps entry n of its group's 16
#pragma unroll
            for (int i = 0; i < NBLK; i++) {
                constexpr float LOG2E = 1.4426950408889634f, LOG2_LOG2E = 0.5287663729448977f;
                const f32x4 wf = to_f32(cur.w.f[i]);
                const f32x4 qf = to_f32(cur.q.f[i]), af = to_f32(cur.a.f[i]), bfl = to_f32(cur.b.f[i]);
                f32x4 kfl;
                if constexpr (FWD) kfl = to_f32(cur.k.f[i]);
                float wq_[4], wa_[4], bwi_[4], bf_[4], kwi_[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    // exp(w) log2(e) as one exponential: 2^(w log2(e) + log2(log2(e))); the prefix sum is then the base-2 log decay
                    const float lc2 = row_prefix_sum(-__builtin_amdgcn_exp2f(fmaf(wf[r], LOG2E, LOG2_LOG2E)));
                    const float P = __builtin_amdgcn_exp2f(lc2);        // decay from the chunk start through token n
                    const float Pi = __builtin_amdgcn_exp2f(-lc2);
                    const float Px = __builtin_bit_cast(                // ... up to but excluding token n
                        float, __builtin_amdgcn_update_dpp(0x3f800000, __builtin_bit_cast(int, P), 0x111, 0xf, 0xf, false));
                    const float fw = row_bcast_last(P);                  // the whole chunk's decay
                    fw1 = (L.n == 4 * i + r) ? fw : fw1;
                    wq_[r] = qf[r] * P;                                 // q * P_t
                    wa_[r] = af[r] * Px;                                // a * P_{t-1}
                    bwi_[r] = bfl[r] * Pi;                              // b / P_t
                    if constexpr (FWD) kwi_[r] = kfl[r] * Pi;
                    else bf_[r] = bwi_[r] * fw;                         // b * P_K / P_t
                }
                wq.f[i] = pack_bf16(wq_[0], wq_[1], wq_[2], wq_[3]);
                wa.f[i] = pack_bf16(wa_[0], wa_[1], wa_[2], wa_[3]);
                bwi.f[i] = pack_bf16(bwi_[0], bwi_[1], bwi_[2], bwi_[3]);
                if constexpr (FWD) kwi.f[i] = pack_bf16(kwi_[0], kwi_[1], kwi_[2], kwi_[3]);
                else bf.f[i] = pack_bf16(bf_[0], bf_[1], bf_[2], bf_[3]);
                if ((CUTS >> i) & 1) STEP_BARRIER();   // cut points 0-3 (the loop is unrolled)
            }
            // ---- segment 2: transposes of V (dY) and the strictly triangular 16x16 products ----
            TileB XT;   // forward: V^T; backward: dY^T   (lane = value ch, reg = token)
#pragma unroll
            for (int ib = 0; ib < NCH; ib++) XT.f[ib] = transpose(cur.v.f[ib], eye);
            const f32x4 AB = mask_lower_strict(tile_xyT(wa, bwi), L);   // [t][s] = wa_t . bwi_s, s < t
            const f32x4 ABT = mask_upper_strict(tile_xyT(bwi, wa), L);
            bf16x4 AK_b, QBT;
            if constexpr (FWD) AK_b = to_bf16(mask_lower_strict(tile_xyT(wa, kwi), L));
            else QBT = to_bf16(mask_upper_incl(tile_xyT(bwi, wq), L));  // [s][t] = wq_t . bwi_s, s <= t
            SEG(4);
            // ---- segments 3, 4: the triangular inverse (matrix instructions in one long dependent chain); the
            //      output's inclusive products ride in the second one ----
            f32x4 Tinv, TinvT;
            tri_inverse_begin(AB, ABT, L, Tinv, TinvT);
            tri_inverse_level<2>(AB, L, Tinv, TinvT);
            SEG(5);
            tri_inverse_level<4>(AB, L, Tinv, TinvT);
            SEG(6);
            tri_inverse_level<8>(AB, L, Tinv, TinvT);
            const bf16x4 Tm = to_bf16(FWD ? Tinv : TinvT);
            bf16x4 QKB0, QKB1;
            if constexpr (FWD && !MAP) {
                QKB0 = to_bf16(mask_lower_incl(tile_xyT(wq, kwi), L));  // QK[t][s] = wq_t . kwi_s, s <= t
                QKB1 = to_bf16(mask_lower_incl(tile_xyT(wq, bwi), L));  // QB
            }
            SEG(7);
            // ---- segment 5: the private operands (forward U0 = Tinv AK V; backward D0 = Tinv^T QB^T dY) and
            //      forward Wm = Tinv wa, backward Bm = Tinv^T bf ----
            TileB ZT;
#pragma unroll
            for (int ib = 0; ib < NCH; ib++) {
                const f32x4 RT = mma(zero4(), FWD ? AK_b : QBT, XT.f[ib]);
                ZT.f[ib] = to_bf16(mma(zero4(), Tm, to_bf16(RT)));
            }
            SEG(8);
            bf16x4 Mm[NBLK];
#pragma unroll
            for (int jb = 0; jb < NBLK; jb++) {
                const bf16x4 xT = transpose(FWD ? wa.f[jb] : bf.f[jb], eye);   // lane = key ch, reg = token
                Mm[jb] = to_bf16(mma(zero4(), xT, Tm));                        // lane = token, reg = key ch
            }
            SEG(9);
            // ---- segment 6: first half of the stores; the next chunk's tiles set out (not earlier: a fetch issued
            //      in segments 2-5 measured 0.4 us slower per step) ----
#pragma unroll
            for (int ib = 0; ib < NCH; ib++) lds_pair(slot + SL_I + ib * 1024, lane, ZT.f[ib], XT.f[ib]);
            if constexpr (FWD && !MAP) {
                lds_pair(slot + SL_Y, lane, wq.f[0], wq.f[1]);
                lds_pair(slot + SL_Y + 1024, lane, wq.f[2], wq.f[3]);
                lds_pair(slot + SL_Y + 2048, lane, QKB0, QKB1);
            }
            *reinterpret_cast<float*>(slot + SL_FW + (16 * (L.n >> 2) + 4 * L.g + (L.n & 3)) * 4) = fw1;
            nxt = fetch(st + P);
            SEG(10);
            // ---- segment 7: the shared operands of the chain ----
#pragma unroll
            for (int jb = 0; jb < NBLK; jb++) {
                if constexpr (FWD)
                    lds_pair(slot + SL_J + (2 + jb) * 1024, lane, transpose(kwi.f[jb], eye), transpose(bwi.f[jb], eye));
                else
                    lds_pair(slot + SL_J + (2 + jb) * 1024, lane, transpose(wq.f[jb], eye), transpose(wa.f[jb], eye));
            }
            lds_pair(slot + SL_J, lane, Mm[0], Mm[1]);
            lds_pair(slot + SL_J + 1024, lane, Mm[2], Mm[3]);
            SEG(11);
            done += P;
        }
        for (; done < STEPS; done++) STEP_BARRIER();
        return;
    }

    if (!MAP && wave == NCW + P + (LN ? LN_WAVES : 0)) {
        // ------------------------------------------------------------------------------------------------
        // store wavefront: after its barrier number P + 3 + st the results of chunk st are in their out slot
        // ------------------------------------------------------------------------------------------------
        unsigned char* const saved = reinterpret_cast<unsigned char*>(A.saved);
        const long row_ld = (long)A.H * HEAD;
        const long y_lane = ((long)(bh / A.H) * A.T + L.n) * row_ld + (long)(bh % A.H) * HEAD + 32 * (vb0 / 2) + 8 * L.g;   // elements
        for (int k = 1; k <= STEPS; k++) {
            STEP_BARRIER();
            const int st = k - (P + 3);
            if (st < 0 || st >= LS) continue;
            const int c = chunk_of(st);
            const unsigned char* o = ring + ORING + (st % OUT_SLOTS) * OSLOT;
            auto piece = [&](int off) { return *reinterpret_cast<const bf16x8*>(o + off + lane * 16); };
            if constexpr (SAVE) {
                long ck, ut;   // byte offsets of this block's part of the kept state and of U^T
                bool keep;
                if (A.paired) {
                    const long pid = (long)bh * SavedPair::pairs(NC) + (c >> 1);
                    ck = SavedPair::ds(pid, vb0) * 2, ut = (SavedPair::ut(pid, c) + vb0 * FRAG_ELEMS) * 2;
                    keep = FWD ? !(c & 1) : SavedPair::keeps(c, NC) && SavedPair::ds_kept(pid, c >> 1, SavedPair::pairs(NC), A.ds_run);
                } else {
                    const long cid = (long)bh * NC + c;
                    ck = Saved::ckpt(cid, vb0) * 2, ut = (Saved::ut(cid) + vb0 * FRAG_ELEMS) * 2;
                    keep = true;
                }
                if (keep) {
#pragma unroll
                    for (int i = 0; i < 2 * NCH; i++) *reinterpret_cast<bf16x8*>(saved + ck + i * 1024 + lane * 16) = piece(out_ck(NCH) + i * 1024);
                }
                if constexpr (NCH == 4) {
#pragma unroll
                    for (int i = 0; i < 2; i++) *reinterpret_cast<bf16x8*>(saved + ut + i * 1024 + lane * 16) = piece(out_ut(NCH) + i * 1024);
                } else {
                    *reinterpret_cast<bf16x8*>(saved + ut + lane * 16) = piece(out_ut(NCH));
                }
            }
            if constexpr (FWD && !LN) {
                // y by rows: a lane's 16 bytes are the fragments of value blocks 2p and 2p + 1 (8 contiguous channels)
#pragma unroll
                for (int pp = 0; pp < NCH / 2; pp++)
                    *reinterpret_cast<bf16x8*>(A.y + y_lane + (long)c * CHUNK * row_ld + 32 * pp) = piece(out_y(NCH) + pp * 1024);
                if (A.centers != nullptr && lane < 16) {   // token `lane`: the centres of this block's value blocks
                    float* dst = A.centers + 4 * (((long)(bh / A.H) * A.T + c * CHUNK + lane) * A.H + bh % A.H) + vb0;
                    const float* src = reinterpret_cast<const float*>(o + out_cen(NCH)) + lane * NCH;
                    if constexpr (NCH == 4) *reinterpret_cast<f32x4*>(dst) = *reinterpret_cast<const f32x4*>(src);
                    else *reinterpret_cast<float2*>(dst) = *reinterpret_cast<const float2*>(src);
                }
            }
        }
        return;
    }
    // ----------------------------------------------------------------------------------------------------
    // chain wavefront ib: value rows 16 ib .. 16 ib + 15 of the state
    // ----------------------------------------------------------------------------------------------------
    // MAP: set 0 runs the recurrence from a zero state (-> N), set 1 the homogeneous recurrence (no V, no U0; backward
    // no dY, no D0) from the identity (-> M); both take the shared operands from the one ring
    const int part = MAP ? wave / NCH : 0;
    const int iw = MAP ? wave % NCH : wave;   // value block within this block (its slot in the ring)
    const int ib = vb0 + iw;                  // value block within the head
    // the chain is the critical path of every step: its wavefronts win the SIMD's issue arbitration against the two
    // producers they share it with, which fill the gaps
    __builtin_amdgcn_s_setprio(3);
    struct Operands {   // read from the ring one step ahead of their use
        bf16x8 j[6];
        bf16x8 iv;
    };
    auto read_ops = [&](Operands& o, int st) {
        const unsigned char* base = ring + (st % FUSE_SLOTS) * SLOT;
#pragma unroll
        for (int i = 0; i < 6; i++) o.j[i] = *reinterpret_cast<const bf16x8*>(base + SL_J + i * 1024 + lane * 16);
        o.iv = *reinterpret_cast<const bf16x8*>(base + SL_I + iw * 1024 + lane * 16);
    };
    // Off the chain: the chunk decay and, forward, the output's operands.  Their producer stored them two steps before
    // the round that uses them, so they too are requested at the end of the round before (into the registers that round
    // has just finished with) and no round starts by waiting for LDS.
    struct Early {
        f32x4 fw[NBLK];
        bf16x8 yp[3];
    };
    auto read_early = [&](Early& e, int st) {
        const unsigned char* base = ring + (st % FUSE_SLOTS) * SLOT;
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) e.fw[jb] = *reinterpret_cast<const f32x4*>(base + SL_FW + jb * 64 + L.g * 16);
        if constexpr (FWD && !MAP) {
#pragma unroll
            for (int i = 0; i < 3; i++) e.yp[i] = *reinterpret_cast<const bf16x8*>(base + SL_Y + i * 1024 + lane * 16);
        }
    };
    f32x4 S[NBLK];
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) {
        if constexpr (MAP) {   // zero, or the rows 16 ib .. + 15 of the identity (fragment order on both sides, as the maps are kept)
#pragma unroll
            for (int r = 0; r < 4; r++) S[jb][r] = (part == 1 && 16 * ib + L.n == 16 * jb + 4 * L.g + r) ? 1.f : 0.f;
        } else {
            S[jb] = load_state_frag(A.s_in, A.s_in_f32, unit, ib, jb, L);   // (one entry per segment when there are several)
        }
    }

    Early early;
    auto round = [&](int st, const Operands& op, Operands& next) {
        const int c = chunk_of(st);
        const f32x4(&fw)[NBLK] = early.fw;
        const bf16x8(&yp)[3] = early.yp;
        const bf16x4 b0 = to_bf16(S[0]), b1 = to_bf16(S[1]), b2 = to_bf16(S[2]), b3 = to_bf16(S[3]);
        const bf16x8 s01 = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
        const bf16x8 s23 = __builtin_shufflevector(b2, b3, 0, 1, 2, 3, 4, 5, 6, 7);
        bf16x8 iv = op.iv;
        if constexpr (MAP) {
            const bf16x8 none = {};
            if (part) iv = none;
        }
        const bf16x4 U0 = __builtin_shufflevector(iv, iv, 0, 1, 2, 3);
        const f32x4 Ua = mma8(to_f32(U0), op.j[0], s01);   // + F(S_ib Wm^T), two independent halves
        const f32x4 Uc = mma8(zero4(), op.j[1], s23);
        f32x4 y;
        if constexpr (FWD && !MAP) {   // F(Y_ib): lane = token, reg = value channel.  wq S_ib^T does not wait for U
            y = mma8(zero4(), s01, yp[0]);
            y = mma8(y, s23, yp[1]);
        }
        const bf16x4 u = to_bf16(Ua + Uc);
        const bf16x8 VU = __builtin_shufflevector(iv, __builtin_shufflevector(u, u, 0, 1, 2, 3, 0, 1, 2, 3), 4, 5, 6, 7, 8, 9, 10, 11);
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            // forward: (S + V_ib^T kwi_jb + U_ib^T bwi_jb) diag(fw), the chunk decay applied to the sum (the producers
            // then need no separately scaled copies of k and b); backward: dS diag(fw) + dY_ib^T wq_jb + dab_u_ib^T wa_jb
            if constexpr (FWD) S[jb] = mma8(S[jb], op.j[2 + jb], VU) * fw[jb];
            else S[jb] = mma8(S[jb] * fw[jb], op.j[2 + jb], VU);
        }
        unsigned char* const out = ring + ORING + (st % OUT_SLOTS) * OSLOT;
        if constexpr (SAVE) {
            // forward: the state only where a pair of chunks begins (the gradient kernel advances it across the pair's
            // first chunk); backward: the dstate only where a pair ends (SavedPair); every chunk when a state per chunk is kept
            bool keep = !A.paired || (FWD ? !(c & 1) : SavedPair::keeps(c, NC));
            if constexpr (!FWD) {
                const int NP = SavedPair::pairs(NC);
                if (A.paired) keep = keep && SavedPair::ds_kept((long)bh * NP + (c >> 1), c >> 1, NP, A.ds_run);
            }
            if (keep) {
                bf16x8* q = reinterpret_cast<bf16x8*>(out + out_ck(NCH) + iw * 2048 + lane * 32);
                q[0] = s01;
                q[1] = s23;
            }
            *reinterpret_cast<bf16x4*>(out + out_ut(NCH) + iw * 512 + lane * 8) = u;
        }
        if constexpr (FWD && !MAP) {
            const f32x4 yo = mma8(y, VU, yp[2]);             // + QK V_ib + QB U_ib
            if constexpr (LN) *reinterpret_cast<f32x4*>(ring + YRING + (st & 1) * 4096 + iw * 1024 + lane * 16) = yo;
            else {
                bf16x4* yq = reinterpret_cast<bf16x4*>(out + out_y(NCH) + ((iw >> 1) * 64 + lane) * 16 + (iw & 1) * 8);
                if (A.centers != nullptr) {   // y is attn_ln's kept output: centred per block (all four lanes of a token hold the same centre)
                    const float cen = row_sum16_bf16(yo) * (1.f / 16);
                    *yq = to_bf16(yo - cen);
                    if (L.g == 0) *reinterpret_cast<float*>(out + out_cen(NCH) + (L.n * NCH + iw) * 4) = cen;
                } else *yq = to_bf16(yo);
            }
        }
        __builtin_amdgcn_sched_barrier(0);   // the next round's operand reads stay behind these writes (see OUT_SLOTS)
        read_ops(next, st + 1);   // complete since the end of the step before this one
        read_early(early, st + 1);
        if constexpr (LN) STEP_BARRIER();   // (publishes the y ring)
        else reader_barrier();
    };

    for (int i = 0; i < P; i++) STEP_BARRIER();
    Operands op0, op1;
    read_ops(op0, 0);
    read_early(early, 0);
    STEP_BARRIER();
    int st = 0;
    for (; st + 2 <= LS; st += 2) {
        round(st, op0, op1);
        round(st + 1, op1, op0);
    }
    if (st < LS) round(st, op0, op1);
    STEP_BARRIER();   // the last round's results are in LDS; the epilogue wavefronts' and the store wavefront's last step
    if constexpr (MAP) {
        float* dst = A.maps + ((long)unit * 2 + part) * HEAD * HEAD;
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            if (part == 0) {
                *reinterpret_cast<f32x4*>(dst + (16 * ib + L.n) * HEAD + 16 * jb + 4 * L.g) = S[jb];
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++) dst[(16 * jb + 4 * L.g + r) * HEAD + 16 * ib + L.n] = S[jb][r];
            }
        }
    } else if (seg == A.NSEG - 1) {   // the segment walked last leaves the sequence's final state
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) store_state_frag(A.s_out, A.s_out_f32, bh, ib, jb, L, S[jb]);
    }
}

// ------------------------------------------------------------------------------------------------
// host launchers
// ------------------------------------------------------------------------------------------------
namespace {
// grid of a launch over `units` (batch, head, segment)s: one block each, or two (halves 8 block ids apart)
inline unsigned fused_grid(int units, int vs) { return vs == 1 ? units : 16 * ((units + 7) / 8); }
inline bool fused_split(int units) { return 2 * units <= compute_units(); }

FusedArgs fused_args(int B, int T, int H, int state_f32, int nseg) {
    FusedArgs A{};
    A.T = T, A.H = H, A.NC = T / CHUNK, A.BH = B * H, A.B = B;
    A.s_in_f32 = A.s_out_f32 = state_f32;
    A.NSEG = nseg, A.LS = A.NC / nseg;
    A.ds_run = 1;
    return A;
}

// Long sequences on few heads (scan_segments > 1): the maps of all segments, then the states entering them.  After
// this A.s_in is the per-segment array and the kernel proper can be launched over B*H*nseg units.
template <bool FWD>
void segment_states(FusedArgs& A, int state_f32, void* seg_ws, hipStream_t stream) {
    const int units = A.BH * A.NSEG;
    float* maps = static_cast<float*>(seg_ws);
    float* s_seg = maps + (size_t)units * 2 * HEAD * HEAD;
    FusedArgs M = A;
    M.maps = maps, M.saved = nullptr, M.y = nullptr, M.centers = nullptr, M.s_in = nullptr, M.s_out = nullptr;
    M.dparams = nullptr, M.dparams_part = nullptr;
    if (fused_split(units))
        hipLaunchKernelGGL((wkv7_fused_kernel<FWD, false, false, CUTS_TEN, 2, true>), dim3(fused_grid(units, 2)),
                           dim3(fused_threads(CUTS_TEN, false, 2, true)), 0, stream, M);
    else
        hipLaunchKernelGGL((wkv7_fused_kernel<FWD, false, false, CUTS_EIGHT_EVEN, 1, true>), dim3(fused_grid(units, 1)),
                           dim3(fused_threads(CUTS_EIGHT_EVEN, false, 1, true)), 0, stream, M);
    launch_segment_carry(A.BH, A.NSEG, state_f32, A.s_in, maps, s_seg, stream);
    A.s_in = s_seg, A.s_in_f32 = 1;
}
}  // namespace

void launch_fused_forward(int B, int T, int H, int state_f32, const void* w, const void* q, const void* k, const void* v,
                          const void* a, const void* b, const void* s_in, void* s_out, void* y, void* saved,
                          int paired, hipStream_t stream, const void* g, const void* params, void* y_wkv, float* centers,
                          void* seg_ws) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    const int nseg = params ? 1 : scan_segments(B, T, H);   // (the one-kernel attn_ln forward is for many heads)
    FusedArgs A = fused_args(B, T, H, state_f32, nseg);
    A.w = c(w), A.q = c(q), A.k = c(k), A.v = c(v), A.a = c(a), A.b = c(b);
    A.saved = static_cast<__bf16*>(saved), A.s_in = s_in, A.s_out = s_out, A.y = static_cast<__bf16*>(y);
    A.g = c(g), A.params = static_cast<const float*>(params), A.y_wkv = static_cast<__bf16*>(y_wkv), A.centers = centers;
    A.paired = paired;
    if (nseg > 1) segment_states<true>(A, state_f32, seg_ws, stream);
    const int units = B * H * nseg;
    auto go = [&](auto kernel, int threads, int vs = 1) {
        hipLaunchKernelGGL(kernel, dim3(fused_grid(units, vs)), dim3(threads), 0, stream, A);
    };
    // Two blocks per (batch, head), two value blocks each, while every block still gets a compute unit of its own: the
    // chain's and the value-side producers' work is halved per block at the price of repeating the key-side producers.
    const bool split = !params && fused_split(units);
    if (params) {
        constexpr int CUTS = CUTS_EIGHT_EVEN;
        if (saved) go(wkv7_fused_kernel<true, true, true, CUTS>, fused_threads(CUTS, true));
        else go(wkv7_fused_kernel<true, false, true, CUTS>, fused_threads(CUTS, true));
    } else {
        if (split) {
            constexpr int CUTS2 = CUTS_TEN;
            if (saved) go(wkv7_fused_kernel<true, true, false, CUTS2, 2>, fused_threads(CUTS2, false, 2), 2);
            else go(wkv7_fused_kernel<true, false, false, CUTS2, 2>, fused_threads(CUTS2, false, 2), 2);
        } else {
            constexpr int CUTS1 = CUTS_EIGHT_EVEN;
            if (saved) go(wkv7_fused_kernel<true, true, false, CUTS1>, fused_threads(CUTS1, false));
            else go(wkv7_fused_kernel<true, false, false, CUTS1>, fused_threads(CUTS1, false));
        }
    }
}

bool fused_backward_scan_takes_dparams(int B, int T, int H) {
    const int units = B * H * scan_segments(B, T, H);
    const int scan_blocks = (int)fused_grid(units, fused_split(units) ? 2 : 1);
    return scan_blocks + 3 * H <= compute_units();
}

void launch_fused_backward_scan(int B, int T, int H, int state_f32, const void* w, const void* q, const void* a,
                                const void* b, const void* dy, const void* ds_in, void* ds_out, void* saved,
                                int paired, hipStream_t stream, const float* dparams_part, float* dparams, void* seg_ws) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    const int nseg = scan_segments(B, T, H);
    FusedArgs A = fused_args(B, T, H, state_f32, nseg);
    A.w = c(w), A.q = c(q), A.a = c(a), A.b = c(b), A.dy = c(dy);
    A.saved = static_cast<__bf16*>(saved), A.s_in = ds_in, A.s_out = ds_out;
    A.paired = paired, A.ds_run = paired ? dstate_run(B, T, H) : 1;
    A.dparams_part = dparams_part, A.dparams = dparams;
    if (nseg > 1) segment_states<false>(A, state_f32, seg_ws, stream);
    const int units = B * H * nseg;
    const unsigned extra = dparams ? 3 * H : 0;
    if (fused_split(units))
        hipLaunchKernelGGL((wkv7_fused_kernel<false, true, false, CUTS_TEN, 2>), dim3(fused_grid(units, 2) + extra), dim3(fused_threads(CUTS_TEN, false, 2)), 0, stream, A);
    else
        hipLaunchKernelGGL((wkv7_fused_kernel<false, true, false, CUTS_EIGHT_EVEN>), dim3(fused_grid(units, 1) + extra), dim3(fused_threads(CUTS_EIGHT_EVEN, false)), 0, stream, A);
}

}  // namespace wkv
