// WKV7 forward for gfx950: chunk-parallel prepare -> state scan that also produces the output.
//
// Replaces forward_kernel of the reference (attn.cu:11-106; attn_ln.cu:106-212 with the epilogue),
// same mathematics (rwkv7_attn_triton.py:27-69), different organisation: the reference runs one
// block per (batch, head) through all chunks with ~60 block barriers per chunk; here each chunk is
// one wavefront's private work and only the 64x64 state update is sequential.
//
// Per chunk (K = 16 tokens), with S0 the state entering the chunk:
//   prepare:  Tinv = inv(I - strict_tril(wa bwi^T)),  U0 = Tinv (strict_tril(wa kwi^T) V),  Wm = Tinv wa
//   scan:     U = U0 + Wm S0^T ;  S' = S0 diag(fw) + V^T kf + U^T bf        (checkpoint S0, keep U)
//             Y = tril(wq kwi^T) V + tril(wq bwi^T) U + wq S0^T             (off the chain, same wavefronts)
//   attn_ln:  a chunk-parallel kernel applies GroupNorm + bonus + gate to Y
#include <type_traits>

#include "ln_epilogue.hpp"
#include "device_info.hpp"
#include "wkv7_common.hpp"
#include "wkv7_kernels.hpp"

namespace wkv {

// ------------------------------------------------------------------------------------------------
// prepare: one wavefront per chunk, four chunks per block.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fwd_prepare_kernel(int T, int H, int nchunks,
                                                          const __bf16* __restrict__ w_, const __bf16* __restrict__ q_,
                                                          const __bf16* __restrict__ k_, const __bf16* __restrict__ v_,
                                                          const __bf16* __restrict__ a_, const __bf16* __restrict__ b_,
                                                          __bf16* __restrict__ rec) {
    using R = RecFwd;
    const int lane = threadIdx.x & 63;
    const int wid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wid >= nchunks) return;
    const int cid = head_major_chunk(wid, nchunks, T);
    const Lane L;
    const ChunkAddr ca(cid, T, H);

    const TileB w = load_rows16(w_ + ca.row0, ca.ld, L);
    const TileB q = load_rows16(q_ + ca.row0, ca.ld, L);
    const TileB k = load_rows16(k_ + ca.row0, ca.ld, L);
    const TileB v = load_rows16(v_ + ca.row0, ca.ld, L);
    const TileB a = load_rows16(a_ + ca.row0, ca.ld, L);
    const TileB b = load_rows16(b_ + ca.row0, ca.ld, L);

    const Decay d = chunk_decay(w);
    const TileB wq = to_bf16(mul(q, d.P));                  // q * P_t
    const TileB wa = to_bf16(mul(a, d.Px));                 // a * P_{t-1}
    const TileF kwi_f = mul(k, d.Pi), bwi_f = mul(b, d.Pi);
    const TileB kwi = to_bf16(kwi_f);                       // k / P_t
    const TileB bwi = to_bf16(bwi_f);                       // b / P_t
    const TileB kf = to_bf16(mul(kwi_f, d.fw));             // k * P_K / P_t
    const TileB bf = to_bf16(mul(bwi_f, d.fw));

    // strictly lower-triangular 16x16 products, in both orientations where the inverse needs them
    const f32x4 AB = mask_lower_strict(tile_xyT(wa, bwi), L);   // F(AB),   AB[t][s] = wa_t . bwi_s, s < t
    const f32x4 ABT = mask_upper_strict(tile_xyT(bwi, wa), L);  // F(AB^T)
    const f32x4 AK = mask_lower_strict(tile_xyT(wa, kwi), L);   // F(AK)
    f32x4 Tinv, TinvT;
    tri_inverse(AB, ABT, L, Tinv, TinvT);
    const bf16x4 Tinv_b = to_bf16(Tinv);
    const bf16x4 AK_b = to_bf16(AK);
    const bf16x4 eye = identity_bf16(L);

    __bf16* J = rec + R::j(cid);
    // the output's intra-chunk operands: QK[t][s] = wq_t . kwi_s, QB[t][s] = wq_t . bwi_s, s <= t
    store_pair(J + 6 * J_PAIR_ELEMS, lane, wq.f[0], wq.f[1]);
    store_pair(J + 7 * J_PAIR_ELEMS, lane, wq.f[2], wq.f[3]);
    store_pair(J + 8 * J_PAIR_ELEMS, lane, to_bf16(mask_lower_incl(tile_xyT(wq, kwi), L)),
               to_bf16(mask_lower_incl(tile_xyT(wq, bwi), L)));
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        const bf16x4 VT = transpose(v.f[ib], eye);                 // F(V_ib^T)        lane = value ch, reg = token
        const f32x4 RT = mma(zero4(), AK_b, VT);                   // F((AK V_ib)^T)
        const f32x4 UT = mma(zero4(), Tinv_b, to_bf16(RT));        // F((Tinv AK V_ib)^T)
        store_pair(rec + R::i(cid, ib), lane, to_bf16(UT), VT);
    }
    bf16x4 Wm[NBLK];
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) {
        const bf16x4 waT = transpose(wa.f[jb], eye);               // F(wa_jb^T)       lane = key ch, reg = token
        Wm[jb] = to_bf16(mma(zero4(), waT, Tinv_b));               // F(Tinv wa_jb)    lane = token, reg = key ch
        store_pair(J + (2 + jb) * J_PAIR_ELEMS, lane, transpose(kf.f[jb], eye), transpose(bf.f[jb], eye));
    }
    store_pair(J, lane, Wm[0], Wm[1]);
    store_pair(J + J_PAIR_ELEMS, lane, Wm[2], Wm[3]);
    if (L.n == 0) {
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            f32x4 fw;
#pragma unroll
            for (int r = 0; r < 4; r++) fw[r] = d.fw.f[jb][r];
            *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(rec + R::fw(cid)) + 16 * jb + 4 * L.g) = fw;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// scan: the only sequential part.  One block of four wavefronts per (batch, head); each wavefront owns 16 of
// the head's 64 value rows, with that slice of the state in its fp32 accumulators (one wavefront per SIMD, so
// each has the whole register file).  The same kernel runs the backward dstate scan (R = RecBwd, reverse = 1,
// no output).
//   per chunk:  U^T = U0^T + S Wm^T               (contraction over key channels)
//               S  <- S diag(fw) + V^T K + U^T B  (contraction over the chunk's tokens)
//   forward:    Y_ib = QK V_ib + QB U_ib + wq S_ib^T   (three more matrix instructions, not on the chain)
// The chain is six matrix instructions per chunk; everything else is about keeping memory latency and
// instruction issue off it.  Measured with cycle stamps: every 64-lane 16-byte LDS instruction costs the
// compute unit's LDS pipe ~16 cycles and every memory instruction costs its address unit ~16 cycles, whoever
// issues them, so the block's work per chunk is split over both pipes and nothing is fetched twice:
//   * the six J pairs of the chain and FW are needed by all four wavefronts: each wavefront loads a quarter
//     of them (DEPTH chunks ahead, in registers) and copies it into a three-slot LDS ring two chunks ahead of
//     the chain; every wavefront reads chunk t+1's slot into a second register set while it works on chunk t
//     (the sets alternate, no moves);
//   * its own (U0^T, V^T) record and, forward, the three output-only pairs come straight from memory into
//     registers, DEPTH chunks ahead;
//   * checkpoint and U^T of chunk t-1 are stored OVER that chunk's record, and the wavefront's 16x16 piece of
//     Y to the output, right after the barrier that ends chunk t-1 - by then every wavefront of the block, the
//     only readers of the record, has consumed it; the stores hit lines that were just read.
// One LDS-only barrier per chunk keeps the four wavefronts in step.
// ------------------------------------------------------------------------------------------------
constexpr int RING_SLOTS = 3;
constexpr int RING_PAIRS = 6;
constexpr int RING_J_BYTES = RING_PAIRS * 1024;
constexpr int RING_PAD = RING_J_BYTES + HEAD * 4;    // after FW: 1 KiB nobody reads
constexpr int RING_BYTES = RING_PAD + 1024;
constexpr int SCAN_THREADS = 4 * 64;
constexpr int SCAN_DEPTH = 8;   // chunks in flight per wavefront; even (two register sets alternate)


// y_: WITH_Y only; [B,T,H,64] bf16.
// LOADER: a fifth wavefront does all the shared loads and ring writes instead of the four splitting them
// (measured: better for the reverse scan, 30 against 35 us at B*H = 96; the forward scan with its larger
// register sets needs one wavefront per SIMD).
//
// Long sequences on few (batch, head) pairs leave most compute units idle, so the chunks of one pair can be cut
// into NSEG segments of LS chunks that run as separate blocks (blockIdx.x = pair * NSEG + segment, segments in
// processing order).  The state entering a segment is then needed up front.  Per segment the chain is an affine
// map of the entering state, S_out = S_in M + N, and the rows of a state evolve independently, so
//   MAP = true   (eight wavefronts, no loader) runs the chain without storing anything: wavefronts 0-3 (part 0)
//                from a zero state (-> N), wavefronts 4-7 (part 1) on the 64 rows of the identity with the
//                inhomogeneous terms switched off (-> M, stored transposed); both parts take the shared
//                operands from the one ring, so a record is read once.  segment_carry_kernel then composes
//                the maps in sequence;
//   MAP = false  is the scan proper, each segment starting from its entry of s_in ([pair][segment][64][64]).
template <typename R, bool WITH_Y, bool LOADER, int DEPTH, bool MAP = false, bool SAVE = true>
__global__ __launch_bounds__(MAP ? 2 * SCAN_THREADS : LOADER ? SCAN_THREADS + 64 : SCAN_THREADS) void state_scan_kernel(
    int NC, int LS, int NSEG, int H, int reverse, int s_in_f32, int s_out_f32, __bf16* __restrict__ rec,
    const void* __restrict__ s_in, void* __restrict__ s_out, __bf16* __restrict__ y_, int scan_blocks, int keep_parity,
    float* __restrict__ centers) {
    static_assert(!MAP || (!WITH_Y && !LOADER), "the map pass produces no output and splits the loads eight ways");
    static_assert(SAVE || WITH_Y, "a scan that keeps neither checkpoints nor the output has nothing to write");
    if (blockIdx.x >= (unsigned)scan_blocks) {
        // Helper blocks on compute units the scan leaves idle: they read the records once, in the order the scan
        // will want them, and throw the data away.  The scan's own loads then find the lines in a cache even when
        // the kernels before it left the memory-side cache full of other dirty data (a forward-only loop: 59 ->
        // 45 us; inside the time-mixer block: 65 -> 48 us).  Pacing the helpers by the clock to stay a few chunks
        // ahead and matching them to the scan blocks of their own XCD (for L2 hits) measured the same.  What
        // remains context-dependent is the scan's stores.  No barrier, no LDS, nothing written.
        const long total = (long)scan_blocks * NC;
        const int nh = gridDim.x - scan_blocks, hid = blockIdx.x - scan_blocks;
        constexpr int PIECES = R::BYTES / 16;
        i32x4 acc = {0, 0, 0, 0};
        for (long o = hid; o < total; o += nh) {
            const long pos = o / scan_blocks, pair = o - pos * scan_blocks;
            const long cid = pair * NC + (reverse ? NC - 1 - pos : pos);
            const i32x4* p = reinterpret_cast<const i32x4*>(rec + cid * R::ELEMS);
            for (int i = threadIdx.x; i < PIECES; i += blockDim.x) acc ^= p[i];
        }
        asm volatile("" ::"v"(acc[0]), "v"(acc[1]), "v"(acc[2]), "v"(acc[3]));
        return;
    }
    static_assert(DEPTH >= 4 && DEPTH % 2 == 0, "two register sets alternate; the prologue uses stages 0, 1 twice");
    static_assert(!WITH_Y || R::NPAIR == 9, "the output needs the wq and (QK, QB) pairs");
    constexpr int NYP = WITH_Y ? 3 : 0;   // output-only pairs
    __shared__ __attribute__((aligned(16))) unsigned char ring[RING_SLOTS * RING_BYTES];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ib = MAP ? wave & 3 : wave;     // the 16 value rows this wavefront carries
    const int part = MAP ? wave >> 2 : 0;
    const int bx = blockIdx.x;
    const int bh = bx / NSEG, seg = bx - bh * NSEG;
    const Lane L;
    auto chunk_of = [&](int step) -> long {
        step = step < LS ? step : LS - 1;
        const int pos = seg * LS + step;
        return (long)bh * NC + (reverse ? NC - 1 - pos : pos);
    };

    if constexpr (LOADER) {
        if (ib == 4) {
            // the loader wavefront: same rounds as the others (a prologue barrier, then one barrier per chunk).
            // invariant at round t: st[(t + 2) % DEPTH] holds J and FW of chunk t+2, which go to slot (t+2) % 3
            struct Stage {
                f32x4 j[RING_PAIRS];
                float fw;
            };
            const char* jsrc = reinterpret_cast<const char*>(rec + R::J) + lane * 16;
            const float* fsrc = reinterpret_cast<const float*>(rec + R::FW) + lane;
            auto issue = [&](Stage& st, int step) {
                const long cid = chunk_of(step);
#pragma unroll
                for (int i = 0; i < RING_PAIRS; i++) st.j[i] = *reinterpret_cast<const f32x4*>(jsrc + cid * R::BYTES + i * 1024);
                st.fw = fsrc[cid * (R::ELEMS / 2)];
            };
            auto to_lds = [&](int step, const Stage& st) {
                unsigned char* base = ring + (step % RING_SLOTS) * RING_BYTES;
#pragma unroll
                for (int i = 0; i < RING_PAIRS; i++) *reinterpret_cast<f32x4*>(base + i * 1024 + lane * 16) = st.j[i];
                *reinterpret_cast<float*>(base + RING_J_BYTES + lane * 4) = st.fw;
            };
            constexpr int DL = 6;
            Stage st[DL];
#pragma unroll
            for (int s = 0; s < DL; s++) issue(st[s], s);
            to_lds(0, st[0]);
            to_lds(1, st[1]);
            issue(st[0], DL);
            issue(st[1], DL + 1);
            lds_barrier();
            int step0 = 0;
            for (; step0 + DL <= LS; step0 += DL) {
#pragma unroll
                for (int s = 0; s < DL; s++) {
                    to_lds(step0 + s + 2, st[(s + 2) % DL]);
                    issue(st[(s + 2) % DL], step0 + s + 2 + DL);
                    lds_barrier();
                }
            }
#pragma unroll
            for (int s = 0; s < DL - 1; s++) {   // the remaining NC % DL rounds; chunks past the end are never read
                if (step0 + s < LS) {
                    to_lds(step0 + s + 2, st[(s + 2) % DL]);
                    lds_barrier();
                }
            }
            return;
        }
    }

    // ---- this wavefront's share of the shared operands: unit A = pair ib; unit B = pair 4, pair 5, FW, nothing;
    //      the eight wavefronts of the map pass take one unit each (pairs 0-5, FW, nothing) ----
    struct Shared {
        f32x4 a, b;
    };
    const char* recb = reinterpret_cast<const char*>(rec);
    // (every wavefront issues the same instructions - a load or store under a condition would make the compiler
    // wait for ALL outstanding memory operations at the join; wavefront 3 re-loads its pair and parks it in a pad)
    const long a_off = wave < RING_PAIRS ? (R::J + wave * J_PAIR_ELEMS) * 2 + lane * 16
                                         : (wave == 6 ? R::FW * 2 + (lane & 15) * 16 : R::J * 2 + lane * 16);
    const int a_dst = wave < RING_PAIRS ? wave * 1024 + lane * 16 : (wave == 6 ? RING_J_BYTES + (lane & 15) * 16 : RING_PAD + lane * 16);
    const long b_off = ib < 2 ? (R::J + (4 + ib) * J_PAIR_ELEMS) * 2 + lane * 16
                              : (ib == 2 ? R::FW * 2 + (lane & 15) * 16 : a_off);
    const int b_dst = ib < 2 ? (4 + ib) * 1024 + lane * 16 : (ib == 2 ? RING_J_BYTES + (lane & 15) * 16 : RING_PAD + lane * 16);
    auto issue_shared = [&](Shared& st, int step) {
        const char* base = recb + chunk_of(step) * R::BYTES;
        st.a = *reinterpret_cast<const f32x4*>(base + a_off);
        if constexpr (!MAP) st.b = *reinterpret_cast<const f32x4*>(base + b_off);
    };
    auto shared_to_lds = [&](int step, const Shared& st) {
        unsigned char* base = ring + (step % RING_SLOTS) * RING_BYTES;
        *reinterpret_cast<f32x4*>(base + a_dst) = st.a;
        if constexpr (!MAP) *reinterpret_cast<f32x4*>(base + b_dst) = st.b;
    };

    struct Operands {   // one chunk's shared operands, in registers
        bf16x8 j[RING_PAIRS];
        f32x4 fw[NBLK];
    };
    struct Private {    // what only this wavefront needs
        bf16x8 iv;                        // this lane's (U0^T, V^T) pair
        bf16x8 yp[NYP > 0 ? NYP : 1];     // forward: (wq0,wq1), (wq2,wq3), (QK,QB)
    };
    struct Outputs {    // what the chunk leaves for the consumers
        bf16x8 s01, s23;
        bf16x4 u, y;
        float c;   // centres != nullptr: the centre y was stored around (this wavefront's 16 channels of this lane's token)
    };
    auto read_ring = [&](Operands& o, int step) {
        const unsigned char* base = ring + (step % RING_SLOTS) * RING_BYTES;
#pragma unroll
        for (int i = 0; i < RING_PAIRS; i++) o.j[i] = *reinterpret_cast<const bf16x8*>(base + i * 1024 + lane * 16);
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) o.fw[jb] = *reinterpret_cast<const f32x4*>(base + RING_J_BYTES + jb * 64 + L.g * 16);
    };
    const __bf16* isrc = rec + R::I + (ib * WAVE + lane) * 8;
    const __bf16* ysrc = rec + R::J + RING_PAIRS * J_PAIR_ELEMS + lane * 8;
    auto issue_private = [&](Private& p, int step) {
        const long off = chunk_of(step) * R::ELEMS;
        if constexpr (MAP) {   // the homogeneous part has no U0 and no V: its load stays on one chunk (a select of
                               // the address and of the value, not a branch)
            const bf16x8 zero = {};
            p.iv = *reinterpret_cast<const bf16x8*>(isrc + (part ? chunk_of(0) * R::ELEMS : off));
            p.iv = part ? zero : p.iv;
        } else {
            p.iv = *reinterpret_cast<const bf16x8*>(isrc + off);
        }
#pragma unroll
        for (int i = 0; i < NYP; i++) p.yp[i] = *reinterpret_cast<const bf16x8*>(ysrc + off + i * J_PAIR_ELEMS);
    };
    const long y_ld = (long)H * HEAD;
    const long y_head = ((long)(bh / H) * NC * CHUNK + L.n) * y_ld + (long)(bh % H) * HEAD + chan16(ib, 4 * L.g);
    const long c_head = 4 * (((long)(bh / H) * NC * CHUNK + L.n) * H + bh % H) + ib;   // centres: [token][head][block of 16 channels]
    auto store_outputs = [&](int step, const Outputs& o) {
        if constexpr (MAP) return;
        const long cid = chunk_of(step);
        if constexpr (SAVE) {   // what the backward pass reads; a forward that nothing differentiates skips it
            __bf16* r = rec + cid * R::ELEMS;
            // keep_parity >= 0: the state only for the chunks of that parity (per pair of chunks: the forward the state
            // entering the even chunk, the reverse scan the dstate arriving at the end of the odd one; the gradient
            // kernel carries both across the pair); a uniform branch
            if (keep_parity < 0 || (int)((cid - (long)bh * NC) & 1) == keep_parity) {
                bf16x8* q = reinterpret_cast<bf16x8*>(r + R::CKPT + ib * TILE_ELEMS + lane * 16);   // 32 bytes per lane
                q[0] = o.s01;
                q[1] = o.s23;
            }
            *reinterpret_cast<bf16x4*>(r + R::UT + ib * FRAG_ELEMS + lane * 4) = o.u;
        }
        if constexpr (WITH_Y)   // this lane's token row of the chunk, 4 of this wavefront's 16 value channels
        {
            *reinterpret_cast<bf16x4*>(y_ + y_head + (cid - (long)bh * NC) * CHUNK * y_ld) = o.y;
            if (centers != nullptr) centers[c_head + (cid - (long)bh * NC) * CHUNK * H * 4] = o.c;   // (the four lanes of a token write the same value)
        }
    };

    f32x4 S[NBLK];
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) {
        if constexpr (MAP) {
#pragma unroll
            for (int r = 0; r < 4; r++) S[jb][r] = (part && 16 * ib + L.n == 16 * jb + 4 * L.g + r) ? 1.f : 0.f;
        } else {
            S[jb] = load_state_frag(s_in, s_in_f32, bx, ib, jb, L);
        }
    }

    auto compute = [&](const Operands& op, const Private& p, Outputs& out) {
        const bf16x4 b0 = to_bf16(S[0]), b1 = to_bf16(S[1]), b2 = to_bf16(S[2]), b3 = to_bf16(S[3]);
        out.s01 = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
        out.s23 = __builtin_shufflevector(b2, b3, 0, 1, 2, 3, 4, 5, 6, 7);
        const bf16x4 U0 = __builtin_shufflevector(p.iv, p.iv, 0, 1, 2, 3);
        const f32x4 Ua = mma8(to_f32(U0), op.j[0], out.s01);   // + F(S_ib Wm^T), two independent halves
        const f32x4 Uc = mma8(zero4(), op.j[1], out.s23);
        f32x4 y;
        if constexpr (WITH_Y) {   // F(Y_ib): lane = token, reg = value channel.  wq S_ib^T does not wait for U
            y = mma8(zero4(), out.s01, p.yp[0]);
            y = mma8(y, out.s23, p.yp[1]);
        }
        out.u = to_bf16(Ua + Uc);
        const bf16x8 VU = __builtin_shufflevector(p.iv, __builtin_shufflevector(out.u, out.u, 0, 1, 2, 3, 0, 1, 2, 3), 4, 5, 6, 7, 8, 9, 10, 11);
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) S[jb] = mma8(S[jb] * op.fw[jb], op.j[2 + jb], VU);   // + F(V_ib^T K_jb + U_ib^T B_jb)
        if constexpr (WITH_Y) {
            f32x4 yo = mma8(y, VU, p.yp[2]);   // + QK V_ib + QB U_ib
            // attn_ln's kept output: centred per token and block of 16 channels, so that its bf16 rounding is relative
            // to the spread GroupNorm divides by and not to the mean (see ln_epilogue.hpp)
            if (centers != nullptr) {
                out.c = row_sum16_bf16(yo) * (1.f / 16);
                yo = yo - out.c;
            }
            out.y = to_bf16(yo);
        }
    };

    // ---- prologue: DEPTH chunks in flight; chunks 0 and 1 of the shared operands go to the ring ----
    Shared sh[LOADER ? 1 : DEPTH];   // invariant at round t: sh[(t + 2) % DEPTH] holds this wavefront's share of chunk t+2
    Private pv[DEPTH];               // pv[t % DEPTH] holds chunk t
    if constexpr (!LOADER) {
#pragma unroll
        for (int s = 0; s < DEPTH; s++) issue_shared(sh[s], s);
    }
#pragma unroll
    for (int s = 0; s < DEPTH; s++) issue_private(pv[s], s);
    if constexpr (!LOADER) {
        shared_to_lds(0, sh[0]);
        shared_to_lds(1, sh[1]);
        issue_shared(sh[0], DEPTH);
        issue_shared(sh[1], DEPTH + 1);
    }
    Operands op[2];
    Outputs out[2];
    lds_barrier();
    read_ring(op[0], 0);
    // one round: chunk `step`, register set s & 1; the previous chunk's outputs go to memory first
    // One round = chunk `step`, register set s & 1: the matrix work of the chunk and the round's memory and LDS
    // traffic (the previous chunk's outputs to memory, chunk step+2's share to the ring, chunk step+1's operands
    // from the ring, refills).  Even wavefronts do the traffic first, odd ones the matrix work first, so that
    // one pair's traffic overlaps the other pair's arithmetic instead of all four queueing on the same pipe.
    auto traffic = [&](int step, int s, bool refill) {
        if (step > 0) store_outputs(step - 1, out[(s & 1) ^ 1]);
        if constexpr (!LOADER) {
            shared_to_lds(step + 2, sh[(s + 2) % DEPTH]);
            if (refill) issue_shared(sh[(s + 2) % DEPTH], step + 2 + DEPTH);
        }
        read_ring(op[(s & 1) ^ 1], step + 1);   // needed a whole chunk from now; written to the ring one round ago
    };
    auto rounds = [&](auto compute_first) {
        constexpr bool CF = decltype(compute_first)::value;
        int step0 = 0;
        for (; step0 + DEPTH <= LS; step0 += DEPTH) {
#pragma unroll
            for (int s = 0; s < DEPTH; s++) {
                if constexpr (!CF) traffic(step0 + s, s, true);
                compute(op[s & 1], pv[s], out[s & 1]);
                if constexpr (CF) traffic(step0 + s, s, true);
                issue_private(pv[s], step0 + s + DEPTH);
                lds_barrier();
            }
        }
#pragma unroll
        for (int s = 0; s < DEPTH - 1; s++) {   // the remaining NC % DEPTH chunks are already in flight or in registers
            if (step0 + s < LS) {
                if constexpr (!CF) traffic(step0 + s, s, false);
                compute(op[s & 1], pv[s], out[s & 1]);
                if constexpr (CF) traffic(step0 + s, s, false);
                lds_barrier();
            }
        }
    };
    if constexpr (LOADER) {
        rounds(std::false_type{});
    } else {
        if (ib & 1) rounds(std::true_type{});
        else rounds(std::false_type{});
    }
    if ((LS - 1) & 1) store_outputs(LS - 1, out[1]);
    else store_outputs(LS - 1, out[0]);
    if constexpr (MAP) {
        // s_out: [pair][segment][2][64][64] floats; N in state order, M transposed (MT[j][j'] = M[j'][j]) so that the
        // carry kernel reads it as the operand fragment it needs
        float* dst = static_cast<float*>(s_out) + ((long)bx * 2 + part) * HEAD * HEAD;
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            if (part == 0) {
                *reinterpret_cast<f32x4*>(dst + (16 * ib + L.n) * HEAD + 16 * jb + 4 * L.g) = S[jb];
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++) dst[(16 * jb + 4 * L.g + r) * HEAD + 16 * ib + L.n] = S[jb][r];
            }
        }
    } else if (seg == NSEG - 1) {
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) store_state_frag(s_out, s_out_f32, bh, ib, jb, L, S[jb]);
    }
}

// ------------------------------------------------------------------------------------------------
// Composes the segment maps in processing order: S_in(0) = s0, S_in(g+1) = S_in(g) M_g + N_g, all in fp32 (fp32
// matrix instructions).  One block per (batch, head), wavefront = 16 value rows.  maps: as written by the MAP
// pass; s_seg: [pair][segment][64][64] floats, the state entering each segment.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void segment_carry_kernel(int NSEG, int s0_f32, const void* __restrict__ s0,
                                                            const float* __restrict__ maps, float* __restrict__ s_seg) {
    const int ib = threadIdx.x >> 6;
    const int bh = blockIdx.x;
    const Lane L;
    f32x4 S[NBLK];
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) S[jb] = load_state_frag(s0, s0_f32, bh, ib, jb, L);
    // the maps of a segment do not depend on the state: those of the next segment are loaded while this one's
    // products run (the chain is 64 dependent matrix instructions per segment; the loads were as long again)
    struct Maps {
        f32x4 n[NBLK], mt[NBLK][NBLK];
    };
    auto issue = [&](Maps& m, int g) {
        g = g < NSEG - 1 ? g : NSEG - 2;
        const long e = (long)bh * NSEG + g;
        const float* N = maps + (e * 2 + 0) * HEAD * HEAD;
        const float* MT = maps + (e * 2 + 1) * HEAD * HEAD;
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            m.n[jb] = *reinterpret_cast<const f32x4*>(N + (16 * ib + L.n) * HEAD + 16 * jb + 4 * L.g);
#pragma unroll
            for (int kb = 0; kb < NBLK; kb++)   // A operand of S[ib][kb] M[kb][jb]: F(M[kb][jb]^T) = the (jb, kb) block of MT
                m.mt[jb][kb] = *reinterpret_cast<const f32x4*>(MT + (16 * jb + L.n) * HEAD + 16 * kb + 4 * L.g);
        }
    };
    auto apply = [&](const Maps& m) {
        f32x4 T[NBLK];
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            f32x4 acc = m.n[jb];
#pragma unroll
            for (int kb = 0; kb < NBLK; kb++) acc = mma_f32(acc, m.mt[jb][kb], S[kb]);
            T[jb] = acc;
        }
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) S[jb] = T[jb];
    };
    auto store = [&](int g) {
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) store_state_frag(s_seg, 1, bh * NSEG + g, ib, jb, L, S[jb]);
    };
    Maps m[2];
    issue(m[0], 0);
    int g = 0;
    for (; g + 2 < NSEG; g += 2) {   // NSEG is a power of two, at least 2
        store(g);
        issue(m[1], g + 1);
        __builtin_amdgcn_sched_barrier(0);   // (the compiler would sink the loads to just before their use)
        apply(m[0]);
        store(g + 1);
        issue(m[0], g + 2);
        __builtin_amdgcn_sched_barrier(0);
        apply(m[1]);
    }
    store(g);
    apply(m[0]);
    store(g + 1);
}


// ------------------------------------------------------------------------------------------------
// attn_ln epilogue: one wavefront per chunk applies GroupNorm + bonus + gate to the WKV7 output the scan
// left in y_wkv (kept, bf16, for the backward pass; centred per block when `centers` is given, see ln_epilogue.hpp).
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ln_epilogue_kernel(int T, int H, int nchunks, const __bf16* __restrict__ y_wkv,
                                                          const float* __restrict__ centers, const __bf16* __restrict__ q_, const __bf16* __restrict__ k_,
                                                          const __bf16* __restrict__ v_, const __bf16* __restrict__ g_,
                                                          const float* __restrict__ params, __bf16* __restrict__ y_) {
    const int cid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (cid >= nchunks) return;
    const Lane L;
    const ChunkAddr ca(cid, T, H);
    const TileB yw = load_rows16(y_wkv + ca.row0, ca.ld, L);
    const TileB q = load_rows16(q_ + ca.row0, ca.ld, L);
    const TileB k = load_rows16(k_ + ca.row0, ca.ld, L);
    const TileB v = load_rows16(v_ + ca.row0, ca.ld, L);
    const TileB g = load_rows16(g_ + ca.row0, ca.ld, L);
    const LnParams p = load_ln_params(params, ca.bh % H, H, L);
    const TileF yf = uncentre(yw, centers, ca.row0 / HEAD + (long)L.n * H);   // (row0 / 64 = token * H + head of the chunk's first token)
    store_rows16(y_ + ca.row0, ca.ld, L, ln_forward(yf, q, k, v, g, p));
}

// ------------------------------------------------------------------------------------------------
// host launchers
// ------------------------------------------------------------------------------------------------
void launch_fwd_prepare(int B, int T, int H, const void* w, const void* q, const void* k, const void* v, const void* a,
                        const void* b, void* rec, hipStream_t stream) {
    const int nchunks = B * H * (T / CHUNK);
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    hipLaunchKernelGGL(fwd_prepare_kernel, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(w), c(q), c(k),
                       c(v), c(a), c(b), static_cast<__bf16*>(rec));
}

// Segments per (batch, head): a power of two that fills an MI355X's 256 compute units when B*H is small and the
// sequence long, leaving at least 64 chunks per segment (the extra pass re-reads the records, which only pays
// while the scan is bound by its chain and not by memory); 1 = the plain one-pass scan, which for head size 64
// means the one-kernel organisation of wkv7_fused.hip.  Only for a fifth of the compute units' worth of (batch, head)
// pairs or fewer: the segmented path moves 3.6 times the caller's bytes at the memory system's rate, the one-kernel
// path runs a chain of T/16 steps of ~0.63 us on two compute units per pair, and the two cross near 55 pairs
// (measured, forward+backward: 56 pairs x 8192 tokens 913 against 905 us, 64 x 4096 562 against 495 us, 96 x 2048
// 440 against 315 us, segmented against one kernel).
int scan_segments(int B, int T, int H) {
    const int BH = B * H, NC = T / CHUNK;
    int g = 1;
    if (BH * 5 > compute_units()) return 1;
    while (g < 8 && BH * g * 2 <= compute_units() && NC % (g * 2) == 0 && NC / (g * 2) >= 64) g *= 2;
    return g;
}
size_t scan_segment_workspace_bytes(int B, int T, int H) {
    const int g = scan_segments(B, T, H);
    return g == 1 ? 0 : (size_t)B * H * g * 3 * HEAD * HEAD * sizeof(float);   // N, M^T and the entering state per segment
}

template <typename R, bool WITH_Y, bool SAVE = true>
static void launch_scan(int B, int T, int H, int reverse, int state_f32, void* rec, const void* s_in, void* s_out, void* y,
                        void* seg_ws, int pairs, hipStream_t stream, float* centers = nullptr) {
    const int keep = pairs ? reverse : -1;   // which chunks' states stay in the records (see the kernel)
    const int BH = B * H, NC = T / CHUNK, g = scan_segments(B, T, H);
    __bf16* r = static_cast<__bf16*>(rec);
    __bf16* yy = static_cast<__bf16*>(y);
    constexpr bool LOADER = !WITH_Y;          // measured best: see the kernel's comment
    constexpr int DEPTH = WITH_Y ? 6 : SCAN_DEPTH;
    constexpr int THREADS = LOADER ? SCAN_THREADS + 64 : SCAN_THREADS;
    if (g == 1) {
        // idle compute units (an MI355X has 256) pre-read the records; see the kernel
        const int cus = compute_units();
        const int helpers = BH < cus - cus / 8 ? (cus - BH < cus * 5 / 8 ? cus - BH : cus * 5 / 8) : 0;
        hipLaunchKernelGGL((state_scan_kernel<R, WITH_Y, LOADER, DEPTH, false, SAVE>), dim3(BH + helpers), dim3(THREADS), 0, stream, NC, NC,
                           1, H, reverse, state_f32, state_f32, r, s_in, s_out, yy, BH, keep, centers);
        return;
    }
    float* maps = static_cast<float*>(seg_ws);
    float* s_seg = maps + (size_t)BH * g * 2 * HEAD * HEAD;
    hipLaunchKernelGGL((state_scan_kernel<R, false, false, 4, true>), dim3(BH * g), dim3(2 * SCAN_THREADS), 0, stream, NC,
                       NC / g, g, H, reverse, 1, 1, r, nullptr, maps, nullptr, BH * g, -1, nullptr);
    hipLaunchKernelGGL(segment_carry_kernel, dim3(BH), dim3(256), 0, stream, g, state_f32, s_in, maps, s_seg);
    hipLaunchKernelGGL((state_scan_kernel<R, WITH_Y, LOADER, DEPTH, false, SAVE>), dim3(BH * g), dim3(THREADS), 0, stream, NC, NC / g, g,
                       H, reverse, 1, state_f32, r, s_seg, s_out, yy, BH * g, keep, centers);
}

void launch_fwd_scan(int B, int T, int H, int state_f32, void* rec, const void* s_in, void* s_out, void* y, void* seg_ws,
                     int save, int pairs, hipStream_t stream, float* centers) {
    if (save) launch_scan<RecFwd, true, true>(B, T, H, 0, state_f32, rec, s_in, s_out, y, seg_ws, pairs, stream, centers);
    else launch_scan<RecFwd, true, false>(B, T, H, 0, state_f32, rec, s_in, s_out, y, seg_ws, 0, stream, centers);
}

void launch_bwd_scan(int B, int T, int H, int state_f32, void* rec, const void* s_in, void* s_out, void* seg_ws,
                     int pairs, hipStream_t stream) {
    launch_scan<RecBwd, false>(B, T, H, 1, state_f32, rec, s_in, s_out, nullptr, seg_ws, pairs, stream);
}

void launch_ln_epilogue(int B, int T, int H, const void* y_wkv, const float* centers, const void* q, const void* k,
                        const void* v, const void* g, const void* params, void* y, hipStream_t stream) {
    const int nchunks = B * H * (T / CHUNK);
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    hipLaunchKernelGGL(ln_epilogue_kernel, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(y_wkv), centers, c(q),
                       c(k), c(v), c(g), static_cast<const float*>(params), static_cast<__bf16*>(y));
}

}  // namespace wkv
