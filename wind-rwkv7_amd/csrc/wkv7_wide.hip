// WKV7 on the matrix cores for head sizes other than 64: C = 16 NB channels per head, NB = 1 .. 8 (16 .. 128).
//
// The reference compiles its CUDA kernel per head size (rwkv7_attn.py:46-51) and serves large heads with
// rwkv7_attn_triton_bighead.py:31-322 (one program per (batch, head) that walks the chunks with the state tiled
// through memory).  Same chunked algebra here (chunks of 16 tokens, rwkv7_attn_triton.py:27-156), organised as
// three phases per direction so that only the state update is sequential:
//
//   forward   prepare (one wavefront per chunk):  Tinv = inv(I - strict_tril(wa bwi^T)),
//                                                 U0 = Tinv strict_tril(wa kwi^T) V,  Wm = Tinv wa, kf, bf, wq, QK, QB
//             scan (one wavefront per 16 value rows, its strip of the state in fp32 registers; blocks of four,
//                   ceil(NB / 4) blocks per (batch, head)):
//                                                 U = U0 + Wm S^T;  Y = QK V + QB U + wq S^T;
//                                                 S <- S diag(fw) + V^T kf + U^T bf        (keeps S and U per chunk)
//   backward  prepare:  D0 = Tinv^T QB^T dY,  Bm = Tinv^T bf, wq^T, wa^T
//             scan (reverse):                     D = D0 + Bm dS^T;  dS <- dS diag(fw) + dY^T wq + D^T wa
//             gradients (one wavefront per chunk) from S, U, dS, D of the chunk.
//
// Everything is a 16x16 fragment (frag.hpp).  The chunk-parallel kernels use v_mfma_f32_16x16x16_bf16 throughout,
// the scan v_mfma_f32_16x16x32_bf16 throughout (two key blocks, or the (V, U) pair, per instruction), so no
// accumulator ever passes between instructions of different shapes.  Channels keep their natural
// order (block jb = channels 16 jb .. 16 jb + 15).  The head-size-64 kernels (wkv7_fused.hip, wkv7_bwd.hip) are
// the tuned form of the same algebra; this file trades their producer/consumer overlap for one template over NB.
// At the end of the file: the single-token step (decoding) for the same head sizes.
#include "wkv7_wide_kernels.hpp"

#include "frag.hpp"

namespace wkv {
namespace wide {
namespace {

template <int NB>
struct TB {
    bf16x4 f[NB];
};

// chunk cid = (b*H + h)*NC + c of a [B,T,H,16 NB] tensor
template <int NB>
struct Addr {
    int bh, c;
    long row0, ld;
    __device__ Addr(int cid, int T, int H) {
        const int NC = T / CHUNK;
        bh = cid / NC;
        c = cid - bh * NC;
        const int b = bh / H, h = bh - b * H;
        ld = (long)H * 16 * NB;
        row0 = ((long)b * T + (long)c * CHUNK) * ld + (long)h * 16 * NB;
    }
};

// fragment jb of the chunk's [16 tokens x C] tile: lane (n, g) holds channels 16 jb + 4g .. + 3 of token n
__device__ __forceinline__ bf16x4 load_frag_rows(const __bf16* __restrict__ p, long ld, int jb, const Lane& L) {
    return *reinterpret_cast<const bf16x4*>(p + (long)L.n * ld + 16 * jb + 4 * L.g);
}
__device__ __forceinline__ void store_frag_rows(__bf16* __restrict__ p, long ld, int jb, const Lane& L, bf16x4 x) {
    *reinterpret_cast<bf16x4*>(p + (long)L.n * ld + 16 * jb + 4 * L.g) = x;
}
template <int NB>
__device__ __forceinline__ TB<NB> load_tile(const __bf16* __restrict__ p, long ld, const Lane& L) {
    TB<NB> t;
#pragma unroll
    for (int i = 0; i < NB; i++) t.f[i] = load_frag_rows(p, ld, i, L);
    return t;
}

// F(X Y^T), contraction over the C channels
template <int NB>
__device__ __forceinline__ f32x4 xyT(const TB<NB>& X, const TB<NB>& Y) {
    f32x4 acc = zero4();
#pragma unroll
    for (int i = 0; i < NB; i++) acc = mma(acc, Y.f[i], X.f[i]);
    return acc;
}

// Decay factors of one block of 16 channels (see chunk_decay in wkv7_common.hpp): lw = -exp(w), P = exp(prefix
// sum of lw over the chunk's tokens), Pi = 1/P as its own exponential, Px = P of the token before (1 at the first),
// fw = P of the last token.
struct DecayF {
    f32x4 lw, P, Pi, Px, fw;
};
__device__ __forceinline__ DecayF decay_frag(bf16x4 w) {
    DecayF d;
    constexpr float LOG2E = 1.4426950408889634f;
    const f32x4 wf = to_f32(w);
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const float lw = -__expf(wf[r]);
        const float lc2 = row_prefix_sum(lw) * LOG2E;
        const float P = __builtin_amdgcn_exp2f(lc2);
        d.lw[r] = lw;
        d.P[r] = P;
        d.Pi[r] = __builtin_amdgcn_exp2f(-lc2);
        d.Px[r] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0x3f800000, __builtin_bit_cast(int, P), 0x111, 0xf, 0xf, false));
        d.fw[r] = row_bcast_last(P);
    }
    return d;
}

// ---- per-chunk records ----
// A fragment is 256 bf16 (512 bytes, lane-major: lane l owns elements 4l .. 4l+3); a PAIR is two fragments side by
// side, lane l owning 16 bytes at element 8l (first fragment, then second), read with one 16-byte load and used as
// the two halves of one 16x16x32 operand.  What a direction's prepare kernel hands to its scan:
//   XZ[jb]  pair, lane = key ch, reg = token     forward (kf^T, bf^T)          backward (wq^T, wa^T)
//   I[ib]   pair, lane = value ch, reg = token   forward (U0^T, V^T)           backward (D0^T, dY^T)
//   forward:   MW[jb] pair, lane = token, reg = key ch: (Wm = Tinv wa, wq);  Q pair (QK, QB), lane = token t, reg = token s
//   backward:  M[jb] fragment, lane = token, reg = key ch: Bm = Tinv^T bf
//   FW      16 NB floats
constexpr long PAIR_ELEMS = 2 * FRAG_ELEMS;
// Order in memory: XZ, MW (backward: M), Q (forward), FW - what every wavefront of a head needs, one contiguous run
// of SHARED_BYTES that the scan copies into LDS as it is - then I, which each wavefront reads for itself.
template <int NB, bool FWD>
struct Rec {
    static constexpr long XZ = 0, MW = NB * PAIR_ELEMS, Q = 2 * NB * PAIR_ELEMS;
    static constexpr long FW = FWD ? (2 * NB + 1) * PAIR_ELEMS : NB * PAIR_ELEMS + NB * FRAG_ELEMS;   // offsets in bf16 elements
    static constexpr long I = FW + 32 * NB;                       // after the 16 NB floats
    static constexpr long ELEMS = I + NB * PAIR_ELEMS;
    static constexpr int SHARED_BYTES = (int)(I * 2);
    // element offsets of a chunk's pieces
    __host__ __device__ static long xz(long cid, int jb) { return cid * ELEMS + XZ + jb * PAIR_ELEMS; }
    __host__ __device__ static long i(long cid, int ib) { return cid * ELEMS + I + ib * PAIR_ELEMS; }
    __host__ __device__ static long mw(long cid, int jb) { return cid * ELEMS + MW + jb * PAIR_ELEMS; }      // forward
    __host__ __device__ static long q(long cid) { return cid * ELEMS + Q; }                                  // forward
    __host__ __device__ static long m(long cid, int jb) { return cid * ELEMS + MW + jb * FRAG_ELEMS; }       // backward
    __device__ static float* fw(__bf16* rec, long cid) { return reinterpret_cast<float*>(rec + cid * ELEMS + FW); }
    __device__ static const float* fw(const __bf16* rec, long cid) { return reinterpret_cast<const float*>(rec + cid * ELEMS + FW); }
};
__device__ __forceinline__ void store_pair(__bf16* __restrict__ p, int lane, bf16x4 u, bf16x4 v) {
    *reinterpret_cast<bf16x8*>(p + 8 * lane) = __builtin_shufflevector(u, v, 0, 1, 2, 3, 4, 5, 6, 7);
}
// one half of a pair: which = 0 first fragment, 1 second
__device__ __forceinline__ void store_half(__bf16* __restrict__ p, int lane, int which, bf16x4 u) {
    *reinterpret_cast<bf16x4*>(p + 8 * lane + 4 * which) = u;
}
__device__ __forceinline__ bf16x8 load_pair(const __bf16* __restrict__ p, int lane) {
    return *reinterpret_cast<const bf16x8*>(p + 8 * lane);
}
__device__ __forceinline__ bf16x8 join(bf16x4 u, bf16x4 v) { return __builtin_shufflevector(u, v, 0, 1, 2, 3, 4, 5, 6, 7); }
__device__ __forceinline__ bf16x4 zero_bf16() { return bf16x4{}; }
// What a scan keeps per chunk for the gradient kernel: the state entering the chunk (backward: the state gradient
// arriving at its end) as bf16 fragments CK[jb][ib] = F(S[16 ib .., 16 jb ..]) (lane = value row, reg = key column;
// all value blocks of one key block side by side, the order the gradient kernel reads them in), then UT[ib] =
// F(U_ib^T) (backward D^T; lane = value ch, reg = token).
template <int NB>
struct Kept {
    static constexpr long UT = (long)NB * NB * FRAG_ELEMS;
    static constexpr long ELEMS = UT + (long)NB * FRAG_ELEMS;
    __device__ static long ck(long cid, int jb, int ib) { return cid * ELEMS + (long)(jb * NB + ib) * FRAG_ELEMS; }
    __device__ static long ut(long cid, int ib) { return cid * ELEMS + UT + (long)ib * FRAG_ELEMS; }
};

// ------------------------------------------------------------------------------------------------
// forward prepare: one wavefront per chunk
// ------------------------------------------------------------------------------------------------
template <int NB>
__global__ __launch_bounds__(256) void fwd_prepare_kernel(int T, int H, int nchunks, const __bf16* __restrict__ w_,
                                                          const __bf16* __restrict__ q_, const __bf16* __restrict__ k_,
                                                          const __bf16* __restrict__ v_, const __bf16* __restrict__ a_,
                                                          const __bf16* __restrict__ b_, __bf16* __restrict__ rec) {
    using R = Rec<NB, true>;
    const int lane = threadIdx.x & 63;
    const int cid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (cid >= nchunks) return;
    const Lane L;
    const Addr<NB> ca(cid, T, H);
    const bf16x4 eye = identity_bf16(L);

    // all of the chunk's rows are requested before any is used (the compiler would place each load next to its
    // use and wait for it there)
    const TB<NB> w = load_tile<NB>(w_ + ca.row0, ca.ld, L), q = load_tile<NB>(q_ + ca.row0, ca.ld, L);
    const TB<NB> k = load_tile<NB>(k_ + ca.row0, ca.ld, L), a = load_tile<NB>(a_ + ca.row0, ca.ld, L);
    const TB<NB> b = load_tile<NB>(b_ + ca.row0, ca.ld, L), v = load_tile<NB>(v_ + ca.row0, ca.ld, L);
    __builtin_amdgcn_sched_barrier(0);
    TB<NB> wq, wa, kwi, bwi;
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
        const DecayF d = decay_frag(w.f[jb]);
        const f32x4 kwi_f = to_f32(k.f[jb]) * d.Pi;
        const f32x4 bwi_f = to_f32(b.f[jb]) * d.Pi;
        wq.f[jb] = to_bf16(to_f32(q.f[jb]) * d.P);
        wa.f[jb] = to_bf16(to_f32(a.f[jb]) * d.Px);
        kwi.f[jb] = to_bf16(kwi_f);
        bwi.f[jb] = to_bf16(bwi_f);
        store_pair(rec + R::xz(cid, jb), lane, transpose(to_bf16(kwi_f * d.fw), eye), transpose(to_bf16(bwi_f * d.fw), eye));
        store_half(rec + R::mw(cid, jb), lane, 1, wq.f[jb]);
        if (L.n == 0) *reinterpret_cast<f32x4*>(R::fw(rec, cid) + 16 * jb + 4 * L.g) = d.fw;
    }
    const f32x4 AB = mask_lower_strict(xyT(wa, bwi), L);     // [t][s] = wa_t . bwi_s, s < t
    const f32x4 ABT = mask_upper_strict(xyT(bwi, wa), L);
    const bf16x4 AK = to_bf16(mask_lower_strict(xyT(wa, kwi), L));
    store_pair(rec + R::q(cid), lane, to_bf16(mask_lower_incl(xyT(wq, kwi), L)), to_bf16(mask_lower_incl(xyT(wq, bwi), L)));
    f32x4 Tinv, TinvT;
    tri_inverse(AB, ABT, L, Tinv, TinvT);
    const bf16x4 Tinv_b = to_bf16(Tinv);
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        const bf16x4 VT = transpose(v.f[ib], eye);                                      // F(V_ib^T)
        const f32x4 RT = mma(zero4(), AK, VT);                                          // F((AK V_ib)^T)
        store_pair(rec + R::i(cid, ib), lane, to_bf16(mma(zero4(), Tinv_b, to_bf16(RT))), VT);
    }
#pragma unroll
    for (int jb = 0; jb < NB; jb++)   // F(Tinv wa_jb): lane = token, reg = key ch
        store_half(rec + R::mw(cid, jb), lane, 0, to_bf16(mma(zero4(), transpose(wa.f[jb], eye), Tinv_b)));
}

// ------------------------------------------------------------------------------------------------
// backward prepare: one wavefront per chunk
// ------------------------------------------------------------------------------------------------
template <int NB>
__global__ __launch_bounds__(256) void bwd_prepare_kernel(int T, int H, int nchunks, const __bf16* __restrict__ w_,
                                                          const __bf16* __restrict__ q_, const __bf16* __restrict__ a_,
                                                          const __bf16* __restrict__ b_, const __bf16* __restrict__ dy_,
                                                          __bf16* __restrict__ rec) {
    using R = Rec<NB, false>;
    const int lane = threadIdx.x & 63;
    const int cid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (cid >= nchunks) return;
    const Lane L;
    const Addr<NB> ca(cid, T, H);
    const bf16x4 eye = identity_bf16(L);

    const TB<NB> w = load_tile<NB>(w_ + ca.row0, ca.ld, L), q = load_tile<NB>(q_ + ca.row0, ca.ld, L);
    const TB<NB> a = load_tile<NB>(a_ + ca.row0, ca.ld, L), b = load_tile<NB>(b_ + ca.row0, ca.ld, L);
    const TB<NB> dy = load_tile<NB>(dy_ + ca.row0, ca.ld, L);
    __builtin_amdgcn_sched_barrier(0);
    TB<NB> wq, wa, bwi, bf;
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
        const DecayF d = decay_frag(w.f[jb]);
        const f32x4 bwi_f = to_f32(b.f[jb]) * d.Pi;
        wq.f[jb] = to_bf16(to_f32(q.f[jb]) * d.P);
        wa.f[jb] = to_bf16(to_f32(a.f[jb]) * d.Px);
        bwi.f[jb] = to_bf16(bwi_f);
        bf.f[jb] = to_bf16(bwi_f * d.fw);
        store_pair(rec + R::xz(cid, jb), lane, transpose(wq.f[jb], eye), transpose(wa.f[jb], eye));
        if (L.n == 0) *reinterpret_cast<f32x4*>(R::fw(rec, cid) + 16 * jb + 4 * L.g) = d.fw;
    }
    const f32x4 AB = mask_lower_strict(xyT(wa, bwi), L);
    const f32x4 ABT = mask_upper_strict(xyT(bwi, wa), L);
    const bf16x4 QBT = to_bf16(mask_upper_incl(xyT(bwi, wq), L));   // [s][t] = wq_t . bwi_s, s <= t
    f32x4 Tinv, TinvT;
    tri_inverse(AB, ABT, L, Tinv, TinvT);
    const bf16x4 TinvT_b = to_bf16(TinvT);
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        const bf16x4 dYT = transpose(dy.f[ib], eye);
        const f32x4 ET = mma(zero4(), QBT, dYT);                                  // F((QB^T dY_ib)^T)
        store_pair(rec + R::i(cid, ib), lane, to_bf16(mma(zero4(), TinvT_b, to_bf16(ET))), dYT);
    }
#pragma unroll
    for (int jb = 0; jb < NB; jb++)   // F(Tinv^T bf_jb): lane = token, reg = key ch
        store_frag(rec + R::m(cid, jb), lane, to_bf16(mma(zero4(), transpose(bf.f[jb], eye), TinvT_b)));
}

// ------------------------------------------------------------------------------------------------
// scan: wavefront ib owns value rows 16 ib .. 16 ib + 15 of the state (NB fp32 fragments); a block is up to four of
// them (one per SIMD, each with the whole register file), a (batch, head) takes ceil(NB / 4) blocks.  Rows of the
// state evolve independently, so the wavefronts never exchange results.  What they share is the chunk's operands
// (all but the (U0, V) pair of their own value block): the block's wavefronts each fetch a quarter of that run of the
// record, three chunks ahead, and hand it on through a ring of three LDS slots two chunks ahead of its use; one
// LDS-only barrier per chunk.  (Each wavefront fetching everything for itself needs three sets of 104 registers at
// C = 128 for the same distance; beyond 256 registers the allocator parks freshly loaded values in accumulator
// registers, which waits for the load: 1.4 us per chunk instead of 0.5.)
// ------------------------------------------------------------------------------------------------
template <int NB, bool FWD>
struct ScanOps {
    bf16x8 xz[NB], mw[FWD ? NB : 1], q;   // pairs
    bf16x4 m[FWD ? 1 : NB];
    f32x4 fw[NB];
};

template <int NB, bool FWD, bool KEEP>
__global__ __launch_bounds__(256) void scan_kernel(int T, int H, int state_f32, const __bf16* __restrict__ rec,
                                                   const void* __restrict__ s_in, void* __restrict__ s_out,
                                                   __bf16* __restrict__ y_, __bf16* __restrict__ kept,
                                                   float* __restrict__ centers) {
    using R = Rec<NB, FWD>;
    using K = Kept<NB>;
    constexpr int C = 16 * NB, NP = (NB + 1) / 2;   // key blocks are contracted two at a time (one 16x16x32 instruction)
    constexpr int NU = (R::SHARED_BYTES + 1023) / 1024;   // units of 1 KiB (16 bytes per lane) of the shared run
    constexpr int UPW = (NU + 3) / 4;                     // units per wavefront in a full block (more in a partial one)
    constexpr int SLOT = NU * 1024, SLOTS = 3, DG = 3;    // ring; chunks a fetch runs ahead of its hand-over
    __shared__ __attribute__((aligned(16))) unsigned char ring[SLOTS * SLOT];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, ib = 4 * blockIdx.y + wave;
    const int bh = blockIdx.x, NC = T / CHUNK;
    const Lane L;

    // chunk of step i (clamped past the end: a fetch beyond the last chunk re-reads it)
    auto chunk_of = [&](int i) {
        const int j = i < NC ? i : NC - 1;
        return (long)bh * NC + (FWD ? j : NC - 1 - j);
    };
    // this wavefront's units of the shared run: wave, wave + 4, ... (indices past the end repeat the last unit: the
    // same bytes to the same place).  Every block has four wavefronts for this; those without a value block of
    // their own (NB no multiple of four) only keep the ring filled.
    struct Stage {
        f32x4 u[UPW];
    };
    auto unit = [&](int k) { const int u = wave + 4 * k; return u < NU ? u : NU - 1; };
    auto issue = [&](Stage& st, int step) {
        const char* base = reinterpret_cast<const char*>(rec + chunk_of(step) * R::ELEMS);
#pragma unroll
        for (int k = 0; k < UPW; k++) st.u[k] = *reinterpret_cast<const f32x4*>(base + unit(k) * 1024 + lane * 16);
    };
    auto to_ring = [&](int step, const Stage& st) {
        unsigned char* slot = ring + (step % SLOTS) * SLOT;
#pragma unroll
        for (int k = 0; k < UPW; k++) *reinterpret_cast<f32x4*>(slot + unit(k) * 1024 + lane * 16) = st.u[k];
    };
    Stage st[DG];
    if (ib >= NB) {   // ring duty only: the same hand-overs and barriers as the working wavefronts below
#pragma unroll
        for (int d = 0; d < DG; d++) issue(st[d], d);
        to_ring(0, st[0]);
        to_ring(1, st[1]);
        issue(st[0], DG);
        issue(st[1], DG + 1);
        lds_barrier();
        int i = 0;
        for (; i + DG <= NC; i += DG) {
#pragma unroll
            for (int d = 0; d < DG; d++) {
                to_ring(i + d + 2, st[(d + 2) % DG]);
                issue(st[(d + 2) % DG], i + d + 2 + DG);
                lds_barrier();
            }
        }
#pragma unroll
        for (int d = 0; d < DG - 1; d++) {
            if (i + d < NC) {
                to_ring(i + d + 2, st[(d + 2) % DG]);
                lds_barrier();
            }
        }
        return;
    }

    auto state_off = [&](int jb) { return ((long)bh * C + 16 * ib + L.n) * C + 16 * jb + 4 * L.g; };
    f32x4 S[NB];
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
        if (s_in == nullptr) S[jb] = zero4();
        else if (state_f32) S[jb] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(s_in) + state_off(jb));
        else S[jb] = to_f32(*reinterpret_cast<const bf16x4*>(static_cast<const __bf16*>(s_in) + state_off(jb)));
    }
    auto read_ring = [&](ScanOps<NB, FWD>& o, int step) {
        const unsigned char* slot = ring + (step % SLOTS) * SLOT;
#pragma unroll
        for (int jb = 0; jb < NB; jb++) {
            if constexpr (FWD) o.mw[jb] = *reinterpret_cast<const bf16x8*>(slot + (R::MW + jb * PAIR_ELEMS) * 2 + lane * 16);
            else o.m[jb] = *reinterpret_cast<const bf16x4*>(slot + (R::MW + jb * FRAG_ELEMS) * 2 + lane * 8);
        }
#pragma unroll
        for (int jb = 0; jb < NB; jb++) {
            o.xz[jb] = *reinterpret_cast<const bf16x8*>(slot + (R::XZ + jb * PAIR_ELEMS) * 2 + lane * 16);
            o.fw[jb] = *reinterpret_cast<const f32x4*>(slot + R::FW * 2 + (16 * jb + 4 * L.g) * 4);
        }
        if constexpr (FWD) o.q = *reinterpret_cast<const bf16x8*>(slot + R::Q * 2 + lane * 16);
    };
    auto load_private = [&](int step) { return load_pair(rec + R::i(chunk_of(step), ib), lane); };
    auto lo = [](bf16x8 p) { return __builtin_shufflevector(p, p, 0, 1, 2, 3); };
    auto hi = [](bf16x8 p) { return __builtin_shufflevector(p, p, 4, 5, 6, 7); };

    auto step = [&](const ScanOps<NB, FWD>& o, bf16x8 iv, int i) {
        const long cid = chunk_of(i);
        bf16x4 Sb[2 * NP];
#pragma unroll
        for (int jb = 0; jb < NB; jb++) {
            Sb[jb] = to_bf16(S[jb]);
            if constexpr (KEEP) store_frag(kept + K::ck(cid, jb, ib), lane, Sb[jb]);
        }
        if constexpr (NB & 1) Sb[NB] = zero_bf16();
        // F(U_ib^T) = F(U0_ib^T + S_ib Wm^T), two partial sums (the products are one dependent chain otherwise)
        f32x4 UT = to_f32(lo(iv)), UT1 = zero4();
#pragma unroll
        for (int p = 0; p < NP; p++) {
            bf16x4 m0, m1;
            if constexpr (FWD) {
                m0 = lo(o.mw[2 * p]);
                m1 = 2 * p + 1 < NB ? lo(o.mw[2 * p + 1 < NB ? 2 * p + 1 : 0]) : zero_bf16();
            } else {
                m0 = o.m[2 * p];
                m1 = 2 * p + 1 < NB ? o.m[2 * p + 1 < NB ? 2 * p + 1 : 0] : zero_bf16();
            }
            if (p & 1) UT1 = mma8(UT1, join(m0, m1), join(Sb[2 * p], Sb[2 * p + 1]));
            else UT = mma8(UT, join(m0, m1), join(Sb[2 * p], Sb[2 * p + 1]));
        }
        const bf16x4 UTb = to_bf16(UT + UT1);
        if constexpr (KEEP) store_frag(kept + K::ut(cid, ib), lane, UTb);
        const bf16x8 VU = join(hi(iv), UTb);      // (V^T, U^T) forward, (dY^T, D^T) backward
        if constexpr (FWD) {
            f32x4 Y = mma8(zero4(), VU, o.q);     // F(QK V_ib + QB U_ib): lane = token, reg = value ch
#pragma unroll
            for (int p = 0; p < NP; p++) {        // + wq S_ib^T
                const bf16x4 w1 = 2 * p + 1 < NB ? hi(o.mw[2 * p + 1 < NB ? 2 * p + 1 : 0]) : zero_bf16();
                Y = mma8(Y, join(Sb[2 * p], Sb[2 * p + 1]), join(hi(o.mw[2 * p]), w1));
            }
            const Addr<NB> ca((int)cid, T, H);
            // centers != nullptr (the output is attn_ln's kept one): written centred per token and block of 16 channels,
            // the centres [token][head][block] beside it, so that its bf16 rounding is relative to the spread GroupNorm
            // divides by and not to the mean
            if (centers != nullptr) {
                const float cen = row_sum16_bf16(Y) * (1.f / 16);
                Y = Y - cen;
                const int bb = ca.bh / H, hh = ca.bh - bb * H;
                centers[(((long)bb * T + (long)ca.c * CHUNK + L.n) * H + hh) * NB + ib] = cen;   // (the four lanes of a token write the same value)
            }
            store_frag_rows(y_ + ca.row0, ca.ld, ib, L, to_bf16(Y));
        }
#pragma unroll
        for (int jb = 0; jb < NB; jb++) S[jb] = mma8(S[jb] * o.fw[jb], o.xz[jb], VU);
    };

    // prologue: chunks 0 and 1 into the ring, chunks 2 .. 4 in flight; this wavefront's own pairs three chunks ahead
    bf16x8 pv[DG];
#pragma unroll
    for (int d = 0; d < DG; d++) {
        issue(st[d], d);
        pv[d] = load_private(d);
    }
    to_ring(0, st[0]);
    to_ring(1, st[1]);
    issue(st[0], DG);
    issue(st[1], DG + 1);
    lds_barrier();
    // round i: chunk i's operands out of the ring, chunk i + 2 into it (fetched three rounds ago), chunk i + 5
    // requested; then the chunk's arithmetic.  The loop body is one basic block (loads are otherwise sunk into
    // the block of their use); the last NC % 3 rounds find everything they need in flight already.
    ScanOps<NB, FWD> o;
    int i = 0;
    for (; i + DG <= NC; i += DG) {
#pragma unroll
        for (int d = 0; d < DG; d++) {
            read_ring(o, i + d);
            to_ring(i + d + 2, st[(d + 2) % DG]);
            issue(st[(d + 2) % DG], i + d + 2 + DG);
            const bf16x8 iv = pv[d];
            pv[d] = load_private(i + d + DG);
            __builtin_amdgcn_sched_barrier(0);
            step(o, iv, i + d);
            lds_barrier();
        }
    }
#pragma unroll
    for (int d = 0; d < DG - 1; d++) {
        if (i + d < NC) {
            read_ring(o, i + d);
            to_ring(i + d + 2, st[(d + 2) % DG]);
            step(o, pv[d], i + d);
            lds_barrier();
        }
    }
    if (s_out != nullptr) {
#pragma unroll
        for (int jb = 0; jb < NB; jb++) {
            if (state_f32) *reinterpret_cast<f32x4*>(static_cast<float*>(s_out) + state_off(jb)) = S[jb];
            else *reinterpret_cast<bf16x4*>(static_cast<__bf16*>(s_out) + state_off(jb)) = to_bf16(S[jb]);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// gradients: one wavefront per chunk (the algebra of bwd_grads_kernel in wkv7_bwd.hip, with the state fragments
// streamed one key block at a time instead of held: at C = 128 both states of a chunk are 128 fragments).
// ------------------------------------------------------------------------------------------------
template <int NB>
__global__ __launch_bounds__(256) void grads_kernel(int T, int H, int nchunks, const __bf16* __restrict__ w_,
                                                    const __bf16* __restrict__ q_, const __bf16* __restrict__ k_,
                                                    const __bf16* __restrict__ v_, const __bf16* __restrict__ a_,
                                                    const __bf16* __restrict__ b_, const __bf16* __restrict__ dy_,
                                                    const __bf16* __restrict__ kept_f, const __bf16* __restrict__ kept_b,
                                                    __bf16* __restrict__ dw_, __bf16* __restrict__ dq_,
                                                    __bf16* __restrict__ dk_, __bf16* __restrict__ dv_,
                                                    __bf16* __restrict__ da_, __bf16* __restrict__ db_) {
    using K = Kept<NB>;
    const int lane = threadIdx.x & 63;
    const int cid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (cid >= nchunks) return;
    const Lane L;
    const Addr<NB> ca(cid, T, H);
    const bf16x4 eye = identity_bf16(L);

    // Everything the chunk needs up front is requested before any of it is used (left to itself the compiler
    // places each load next to its use and waits for it there: one memory latency per fragment).
    const TB<NB> w = load_tile<NB>(w_ + ca.row0, ca.ld, L);
    const TB<NB> q = load_tile<NB>(q_ + ca.row0, ca.ld, L);
    const TB<NB> k = load_tile<NB>(k_ + ca.row0, ca.ld, L);
    const TB<NB> a = load_tile<NB>(a_ + ca.row0, ca.ld, L);
    const TB<NB> b = load_tile<NB>(b_ + ca.row0, ca.ld, L);
    const TB<NB> v = load_tile<NB>(v_ + ca.row0, ca.ld, L);
    const TB<NB> dy = load_tile<NB>(dy_ + ca.row0, ca.ld, L);
    TB<NB> UT, DT, Ur, Dr, dYT;
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        UT.f[ib] = load_frag(kept_f + K::ut(cid, ib), lane);   // F(U_ib^T)   lane = value ch
        DT.f[ib] = load_frag(kept_b + K::ut(cid, ib), lane);   // F(D_ib^T)
    }
    // the state fragments of key block jb + 1 are requested while block jb is worked on
    bf16x4 s0n[NB], dsn[NB];
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        s0n[ib] = load_frag(kept_f + K::ck(cid, 0, ib), lane);
        dsn[ib] = load_frag(kept_b + K::ck(cid, 0, ib), lane);
    }
    __builtin_amdgcn_sched_barrier(0);

    // key side: the decayed operands of all key blocks (needed whole for the 16x16 products)
    TB<NB> wq, wa, kwi, bwi, kf;
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
        const DecayF d = decay_frag(w.f[jb]);
        const f32x4 kwi_f = to_f32(k.f[jb]) * d.Pi;
        wq.f[jb] = to_bf16(to_f32(q.f[jb]) * d.P);
        wa.f[jb] = to_bf16(to_f32(a.f[jb]) * d.Px);
        kwi.f[jb] = to_bf16(kwi_f);
        bwi.f[jb] = to_bf16(to_f32(b.f[jb]) * d.Pi);
        kf.f[jb] = to_bf16(kwi_f * d.fw);
    }
    // value side
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        Ur.f[ib] = transpose(UT.f[ib], eye);                   // F(U_ib)     lane = token
        Dr.f[ib] = transpose(DT.f[ib], eye);
        dYT.f[ib] = transpose(dy.f[ib], eye);
    }
    // 16x16 products over the value channels, each in both orientations
    const bf16x4 dab = to_bf16(mask_lower_strict(xyT(Dr, Ur), L));   // [t][s] = D_t . U_s,  s < t
    const bf16x4 dabT = to_bf16(mask_upper_strict(xyT(Ur, Dr), L));
    const bf16x4 dak = to_bf16(mask_lower_strict(xyT(Dr, v), L));    // [t][s] = D_t . v_s
    const bf16x4 dakT = to_bf16(mask_upper_strict(xyT(v, Dr), L));
    const bf16x4 dqb = to_bf16(mask_lower_incl(xyT(dy, Ur), L));     // [t][s] = dY_t . U_s,  s <= t
    const bf16x4 dqbT = to_bf16(mask_upper_incl(xyT(Ur, dy), L));
    const bf16x4 dqk = to_bf16(mask_lower_incl(xyT(dy, v), L));      // [t][s] = dY_t . v_s
    const bf16x4 dqkT = to_bf16(mask_upper_incl(xyT(v, dy), L));
    // over the key channels (rows = the token being written)
    const bf16x4 QKT = to_bf16(mask_upper_incl(xyT(kwi, wq), L));    // [t][s] = kwi_t . wq_s, s >= t
    const bf16x4 AKT = to_bf16(mask_upper_strict(xyT(kwi, wa), L));  // [t][s] = kwi_t . wa_s, s >  t

    // dv = QK^T dY + AK^T D + kf dS^T: the last term is gathered key block by key block below
    f32x4 dv[NB];
#pragma unroll
    for (int ib = 0; ib < NB; ib++) dv[ib] = mma(mma(zero4(), dYT.f[ib], QKT), DT.f[ib], AKT);

#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
        bf16x4 s0c[NB], dsc[NB];   // F(S0[16 ib.., 16 jb..]), F(dS[16 ib.., 16 jb..]): lane = value row
#pragma unroll
        for (int ib = 0; ib < NB; ib++) {
            s0c[ib] = s0n[ib];
            dsc[ib] = dsn[ib];
        }
        if (jb + 1 < NB) {
#pragma unroll
            for (int ib = 0; ib < NB; ib++) {
                s0n[ib] = load_frag(kept_f + K::ck(cid, jb + 1, ib), lane);
                dsn[ib] = load_frag(kept_b + K::ck(cid, jb + 1, ib), lane);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        f32x4 sds = zero4();                       // sum over the value rows of S0 * dS, this key block
        f32x4 Bq = mma(mma(zero4(), transpose(bwi.f[jb], eye), dqb), transpose(kwi.f[jb], eye), dqk);
        f32x4 Ba = mma(mma(zero4(), transpose(bwi.f[jb], eye), dab), transpose(kwi.f[jb], eye), dak);
        const f32x4 Bb = mma(mma(zero4(), transpose(wa.f[jb], eye), dabT), transpose(wq.f[jb], eye), dqbT);
        const f32x4 Bk = mma(mma(zero4(), transpose(wa.f[jb], eye), dakT), transpose(wq.f[jb], eye), dqkT);
        f32x4 UdS = zero4(), VdS = zero4();
#pragma unroll
        for (int ib = 0; ib < NB; ib++) {
            const bf16x4 s0 = s0c[ib], ds = dsc[ib];
            sds += to_f32(s0) * to_f32(ds);
            const bf16x4 s0T = transpose(s0, eye), dsT = transpose(ds, eye);  // lane = key column, reg = value row
            dv[ib] = mma(dv[ib], ds, kf.f[jb]);
            Bq = mma(Bq, s0T, dy.f[ib]);          // + dY S0
            Ba = mma(Ba, s0T, Dr.f[ib]);          // + D S0
            UdS = mma(UdS, dsT, Ur.f[ib]);        // U dS
            VdS = mma(VdS, dsT, v.f[ib]);         // V dS
        }
        const DecayF d = decay_frag(w.f[jb]);
        const f32x4 wqf = to_f32(wq.f[jb]), waf = to_f32(wa.f[jb]), kwif = to_f32(kwi.f[jb]), bwif = to_f32(bwi.f[jb]);
        f32x4 dq, da, dk, db, dw;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float fw = d.fw[r];
            const float fwU = fw * UdS[r], fwV = fw * VdS[r];
            const float bb = Bb[r] + fwU, bk = Bk[r] + fwV;
            dq[r] = d.P[r] * Bq[r];
            da[r] = d.Px[r] * Ba[r];
            db[r] = d.Pi[r] * bb;
            dk[r] = d.Pi[r] * bk;
            // gradient of the log decays: what every later token's factors contribute, plus the chunk's whole decay
            const float g_incl = wqf[r] * Bq[r] - kwif[r] * bk - bwif[r] * bb;
            const float g_strict = waf[r] * Ba[r];
            const float tail = row_sum(kwif[r] * fwV + bwif[r] * fwU + fw * sds[r]);
            const float dlogw = row_suffix_sum(g_incl + g_strict) - g_strict + tail;
            dw[r] = dlogw * d.lw[r];
        }
        store_frag_rows(dq_ + ca.row0, ca.ld, jb, L, to_bf16(dq));
        store_frag_rows(da_ + ca.row0, ca.ld, jb, L, to_bf16(da));
        store_frag_rows(dk_ + ca.row0, ca.ld, jb, L, to_bf16(dk));
        store_frag_rows(db_ + ca.row0, ca.ld, jb, L, to_bf16(db));
        store_frag_rows(dw_ + ca.row0, ca.ld, jb, L, to_bf16(dw));
    }
#pragma unroll
    for (int ib = 0; ib < NB; ib++) store_frag_rows(dv_ + ca.row0, ca.ld, ib, L, to_bf16(dv[ib]));
}

// ------------------------------------------------------------------------------------------------
// one token per sequence on a resident state (decoding), with the optional attn_ln epilogue: the step of
// wkv7_decode.hip for C = 16 NB.  One wavefront owns the C x C state of a (batch, head) pair and walks its NB row
// blocks; lane (n, g) holds four columns of each of the NB column blocks of row 16 ib + n.
//     sa = S a ;   S <- S diag(exp(-exp(w))) + sa b^T + v k^T ;   y = S q            (time_mixer.py:6-16)
// ------------------------------------------------------------------------------------------------
template <int NB, bool LN>
__global__ __launch_bounds__(256) void decode_kernel(int BH, int H, int state_f32, const __bf16* __restrict__ w_,
                                                     const __bf16* __restrict__ q_, const __bf16* __restrict__ k_,
                                                     const __bf16* __restrict__ v_, const __bf16* __restrict__ a_,
                                                     const __bf16* __restrict__ b_, void* __restrict__ state,
                                                     __bf16* __restrict__ y_, const __bf16* __restrict__ g_,
                                                     const float* __restrict__ params) {
    constexpr int C = 16 * NB;
    constexpr float EPS = 64e-5f;   // GroupNorm eps of the block (time_mixer.py:154)
    const int bh = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (bh >= BH) return;
    const Lane L;
    const long row = (long)bh * C;   // this head's channels in a [B, H*C] tensor

    f32x4 decay[NB], qv[NB], kv[NB], av[NB], bv[NB];
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
        const long c = row + 16 * jb + 4 * L.g;
        const f32x4 wv = to_f32(*reinterpret_cast<const bf16x4*>(w_ + c));
#pragma unroll
        for (int r = 0; r < 4; r++) decay[jb][r] = __expf(-__expf(wv[r]));
        qv[jb] = to_f32(*reinterpret_cast<const bf16x4*>(q_ + c));
        kv[jb] = to_f32(*reinterpret_cast<const bf16x4*>(k_ + c));
        av[jb] = to_f32(*reinterpret_cast<const bf16x4*>(a_ + c));
        bv[jb] = to_f32(*reinterpret_cast<const bf16x4*>(b_ + c));
    }
    float y[NB], vrow[NB];
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        vrow[ib] = (float)v_[row + 16 * ib + L.n];
        const long s_off = ((long)bh * C + 16 * ib + L.n) * C + 4 * L.g;
        f32x4 S[NB];
        float sa = 0.f;
#pragma unroll
        for (int jb = 0; jb < NB; jb++) {
            if (state_f32) S[jb] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(state) + s_off + 16 * jb);
            else S[jb] = to_f32(*reinterpret_cast<const bf16x4*>(static_cast<const __bf16*>(state) + s_off + 16 * jb));
#pragma unroll
            for (int r = 0; r < 4; r++) sa += S[jb][r] * av[jb][r];
        }
        sa = group_sum(sa);   // over the four lanes that share the row
        float acc = 0.f;
#pragma unroll
        for (int jb = 0; jb < NB; jb++) {
            S[jb] = S[jb] * decay[jb] + sa * bv[jb] + vrow[ib] * kv[jb];
#pragma unroll
            for (int r = 0; r < 4; r++) acc += S[jb][r] * qv[jb][r];
            if (state_f32) *reinterpret_cast<f32x4*>(static_cast<float*>(state) + s_off + 16 * jb) = S[jb];
            else *reinterpret_cast<bf16x4*>(static_cast<__bf16*>(state) + s_off + 16 * jb) = to_bf16(S[jb]);
        }
        y[ib] = group_sum(acc);
    }
    if constexpr (LN) {
        // GroupNorm over the head's C outputs: lane (n, g) holds rows 16 ib + n, replicated over g
        auto head_sum = [&](float x) {
            x += __shfl_xor(x, 1);
            x += __shfl_xor(x, 2);
            x += __shfl_xor(x, 4);
            x += __shfl_xor(x, 8);
            return x;
        };
        float part = 0.f;
#pragma unroll
        for (int ib = 0; ib < NB; ib++) part += y[ib];
        const float mean = head_sum(part) * (1.f / C);
        float sq = 0.f;
#pragma unroll
        for (int ib = 0; ib < NB; ib++) sq += (y[ib] - mean) * (y[ib] - mean);
        const float istd = rsqrtf(head_sum(sq) * (1.f / C) + EPS);
        const int h = bh % H;
        const long HC = (long)H * C;
        float dot = 0.f;   // sum_c q_c k_c bonus_c
#pragma unroll
        for (int jb = 0; jb < NB; jb++) {
            const f32x4 bonus = *reinterpret_cast<const f32x4*>(params + 2 * HC + (long)h * C + 16 * jb + 4 * L.g);
#pragma unroll
            for (int r = 0; r < 4; r++) dot += qv[jb][r] * kv[jb][r] * bonus[r];
        }
        dot = group_sum(dot);
#pragma unroll
        for (int ib = 0; ib < NB; ib++) {
            const long ch = (long)h * C + 16 * ib + L.n;
            const float x1 = (y[ib] - mean) * istd * params[ch] + params[HC + ch];
            y[ib] = (x1 + dot * vrow[ib]) * (float)g_[row + 16 * ib + L.n];
        }
    }
    if (L.g == 0) {
#pragma unroll
        for (int ib = 0; ib < NB; ib++) y_[row + 16 * ib + L.n] = (__bf16)y[ib];
    }
}

template <int NB>
constexpr size_t rec_bytes(bool fwd) {
    return (size_t)(fwd ? Rec<NB, true>::ELEMS : Rec<NB, false>::ELEMS) * sizeof(__bf16);
}
template <int NB>
constexpr size_t kept_bytes() { return (size_t)Kept<NB>::ELEMS * sizeof(__bf16); }

inline const __bf16* c(const void* p) { return static_cast<const __bf16*>(p); }
inline __bf16* m(void* p) { return static_cast<__bf16*>(p); }

template <int NB>
void forward(int B, int T, int H, int state_f32, const void* w, const void* q, const void* k, const void* v, const void* a,
             const void* b, const void* s_in, void* s_out, void* y, void* rec, void* kept, float* centers, hipStream_t stream) {
    const int nchunks = B * H * (T / CHUNK);
    hipLaunchKernelGGL(fwd_prepare_kernel<NB>, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(w), c(q),
                       c(k), c(v), c(a), c(b), m(rec));
    const dim3 grid(B * H, (NB + 3) / 4), block(256);
    if (kept) hipLaunchKernelGGL((scan_kernel<NB, true, true>), grid, block, 0, stream, T, H, state_f32, c(rec), s_in, s_out, m(y), m(kept), centers);
    else hipLaunchKernelGGL((scan_kernel<NB, true, false>), grid, block, 0, stream, T, H, state_f32, c(rec), s_in, s_out, m(y), m(kept), centers);
}
template <int NB>
void backward(int B, int T, int H, int state_f32, const void* w, const void* q, const void* k, const void* v, const void* a,
              const void* b, const void* dy, const void* kept_f, const void* ds_in, void* ds_out, void* dw, void* dq,
              void* dk, void* dv, void* da, void* db, void* rec, void* kept_b, hipStream_t stream) {
    const int nchunks = B * H * (T / CHUNK);
    hipLaunchKernelGGL(bwd_prepare_kernel<NB>, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(w), c(q),
                       c(a), c(b), c(dy), m(rec));
    hipLaunchKernelGGL((scan_kernel<NB, false, true>), dim3(B * H, (NB + 3) / 4), dim3(256), 0, stream, T, H,
                       state_f32, c(rec), ds_in, ds_out, static_cast<__bf16*>(nullptr), m(kept_b), static_cast<float*>(nullptr));
    hipLaunchKernelGGL(grads_kernel<NB>, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(w), c(q), c(k),
                       c(v), c(a), c(b), c(dy), c(kept_f), c(kept_b), m(dw), m(dq), m(dk), m(dv), m(da), m(db));
}

// calls f.template operator()<NB>() for the head size's NB
template <class F>
bool dispatch(int C, F&& f) {
    switch (C / 16) {
        case 1: f.template operator()<1>(); return true;
        case 2: f.template operator()<2>(); return true;
        case 3: f.template operator()<3>(); return true;
        case 4: f.template operator()<4>(); return true;
        case 5: f.template operator()<5>(); return true;
        case 6: f.template operator()<6>(); return true;
        case 7: f.template operator()<7>(); return true;
        case 8: f.template operator()<8>(); return true;
        default: return false;
    }
}

struct SizeQuery {
    size_t rec_f = 0, rec_b = 0, kept = 0;
    template <int NB>
    void operator()() {
        rec_f = rec_bytes<NB>(true);
        rec_b = rec_bytes<NB>(false);
        kept = kept_bytes<NB>();
    }
};

}  // namespace

bool head_size_supported(int C) { return C >= 16 && C <= 128 && C % 16 == 0; }

static size_t A256(size_t n) { return (n + 255) & ~(size_t)255; }

size_t kept_bytes(int B, int T, int H, int C) {
    SizeQuery s;
    if (!head_size_supported(C) || !dispatch(C, s)) return 0;
    return A256((size_t)B * H * (T / CHUNK) * s.kept);
}
size_t record_bytes(int B, int T, int H, int C, bool fwd) {
    SizeQuery s;
    if (!head_size_supported(C) || !dispatch(C, s)) return 0;
    return A256((size_t)B * H * (T / CHUNK) * (fwd ? s.rec_f : s.rec_b));
}

namespace {
struct Forward {
    int B, T, H, state_f32;
    const void *w, *q, *k, *v, *a, *b, *s_in;
    void *s_out, *y, *rec, *kept;
    float* centers;
    hipStream_t stream;
    template <int NB>
    void operator()() { forward<NB>(B, T, H, state_f32, w, q, k, v, a, b, s_in, s_out, y, rec, kept, centers, stream); }
};
struct Backward {
    int B, T, H, state_f32;
    const void *w, *q, *k, *v, *a, *b, *dy, *kept_f, *ds_in;
    void *ds_out, *dw, *dq, *dk, *dv, *da, *db, *rec, *kept_b;
    hipStream_t stream;
    template <int NB>
    void operator()() {
        backward<NB>(B, T, H, state_f32, w, q, k, v, a, b, dy, kept_f, ds_in, ds_out, dw, dq, dk, dv, da, db, rec, kept_b, stream);
    }
};
}  // namespace

namespace {
struct Decode {
    int B, H, state_f32;
    const void *w, *q, *k, *v, *a, *b;
    void *state, *y;
    const void *g, *params;
    hipStream_t stream;
    template <int NB>
    void operator()() {
        const int BH = B * H;
        const dim3 grid((BH + 3) / 4), block(256);
        if (params != nullptr)
            hipLaunchKernelGGL((decode_kernel<NB, true>), grid, block, 0, stream, BH, H, state_f32, c(w), c(q), c(k), c(v), c(a),
                               c(b), state, m(y), c(g), static_cast<const float*>(params));
        else
            hipLaunchKernelGGL((decode_kernel<NB, false>), grid, block, 0, stream, BH, H, state_f32, c(w), c(q), c(k), c(v), c(a),
                               c(b), state, m(y), c(g), static_cast<const float*>(params));
    }
};
}  // namespace

void launch_decode(int B, int H, int C, int state_f32, const void* w, const void* q, const void* k, const void* v,
                   const void* a, const void* b, void* state, void* y, hipStream_t stream, const void* g, const void* params) {
    Decode f{B, H, state_f32, w, q, k, v, a, b, state, y, g, params, stream};
    dispatch(C, f);
}

void launch_forward(int B, int T, int H, int C, int state_f32, const void* w, const void* q, const void* k, const void* v,
                    const void* a, const void* b, const void* s_in, void* s_out, void* y, void* rec, void* kept,
                    hipStream_t stream, float* centers) {
    Forward f{B, T, H, state_f32, w, q, k, v, a, b, s_in, s_out, y, rec, kept, centers, stream};
    dispatch(C, f);
}

void launch_backward(int B, int T, int H, int C, int state_f32, const void* w, const void* q, const void* k, const void* v,
                     const void* a, const void* b, const void* dy, const void* kept_f, const void* ds_in, void* ds_out,
                     void* dw, void* dq, void* dk, void* dv, void* da, void* db, void* rec, void* kept_b, hipStream_t stream) {
    Backward f{B, T, H, state_f32, w, q, k, v, a, b, dy, kept_f, ds_in, ds_out, dw, dq, dk, dv, da, db, rec, kept_b, stream};
    dispatch(C, f);
}

}  // namespace wide
}  // namespace wkv
