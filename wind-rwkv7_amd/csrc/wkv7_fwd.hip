// WKV7 forward for gfx950: chunk-parallel prepare -> state scan -> chunk-parallel output.
//
// Replaces forward_kernel of the reference (attn.cu:11-106; attn_ln.cu:106-212 with the epilogue),
// same mathematics (rwkv7_attn_triton.py:27-69), different organisation: the reference runs one
// block per (batch, head) through all chunks with ~60 block barriers per chunk; here each chunk is
// one wavefront's private work and only the 64x64 state update is sequential.
//
// Per chunk (K = 16 tokens), with S0 the state entering the chunk:
//   prepare:  Tinv = inv(I - strict_tril(wa bwi^T)),  U0 = Tinv (strict_tril(wa kwi^T) V),  Wm = Tinv wa
//   scan:     U = U0 + Wm S0^T ;  S' = S0 diag(fw) + V^T kf + U^T bf        (checkpoint S0, keep U)
//   output:   Y = tril(wq kwi^T) V + tril(wq bwi^T) U + wq S0^T
#include "ln_epilogue.hpp"
#include "wkv7_common.hpp"
#include "wkv7_kernels.hpp"

namespace wkv {

// ------------------------------------------------------------------------------------------------
// prepare: one wavefront per chunk, four chunks per block.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fwd_prepare_kernel(int T, int H, int nchunks,
                                                          const __bf16* __restrict__ w_, const __bf16* __restrict__ k_,
                                                          const __bf16* __restrict__ v_, const __bf16* __restrict__ a_,
                                                          const __bf16* __restrict__ b_, __bf16* __restrict__ rec) {
    const int lane = threadIdx.x & 63;
    const int cid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (cid >= nchunks) return;
    const Lane L;
    const ChunkAddr ca(cid, T, H);

    const TileB w = load_rows(w_ + ca.row0, ca.ld, L);
    const TileB k = load_rows(k_ + ca.row0, ca.ld, L);
    const TileB v = load_rows(v_ + ca.row0, ca.ld, L);
    const TileB a = load_rows(a_ + ca.row0, ca.ld, L);
    const TileB b = load_rows(b_ + ca.row0, ca.ld, L);

    const Decay d = chunk_decay(w);
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

    __bf16* J = rec + rec_j(cid);
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        const bf16x4 VT = transpose(v.f[ib], eye);                 // F(V_ib^T)        lane = value ch, reg = token
        const f32x4 RT = mma(zero4(), AK_b, VT);                   // F((AK V_ib)^T)
        const f32x4 UT = mma(zero4(), Tinv_b, to_bf16(RT));        // F((Tinv AK V_ib)^T)
        store_pair(rec + rec_i(cid, ib), lane, to_bf16(UT), VT);
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
            *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(rec + rec_fw(cid)) + 16 * jb + 4 * L.g) = fw;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// scan: the only sequential part.  One block per (batch, head): four compute wavefronts (16 of the head's
// 64 value rows each, one per SIMD, the state in their fp32 accumulators) and one loader.  The same kernel
// runs the backward dstate scan (reverse = 1).
//   per chunk:  U^T = U0^T + S Wm^T               (contraction over key channels)
//               S  <- S diag(fw) + V^T K + U^T B  (contraction over the chunk's tokens)
// The chain is six matrix instructions per chunk; everything else is about keeping memory latency and
// instruction issue off it.  A compute unit's address unit takes 16 cycles per 64-lane memory instruction,
// whoever issues it, so the block as a whole must issue few of them per chunk:
//   loader   loads J and FW (shared by the four compute wavefronts) once, DEPTH_L chunks ahead, and keeps a
//            three-slot LDS ring filled two chunks ahead of the chain;
//   compute  reads chunk t+1's slot into registers while it works on chunk t; loads only its own
//            (U0^T, V^T) record from memory (DEPTH_C chunks ahead); stores the checkpoint and U^T of chunk
//            t-1 over that chunk's record right after the barrier that ends chunk t-1 - by then every
//            wavefront of the block, the only readers of the record, has consumed it.
// One LDS-only barrier per chunk keeps the five wavefronts in step.
// ------------------------------------------------------------------------------------------------
constexpr int RING_SLOTS = 3;
constexpr int RING_J_BYTES = FRAGS_J * FRAG_ELEMS * 2;   // 6144
constexpr int RING_BYTES = RING_J_BYTES + HEAD * 4;      // + FW
constexpr int SCAN_THREADS = 5 * 64;
constexpr int SCAN_DEPTH_L = 6;   // loader: 25 registers per chunk in flight
constexpr int SCAN_DEPTH_C = 8;   // compute: 4 registers per chunk in flight; must be even (register sets alternate)

__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int DEPTH_L, int DEPTH_C>
__global__ __launch_bounds__(SCAN_THREADS) void state_scan_kernel(int NC, int reverse, int state_f32, __bf16* __restrict__ rec,
                                                                  const void* __restrict__ s_in, void* __restrict__ s_out) {
    static_assert(DEPTH_L >= 3, "the loader prologue uses st[0], st[1] twice");
    static_assert(DEPTH_C % 2 == 0, "the compute wavefronts alternate two register sets");
    __shared__ __attribute__((aligned(16))) unsigned char ring[RING_SLOTS * RING_BYTES];
    const int lane = threadIdx.x & 63;
    const int role = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // 0..3 compute; 4 loader
    const int bh = blockIdx.x;
    // both roles run the same rounds: a prologue barrier, then one barrier per chunk
    auto chunk_of = [&](int step) -> long {
        step = step < NC ? step : NC - 1;
        return (long)bh * NC + (reverse ? NC - 1 - step : step);
    };

    if (role == 4) {
        // ---------------- loader ----------------
        // invariant at round t: st[(t + 2) % DEPTH_L] holds J and FW of chunk t+2, which go to slot (t+2) % 3
        struct Stage {
            f32x4 j[6];
            float fw;
        };
        const char* jsrc = reinterpret_cast<const char*>(rec + REC_J) + lane * 16;
        const float* fsrc = reinterpret_cast<const float*>(rec + REC_FW) + lane;
        auto issue = [&](Stage& st, int step) {
            const long cid = chunk_of(step);
#pragma unroll
            for (int i = 0; i < 6; i++) st.j[i] = *reinterpret_cast<const f32x4*>(jsrc + cid * REC_BYTES + i * 1024);
            st.fw = fsrc[cid * (REC_ELEMS / 2)];
        };
        auto to_lds = [&](int step, const Stage& st) {
            unsigned char* base = ring + (step % RING_SLOTS) * RING_BYTES;
#pragma unroll
            for (int i = 0; i < 6; i++) *reinterpret_cast<f32x4*>(base + i * 1024 + lane * 16) = st.j[i];
            *reinterpret_cast<float*>(base + RING_J_BYTES + lane * 4) = st.fw;
        };
        Stage st[DEPTH_L];
#pragma unroll
        for (int s = 0; s < DEPTH_L; s++) issue(st[s], s);
        to_lds(0, st[0]);
        to_lds(1, st[1]);
        issue(st[0], DEPTH_L);
        issue(st[1], DEPTH_L + 1);
        lds_barrier();
        int step0 = 0;
        for (; step0 + DEPTH_L <= NC; step0 += DEPTH_L) {
#pragma unroll
            for (int s = 0; s < DEPTH_L; s++) {
                to_lds(step0 + s + 2, st[(s + 2) % DEPTH_L]);
                issue(st[(s + 2) % DEPTH_L], step0 + s + 2 + DEPTH_L);
                lds_barrier();
            }
        }
#pragma unroll
        for (int s = 0; s < DEPTH_L - 1; s++) {   // the remaining NC % DEPTH_L rounds; chunks past the end are never read
            if (step0 + s < NC) {
                to_lds(step0 + s + 2, st[(s + 2) % DEPTH_L]);
                lds_barrier();
            }
        }
        return;
    }
    // ---------------- compute ----------------
    const Lane L;
    const int ib = role;
    f32x4 S[NBLK];
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) S[jb] = load_state_frag(s_in, state_f32, bh, ib, jb, L);

    struct Operands {   // one chunk's shared operands, in registers
        bf16x8 j[6];
        f32x4 fw[NBLK];
    };
    struct Outputs {    // what the chunk leaves for the consumers
        bf16x8 s01, s23;
        bf16x4 u;
    };
    auto read_ring = [&](Operands& o, int step) {
        const unsigned char* base = ring + (step % RING_SLOTS) * RING_BYTES;
#pragma unroll
        for (int i = 0; i < 6; i++) o.j[i] = *reinterpret_cast<const bf16x8*>(base + i * 1024 + lane * 16);
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) o.fw[jb] = *reinterpret_cast<const f32x4*>(base + RING_J_BYTES + jb * 64 + L.g * 16);
    };
    const __bf16* isrc = rec + REC_I + (ib * WAVE + lane) * 8;
    auto issue = [&](bf16x8& iv, int step) { iv = *reinterpret_cast<const bf16x8*>(isrc + chunk_of(step) * REC_ELEMS); };
    auto store_outputs = [&](int step, const Outputs& o) {
        __bf16* r = rec + chunk_of(step) * REC_ELEMS;
        bf16x8* q = reinterpret_cast<bf16x8*>(r + REC_CKPT + ib * TILE_ELEMS + lane * 16);   // 32 bytes per lane
        q[0] = o.s01;
        q[1] = o.s23;
        *reinterpret_cast<bf16x4*>(r + REC_UT + ib * FRAG_ELEMS + lane * 4) = o.u;
    };
    auto compute = [&](const Operands& op, bf16x8 iv, Outputs& out) {
        const bf16x4 b0 = to_bf16(S[0]), b1 = to_bf16(S[1]), b2 = to_bf16(S[2]), b3 = to_bf16(S[3]);
        out.s01 = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
        out.s23 = __builtin_shufflevector(b2, b3, 0, 1, 2, 3, 4, 5, 6, 7);
        const bf16x4 U0 = __builtin_shufflevector(iv, iv, 0, 1, 2, 3);
        const f32x4 Ua = mma8(to_f32(U0), op.j[0], out.s01);   // + F(S_ib Wm^T), two independent halves
        const f32x4 Uc = mma8(zero4(), op.j[1], out.s23);
        out.u = to_bf16(Ua + Uc);
        const bf16x8 VU = __builtin_shufflevector(iv, __builtin_shufflevector(out.u, out.u, 0, 1, 2, 3, 0, 1, 2, 3), 4, 5, 6, 7, 8, 9, 10, 11);
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) S[jb] = mma8(S[jb] * op.fw[jb], op.j[2 + jb], VU);   // + F(V_ib^T K_jb + U_ib^T B_jb)
    };

    bf16x8 iv[DEPTH_C];
#pragma unroll
    for (int s = 0; s < DEPTH_C; s++) issue(iv[s], s);
    Operands op[2];
    Outputs out[2];
    lds_barrier();
    read_ring(op[0], 0);
    // one round: chunk `step` with register set `cur`; the previous chunk's outputs go to memory first
    auto round = [&](int step, int cur, bf16x8& ivs, bool refill) {
        if (step > 0) store_outputs(step - 1, out[cur ^ 1]);
        read_ring(op[cur ^ 1], step + 1);   // needed a whole chunk from now
        compute(op[cur], ivs, out[cur]);
        if (refill) issue(ivs, step + DEPTH_C);
        lds_barrier();
    };
    int step0 = 0;
    for (; step0 + DEPTH_C <= NC; step0 += DEPTH_C) {
#pragma unroll
        for (int s = 0; s < DEPTH_C; s++) round(step0 + s, s & 1, iv[s], true);
    }
#pragma unroll
    for (int s = 0; s < DEPTH_C - 1; s++) {   // the remaining NC % DEPTH_C chunks are already in iv[0..]
        if (step0 + s < NC) round(step0 + s, s & 1, iv[s], false);
    }
    if ((NC - 1) & 1) store_outputs(NC - 1, out[1]);
    else store_outputs(NC - 1, out[0]);
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) store_state_frag(s_out, state_f32, bh, ib, jb, L, S[jb]);
}

// ------------------------------------------------------------------------------------------------
// output: one wavefront per chunk.  With LN the GroupNorm + bonus + gate epilogue of attn_ln runs on the
// accumulators before the store, and the plain WKV7 output is kept (bf16) for the backward pass.
// ------------------------------------------------------------------------------------------------
struct LnFwdArgs {
    const __bf16* g;        // [B,T,H,64]
    const float* params;    // [3][H*64]
    __bf16* y_wkv;          // [B,T,H,64] saved for backward
};

template <bool LN>
__global__ __launch_bounds__(256) void fwd_output_kernel(int T, int H, int nchunks,
                                                         const __bf16* __restrict__ w_, const __bf16* __restrict__ q_,
                                                         const __bf16* __restrict__ k_, const __bf16* __restrict__ v_,
                                                         const __bf16* __restrict__ b_, const __bf16* __restrict__ rec,
                                                         __bf16* __restrict__ y_, LnFwdArgs ln) {
    const int lane = threadIdx.x & 63;
    const int cid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (cid >= nchunks) return;
    const Lane L;
    const ChunkAddr ca(cid, T, H);

    const TileB w = load_rows(w_ + ca.row0, ca.ld, L);
    const TileB q = load_rows(q_ + ca.row0, ca.ld, L);
    const TileB k = load_rows(k_ + ca.row0, ca.ld, L);
    const TileB v = load_rows(v_ + ca.row0, ca.ld, L);
    const TileB b = load_rows(b_ + ca.row0, ca.ld, L);
    const TileB UT = load_frags(rec + rec_ut(cid), lane);
    const bf16x4 eye = identity_bf16(L);
    TileB VT;   // F(V_ib^T): lane = value channel, reg = token
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) VT.f[ib] = transpose(v.f[ib], eye);

    const Decay d = chunk_decay(w);
    const TileB wq = to_bf16(mul(q, d.P));
    const TileB kwi = to_bf16(mul(k, d.Pi));
    const TileB bwi = to_bf16(mul(b, d.Pi));
    const bf16x4 QK = to_bf16(mask_lower_incl(tile_xyT(wq, kwi), L));  // F(QK), QK[t][s], s <= t
    const bf16x4 QB = to_bf16(mask_lower_incl(tile_xyT(wq, bwi), L));

    TileF yf;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        const TileB S0 = load_lane16(rec + rec_ckpt(cid, ib), lane);   // F(S0[16ib.., 16jb..])
        f32x4 acc = mma2(zero4(), VT.f[ib], UT.f[ib], QK, QB);         // F(QK V_ib + QB U_ib)   lane = token
        acc = mma2(acc, S0.f[0], S0.f[1], wq.f[0], wq.f[1]);           // + F(wq S0_ib^T)
        acc = mma2(acc, S0.f[2], S0.f[3], wq.f[2], wq.f[3]);
        yf.f[ib] = acc;
    }
    if constexpr (LN) {
        const int h = ca.bh % H;
        const LnParams p = load_ln_params(ln.params, h, H, L);
        const TileB g = load_rows(ln.g + ca.row0, ca.ld, L);
        store_rows(ln.y_wkv + ca.row0, ca.ld, L, to_bf16(yf));
        store_rows(y_ + ca.row0, ca.ld, L, ln_forward(yf, q, k, v, g, p));
    } else {
        store_rows(y_ + ca.row0, ca.ld, L, to_bf16(yf));
    }
}

// ------------------------------------------------------------------------------------------------
// host launchers
// ------------------------------------------------------------------------------------------------
void launch_fwd_prepare(int B, int T, int H, const void* w, const void* k, const void* v, const void* a, const void* b,
                        void* rec, hipStream_t stream) {
    const int nchunks = B * H * (T / CHUNK);
    hipLaunchKernelGGL(fwd_prepare_kernel, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks,
                       static_cast<const __bf16*>(w), static_cast<const __bf16*>(k), static_cast<const __bf16*>(v),
                       static_cast<const __bf16*>(a), static_cast<const __bf16*>(b), static_cast<__bf16*>(rec));
}

void launch_state_scan(int B, int T, int H, int reverse, int state_f32, void* rec, const void* s_in, void* s_out,
                       hipStream_t stream) {
    hipLaunchKernelGGL((state_scan_kernel<SCAN_DEPTH_L, SCAN_DEPTH_C>), dim3(B * H), dim3(SCAN_THREADS), 0, stream, T / CHUNK, reverse,
                       state_f32, static_cast<__bf16*>(rec), s_in, s_out);
}

void launch_fwd_output(int B, int T, int H, const void* w, const void* q, const void* k, const void* v, const void* b,
                       const void* rec, void* y, hipStream_t stream, const void* g, const void* params, void* y_wkv) {
    const int nchunks = B * H * (T / CHUNK);
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    const LnFwdArgs ln{c(g), static_cast<const float*>(params), static_cast<__bf16*>(y_wkv)};
    if (params != nullptr)
        hipLaunchKernelGGL(fwd_output_kernel<true>, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(w),
                           c(q), c(k), c(v), c(b), c(rec), static_cast<__bf16*>(y), ln);
    else
        hipLaunchKernelGGL(fwd_output_kernel<false>, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(w),
                           c(q), c(k), c(v), c(b), c(rec), static_cast<__bf16*>(y), ln);
}

}  // namespace wkv
