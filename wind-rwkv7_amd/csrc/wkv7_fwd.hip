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
                                                          const __bf16* __restrict__ b_, ScanWs ws) {
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

    __bf16* J = ws.J + (long)cid * J_ELEMS;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        const bf16x4 VT = transpose(v.f[ib], eye);                 // F(V_ib^T)        lane = value ch, reg = token
        const f32x4 RT = mma(zero4(), AK_b, VT);                   // F((AK V_ib)^T)
        const f32x4 UT = mma(zero4(), Tinv_b, to_bf16(RT));        // F((Tinv AK V_ib)^T)
        store_pair(ws.I + i_record(cid, ib), lane, to_bf16(UT), VT);
    }
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) {
        const bf16x4 waT = transpose(wa.f[jb], eye);               // F(wa_jb^T)       lane = key ch, reg = token
        const f32x4 Wm = mma(zero4(), waT, Tinv_b);                // F(Tinv wa_jb)    lane = token, reg = key ch
        store_frag(J + (0 + jb) * FRAG_ELEMS, lane, to_bf16(Wm));
        store_frag(J + (4 + jb) * FRAG_ELEMS, lane, transpose(kf.f[jb], eye));
        store_frag(J + (8 + jb) * FRAG_ELEMS, lane, transpose(bf.f[jb], eye));
    }
    if (L.n == 0) {
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            f32x4 fw;
#pragma unroll
            for (int r = 0; r < 4; r++) fw[r] = d.fw.f[jb][r];
            *reinterpret_cast<f32x4*>(ws.FW + (long)cid * HEAD + 16 * jb + 4 * L.g) = fw;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// scan: one block per (batch, head); wavefront ib carries the 16 value rows 16*ib .. 16*ib+15 of
// the state in fp32 accumulators.  The same kernel runs the backward dstate scan (reverse = 1).
//   per chunk:  U^T = U0^T + S Wm^T               (contraction over key channels)
//               S  <- S diag(fw) + V^T K + U^T B  (contraction over the chunk's tokens)
// The step is short (six matrix instructions per wavefront) and strictly sequential, so everything is
// about never waiting for memory: each thread keeps SCAN_DEPTH chunks of its share of the operands in
// flight in registers; the key-channel operands, which all four wavefronts need, are copied
// cooperatively (a quarter each) into a double-buffered LDS slot one step ahead of use.  One workgroup
// barrier per step, waiting on LDS traffic only.
// ------------------------------------------------------------------------------------------------
constexpr int SLOT_BYTES = 8192;   // 6144 J + 256 FW, padded to 512 16-byte units
constexpr int SLOT_FW = 6144;

template <int UNITS>
struct ScanStage {
    f32x4 j[UNITS];   // this thread's 16-byte units of the chunk's J/FW record (raw bits)
    bf16x8 iv;        // this lane's (U0^T, V^T) pair
};

__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// WPB wavefronts per block (each owns 16 value rows; 4/WPB blocks share one (batch, head)), DEPTH chunks in
// flight per thread.  Fewer wavefronts per block spread one head's scan over more compute units: the scan
// is bound by how many bytes it keeps in flight, and every block brings its own registers for that.
template <int WPB, int DEPTH>
__global__ __launch_bounds__(64 * WPB) void state_scan_kernel(int NC, int BH, int reverse, int state_f32, ScanWs ws,
                                                              const void* __restrict__ s_in, void* __restrict__ s_out,
                                                              __bf16* __restrict__ ckpt, __bf16* __restrict__ u_out) {
    constexpr int NT = 64 * WPB;
    constexpr int UNITS = 512 / NT;   // 16-byte units of the padded slot copied by each thread
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * SLOT_BYTES];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // blocks of one (batch, head) are BH apart, so that they share an L2 slice when BH is a multiple of 8
    const int bh = blockIdx.x % BH;
    const int ib = (blockIdx.x / BH) * WPB + (tid >> 6);
    const Lane L;

    f32x4 S[NBLK];
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) S[jb] = load_state_frag(s_in, state_f32, bh, ib, jb, L);

    // per-thread sources of the cooperative copy: units tid, tid+NT, ... of the 512-unit slot
    // (units 0..383 = J record, 384..399 = FW, the rest is padding and re-reads unit 399)
    const char* src[UNITS];
    long stride[UNITS];
#pragma unroll
    for (int u = 0; u < UNITS; u++) {
        const int unit = tid + u * NT;
        const bool is_j = unit < 384;
        const int fw_unit = unit - 384 < 15 ? (unit - 384 < 0 ? 0 : unit - 384) : 15;
        src[u] = is_j ? reinterpret_cast<const char*>(ws.J) + unit * 16 : reinterpret_cast<const char*>(ws.FW) + fw_unit * 16;
        stride[u] = is_j ? J_ELEMS * 2 : HEAD * 4;
    }
    const char* srcI = reinterpret_cast<const char*>(ws.I) + (ib * WAVE + lane) * 16;
    const long strideI = I_ELEMS * 2;

    auto chunk_of = [&](int step) -> long {
        step = step < NC ? step : NC - 1;
        return (long)bh * NC + (reverse ? NC - 1 - step : step);
    };
    auto issue = [&](ScanStage<UNITS>& st, int step) {
        const long cid = chunk_of(step);
#pragma unroll
        for (int u = 0; u < UNITS; u++) st.j[u] = *reinterpret_cast<const f32x4*>(src[u] + cid * stride[u]);
        st.iv = *reinterpret_cast<const bf16x8*>(srcI + cid * strideI);
    };
    auto to_lds = [&](int slot, const ScanStage<UNITS>& st) {
        unsigned char* base = lds + slot * SLOT_BYTES;
#pragma unroll
        for (int u = 0; u < UNITS; u++) *reinterpret_cast<f32x4*>(base + (tid + u * NT) * 16) = st.j[u];
    };
    auto compute = [&](int step, int slot, bf16x8 iv) {
        const long cid = chunk_of(step);
        const unsigned char* base = lds + slot * SLOT_BYTES;
        bf16x4 A[NBLK], KT[NBLK], BT[NBLK];
        f32x4 fw[NBLK];
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            A[jb] = *reinterpret_cast<const bf16x4*>(base + (0 + jb) * 512 + lane * 8);
            KT[jb] = *reinterpret_cast<const bf16x4*>(base + (4 + jb) * 512 + lane * 8);
            BT[jb] = *reinterpret_cast<const bf16x4*>(base + (8 + jb) * 512 + lane * 8);
            fw[jb] = *reinterpret_cast<const f32x4*>(base + SLOT_FW + jb * 64 + L.g * 16);
        }
        TileB Sb;
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) Sb.f[jb] = to_bf16(S[jb]);
        store_lane16(ckpt + state_record(cid, ib), lane, Sb);
        const bf16x4 U0 = __builtin_shufflevector(iv, iv, 0, 1, 2, 3);
        const bf16x4 VT = __builtin_shufflevector(iv, iv, 4, 5, 6, 7);
        const f32x4 Ua = mma2(to_f32(U0), A[0], A[1], Sb.f[0], Sb.f[1]);   // + F(S_ib Wm^T), two independent halves
        const f32x4 Uc = mma2(zero4(), A[2], A[3], Sb.f[2], Sb.f[3]);
        const bf16x4 Ub = to_bf16(Ua + Uc);
        store_frag(u_out + cid * TILE_ELEMS + ib * FRAG_ELEMS, lane, Ub);
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++)
            S[jb] = mma2(S[jb] * fw[jb], KT[jb], BT[jb], VT, Ub);          // + F(V_ib^T K_jb + U_ib^T B_jb)
    };

    ScanStage<UNITS> st[DEPTH];
#pragma unroll
    for (int s = 0; s < DEPTH; s++) issue(st[s], s);
    to_lds(0, st[0]);
    lds_barrier();

    int step0 = 0;
    for (; step0 + DEPTH <= NC; step0 += DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; s++) {
            const int step = step0 + s;
            const bf16x8 iv = st[s].iv;
            to_lds((step + 1) & 1, st[(s + 1) % DEPTH]);   // chunk step+1 -> the slot nobody reads now
            issue(st[s], step + DEPTH);
            compute(step, step & 1, iv);
            lds_barrier();
        }
    }
    // remaining NC % DEPTH steps: same step, no register pipeline.  The J record of chunk step0 is already in
    // slot step0 & 1 (copied by the last pipelined step, or by the prologue when NC < DEPTH).
    for (int step = step0; step < NC; step++) {
        ScanStage<UNITS> cur, nxt;
        issue(cur, step);
        issue(nxt, step + 1);
        to_lds((step + 1) & 1, nxt);
        compute(step, step & 1, cur.iv);
        lds_barrier();
    }
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) store_state_frag(s_out, state_f32, bh, ib, jb, L, S[jb]);
}

// ------------------------------------------------------------------------------------------------
// output: one wavefront per chunk.  With LN the GroupNorm + bonus + gate epilogue of attn_ln runs on the
// accumulators before the store, and the plain WKV7 output is kept (bf16) for the backward pass.
// ------------------------------------------------------------------------------------------------
struct LnFwdArgs {
    const __bf16 *v, *g;    // [B,T,H,64]
    const float* params;    // [3][H*64]
    __bf16* y_wkv;          // [B,T,H,64] saved for backward
};

template <bool LN>
__global__ __launch_bounds__(256) void fwd_output_kernel(int T, int H, int nchunks,
                                                         const __bf16* __restrict__ w_, const __bf16* __restrict__ q_,
                                                         const __bf16* __restrict__ k_, const __bf16* __restrict__ b_,
                                                         const __bf16* __restrict__ wsI, const __bf16* __restrict__ ckpt,
                                                         const __bf16* __restrict__ u_, __bf16* __restrict__ y_,
                                                         LnFwdArgs ln) {
    const int lane = threadIdx.x & 63;
    const int cid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (cid >= nchunks) return;
    const Lane L;
    const ChunkAddr ca(cid, T, H);

    const TileB w = load_rows(w_ + ca.row0, ca.ld, L);
    const TileB q = load_rows(q_ + ca.row0, ca.ld, L);
    const TileB k = load_rows(k_ + ca.row0, ca.ld, L);
    const TileB b = load_rows(b_ + ca.row0, ca.ld, L);
    const TileB UT = load_frags(u_ + (long)cid * TILE_ELEMS, lane);
    TileB VT;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) VT.f[ib] = *reinterpret_cast<const bf16x4*>(wsI + i_record(cid, ib) + lane * 8 + 4);

    const Decay d = chunk_decay(w);
    const TileB wq = to_bf16(mul(q, d.P));
    const TileB kwi = to_bf16(mul(k, d.Pi));
    const TileB bwi = to_bf16(mul(b, d.Pi));
    const bf16x4 QK = to_bf16(mask_lower_incl(tile_xyT(wq, kwi), L));  // F(QK), QK[t][s], s <= t
    const bf16x4 QB = to_bf16(mask_lower_incl(tile_xyT(wq, bwi), L));

    TileF yf;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        const TileB S0 = load_lane16(ckpt + state_record(cid, ib), lane);   // F(S0[16ib.., 16jb..])
        f32x4 acc = mma2(zero4(), VT.f[ib], UT.f[ib], QK, QB);         // F(QK V_ib + QB U_ib)   lane = token
        acc = mma2(acc, S0.f[0], S0.f[1], wq.f[0], wq.f[1]);           // + F(wq S0_ib^T)
        acc = mma2(acc, S0.f[2], S0.f[3], wq.f[2], wq.f[3]);
        yf.f[ib] = acc;
    }
    if constexpr (LN) {
        const int h = ca.bh % H;
        const LnParams p = load_ln_params(ln.params, h, H, L);
        const TileB v = load_rows(ln.v + ca.row0, ca.ld, L);
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
                        void* scan_ws, hipStream_t stream) {
    const int nchunks = B * H * (T / CHUNK);
    ScanWs ws = carve_scan_ws(scan_ws, nchunks);
    hipLaunchKernelGGL(fwd_prepare_kernel, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks,
                       static_cast<const __bf16*>(w), static_cast<const __bf16*>(k), static_cast<const __bf16*>(v),
                       static_cast<const __bf16*>(a), static_cast<const __bf16*>(b), ws);
}

void launch_state_scan(int B, int T, int H, int reverse, int state_f32, void* scan_ws, const void* s_in, void* s_out,
                       void* ckpt, void* u_out, hipStream_t stream) {
    const int NC = T / CHUNK;
    ScanWs ws = carve_scan_ws(scan_ws, (long)B * H * NC);
    // Two wavefronts per block, eight chunks in flight per thread: measured best on MI355X at B*H = 96
    // (four wavefronts per block: +4 us forward, +10 us backward; one: +9 / +6 us).
    const int BH = B * H;
    hipLaunchKernelGGL((state_scan_kernel<2, 8>), dim3(BH * 2), dim3(128), 0, stream, NC, BH, reverse, state_f32, ws, s_in,
                       s_out, static_cast<__bf16*>(ckpt), static_cast<__bf16*>(u_out));
}

void launch_fwd_output(int B, int T, int H, const void* w, const void* q, const void* k, const void* b,
                       const void* scan_ws, const void* ckpt, const void* u, void* y, hipStream_t stream,
                       const void* v, const void* g, const void* params, void* y_wkv) {
    const int nchunks = B * H * (T / CHUNK);
    ScanWs ws = carve_scan_ws(const_cast<void*>(scan_ws), nchunks);
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    const LnFwdArgs ln{c(v), c(g), static_cast<const float*>(params), static_cast<__bf16*>(y_wkv)};
    if (params != nullptr)
        hipLaunchKernelGGL(fwd_output_kernel<true>, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(w),
                           c(q), c(k), c(b), ws.I, c(ckpt), c(u), static_cast<__bf16*>(y), ln);
    else
        hipLaunchKernelGGL(fwd_output_kernel<false>, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(w),
                           c(q), c(k), c(b), ws.I, c(ckpt), c(u), static_cast<__bf16*>(y), ln);
}

}  // namespace wkv
