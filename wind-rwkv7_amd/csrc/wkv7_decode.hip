// WKV7 for ONE token per sequence (autoregressive decoding), with the optional attn_ln epilogue.
//
// The reference has no single-token kernel: its decode path is the token loop of ref_attn (time_mixer.py:6-16,
// the same recurrence as tests/test_attn.py:13-17), which this kernel evaluates for one step on a state that
// stays resident in HBM between calls:
//     sa = S a ;   S <- S diag(exp(-exp(w))) + sa b^T + v k^T ;   y = S q
// One wavefront owns the 64x64 state of one (batch, head) pair, in the same fragment order as the training
// kernels' state I/O (lane (n, g) holds one row piece of each of the sixteen (ib, jb) blocks), so each
// row-times-vector product is a 16-term register sum plus two cross-lane adds.  The step is pure state traffic
// (read and write 16 KiB fp32 per head) - no matrix instructions, no LDS.
#include "ln_epilogue.hpp"
#include "wkv7_common.hpp"
#include "wkv7_kernels.hpp"

namespace wkv {

struct DecodeLn {
    const __bf16* g;       // [B, H*64]
    const float* params;   // [3][H*64]
};

template <bool LN>
__global__ __launch_bounds__(256) void decode_kernel(int BH, int H, int state_f32, const __bf16* __restrict__ w_,
                                                     const __bf16* __restrict__ q_, const __bf16* __restrict__ k_,
                                                     const __bf16* __restrict__ v_, const __bf16* __restrict__ a_,
                                                     const __bf16* __restrict__ b_, void* __restrict__ state,
                                                     __bf16* __restrict__ y_, DecodeLn ln) {
    const int bh = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (bh >= BH) return;
    const Lane L;
    const long row = (long)bh * HEAD;   // this head's 64 channels in a [B, H*64] tensor

    // key-channel vectors: this lane's 4 columns of each of the 4 column blocks
    f32x4 decay[NBLK], qv[NBLK], kv[NBLK], av[NBLK], bv[NBLK];
#pragma unroll
    for (int jb = 0; jb < NBLK; jb++) {
        const long c = row + chan16(jb, 4 * L.g);
        const f32x4 wv = to_f32(*reinterpret_cast<const bf16x4*>(w_ + c));
#pragma unroll
        for (int r = 0; r < 4; r++) decay[jb][r] = __expf(-__expf(wv[r]));
        qv[jb] = to_f32(*reinterpret_cast<const bf16x4*>(q_ + c));
        kv[jb] = to_f32(*reinterpret_cast<const bf16x4*>(k_ + c));
        av[jb] = to_f32(*reinterpret_cast<const bf16x4*>(a_ + c));
        bv[jb] = to_f32(*reinterpret_cast<const bf16x4*>(b_ + c));
    }
    float y[NBLK], vrow[NBLK];
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        vrow[ib] = (float)v_[row + chan16(ib, L.n)];   // value channel of this lane's row
        f32x4 S[NBLK];
        float sa = 0.f;
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            S[jb] = load_state_frag(state, state_f32, bh, ib, jb, L);
#pragma unroll
            for (int r = 0; r < 4; r++) sa += S[jb][r] * av[jb][r];
        }
        sa = group_sum(sa);   // over the four lanes that share the row
        float acc = 0.f;
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            S[jb] = S[jb] * decay[jb] + sa * bv[jb] + vrow[ib] * kv[jb];
#pragma unroll
            for (int r = 0; r < 4; r++) acc += S[jb][r] * qv[jb][r];
            store_state_frag(state, state_f32, bh, ib, jb, L, S[jb]);
        }
        y[ib] = group_sum(acc);
    }

    if constexpr (LN) {
        // GroupNorm over the head's 64 outputs: lane (n, g) holds rows 16 ib + n, replicated over g
        auto head_sum = [&](float x) {   // sum over n (the 16 row lanes of one g), then the value is the same in every lane
            x += __shfl_xor(x, 1);
            x += __shfl_xor(x, 2);
            x += __shfl_xor(x, 4);
            x += __shfl_xor(x, 8);
            return x;
        };
        const float mean = head_sum((y[0] + y[1]) + (y[2] + y[3])) * (1.f / HEAD);
        float sq = 0.f;
#pragma unroll
        for (int ib = 0; ib < NBLK; ib++) sq += (y[ib] - mean) * (y[ib] - mean);
        const float istd = rsqrtf(head_sum(sq) * (1.f / HEAD) + LN_EPS);
        const int h = bh % H;
        const long HC = (long)H * HEAD;
        float dot = 0.f;   // sum_c q_c k_c bonus_c, over this lane's 16 key channels then across the four g lanes
#pragma unroll
        for (int jb = 0; jb < NBLK; jb++) {
            const f32x4 bonus = *reinterpret_cast<const f32x4*>(ln.params + 2 * HC + (long)h * HEAD + chan16(jb, 4 * L.g));
#pragma unroll
            for (int r = 0; r < 4; r++) dot += qv[jb][r] * kv[jb][r] * bonus[r];
        }
        dot = group_sum(dot);
#pragma unroll
        for (int ib = 0; ib < NBLK; ib++) {
            const long ch = (long)h * HEAD + chan16(ib, L.n);
            const float x1 = (y[ib] - mean) * istd * ln.params[ch] + ln.params[HC + ch];
            y[ib] = (x1 + dot * vrow[ib]) * (float)ln.g[row + chan16(ib, L.n)];
        }
    }
    if (L.g == 0) {
#pragma unroll
        for (int ib = 0; ib < NBLK; ib++) y_[row + chan16(ib, L.n)] = (__bf16)y[ib];
    }
}

void launch_decode(int B, int H, int state_f32, const void* w, const void* q, const void* k, const void* v, const void* a,
                   const void* b, void* state, void* y, hipStream_t stream, const void* g, const void* params) {
    const int BH = B * H;
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    const DecodeLn ln{c(g), static_cast<const float*>(params)};
    if (params != nullptr)
        hipLaunchKernelGGL(decode_kernel<true>, dim3((BH + 3) / 4), dim3(256), 0, stream, BH, H, state_f32, c(w), c(q), c(k),
                           c(v), c(a), c(b), state, static_cast<__bf16*>(y), ln);
    else
        hipLaunchKernelGGL(decode_kernel<false>, dim3((BH + 3) / 4), dim3(256), 0, stream, BH, H, state_f32, c(w), c(q), c(k),
                           c(v), c(a), c(b), state, static_cast<__bf16*>(y), ln);
}

}  // namespace wkv
