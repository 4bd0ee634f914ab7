// Device self-test of the fragment primitives (built into its own small library, used by the GPU
// tests only).  Each entry runs one wavefront and writes plain row-major 16x16 results so the host can
// compare with ordinary matrix arithmetic.
#include "frag.hpp"

namespace wkv {

// writes F(M) as a row-major 16x16 float matrix
__device__ void dump_frag(float* out, f32x4 x, const Lane& L) {
#pragma unroll
    for (int r = 0; r < 4; r++) out[L.n * 16 + 4 * L.g + r] = x[r];
}
__device__ f32x4 read_frag(const float* in, const Lane& L) {
    f32x4 x;
#pragma unroll
    for (int r = 0; r < 4; r++) x[r] = in[L.n * 16 + 4 * L.g + r];
    return x;
}

// in: X, Y (16x16 row-major floats).  out: 8 matrices of 16x16:
//  0: X*Y^T via bf16 mma   1: X*Y^T via fp32 mma   2: X^T via identity product
//  3: prefix sum of X over rows   4: suffix sum over rows   5: row 15 broadcast   6: sum over rows   7: inv(I - strict_tril(X))
//  8: transpose of 7 as returned by tri_inverse   9: group_sum of X (sum over the four column groups, per register)
__global__ void selftest_kernel(const float* X_, const float* Y_, float* out) {
    const Lane L;
    f32x4 X = read_frag(X_, L), Y = read_frag(Y_, L);
    dump_frag(out + 0 * 256, mma(zero4(), to_bf16(Y), to_bf16(X)), L);
    dump_frag(out + 1 * 256, mma_f32(zero4(), Y, X), L);
    dump_frag(out + 2 * 256, to_f32(transpose(to_bf16(X), identity_bf16(L))), L);
    f32x4 p, s, bc, rs, gs;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        p[r] = row_prefix_sum(X[r]);
        s[r] = row_suffix_sum(X[r]);
        bc[r] = row_bcast(X[r], 15);
        rs[r] = row_sum(X[r]);
        gs[r] = group_sum(X[r]);
    }
    dump_frag(out + 3 * 256, p, L);
    dump_frag(out + 4 * 256, s, L);
    dump_frag(out + 5 * 256, bc, L);
    dump_frag(out + 6 * 256, rs, L);
    f32x4 Xl = mask_lower_strict(X, L);
    f32x4 XT = mma_f32(zero4(), Xl, identity_f32(L));  // F(Xl^T)
    f32x4 M, MT;
    tri_inverse(Xl, XT, L, M, MT);
    dump_frag(out + 7 * 256, M, L);
    dump_frag(out + 8 * 256, MT, L);
    dump_frag(out + 9 * 256, gs, L);
}

// Dense matrix-instruction loop for a measured bf16 peak: eight independent accumulator chains of
// v_mfma_f32_16x16x32_bf16 per wavefront, operands in registers, nothing else in the loop.
__global__ __launch_bounds__(256) void mfma_loop_kernel(int iters, float* out) {
    const Lane L;
    bf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = (__bf16)(0.001f * (float)(L.n + i));
        b[i] = (__bf16)(0.002f * (float)(L.g + i));
    }
    f32x4 acc[8];
#pragma unroll
    for (int c = 0; c < 8; c++) acc[c] = zero4();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int c = 0; c < 8; c++) acc[c] = mma8(acc[c], a, b);
    }
    f32x4 s = zero4();
#pragma unroll
    for (int c = 0; c < 8; c++) s += acc[c];
    if (s[0] == 12345.678f) out[0] = s[1];   // keeps the loop alive; never true for these operands
}

}  // namespace wkv

// Launches `blocks` blocks of four wavefronts, each running iters * 8 matrix instructions of 16*16*32*2 flop.
extern "C" int wind_rwkv7_selftest_mfma_loop(int blocks, int iters, float* out, void* stream) {
    hipLaunchKernelGGL(wkv::mfma_loop_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), iters, out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

extern "C" int wind_rwkv7_selftest_primitives(const float* X, const float* Y, float* out, void* stream) {
    hipLaunchKernelGGL(wkv::selftest_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), X, Y, out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}
