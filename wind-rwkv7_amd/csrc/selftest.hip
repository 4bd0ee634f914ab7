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
//  10: the sum over all sixteen columns by row_sum16_bf16 (on bf16-rounded values)
__global__ void selftest_kernel(const float* X_, const float* Y_, float* out) {
    const Lane L;
    f32x4 X = read_frag(X_, L), Y = read_frag(Y_, L);
    dump_frag(out + 0 * 256, mma(zero4(), to_bf16(Y), to_bf16(X)), L);
    dump_frag(out + 1 * 256, mma_f32(zero4(), Y, X), L);
    dump_frag(out + 2 * 256, to_f32(transpose(to_bf16(X), identity_bf16(L))), L);
    f32x4 p, s, bc, rs, gs, gw;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        p[r] = row_prefix_sum(X[r]);
        s[r] = row_suffix_sum(X[r]);
        bc[r] = row_bcast(X[r], 15);
        rs[r] = row_sum(X[r]);
        gs[r] = group_sum(X[r]);
        gw[r] = row_sum16_bf16(X);
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
    dump_frag(out + 10 * 256, gw, L);
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

// Dumps what ds_read_b64_tr_b16 returns when LDS holds its own element index and lane l points at
// element stride*l: out[4*l + r] = the 16-bit value register r of lane l received.
__global__ __launch_bounds__(64) void lds_transpose_read_kernel(int stride, short* out) {
    __shared__ short lds[4096];
    for (int i = threadIdx.x; i < 4096; i += 64) lds[i] = (short)i;
    __syncthreads();
    typedef short __attribute__((address_space(3))) lds_short;
    typedef s16x4 __attribute__((address_space(3))) lds_s16x4;
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)((lds_short*)lds + stride * threadIdx.x));
#pragma unroll
    for (int r = 0; r < 4; r++) out[4 * threadIdx.x + r] = v[r];
}

// Issue rate of LDS reads: every wavefront of the block runs `iters` rounds of 16 independent reads of one
// kind (0: ds_read_b64_tr_b16, 1: ds_read_b64, 2: ds_read_b128, 3: ds_write_b128) at the row pitch given in
// elements, and lane 0 of each wavefront reports the shader-clock cycles it took.
typedef short s16x8 __attribute__((ext_vector_type(8)));
template <int mode>
__global__ __launch_bounds__(256) void lds_rate_kernel(int iters, int pitch, long long* out) {
    __shared__ __attribute__((aligned(16))) short lds[16384];
    for (int i = threadIdx.x; i < 16384; i += blockDim.x) lds[i] = (short)i;
    __syncthreads();
    typedef short __attribute__((address_space(3))) lds_short;
    typedef s16x4 __attribute__((address_space(3))) lds_s16x4;
    const int lane = threadIdx.x & 63, kg = lane >> 4, p = lane & 15;
    typedef s16x8 __attribute__((address_space(3))) lds_s16x8;
    lds_short* const L = (lds_short*)lds;
    lds_short* base = L + (4 * kg + (p >> 2)) * pitch + 4 * (p & 3);
    lds_short* wbase = L + (lane >> 3) * pitch + 8 * (lane & 7) + 1024 * (threadIdx.x >> 6);
    s16x4 acc = {0, 0, 0, 0};
    s16x8 acc8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const long long w0 = wall_clock64();
    const long long t0 = clock64();
    for (int it = 0; it < iters; it++) {
        s16x4 v[16];
        s16x8 v8[16];
#pragma unroll
        for (int k = 0; k < 16; k++) {
            lds_short* q = base + 16 * (k & 7) + 16 * pitch * (k >> 3);
            if (mode == 0) v[k] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)q);
            else if (mode == 1) v[k] = *(volatile lds_s16x4*)q;
            else if (mode == 2) v8[k] = *(volatile lds_s16x8*)(L + 8 * ((lane + 64 * k) & 1023));
            else *(volatile lds_s16x8*)(wbase + 64 * (k & 7)) = acc8;
        }
#pragma unroll
        for (int k = 0; k < 16; k++) {
            if (mode < 2) acc ^= v[k];
            else if (mode == 2) acc8 ^= v8[k];
        }
    }
    const long long t1 = clock64();
    acc ^= __builtin_shufflevector(acc8, acc8, 0, 1, 2, 3) ^ __builtin_shufflevector(acc8, acc8, 4, 5, 6, 7);
    if (acc[0] == 12345 && acc[1] == 23456 && acc[2] == 1 && acc[3] == 2) out[63] = 1;
    const long long w1 = wall_clock64();
    if (lane == 0) out[threadIdx.x >> 6] = t1 - t0;
    if (lane == 0) out[8 + (threadIdx.x >> 6)] = w1 - w0;   // 100 MHz ticks
}

// The matrix-instruction loop with v_mfma_f32_32x32x16_bf16 (twice the flop per instruction, four accumulator
// sets of 16 registers).
typedef float f32x16 __attribute__((ext_vector_type(16)));
__global__ __launch_bounds__(256) void mfma_loop32_kernel(int iters, float* out) {
    const Lane L;
    bf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = (__bf16)(0.001f * (float)(L.n + i));
        b[i] = (__bf16)(0.002f * (float)(L.g + i));
    }
    f32x16 acc[4];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[c][r] = 0.f;
    if (iters < 0) {
        // variant: nine accumulators and three distinct operands on either side, as in a 96 x 96 output tile
        f32x16 acc9[9];
        bf16x8 av[3], bv[3];
#pragma unroll
        for (int c = 0; c < 9; c++) acc9[c] = acc[c & 3];
#pragma unroll
        for (int c = 0; c < 3; c++) {
            av[c] = a;
            bv[c] = b;
            av[c][c] = (__bf16)1.f;
            bv[c][c + 1] = (__bf16)2.f;
        }
        for (int it = 0; it < -iters; it++) {
#pragma unroll
            for (int c = 0; c < 9; c++)
                acc9[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[c / 3], bv[c % 3], acc9[c], 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < 9; c++) acc[c & 3] += acc9[c];
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int c = 0; c < 4; c++) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 4; c++) s += acc[c][0] + acc[c][7];
    if (s == 12345.678f) out[0] = s;
}

// Register layout of v_mfma_f32_32x32x16_bf16.  Operands are built assuming lane l holds row (column) l % 32 and
// contraction indices 8 (l / 32) .. + 7: A[i][0] = i + 1, A[i][1] = 1, B[0][j] = 1, B[1][j] = 64 (j + 1), so that
// D[i][j] = (i + 1) + 64 (j + 1) names its own position; out[16 l + r] = register r of lane l.
__global__ __launch_bounds__(64) void mfma32_layout_kernel(float* out) {
    const int l = threadIdx.x;
    bf16x8 a = {}, b = {};
    if (l < 32) {
        a[0] = (__bf16)(float)(l + 1);
        a[1] = (__bf16)1.f;
        b[0] = (__bf16)1.f;
        b[1] = (__bf16)(float)(64 * (l + 1));
    }
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 16; r++) out[16 * l + r] = acc[r];
}


// Global -> LDS loads without a trip through registers (buffer_load_dwordx4 ... lds / global_load_lds_dwordx4).  Every
// lane names its own 16 bytes of memory; the destination is NOT per lane: the instruction writes lane l's piece at
// (wave-uniform LDS base) + 16 l.  The instruction's immediate offset is added to BOTH addresses (the global form's is
// 13 bits, signed, and the compiler wraps larger constants silently); a buffer load's scalar offset moves the memory
// address only.  Four wavefronts, each with its own base (1 KiB apart); lane l of wavefront w fetches piece
// 128 + perm(64 w + l), perm(t) = (37 t + 11) mod 256, of src with the buffer form, the 128 pieces through the scalar
// offset; the second load, global form, names piece 255 - perm with an immediate offset of 2048 bytes, so
// it fetches the piece 128 further up and lands 2 KiB above the base it is given.  The whole LDS image is copied out.
// src: 384 pieces.
__global__ __launch_bounds__(256) void lds_dma_kernel(const int* __restrict__ src, int* __restrict__ out) {
    __shared__ __attribute__((aligned(16))) int buf[2 * 256 * 4];
    const int t = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int piece = (37 * t + 11) & 255;
    const auto r = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(src), 0, 0x7fffffff, 0x00020000);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, buf + wave * 256, 16, 16 * piece, 128 * 16, 0, 0);
    __builtin_amdgcn_global_load_lds(src + 4 * (255 - piece), buf + wave * 256 + 512, 16, 2048, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (int i = t; i < 2 * 256 * 4; i += 256) out[i] = buf[i];
}

}  // namespace wkv

extern "C" int wind_rwkv7_selftest_mfma32_layout(float* out, void* stream) {
    hipLaunchKernelGGL(wkv::mfma32_layout_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// blocks x four wavefronts, each running iters * 4 matrix instructions of 32*32*16*2 flop
extern "C" int wind_rwkv7_selftest_mfma_loop32(int blocks, int iters, float* out, void* stream) {
    hipLaunchKernelGGL(wkv::mfma_loop32_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), iters, out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

extern "C" int wind_rwkv7_selftest_lds_rate(int mode, int waves, int iters, int pitch, long long* out, void* stream) {
    if (mode < 0 || mode > 3 || waves < 1 || waves > 4 || iters < 1 || pitch < 64 || pitch > 448 || pitch % 8) return 1;
    const dim3 grid(1), block(64 * waves);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (mode) {
        case 0: hipLaunchKernelGGL(wkv::lds_rate_kernel<0>, grid, block, 0, st, iters, pitch, out); break;
        case 1: hipLaunchKernelGGL(wkv::lds_rate_kernel<1>, grid, block, 0, st, iters, pitch, out); break;
        case 2: hipLaunchKernelGGL(wkv::lds_rate_kernel<2>, grid, block, 0, st, iters, pitch, out); break;
        default: hipLaunchKernelGGL(wkv::lds_rate_kernel<3>, grid, block, 0, st, iters, pitch, out); break;
    }
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

extern "C" int wind_rwkv7_selftest_lds_transpose_read(int stride, short* out, void* stream) {
    if (stride < 4 || stride > 64 || stride % 4) return 1;
    hipLaunchKernelGGL(wkv::lds_transpose_read_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), stride, out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// Launches `blocks` blocks of four wavefronts, each running iters * 8 matrix instructions of 16*16*32*2 flop.
extern "C" int wind_rwkv7_selftest_mfma_loop(int blocks, int iters, float* out, void* stream) {
    hipLaunchKernelGGL(wkv::mfma_loop_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), iters, out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

extern "C" int wind_rwkv7_selftest_primitives(const float* X, const float* Y, float* out, void* stream) {
    hipLaunchKernelGGL(wkv::selftest_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), X, Y, out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// src: 1536 ints (384 pieces of 16 bytes); out: 2048 ints, the LDS image after the two loads of lds_dma_kernel
extern "C" int wind_rwkv7_selftest_lds_dma(const int* src, int* out, void* stream) {
    hipLaunchKernelGGL(wkv::lds_dma_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream), src, out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}
