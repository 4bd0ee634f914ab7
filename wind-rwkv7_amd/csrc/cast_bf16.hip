// Many tensors to bf16 in one launch: the bf16 working copies of a block's projection weights.
//
// The reference casts each weight on its own before every matmul (time_mixer.py:120-131, `.to(bf16)` per
// operand).  A framework multi-tensor copy does this in chunks of 65 536 elements per block - 46 blocks for the
// 3 M weights of a 768-channel time mixer, on a chip with 256 compute units - and took 48 us per step in three
// launches.  Here a block takes 2048 elements (8 per thread, 16-byte stores), and one launch covers up to
// CAST_MAX_TENSORS tensors whose copies go to given offsets of one destination buffer (back to back, so that
// weights used together form one matrix, or padded to an alignment).
#include "linear_kernels.hpp"

#include <hip/hip_runtime.h>

#include "frag.hpp"

namespace wkv {
namespace {

constexpr int UNIT = 2048;   // elements per block

struct CastArgs {
    const void* src[CAST_MAX_TENSORS];
    long long unit_begin[CAST_MAX_TENSORS + 1];   // first block of tensor t
    long long dst_off[CAST_MAX_TENSORS];          // first destination element of tensor t
    long long numel[CAST_MAX_TENSORS];
    int src_f32[CAST_MAX_TENSORS];                // 1: float32 source, 0: bf16 source (a plain copy)
    int n;
};

__global__ __launch_bounds__(256) void cast_to_bf16_kernel(CastArgs g, __bf16* __restrict__ dst) {
    const long long unit = blockIdx.x;
    int t = 0;
    while (t + 1 < g.n && unit >= g.unit_begin[t + 1]) t++;   // the same for every thread of the block
    const long long numel = g.numel[t];
    const long long local = (unit - g.unit_begin[t]) * UNIT + threadIdx.x * 8;
    if (local >= numel) return;
    __bf16* out = dst + g.dst_off[t] + local;
    const bool whole = local + 8 <= numel && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    if (g.src_f32[t]) {
        const float* in = static_cast<const float*>(g.src[t]) + local;
        if (whole && reinterpret_cast<uintptr_t>(in) % 16 == 0) {
            const f32x4 lo = *reinterpret_cast<const f32x4*>(in), hi = *reinterpret_cast<const f32x4*>(in + 4);
            const bf16x4 a = to_bf16(lo), b = to_bf16(hi);
            *reinterpret_cast<bf16x8*>(out) = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
            for (int e = 0; e < 8 && local + e < numel; e++) out[e] = (__bf16)in[e];
        }
    } else {
        const __bf16* in = static_cast<const __bf16*>(g.src[t]) + local;
        if (whole && reinterpret_cast<uintptr_t>(in) % 16 == 0) {
            *reinterpret_cast<bf16x8*>(out) = *reinterpret_cast<const bf16x8*>(in);
        } else {
            for (int e = 0; e < 8 && local + e < numel; e++) out[e] = in[e];
        }
    }
}

}  // namespace

void launch_cast_to_bf16(int n, const void* const* src, const int* src_f32, const long long* numel,
                         const long long* dst_offset, void* dst, hipStream_t stream) {
    long long next = 0;   // where a tensor goes when no offsets are given: right after the one before
    for (int first = 0; first < n; first += CAST_MAX_TENSORS) {
        CastArgs g;
        g.n = n - first < CAST_MAX_TENSORS ? n - first : CAST_MAX_TENSORS;
        g.unit_begin[0] = 0;
        for (int t = 0; t < g.n; t++) {
            g.src[t] = src[first + t];
            g.src_f32[t] = src_f32[first + t];
            g.numel[t] = numel[first + t];
            g.dst_off[t] = dst_offset ? dst_offset[first + t] : next;
            next += numel[first + t];
            g.unit_begin[t + 1] = g.unit_begin[t] + (numel[first + t] + UNIT - 1) / UNIT;
        }
        if (g.unit_begin[g.n] > 0)
            hipLaunchKernelGGL(cast_to_bf16_kernel, dim3((unsigned)g.unit_begin[g.n]), dim3(256), 0, stream, g,
                               static_cast<__bf16*>(dst));
    }
}

}  // namespace wkv
