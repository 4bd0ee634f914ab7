// Column blocks of token-major matrices, moved (and passed through tanh or its derivative) in one launch.
//
// The reference concatenates the first halves of several LoRAs into one product and splits the result
// (time_mixer.py:124-131: `w1,a1,ma1 = (xwa @ cat(...).mT).split(...)`, `tanh(w1) @ w2.mT`); the framework then
// copies every slice to a contiguous tensor for the next kernel, runs tanh on a strided view, and in the
// backward pass rebuilds the gradient of the wide tensor with tanh-backward and concatenation kernels - eleven
// small launches around five slices.  Here a "piece" is `width` columns of M rows, read at (src, src_ld,
// src_col0) and written at (dst, dst_ld, dst_col0), optionally through tanh (forward) or multiplied by
// 1 - y^2 with y the saved tanh output (backward); up to COLS_MAX_PIECES pieces per launch.
#include "linear_kernels.hpp"

#include <hip/hip_runtime.h>

#include "frag.hpp"

namespace wkv {
namespace {

struct Piece {
    const __bf16* src;   // null: zeros
    const __bf16* aux;   // COLS_TANH_GRAD: the tanh output, rows of `width` elements
    __bf16* dst;
    long long src_ld, dst_ld, vec_begin;   // vec_begin: first 8-element vector of this piece in the launch
    int src_col0, dst_col0, width, op;
};
struct ColsArgs {
    Piece p[COLS_MAX_PIECES];
    long long vec_end;
    int n;
};

__global__ __launch_bounds__(256) void copy_columns_kernel(ColsArgs g) {
    const long long v = (long long)blockIdx.x * 256 + threadIdx.x;
    if (v >= g.vec_end) return;
    int t = 0;
    while (t + 1 < g.n && v >= g.p[t + 1].vec_begin) t++;
    const Piece& p = g.p[t];
    const long long local = v - p.vec_begin;
    const int per_row = p.width / 8;
    const long long m = local / per_row;
    const int c = (int)(local - m * per_row) * 8;
    bf16x8 x = {};
    if (p.src) x = *reinterpret_cast<const bf16x8*>(p.src + m * p.src_ld + p.src_col0 + c);
    if (p.op != COLS_COPY) {
        bf16x8 y = {};
        if (p.op == COLS_TANH_GRAD) y = *reinterpret_cast<const bf16x8*>(p.aux + m * p.width + c);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float xf = (float)x[e];
            if (p.op == COLS_TANH) {
                x[e] = (__bf16)tanhf(xf);
            } else {
                const float yf = (float)y[e];
                x[e] = (__bf16)(xf * (1.f - yf * yf));
            }
        }
    }
    *reinterpret_cast<bf16x8*>(p.dst + m * p.dst_ld + p.dst_col0 + c) = x;
}

}  // namespace

void launch_copy_columns(long long M, int n, const ColumnPiece* pieces, hipStream_t stream) {
    for (int first = 0; first < n; first += COLS_MAX_PIECES) {
        ColsArgs g;
        g.n = n - first < COLS_MAX_PIECES ? n - first : COLS_MAX_PIECES;
        long long v = 0;
        for (int t = 0; t < g.n; t++) {
            const ColumnPiece& c = pieces[first + t];
            g.p[t] = Piece{static_cast<const __bf16*>(c.src), static_cast<const __bf16*>(c.aux), static_cast<__bf16*>(c.dst),
                           c.src_ld, c.dst_ld, v, c.src_col0, c.dst_col0, c.width, c.op};
            v += M * (c.width / 8);
        }
        g.vec_end = v;
        if (v > 0) hipLaunchKernelGGL(copy_columns_kernel, dim3((unsigned)((v + 255) / 256)), dim3(256), 0, stream, g);
    }
}

}  // namespace wkv
