// Host-side launcher of the projection weight-gradient kernel (internal; public surface is include/wind_rwkv7.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace wkv {

// How a [tokens] x (O, I) problem is cut: tile shape (index into the kernel's table), ntn tiles across the
// narrower dimension, ntiles in all, ksplit token ranges; swap = the input channels take the wider side.
struct WgradPlan {
    int shape, ntn, ntiles, ksplit;
    bool swap;
    size_t partial_bytes;
};
WgradPlan linear_wgrad_plan(long tokens, int O, int I);
// dW[o][i] = sum_t dy[t][o] x[t][i];  dy [tokens, O] (row stride ld_dy), x [tokens, I] (row stride ld_x), bf16;
// dW [O, I] contiguous, fp32 or bf16, overwritten.  O, I multiples of 16; strides multiples of 8 elements.
void launch_linear_wgrad(long tokens, int O, int I, const void* dy, long ld_dy, const void* x, long ld_x, void* dW,
                         bool out_f32, void* workspace, hipStream_t stream);

// Up to eight problems with the same token count, each with the tile shape that suits it: one launch for the products
// and one for the sums of the partial tiles.  Returns false (nothing launched) for n outside 1 .. 8 or no tokens;
// workspace bytes 0 likewise.
size_t linear_wgrad_group_workspace_bytes(int n, long tokens, const int* O, const int* I);
bool launch_linear_wgrad_group(int n, long tokens, const int* O, const int* I, const void* const* dy, const long* ld_dy,
                               const void* const* x, const long* ld_x, void* const* dW, bool out_f32, void* workspace,
                               hipStream_t stream);

// Column blocks of token-major bf16 matrices (csrc/cols.hip): piece = `width` columns (a multiple of 8) of M rows
// from (src, src_ld, src_col0) to (dst, dst_ld, dst_col0); offsets and strides multiples of 8 elements.
enum { COLS_COPY = 0, COLS_TANH = 1, COLS_TANH_GRAD = 2 };   // TANH_GRAD: src * (1 - aux^2), aux [M, width] contiguous
constexpr int COLS_MAX_PIECES = 8;   // per launch; longer lists take several
struct ColumnPiece {
    const void* src;   // null: zeros
    const void* aux;
    void* dst;
    long long src_ld, dst_ld;
    int src_col0, dst_col0, width, op;
};
void launch_copy_columns(long long M, int n, const ColumnPiece* pieces, hipStream_t stream);

// bf16 copies of n tensors (float32 or bf16, contiguous, numel[t] elements each) written to element offsets
// dst_offset[t] of dst (null: back to back)
constexpr int CAST_MAX_TENSORS = 32;   // per launch; longer lists take several
void launch_cast_to_bf16(int n, const void* const* src, const int* src_f32, const long long* numel,
                         const long long* dst_offset, void* dst, hipStream_t stream);

}  // namespace wkv
