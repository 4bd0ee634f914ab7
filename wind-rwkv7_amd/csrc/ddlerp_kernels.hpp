// Host-side launchers of the ddlerp kernels (internal; public surface is include/wind_rwkv7.h).
// M = B*T tokens; T and C must be multiples of 16 and 64; parameters are bf16 device arrays.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace wkv {

bool ddlerp_rank_supported(int D);
size_t ddlerp_bwd_workspace_bytes(long M, int C, int D);
// bmid, bder: [M, 4D] bf16 (tanh and its derivative, saved for backward); y: [4, M, C] bf16
void launch_ddlerp_forward(long M, int T, int C, int D, const void* x, const void* alpha, const void* Lw, const void* R,
                           const void* beta, void* bmid, void* bder, void* y, hipStream_t stream);
// dy4: four [M, C] bf16 gradients; dx: [M, C] bf16; dalpha [C], dL [4D, C], dR [4, C, D], dbeta [4, C]: fp32
void launch_ddlerp_backward(long M, int T, int C, int D, const void* x, const void* alpha, const void* Lw, const void* R,
                            const void* beta, const void* bmid, const void* bder, const void* const dy4[4], void* dx,
                            void* dalpha,
                            void* dL, void* dR, void* dbeta, void* workspace, hipStream_t stream);

}  // namespace wkv
