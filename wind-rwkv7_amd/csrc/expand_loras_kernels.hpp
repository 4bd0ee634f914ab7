// Host-side launchers of the expand_loras kernels (internal; public surface is include/wind_rwkv7.h).
// M = B*T tokens (multiple of 16); C a multiple of 64 and of the head size HS (itself a multiple of 16); all
// tensors bf16 unless noted.
// Index order of the four LoRAs everywhere: 0 = z (kk), 1 = a, 2 = ma, 3 = mk; biases: 0 = w_bias.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace wkv {

bool expand_loras_rank_supported(int D);
bool expand_loras_head_size_supported(int C, int HS);
size_t expand_loras_bwd_workspace_bytes(long M, int C, int D);
// outs: w_out, k_out, kk_out, b_out [M, C]
void launch_expand_loras_forward(long M, int C, int D, int HS, const void* w_in, const void* k_in, const void* const acts[4],
                                 const void* const Ws[4], const void* const biases[4], void* const outs[4],
                                 hipStream_t stream);
// dys: dw_out, dk_out, dkk_out, db_out [M, C]; dacts: [M, D] bf16; dWs [C, D] and dbiases [C]: fp32
void launch_expand_loras_backward(long M, int C, int D, int HS, const void* w_in, const void* k_in, const void* const acts[4],
                                  const void* const Ws[4], const void* const biases[4], const void* const dys[4],
                                  void* dw_in, void* dk_in, void* const dacts[4], void* const dWs[4],
                                  void* const dbiases[4], void* workspace, hipStream_t stream);

}  // namespace wkv
