// Host-side launchers of the fp32 WKV7 kernels (internal; public surface is include/wind_rwkv7.h).
// All tensors fp32: sequences [B,T,H,64], states [B,H,64,64], checkpoints [B,H,T/F32_CHUNK,64,64].
#pragma once
#include <hip/hip_runtime.h>

namespace wkv {

constexpr int F32_CHUNK = 8;   // tokens between saved states; T must be a multiple

void launch_wkv7_f32_forward(int B, int T, int H, const float* w, const float* q, const float* k, const float* v,
                             const float* a, const float* b, const float* s0, float* y, float* ckpt, float* sT,
                             hipStream_t stream);
void launch_wkv7_f32_backward(int B, int T, int H, const float* w, const float* q, const float* k, const float* v,
                              const float* a, const float* b, const float* dy, const float* ckpt, const float* dsT,
                              float* dw, float* dq, float* dk, float* dv, float* da, float* db, float* ds0,
                              hipStream_t stream);

}  // namespace wkv
