// Host-side launchers of the fp32 WKV7 kernels (internal; public surface is include/wind_rwkv7.h).
// All tensors fp32: sequences [B,T,H,C], states [B,H,C,C]; what the forward keeps for the backward: wkv7_f32_saved_bytes;
// C a multiple of 16 up to WKV7_F32_MAX_HEAD.
#pragma once
#include <hip/hip_runtime.h>

namespace wkv {

constexpr int WKV7_F32_MAX_HEAD = 128;
constexpr int WKV7_F32_CHUNK = 16;   // tokens between saved states; T must be a multiple
size_t wkv7_f32_saved_bytes(int B, int T, int H, int C);   // what `ckpt` must hold: the states [B,H,T/16,C,C] and [B,T,H,C] floats

// ckpt may be null: then no state is saved (a forward that nothing differentiates)

void launch_wkv7_f32_forward(int B, int T, int H, int C, const float* w, const float* q, const float* k, const float* v,
                             const float* a, const float* b, const float* s0, float* y, float* ckpt, float* sT,
                             hipStream_t stream);
void launch_wkv7_f32_backward(int B, int T, int H, int C, const float* w, const float* q, const float* k, const float* v,
                              const float* a, const float* b, const float* dy, const float* ckpt, const float* dsT,
                              float* dw, float* dq, float* dk, float* dv, float* da, float* db, float* ds0,
                              hipStream_t stream);

}  // namespace wkv
