// Host-side launchers of the fp32 WKV7 kernels (internal; public surface is include/wind_rwkv7.h).
// All tensors fp32: sequences [B,T,H,C], states [B,H,C,C], checkpoints [B,H,T/wkv7_f32_chunk(C),C,C] (wkv7_f32_saved_bytes);
// C a multiple of 16 up to WKV7_F32_MAX_HEAD.
#pragma once
#include <hip/hip_runtime.h>

namespace wkv {

constexpr int WKV7_F32_MAX_HEAD = 128;
int wkv7_f32_chunk(int C);   // tokens between saved states (16 at C = 64 and 128, 8 below 64, 2 at 80 .. 112); T must be a multiple
size_t wkv7_f32_saved_bytes(int B, int T, int H, int C);   // what `ckpt` must hold: those states; at C = 64 and 128 also [B,T,H,C] floats

// ckpt may be null: then no state is saved (a forward that nothing differentiates)

void launch_wkv7_f32_forward(int B, int T, int H, int C, const float* w, const float* q, const float* k, const float* v,
                             const float* a, const float* b, const float* s0, float* y, float* ckpt, float* sT,
                             hipStream_t stream);
void launch_wkv7_f32_backward(int B, int T, int H, int C, const float* w, const float* q, const float* k, const float* v,
                              const float* a, const float* b, const float* dy, const float* ckpt, const float* dsT,
                              float* dw, float* dq, float* dk, float* dv, float* da, float* db, float* ds0,
                              hipStream_t stream);

}  // namespace wkv
