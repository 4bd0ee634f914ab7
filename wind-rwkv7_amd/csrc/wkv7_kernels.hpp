// Host-side launchers of the WKV7 device kernels (internal to the library; the public surface is
// include/wind_rwkv7.h).  All pointers are device pointers; nothing here allocates or synchronises.
#pragma once
#include <hip/hip_runtime.h>

namespace wkv {

void launch_fwd_prepare(int B, int T, int H, const void* w, const void* k, const void* v, const void* a, const void* b,
                        void* scan_ws, hipStream_t stream);
void launch_state_scan(int B, int T, int H, int reverse, int state_f32, void* scan_ws, const void* s_in, void* s_out,
                       void* ckpt, void* u_out, hipStream_t stream);
void launch_fwd_output(int B, int T, int H, const void* w, const void* q, const void* k, const void* b,
                       const void* scan_ws, const void* ckpt, const void* u, void* y, hipStream_t stream);

void launch_bwd_prepare(int B, int T, int H, const void* w, const void* q, const void* a, const void* b, const void* dy,
                        void* scan_ws, hipStream_t stream);
void launch_bwd_grads(int B, int T, int H, const void* w, const void* q, const void* k, const void* v, const void* a,
                      const void* b, const void* dy, const void* s0ckpt, const void* u, const void* dsckpt,
                      const void* dabu, void* dw, void* dq, void* dk, void* dv, void* da, void* db, hipStream_t stream);

}  // namespace wkv
