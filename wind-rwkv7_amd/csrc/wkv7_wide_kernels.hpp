// Host-side launchers of the WKV7 kernels for head sizes other than 64 (wkv7_wide.hip): bf16 sequences, the
// state in fp32 or bf16, head size C a multiple of 16 up to 128.  All pointers are device pointers; nothing here
// allocates or synchronises.
#pragma once
#include <hip/hip_runtime.h>

namespace wkv {
namespace wide {

bool head_size_supported(int C);
// what the forward keeps for the backward pass (and the backward scan for its gradient kernel), 256-byte multiple
size_t kept_bytes(int B, int T, int H, int C);
// one direction's chunk records: written by its prepare kernel, read by its scan
size_t record_bytes(int B, int T, int H, int C, bool forward);

// y, s_out = WKV7(..., s_in).  rec: record_bytes(forward); kept: kept_bytes, or null when no backward pass follows.
// s_in may be null (zero state).  centers != nullptr: y is written centred per token and block of 16 channels and the
// centres go there ([B*T*H][C/16] floats) - the form in which attn_ln keeps the WKV7 output.
void launch_forward(int B, int T, int H, int C, int state_f32, const void* w, const void* q, const void* k, const void* v,
                    const void* a, const void* b, const void* s_in, void* s_out, void* y, void* rec, void* kept,
                    hipStream_t stream, float* centers = nullptr);
// Gradients.  kept_f: what launch_forward kept; rec: record_bytes(backward); kept_b: kept_bytes of scratch.
// ds_in (gradient of the final state) may be null (zero), ds_out (gradient of the initial state) may be null.
void launch_backward(int B, int T, int H, int C, int state_f32, const void* w, const void* q, const void* k, const void* v,
                     const void* a, const void* b, const void* dy, const void* kept_f, const void* ds_in, void* ds_out,
                     void* dw, void* dq, void* dk, void* dv, void* da, void* db, void* rec, void* kept_b,
                     hipStream_t stream);

// One token per sequence on a resident state [B,H,C,C] (updated in place); params != nullptr adds the attn_ln
// epilogue (g: [B, H*C] bf16, params: [3, H*C] float).
void launch_decode(int B, int H, int C, int state_f32, const void* w, const void* q, const void* k, const void* v,
                   const void* a, const void* b, void* state, void* y, hipStream_t stream, const void* g = nullptr,
                   const void* params = nullptr);

}  // namespace wide
}  // namespace wkv
