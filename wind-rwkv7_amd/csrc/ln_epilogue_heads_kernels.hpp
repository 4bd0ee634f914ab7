// Host-side launchers of the stand-alone attn_ln epilogue kernels (internal; public surface is include/wind_rwkv7.h).
// M = B*T tokens (multiple of 16); sequences [M, H, C] bf16; params [3][H*C] fp32 (ln weight, ln bias, bonus).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace wkv {
namespace lnheads {

bool head_size_supported(int C);   // multiples of 16 up to 128
size_t bwd_workspace_bytes(long M, int H, int C);
// centers != nullptr: y is centred per token and block of 16 contiguous channels, the centres [M*H][C/16] floats there
// (the form in which the WKV7 kernels of these head sizes hand attn_ln's output over); null: a plain bf16 y.
void launch_forward(long M, int H, int C, const void* y, const void* q, const void* k, const void* v, const void* g,
                    const void* params, void* out, hipStream_t stream, const float* centers = nullptr);
// dy: gradient of the WKV7 output; dq, dk, dv: the epilogue's own contributions (bonus term); dparams [3][H*C] fp32,
// overwritten, summed in a fixed order
void launch_backward(long M, int H, int C, const void* y, const void* q, const void* k, const void* v, const void* g,
                     const void* params, const void* dout, void* dy, void* dq, void* dk, void* dv, void* dg, void* dparams,
                     void* workspace, hipStream_t stream, const float* centers = nullptr);

// dst[i] += src[i] for three bf16 arrays of n elements (n a multiple of 8), summed in fp32 and rounded once
void launch_accumulate(long n, void* const dst[3], const void* const src[3], hipStream_t stream);

}  // namespace lnheads
}  // namespace wkv
