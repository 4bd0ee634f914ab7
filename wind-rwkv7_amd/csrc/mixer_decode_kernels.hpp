// Host-side launcher of the single-token time-mixer step (internal; public surface is include/wind_rwkv7.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace wkv {

// The block's parameters (names as in time_mixer.py:42-104), bf16 device arrays except ln_params.
struct MixerWeights {
    const void *time_maa_x, *time_maa, *time_maa_w1, *time_maa_w2;            // [C], [4,C], [128,C], [4,C,32]
    const void *Wr, *Wk, *Wv, *Wo;                                            // [C,C]
    const void *gate_w1, *time_decay_w1, *time_kkk_w1, *mk_w1, *time_aaa_w1, *ma_w1;   // [rank,C]
    const void *gate_w2, *time_decay_w2, *time_kkk_w2, *mk_w2, *time_aaa_w2, *ma_w2;   // [C,rank]
    const void *time_decay, *time_aaaaa, *time_misc_a, *time_misc_k;          // [C]
    const void* ln_params;                                                    // [3,C] fp32: GroupNorm weight, bias, bonus
};

size_t mixer_decode_workspace_bytes(int B, int C);
// x, x_prev [B,C] bf16; state [B,H,64,64] (bf16 or fp32), updated in place; y [B,C] bf16; x_carry: null or [B,C] bf16
// that receives a copy of x (the next step's x_prev; must not alias x_prev)
void launch_mixer_decode(int B, int C, int H, int state_f32, const MixerWeights& w, const void* x, const void* x_prev,
                         void* state, void* y, void* x_carry, void* workspace, hipStream_t stream);

}  // namespace wkv
