// Per-head GroupNorm + bonus + gate epilogue of attn_ln, forward and backward, on token-major tiles.
//
// Semantics follow the reference's fw_post_process / bw_post_process (attn_ln.cu:11-37, :40-104;
// spec tests/test_attn_ln.py:18-21):
//     x1  = (y - mean(y)) * rsqrt(var(y) + 64e-5) * ln_w + ln_b        (biased variance over the head's 64 channels)
//     x2  = x1 + (sum_c q_c k_c bonus_c) * v
//     out = x2 * g
// A token row of a 16x64 tile is spread over the four lanes (n, 0..3), 16 channels each, so every
// per-token reduction is a 16-term sum in registers followed by two cross-lane exchanges (group_sum);
// the reference needs a shared-memory reduction across warps with four block barriers for each.
#pragma once
#include "frag.hpp"

namespace wkv {

constexpr float LN_EPS = 64e-5f;

struct LnParams {  // this lane's 16 channels of the head's parameters
    TileF w, b, bonus;
};
// params: [3][H*64] fp32 (ln weight, ln bias, bonus), as the reference stacks them (rwkv7_attn_ln.py:26).
__device__ __forceinline__ LnParams load_ln_params(const float* __restrict__ params, int h, int H, const Lane& L) {
    LnParams p;
    const long HC = (long)H * HEAD;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        const long ch = (long)h * HEAD + chan16(ib, 4 * L.g);   // tiles come from load_rows16
        p.w.f[ib] = *reinterpret_cast<const f32x4*>(params + ch);
        p.b.f[ib] = *reinterpret_cast<const f32x4*>(params + HC + ch);
        p.bonus.f[ib] = *reinterpret_cast<const f32x4*>(params + 2 * HC + ch);
    }
    return p;
}

__device__ __forceinline__ float tile_row_sum(const TileF& x) {  // sum over the token's 64 channels
    float s = 0.f;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) s += (x.f[ib][0] + x.f[ib][1]) + (x.f[ib][2] + x.f[ib][3]);
    return group_sum(s);
}

// How the plain WKV7 output is kept between kernels (for the epilogue as a kernel of its own, and for the backward
// pass): bf16, but CENTRED per token and block of 16 channels - y' = y - c with c the fp32 mean of the block, kept
// beside it (16 bytes per token and head).  GroupNorm subtracts the head's mean and divides by its spread, so an error
// in y counts relative to the spread; rounding y itself to bf16 makes an error relative to |y|, which with a large
// common offset (|mean| >> spread) is many times larger, while the rounding error of y' is relative to the spread.
// The reference's epilogue works on the fp32 accumulator tile (attn_ln.cu:11-22); this keeps its accuracy at bf16
// traffic.  centers: [tokens x heads][4] floats, block ib of a token's head at index 4 * (token * H + head) + ib.  Any
// value near the mean serves as a centre (the reader adds back exactly what the writer took off): the forward with the
// epilogue inside uses the head's mean, which its statistics have anyway, for all four blocks; where the plain
// forward's chain wavefronts write the output, each knows only its own 16 channels and takes their mean.
struct Centred {
    TileB y;      // y - c, bf16
    f32x4 c;      // per block of 16 channels
};
// centers == nullptr: y was kept uncentred (callers that hand in a plain bf16 output, e.g. the standalone epilogue entry point)
__device__ __forceinline__ TileF uncentre(const TileB& y, const float* __restrict__ centers, long token_head) {
    TileF r = to_f32(y);
    if (centers != nullptr) {
        const f32x4 c = *reinterpret_cast<const f32x4*>(centers + 4 * token_head);
#pragma unroll
        for (int ib = 0; ib < NBLK; ib++) r.f[ib] += c[ib];
    }
    return r;
}

struct LnStats {
    TileF xhat;   // (y - mean) * istd
    float istd;
    float dot;    // sum_c q k bonus
    float mean;
};
__device__ __forceinline__ LnStats ln_stats(const TileF& y, const TileB& q, const TileB& k, const LnParams& p) {
    LnStats s;
    const float mean = tile_row_sum(y) * (1.f / HEAD);
    s.mean = mean;
    TileF c, sq, qk;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        c.f[ib] = y.f[ib] - mean;
        sq.f[ib] = c.f[ib] * c.f[ib];
        qk.f[ib] = to_f32(q.f[ib]) * to_f32(k.f[ib]) * p.bonus.f[ib];
    }
    s.istd = rsqrtf(tile_row_sum(sq) * (1.f / HEAD) + LN_EPS);
    s.dot = tile_row_sum(qk);
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) s.xhat.f[ib] = c.f[ib] * s.istd;
    return s;
}

// forward: out = ((xhat*ln_w + ln_b) + dot*v) * g.  kept != nullptr: also the output as it is kept for the backward
// pass, centred on the head's mean, which the statistics have anyway (one centre for all four blocks).
__device__ __forceinline__ TileB ln_forward(const TileF& y, const TileB& q, const TileB& k, const TileB& v,
                                            const TileB& g, const LnParams& p, Centred* kept = nullptr) {
    const LnStats s = ln_stats(y, q, k, p);
    if (kept != nullptr) {
#pragma unroll
        for (int ib = 0; ib < NBLK; ib++) {
            kept->y.f[ib] = to_bf16(y.f[ib] - s.mean);
            kept->c[ib] = s.mean;
        }
    }
    TileB out;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        const f32x4 x2 = s.xhat.f[ib] * p.w.f[ib] + p.b.f[ib] + s.dot * to_f32(v.f[ib]);
        out.f[ib] = to_bf16(x2 * to_f32(g.f[ib]));
    }
    return out;
}

// backward of the epilogue for one chunk.  y is the saved WKV7 output.
struct LnBackward {
    TileB dy;        // gradient w.r.t. the WKV7 output (what the WKV7 backward consumes)
    TileB dg;        // gradient w.r.t. the gate
    TileB dv_bonus;  // dot * dx2                       (added to dv)
    float ddot;      // sum_c dx2_c v_c ; dq += k*bonus*ddot, dk += q*bonus*ddot
    TileF dw, db, dbonus;  // this token's contribution to the parameter gradients (sum over tokens is the caller's)
};
__device__ __forceinline__ LnBackward ln_backward(const TileF& y, const TileB& q, const TileB& k, const TileB& v,
                                                  const TileB& g, const TileB& dout, const LnParams& p) {
    LnBackward r;
    const LnStats s = ln_stats(y, q, k, p);
    TileF dx2, t1, t2, t3;
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        const f32x4 dof = to_f32(dout.f[ib]), vf = to_f32(v.f[ib]);
        const f32x4 x2 = s.xhat.f[ib] * p.w.f[ib] + p.b.f[ib] + s.dot * vf;
        r.dg.f[ib] = to_bf16(dof * x2);
        dx2.f[ib] = dof * to_f32(g.f[ib]);
        r.dv_bonus.f[ib] = to_bf16(s.dot * dx2.f[ib]);
        t1.f[ib] = dx2.f[ib] * vf;                       // -> ddot
        r.db.f[ib] = dx2.f[ib];
        r.dw.f[ib] = dx2.f[ib] * s.xhat.f[ib];
        t2.f[ib] = dx2.f[ib] * p.w.f[ib];                // dxhat
        t3.f[ib] = t2.f[ib] * s.xhat.f[ib];
    }
    r.ddot = tile_row_sum(t1);
    const float m1 = tile_row_sum(t2) * (1.f / HEAD);    // mean(dxhat)
    const float m2 = tile_row_sum(t3) * (1.f / HEAD);    // mean(dxhat * xhat)
#pragma unroll
    for (int ib = 0; ib < NBLK; ib++) {
        r.dbonus.f[ib] = to_f32(q.f[ib]) * to_f32(k.f[ib]) * r.ddot;
        r.dy.f[ib] = to_bf16(s.istd * (t2.f[ib] - m1 - s.xhat.f[ib] * m2));
    }
    return r;
}

}  // namespace wkv
