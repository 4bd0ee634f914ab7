// The GroupNorm + bonus + gate epilogue of attn_ln as kernels of their own, forward and backward, for any head
// size that is a multiple of 16 up to 128, for gfx950.
//
// Semantics follow the reference's fw_post_process / bw_post_process (attn_ln.cu:11-37, :40-104; spec
// tests/test_attn_ln.py:18-21), which the reference instantiates for whatever head size its extension is built
// with (rwkv7_attn_ln.py:11-17):
//     x1  = (y - mean(y)) * rsqrt(var(y) + 64e-5) * ln_w + ln_b        (biased variance over the head's channels)
//     x2  = x1 + (sum_c q_c k_c bonus_c) * v
//     out = x2 * g
// At head size 64 the epilogue lives inside the WKV7 kernels (ln_epilogue.hpp).  The other head sizes run the
// plain WKV7 operator followed by these kernels; written with framework operators the same arithmetic is some
// forty elementwise and reduction launches per step, several times the cost of the recurrence itself.
// The work is elementwise with three per-token sums, hence bound by its bytes: one wavefront holds 16 tokens x
// one head in registers, lane (n, g) the channels 16 ib + 4g .. + 3 of token n for every block ib, so a per-token
// sum is a register sum and two cross-lane adds.
#include "frag.hpp"
#include "device_info.hpp"
#include "ln_epilogue_heads_kernels.hpp"
#include <type_traits>

namespace wkv {
namespace lnheads {

namespace {

constexpr int TOK = 16;
constexpr float EPS = 64e-5f;
constexpr int MAX_HEAD = 128;

__device__ __forceinline__ float sum4(const f32x4& x) { return (x[0] + x[1]) + (x[2] + x[3]); }

// Which channels a lane holds.  Nothing here cares which 16 channels form a block (per-token sums run over all of
// them, the rest is elementwise), so with an even number of blocks the blocks 2p and 2p+1 interleave in groups of
// four and a lane's pieces of the two are 8 contiguous channels, one 16-byte access: with 8-byte pieces every
// access uses a quarter of each 128-byte line it touches, and the lines travel from L2 once per access.
template <int NB>
struct Map {
    static constexpr bool PAIRS = NB % 2 == 0;
    // offset inside the head of the four channels this lane holds of block ib
    static __device__ __forceinline__ int off(int ib, int g) {
        return PAIRS ? 32 * (ib >> 1) + 8 * g + 4 * (ib & 1) : 16 * ib + 4 * g;
    }
    // p: the head's first channel in this lane's token row
    static __device__ __forceinline__ void load(bf16x4 (&x)[NB], const __bf16* __restrict__ p, int g) {
        if constexpr (PAIRS) {
#pragma unroll
            for (int pr = 0; pr < NB / 2; pr++) {
                const bf16x8 v = *reinterpret_cast<const bf16x8*>(p + 32 * pr + 8 * g);
                x[2 * pr] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
                x[2 * pr + 1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
            }
        } else {
#pragma unroll
            for (int ib = 0; ib < NB; ib++) x[ib] = *reinterpret_cast<const bf16x4*>(p + 16 * ib + 4 * g);
        }
    }
    static __device__ __forceinline__ void store(__bf16* __restrict__ p, int g, const bf16x4 (&x)[NB]) {
        if constexpr (PAIRS) {
#pragma unroll
            for (int pr = 0; pr < NB / 2; pr++)
                *reinterpret_cast<bf16x8*>(p + 32 * pr + 8 * g) = __builtin_shufflevector(x[2 * pr], x[2 * pr + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
#pragma unroll
            for (int ib = 0; ib < NB; ib++) *reinterpret_cast<bf16x4*>(p + 16 * ib + 4 * g) = x[ib];
        }
    }
    // which contiguous block of 16 channels the four channels at off(ib, g) belong to
    static __device__ __forceinline__ int block(int ib, int g) { return PAIRS ? 2 * (ib >> 1) + (g >> 1) : ib; }
    static __device__ __forceinline__ f32x4 param(const float* __restrict__ p, int ib, int g) {   // p: the head's first channel
        return *reinterpret_cast<const f32x4*>(p + off(ib, g));
    }
};

// what both directions need of one token: the normalised output, 1/std and the bonus dot product
template <int NB>
struct Stats {
    f32x4 xhat[NB];
    float istd, dot;
};
// cen: the NB centres of this lane's token and head when y was kept centred per block of 16 channels (the form in
// which the WKV7 kernels of these head sizes hand attn_ln's output over, so that its bf16 rounding is relative to the
// spread and not to the mean), or null for a plain bf16 y
template <int NB>
__device__ __forceinline__ Stats<NB> stats(const bf16x4 (&y)[NB], const bf16x4 (&q)[NB], const bf16x4 (&k)[NB],
                                           const float* __restrict__ bonus, int g, const float* __restrict__ cen) {
    constexpr float INV = 1.f / (16 * NB);
    Stats<NB> s;
    float sy = 0.f, sd = 0.f;
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        s.xhat[ib] = to_f32(y[ib]);
        if (cen != nullptr) s.xhat[ib] = s.xhat[ib] + cen[Map<NB>::block(ib, g)];
        sy += sum4(s.xhat[ib]);
        sd += sum4(to_f32(q[ib]) * to_f32(k[ib]) * Map<NB>::param(bonus, ib, g));
    }
    const float mean = group_sum(sy) * INV;
    float sq = 0.f;
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        s.xhat[ib] = s.xhat[ib] - mean;
        sq += sum4(s.xhat[ib] * s.xhat[ib]);
    }
    s.istd = rsqrtf(group_sum(sq) * INV + EPS);
    s.dot = group_sum(sd);
#pragma unroll
    for (int ib = 0; ib < NB; ib++) s.xhat[ib] = s.xhat[ib] * s.istd;
    return s;
}

// forward: one wavefront per (16 tokens, head)
template <int NB>
__global__ __launch_bounds__(256) void forward_kernel(long ntiles, int H, const __bf16* __restrict__ y_,
                                                      const __bf16* __restrict__ q_, const __bf16* __restrict__ k_,
                                                      const __bf16* __restrict__ v_, const __bf16* __restrict__ g_,
                                                      const float* __restrict__ params, __bf16* __restrict__ out_,
                                                      const float* __restrict__ centers) {
    constexpr int C = 16 * NB;
    using M = Map<NB>;
    const Lane L;
    const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= ntiles * H) return;
    const long HC = (long)H * C;
    const int h = (int)(item % H);
    const long row = ((item / H) * TOK + L.n) * HC + h * C;   // the head's first channel in this lane's token row
    const float* pw = params + h * C;
    bf16x4 y[NB], q[NB], k[NB], v[NB], g[NB], out[NB];
    M::load(y, y_ + row, L.g);
    M::load(q, q_ + row, L.g);
    M::load(k, k_ + row, L.g);
    M::load(v, v_ + row, L.g);
    M::load(g, g_ + row, L.g);
    const float* cen = centers ? centers + (((item / H) * TOK + L.n) * H + h) * NB : nullptr;
    const Stats<NB> s = stats<NB>(y, q, k, pw + 2 * HC, L.g, cen);
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        const f32x4 x2 = s.xhat[ib] * M::param(pw, ib, L.g) + M::param(pw + HC, ib, L.g) + s.dot * to_f32(v[ib]);
        out[ib] = to_bf16(x2 * to_f32(g[ib]));
    }
    M::store(out_ + row, L.g, out);
}

// backward: block = (head, range of token tiles), its four wavefronts take every fourth tile and keep their share
// of the three parameter gradients in registers (lane = token partial sums); the four are combined through LDS and
// the block writes one partial record, [3][C] floats at partial[split * 3 * H * C + i * H * C + h * C ..].
struct BwdOut {
    __bf16 *dy, *dq, *dk, *dv, *dg;
};
template <int NB>
__global__ __launch_bounds__(256) void backward_kernel(long ntiles, int H, int tiles_per_split, const __bf16* __restrict__ y_,
                                                       const __bf16* __restrict__ q_, const __bf16* __restrict__ k_,
                                                       const __bf16* __restrict__ v_, const __bf16* __restrict__ g_,
                                                       const float* __restrict__ params, const __bf16* __restrict__ dout_,
                                                       BwdOut o, float* __restrict__ partial,
                                                       const float* __restrict__ centers) {
    constexpr int C = 16 * NB;
    constexpr float INV = 1.f / C;
    using M = Map<NB>;
    __shared__ float comb[4][3][C];
    const Lane L;
    const int wave = threadIdx.x >> 6;
    const int h = blockIdx.x, split = blockIdx.y;
    const long HC = (long)H * C;
    const long tile_begin = (long)split * tiles_per_split;
    const long tile_end = tile_begin + tiles_per_split < ntiles ? tile_begin + tiles_per_split : ntiles;
    const float* pw = params + h * C;
    f32x4 aw[NB], ab[NB], abo[NB];
#pragma unroll
    for (int ib = 0; ib < NB; ib++) aw[ib] = ab[ib] = abo[ib] = zero4();
    for (long tile = tile_begin + wave; tile < tile_end; tile += 4) {
        const long row = (tile * TOK + L.n) * HC + h * C;
        bf16x4 y[NB], q[NB], k[NB], v[NB], g[NB], dout[NB];
        M::load(y, y_ + row, L.g);
        M::load(q, q_ + row, L.g);
        M::load(k, k_ + row, L.g);
        M::load(v, v_ + row, L.g);
        M::load(g, g_ + row, L.g);
        M::load(dout, dout_ + row, L.g);
        const float* cen = centers ? centers + ((tile * TOK + L.n) * H + h) * NB : nullptr;
        const Stats<NB> s = stats<NB>(y, q, k, pw + 2 * HC, L.g, cen);
        f32x4 dxh[NB];
        bf16x4 dg[NB], dv[NB];
        float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
        for (int ib = 0; ib < NB; ib++) {
            const f32x4 w = M::param(pw, ib, L.g);
            const f32x4 dof = to_f32(dout[ib]), vf = to_f32(v[ib]);
            const f32x4 x2 = s.xhat[ib] * w + M::param(pw + HC, ib, L.g) + s.dot * vf;
            dg[ib] = to_bf16(dof * x2);
            const f32x4 dx2 = dof * to_f32(g[ib]);
            dv[ib] = to_bf16(s.dot * dx2);
            ab[ib] += dx2;
            aw[ib] += dx2 * s.xhat[ib];
            dxh[ib] = dx2 * w;
            s1 += sum4(dx2 * vf);
            s2 += sum4(dxh[ib]);
            s3 += sum4(dxh[ib] * s.xhat[ib]);
        }
        M::store(o.dg + row, L.g, dg);
        M::store(o.dv + row, L.g, dv);
        const float ddot = group_sum(s1);           // d/d(sum_c q k bonus)
        const float m1 = group_sum(s2) * INV;       // mean(dxhat)
        const float m2 = group_sum(s3) * INV;       // mean(dxhat * xhat)
        bf16x4 dy[NB], dq[NB], dk[NB];
#pragma unroll
        for (int ib = 0; ib < NB; ib++) {
            const f32x4 qf = to_f32(q[ib]), kf = to_f32(k[ib]);
            const f32x4 bo = M::param(pw + 2 * HC, ib, L.g) * ddot;
            dy[ib] = to_bf16(s.istd * (dxh[ib] - m1 - s.xhat[ib] * m2));
            dq[ib] = to_bf16(kf * bo);
            dk[ib] = to_bf16(qf * bo);
            abo[ib] += qf * kf * ddot;
        }
        M::store(o.dy + row, L.g, dy);
        M::store(o.dq + row, L.g, dq);
        M::store(o.dk + row, L.g, dk);
    }
    // sum over the 16 token lanes (total in lane n = 15), then over the four wavefronts in a fixed order; a
    // wavefront without tiles contributes zeros
#pragma unroll
    for (int ib = 0; ib < NB; ib++) {
        f32x4 sw, sb, sbo;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            sw[r] = row_prefix_sum(aw[ib][r]);
            sb[r] = row_prefix_sum(ab[ib][r]);
            sbo[r] = row_prefix_sum(abo[ib][r]);
        }
        if (L.n == 15) {
            *reinterpret_cast<f32x4*>(&comb[wave][0][M::off(ib, L.g)]) = sw;
            *reinterpret_cast<f32x4*>(&comb[wave][1][M::off(ib, L.g)]) = sb;
            *reinterpret_cast<f32x4*>(&comb[wave][2][M::off(ib, L.g)]) = sbo;
        }
    }
    __syncthreads();
    float* rec = partial + (long)split * 3 * HC + h * C;
    for (int e = threadIdx.x; e < 3 * C; e += 256) {
        const int i = e / C, c = e % C;
        rec[i * HC + c] = ((comb[0][i][c] + comb[1][i][c]) + comb[2][i][c]) + comb[3][i][c];
    }
}

// dparams [3][H*C] = sum of the nrec records, in a fixed order.  A block of 256 threads: 16 groups of four
// elements x 16 interleaved shares of the records, combined through LDS.
__global__ __launch_bounds__(256) void reduce_kernel(int n4, int nrec, const float* __restrict__ partial,
                                                     float* __restrict__ dparams) {
    __shared__ f32x4 sh[16][16];
    const int el = threadIdx.x & 15, share = threadIdx.x >> 4;
    const int e = blockIdx.x * 16 + el;
    f32x4 s = zero4();
    if (e < n4)
        for (int r = share; r < nrec; r += 16) s += *reinterpret_cast<const f32x4*>(partial + ((long)r * n4 + e) * 4);
    sh[share][el] = s;
    __syncthreads();
    if (share == 0 && e < n4) {
        f32x4 t = sh[0][el];
#pragma unroll
        for (int i = 1; i < 16; i++) t += sh[i][el];
        *reinterpret_cast<f32x4*>(dparams + 4L * e) = t;
    }
}

struct Acc3 {
    __bf16* dst[3];
    const __bf16* src[3];
};
__global__ __launch_bounds__(256) void accumulate_kernel(long n8, Acc3 a) {
    const long e = (long)blockIdx.x * 256 + threadIdx.x;
    if (e >= n8) return;
    const int i = blockIdx.y;
    const bf16x8 x = *reinterpret_cast<const bf16x8*>(a.dst[i] + 8 * e), y = *reinterpret_cast<const bf16x8*>(a.src[i] + 8 * e);
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; j++) o[j] = (__bf16)((float)x[j] + (float)y[j]);
    *reinterpret_cast<bf16x8*>(a.dst[i] + 8 * e) = o;
}

constexpr size_t A256(size_t x) { return (x + 255) / 256 * 256; }
// token ranges of the backward: about two blocks per compute unit over the heads, at least four tiles (one per
// wavefront) each
int splits(long ntiles, int H) {
    long s = 2 * compute_units() / H;
    if (s > ntiles / 4) s = ntiles / 4;
    if (s < 1) s = 1;
    return (int)s;
}

template <typename F>
void dispatch(int C, F&& f) {
    switch (C / 16) {
        case 1: f(std::integral_constant<int, 1>{}); break;
        case 2: f(std::integral_constant<int, 2>{}); break;
        case 3: f(std::integral_constant<int, 3>{}); break;
        case 4: f(std::integral_constant<int, 4>{}); break;
        case 5: f(std::integral_constant<int, 5>{}); break;
        case 6: f(std::integral_constant<int, 6>{}); break;
        case 7: f(std::integral_constant<int, 7>{}); break;
        default: f(std::integral_constant<int, 8>{}); break;
    }
}

}  // namespace

bool head_size_supported(int C) { return C >= 16 && C <= MAX_HEAD && C % 16 == 0; }

size_t bwd_workspace_bytes(long M, int H, int C) {
    return A256((size_t)splits(M / TOK, H) * 3 * H * C * sizeof(float));
}

void launch_forward(long M, int H, int C, const void* y, const void* q, const void* k, const void* v, const void* g,
                    const void* params, void* out, hipStream_t stream, const float* centers) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    const long ntiles = M / TOK;
    const dim3 grid((unsigned)((ntiles * H + 3) / 4));
    dispatch(C, [&](auto nb) {
        hipLaunchKernelGGL(forward_kernel<decltype(nb)::value>, grid, dim3(256), 0, stream, ntiles, H, c(y), c(q), c(k), c(v),
                           c(g), static_cast<const float*>(params), static_cast<__bf16*>(out), centers);
    });
}

void launch_backward(long M, int H, int C, const void* y, const void* q, const void* k, const void* v, const void* g,
                     const void* params, const void* dout, void* dy, void* dq, void* dk, void* dv, void* dg, void* dparams,
                     void* workspace, hipStream_t stream, const float* centers) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    auto m = [](void* p) { return static_cast<__bf16*>(p); };
    const long ntiles = M / TOK;
    const int ns = splits(ntiles, H);
    const int tiles_per_split = (int)((ntiles + ns - 1) / ns);
    float* partial = static_cast<float*>(workspace);
    const BwdOut o{m(dy), m(dq), m(dk), m(dv), m(dg)};
    dispatch(C, [&](auto nb) {
        hipLaunchKernelGGL(backward_kernel<decltype(nb)::value>, dim3(H, ns), dim3(256), 0, stream, ntiles, H, tiles_per_split,
                           c(y), c(q), c(k), c(v), c(g), static_cast<const float*>(params), c(dout), o, partial, centers);
    });
    const int n4 = 3 * H * C / 4;
    hipLaunchKernelGGL(reduce_kernel, dim3((n4 + 15) / 16), dim3(256), 0, stream, n4, ns, partial,
                       static_cast<float*>(dparams));
}

void launch_accumulate(long n, void* const dst[3], const void* const src[3], hipStream_t stream) {
    Acc3 a;
    for (int i = 0; i < 3; i++) {
        a.dst[i] = static_cast<__bf16*>(dst[i]);
        a.src[i] = static_cast<const __bf16*>(src[i]);
    }
    const long n8 = n / 8;
    hipLaunchKernelGGL(accumulate_kernel, dim3((unsigned)((n8 + 255) / 256), 3), dim3(256), 0, stream, n8, a);
}

}  // namespace lnheads
}  // namespace wkv
