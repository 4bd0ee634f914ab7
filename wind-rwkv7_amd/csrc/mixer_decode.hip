// One token per sequence through the whole RWKV-7 time mixer (decoding), for gfx950: five launches.
//
// The reference's block has no single-token form: its forward (time_mixer.py:96-167) is the specification, taken at
// T = 1 with the previous token and the WKV7 state carried by the caller.  A step through the sequence kernels is some
// twenty launches of kernels built for thousands of tokens, each waiting out its own launch and drain; here the B
// tokens are the rows of 16-row tiles (rows past B are zero and never stored) and every stage is a kernel whose grid
// is as wide as the stage's OUTPUT, so the weights (6 MB) stream once through many compute units:
//   1. mix      the four token-shifted streams (rwkv7_ddlerp.py:20-84): one block per tile, a wavefront per 64
//               channels, the contraction over the channels added in LDS
//   2. linear   all first-half products (time_mixer.py:120-131) - r, k, v and the six LoRA first halves, nine weight
//               matrices - in one launch: a block per 16 output columns, its wavefronts splitting the contraction
//   3. expand   the LoRA second halves with the elementwise tail (rwkv7_expand_loras.py:33-70) and the gate's and the
//               decay's second halves, one wavefront per (tile, head)
//   4. the single-token WKV7 recurrence with GroupNorm, bonus and gate (wkv7_decode.hip)
//   5. linear   the output projection
// Rounding follows the sequence path: every tensor that path keeps in bf16 between its kernels is rounded to bf16
// here at the same place.
#include "mixer_decode_kernels.hpp"

#include "frag.hpp"
#include "wkv7_kernels.hpp"

namespace wkv {

namespace {

constexpr int TOK = 16;
// LoRA ranks of the block (time_mixer.py:42-104)
constexpr int R_MIX = 32, R_DECAY = 64, R_AAA = 16, R_KKK = 16, R_GATE = 128, R_MA = 16, R_MK = 16;

__device__ __forceinline__ float sigmoidf_(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }
// log(1 + exp(-|u|)): the argument of the logarithm lies in [1, 2], so the bare v_log_f32 needs none of the
// denormal handling that __logf wraps around it (four instructions per element)
__device__ __forceinline__ float log1pexp_(float u) {
    return 0.6931471805599453f * __builtin_amdgcn_logf(1.f + __expf(-fabsf(u)));
}
__device__ __forceinline__ float tanhf_(float x) {
    const float e = __expf(2.f * fminf(x, 40.f));
    return 1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f);
}
__device__ __forceinline__ bf16x4 lo4(bf16x8 v) { return __builtin_shufflevector(v, v, 0, 1, 2, 3); }
__device__ __forceinline__ bf16x4 hi4(bf16x8 v) { return __builtin_shufflevector(v, v, 4, 5, 6, 7); }
__device__ __forceinline__ bf16x8 cat8(bf16x4 a, bf16x4 b) { return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7); }

// In every 32-wide product below a lane group g holds contraction indices 8g .. 8g+7 of BOTH operands (one 16-byte
// load each): the order of the summed index is free as long as the operands agree.

// ------------------------------------------------------------------------------------------------
// 1. mix: y_k = x + xx (tanh((x + xx alpha) L^T)_k R_k^T + beta_k),  xx = x_prev - x
// ------------------------------------------------------------------------------------------------
constexpr int MIX_MAX_WAVES = 12;   // one wavefront per 64-channel block up to C = 768; 8 KiB of partial sums each
__global__ __launch_bounds__(64 * MIX_MAX_WAVES) void decode_mix_kernel(int B, int Bp, int C, const __bf16* __restrict__ x,
                                                         const __bf16* __restrict__ x_prev,
                                                         const __bf16* __restrict__ alpha, const __bf16* __restrict__ beta,
                                                         const __bf16* __restrict__ Lw, const __bf16* __restrict__ R,
                                                         __bf16* __restrict__ streams, __bf16* __restrict__ x_carry) {
    constexpr int NOB = 4 * R_MIX / 16;               // 8 blocks of 16 mid values
    __shared__ f32x4 part[MIX_MAX_WAVES][NOB][WAVE];  // the wavefronts' partial sums of the first product
    __shared__ __attribute__((aligned(16))) __bf16 s_bm[4][WAVE * 8];   // tanh(...)_k as the second product's operand
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const Lane L;
    const int row = blockIdx.x * TOK + L.n;
    const bool valid = row < B;
    const long xrow = (long)(valid ? row : B - 1) * C;
    const int ncb = C / 64;

    f32x4 acc[NOB];
#pragma unroll
    for (int ob = 0; ob < NOB; ob++) acc[ob] = zero4();
    for (int cb = wave; cb < ncb; cb += nw) {
        // every load of the channel block is issued before the first product (left to itself the compiler loads
        // each weight fragment right before its use and waits for it: sixteen memory latencies in a row)
        bf16x8 xc[2], xp[2], al[2], lw[2][NOB];
#pragma unroll
        for (int pr = 0; pr < 2; pr++) {
            const int c = 64 * cb + 32 * pr + 8 * L.g;
            xc[pr] = *reinterpret_cast<const bf16x8*>(x + xrow + c);
            xp[pr] = *reinterpret_cast<const bf16x8*>(x_prev + xrow + c);
            al[pr] = *reinterpret_cast<const bf16x8*>(alpha + c);
#pragma unroll
            for (int ob = 0; ob < NOB; ob++) lw[pr][ob] = *reinterpret_cast<const bf16x8*>(Lw + (long)(16 * ob + L.n) * C + c);   // lane = mid index
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int pr = 0; pr < 2; pr++) {
            // the interpolated input as a bf16 pair (hi + lo), as the sequence kernel has it: it feeds tanh', which
            // is steep, and must not be rounded to 8 bits before the C-term sum
            bf16x4 h[2], l[2];
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const f32x4 cv = to_f32(hf ? hi4(xc[pr]) : lo4(xc[pr]));
                const f32x4 av = cv + (to_f32(hf ? hi4(xp[pr]) : lo4(xp[pr])) - cv) * to_f32(hf ? hi4(al[pr]) : lo4(al[pr]));
                h[hf] = to_bf16(av);
                l[hf] = to_bf16(av - to_f32(h[hf]));
            }
            const bf16x8 a_hi = cat8(h[0], h[1]), a_lo = cat8(l[0], l[1]);
#pragma unroll
            for (int ob = 0; ob < NOB; ob++) {
                acc[ob] = mma8(acc[ob], lw[pr][ob], a_hi);   // lane = token
                acc[ob] = mma8(acc[ob], lw[pr][ob], a_lo);
            }
        }
    }
#pragma unroll
    for (int ob = 0; ob < NOB; ob++) part[wave][ob][lane] = acc[ob];
    __syncthreads();
    // wavefront w < 8 adds block w in a fixed order, applies tanh and files the result where the second product's lane
    // group 2(ob&1) + (g>>1) of interpolation k = ob/2 looks for mid indices 8g' .. 8g'+7
    if (wave < NOB) {
        const int ob = wave;
        f32x4 s = part[0][ob][lane];
        for (int w = 1; w < nw; w++) s += part[w][ob][lane];
        f32x4 t;
#pragma unroll
        for (int r = 0; r < 4; r++) t[r] = tanhf_(s[r]);
        const int k = ob >> 1, gq = 2 * (ob & 1) + (L.g >> 1);
        *reinterpret_cast<bf16x4*>(&s_bm[k][(16 * gq + L.n) * 8 + 4 * (L.g & 1)]) = to_bf16(t);
    }
    __syncthreads();
    bf16x8 bm[4];
#pragma unroll
    for (int k = 0; k < 4; k++) bm[k] = *reinterpret_cast<const bf16x8*>(&s_bm[k][lane * 8]);
    for (int cb = wave; cb < ncb; cb += nw) {
        bf16x8 rw[4][4];      // [s][k]: lane = channel
        bf16x4 xq[4], xpq[4], bq[4][4];
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const int c = 64 * cb + 16 * s;
            xq[s] = *reinterpret_cast<const bf16x4*>(x + xrow + c + 4 * L.g);
            xpq[s] = *reinterpret_cast<const bf16x4*>(x_prev + xrow + c + 4 * L.g);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                rw[s][k] = *reinterpret_cast<const bf16x8*>(R + ((long)k * C + c + L.n) * R_MIX + 8 * L.g);
                bq[s][k] = *reinterpret_cast<const bf16x4*>(beta + (long)k * C + c + 4 * L.g);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const int c = 64 * cb + 16 * s;
            const f32x4 xv = to_f32(xq[s]);
            const f32x4 xxv = to_f32(xpq[s]) - xv;
            if (x_carry && valid) *reinterpret_cast<bf16x4*>(x_carry + (long)row * C + c + 4 * L.g) = xq[s];   // the next step's x_prev
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const f32x4 coef = mma8(to_f32(bq[s][k]), rw[s][k], bm[k]);   // lane = token
                const bf16x4 y = valid ? to_bf16(xv + xxv * coef) : bf16x4{};
                *reinterpret_cast<bf16x4*>(streams + ((long)k * Bp + row) * C + c + 4 * L.g) = y;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// 2./5. linear: out_s = in_s W_s^T for up to nine (input, weight) pairs.  Block = 16 output columns of one pair
// x one 16-row tile; its four wavefronts take every fourth 32-channel step of the contraction.
// ------------------------------------------------------------------------------------------------
struct LinSeg {
    const __bf16* in;    // [Bp, C]
    const __bf16* W;     // [N, C]
    __bf16* out;         // [rows, N]
    int N;               // multiple of 16
    int tanh_out;        // the output is tanh of the (bf16-rounded) product
};
constexpr int MAX_SEGS = 9;
struct LinArgs {
    LinSeg seg[MAX_SEGS];
    int nseg, C, rows;   // rows: output rows that exist (stores beyond are dropped)
};

__global__ __launch_bounds__(256) void decode_linear_kernel(const LinArgs A) {
    __shared__ f32x4 part[4][WAVE];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    // which pair this block belongs to (the descriptor fields through scalar selects, not an indexed copy of the
    // argument struct)
    int blk = blockIdx.x;
    const __bf16* __restrict__ in = nullptr;
    const __bf16* __restrict__ W = nullptr;
    __bf16* __restrict__ out = nullptr;
    int N = 0, act = 0;
    bool found = false;
#pragma unroll
    for (int i = 0; i < MAX_SEGS; i++) {
        if (!found && i < A.nseg) {
            const int nb = A.seg[i].N / 16;
            if (blk < nb) {
                found = true;
                in = A.seg[i].in;
                W = A.seg[i].W;
                out = A.seg[i].out;
                N = A.seg[i].N;
                act = A.seg[i].tanh_out;
            } else {
                blk -= nb;
            }
        }
    }
    if (!found) return;   // (whole block; the grid is exactly the sum of the pairs' blocks)
    const int C = A.C;
    const int row = blockIdx.y * TOK + L.n;
    const __bf16* wrow = W + (long)(16 * blk + L.n) * C + 8 * L.g;   // lane = output column
    const __bf16* irow = in + (long)row * C + 8 * L.g;               // lane = token
    f32x4 acc0 = zero4(), acc1 = zero4();
    const int nk = C / 32;
    for (int s0 = wave; s0 < nk; s0 += 32) {   // eight steps of this wavefront at a time, all loads before the products
        bf16x8 wv[8], iv[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int s = s0 + 4 * u < nk ? s0 + 4 * u : s0;   // (past the end: the first step again, not used)
            wv[u] = *reinterpret_cast<const bf16x8*>(wrow + 32 * s);
            iv[u] = *reinterpret_cast<const bf16x8*>(irow + 32 * s);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 8; u += 2) {
            if (s0 + 4 * u < nk) acc0 = mma8(acc0, wv[u], iv[u]);
            if (s0 + 4 * (u + 1) < nk) acc1 = mma8(acc1, wv[u + 1], iv[u + 1]);
        }
    }
    part[wave][lane] = acc0 + acc1;
    __syncthreads();
    if (wave != 0) return;
    f32x4 r = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);   // lane = token, reg = column 4g + r
    if (act) {
        r = to_f32(to_bf16(r));
#pragma unroll
        for (int q = 0; q < 4; q++) r[q] = tanhf_(r[q]);
    }
    if (row < A.rows) *reinterpret_cast<bf16x4*>(out + (long)row * N + 16 * blk + 4 * L.g) = to_bf16(r);
}

// ------------------------------------------------------------------------------------------------
// 3. expand: one wavefront per (16-row tile, head of 64 channels)
//     g  = tanh(g1) Wg2^T ;   w2 = tanh(w1) Ww2^T ;   w = -softplus(-(w_bias + w2)) - 0.5
//     z  = tanh(kk1) Wz^T + k ;   kk = z / sqrt(max(sum_head z^2, 1e-12))
//     a  = sigmoid(a1 Wa^T + a_bias) ;  ma, mk likewise ;   k' = k (ma + a - ma a) exp(w mk) ;   b = -kk a
// ------------------------------------------------------------------------------------------------
struct ExpandArgs {
    int Bp, C;
    const __bf16 *k, *tg1, *tw1, *kk1, *mk1, *a1, *ma1;                 // [Bp, C], [Bp, 128], [Bp, 64], 4 x [Bp, 16]
    const __bf16 *gate_w2, *decay_w2, *kkk_w2, *aaa_w2, *ma_w2, *mk_w2;   // [C, rank]
    const __bf16 *time_decay, *time_aaaaa, *time_misc_a, *time_misc_k;   // [C]
    __bf16 *w, *k2, *kk, *b, *g;                                          // [Bp, C]
};

__global__ __launch_bounds__(64) void decode_expand_kernel(const ExpandArgs A) {
    const Lane L;
    const int h = blockIdx.x;
    const int row = blockIdx.y * TOK + L.n;
    const int C = A.C;
    bf16x8 tg1[R_GATE / 32], tw1[R_DECAY / 32];
#pragma unroll
    for (int j = 0; j < R_GATE / 32; j++) tg1[j] = *reinterpret_cast<const bf16x8*>(A.tg1 + (long)row * R_GATE + 32 * j + 8 * L.g);
#pragma unroll
    for (int j = 0; j < R_DECAY / 32; j++) tw1[j] = *reinterpret_cast<const bf16x8*>(A.tw1 + (long)row * R_DECAY + 32 * j + 8 * L.g);
    auto act16 = [&](const __bf16* p) { return *reinterpret_cast<const bf16x4*>(p + (long)row * 16 + 4 * L.g); };
    bf16x4 tz;
    {
        f32x4 t = to_f32(act16(A.kk1));
#pragma unroll
        for (int q = 0; q < 4; q++) t[q] = tanhf_(t[q]);
        tz = to_bf16(t);
    }
    const bf16x4 a1 = act16(A.a1), ma1 = act16(A.ma1), mk1 = act16(A.mk1);

    // every weight fragment of the head is requested before the first product (else each is loaded right before its
    // use and waited for)
    bf16x8 gw[NBLK][R_GATE / 32], dw[NBLK][R_DECAY / 32];
    bf16x4 wz[NBLK], wa[NBLK], wma[NBLK], wmk[NBLK], bias[NBLK][4], kq[NBLK];
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) {
        const int c = h * HEAD + 16 * cb;            // lane n: channel c + n as a weight row; column 4g + r of the result
#pragma unroll
        for (int j = 0; j < R_GATE / 32; j++)
            gw[cb][j] = *reinterpret_cast<const bf16x8*>(A.gate_w2 + (long)(c + L.n) * R_GATE + 32 * j + 8 * L.g);
#pragma unroll
        for (int j = 0; j < R_DECAY / 32; j++)
            dw[cb][j] = *reinterpret_cast<const bf16x8*>(A.decay_w2 + (long)(c + L.n) * R_DECAY + 32 * j + 8 * L.g);
        auto w16 = [&](const __bf16* W) { return *reinterpret_cast<const bf16x4*>(W + (long)(c + L.n) * 16 + 4 * L.g); };
        wz[cb] = w16(A.kkk_w2);
        wa[cb] = w16(A.aaa_w2);
        wma[cb] = w16(A.ma_w2);
        wmk[cb] = w16(A.mk_w2);
        bias[cb][0] = *reinterpret_cast<const bf16x4*>(A.time_decay + c + 4 * L.g);
        bias[cb][1] = *reinterpret_cast<const bf16x4*>(A.time_aaaaa + c + 4 * L.g);
        bias[cb][2] = *reinterpret_cast<const bf16x4*>(A.time_misc_a + c + 4 * L.g);
        bias[cb][3] = *reinterpret_cast<const bf16x4*>(A.time_misc_k + c + 4 * L.g);
        kq[cb] = *reinterpret_cast<const bf16x4*>(A.k + (long)row * C + c + 4 * L.g);
    }
    __builtin_amdgcn_sched_barrier(0);
    f32x4 z[NBLK], av[NBLK];
    float ss = 0.f;
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) {
        const long o = (long)row * C + h * HEAD + 16 * cb + 4 * L.g;
        f32x4 gacc = zero4(), w2 = zero4();
#pragma unroll
        for (int j = 0; j < R_GATE / 32; j++) gacc = mma8(gacc, gw[cb][j], tg1[j]);
#pragma unroll
        for (int j = 0; j < R_DECAY / 32; j++) w2 = mma8(w2, dw[cb][j], tw1[j]);
        *reinterpret_cast<bf16x4*>(A.g + o) = to_bf16(gacc);
        const f32x4 kin = to_f32(kq[cb]);
        z[cb] = mma(kin, wz[cb], tz);
        const f32x4 pa = mma(to_f32(bias[cb][1]), wa[cb], a1);
        const f32x4 pma = mma(to_f32(bias[cb][2]), wma[cb], ma1);
        const f32x4 pmk = mma(to_f32(bias[cb][3]), wmk[cb], mk1);
        const f32x4 u = to_f32(bias[cb][0]) + to_f32(to_bf16(w2));   // (w2 is a bf16 tensor in the sequence path)
        f32x4 w, k;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const float a = sigmoidf_(pa[q]), ma = sigmoidf_(pma[q]), mk = sigmoidf_(pmk[q]);
            w[q] = -(fmaxf(-u[q], 0.f) + log1pexp_(u[q])) - 0.5f;
            k[q] = kin[q] * (ma + a - ma * a) * __expf(w[q] * mk);
            av[cb][q] = a;
            ss += z[cb][q] * z[cb][q];
        }
        *reinterpret_cast<bf16x4*>(A.w + o) = to_bf16(w);
        *reinterpret_cast<bf16x4*>(A.k2 + o) = to_bf16(k);
    }
    const float inorm = rsqrtf(fmaxf(group_sum(ss), 1e-12f));
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) {
        const long o = (long)row * C + h * HEAD + 16 * cb + 4 * L.g;
        const f32x4 kk = z[cb] * inorm;
        *reinterpret_cast<bf16x4*>(A.kk + o) = to_bf16(kk);
        *reinterpret_cast<bf16x4*>(A.b + o) = to_bf16(-kk * av[cb]);
    }
}

constexpr size_t A256(size_t x) { return (x + 255) / 256 * 256; }
int padded_rows(int B) { return (B + TOK - 1) / TOK * TOK; }

}  // namespace

size_t mixer_decode_workspace_bytes(int B, int C) {
    const size_t Bp = padded_rows(B);
    return 13 * A256(Bp * C * 2) + A256(Bp * R_GATE * 2) + A256(Bp * R_DECAY * 2) + 4 * A256(Bp * 16 * 2);
}

void launch_mixer_decode(int B, int C, int H, int state_f32, const MixerWeights& mw, const void* x, const void* x_prev,
                         void* state, void* y, void* x_carry, void* workspace, hipStream_t stream) {
    const int Bp = padded_rows(B);
    char* p = static_cast<char*>(workspace);
    auto take = [&](size_t elems) {
        __bf16* r = reinterpret_cast<__bf16*>(p);
        p += A256(elems * 2);
        return r;
    };
    const size_t BC = (size_t)Bp * C;
    __bf16* streams = take(4 * BC);   // (4 x A256(BC*2) >= A256(4*BC*2): the budget above covers it)
    __bf16 *r = take(BC), *k = take(BC), *v = take(BC);
    __bf16 *w = take(BC), *k2 = take(BC), *kk = take(BC), *b = take(BC), *g = take(BC), *ya = take(BC);
    __bf16 *tg1 = take((size_t)Bp * R_GATE), *tw1 = take((size_t)Bp * R_DECAY);
    __bf16 *kk1 = take((size_t)Bp * 16), *mk1 = take((size_t)Bp * 16), *a1 = take((size_t)Bp * 16), *ma1 = take((size_t)Bp * 16);
    auto c = [](const void* q) { return static_cast<const __bf16*>(q); };
    const dim3 tiles(Bp / TOK);

    // at least eight wavefronts (the eight 16-wide blocks of the first product are added by one each)
    const int mix_waves = C / 64 < 8 ? 8 : (C / 64 < MIX_MAX_WAVES ? C / 64 : MIX_MAX_WAVES);
    hipLaunchKernelGGL(decode_mix_kernel, tiles, dim3(64 * mix_waves), 0, stream, B, Bp, C, c(x), c(x_prev), c(mw.time_maa_x),
                       c(mw.time_maa), c(mw.time_maa_w1), c(mw.time_maa_w2), streams, static_cast<__bf16*>(x_carry));
    const __bf16 *xrg = streams, *xwa = streams + BC, *xk = streams + 2 * BC, *xv = streams + 3 * BC;
    {
        LinArgs a{};
        a.seg[0] = {xrg, c(mw.Wr), r, C, 0};
        a.seg[1] = {xk, c(mw.Wk), k, C, 0};
        a.seg[2] = {xv, c(mw.Wv), v, C, 0};
        a.seg[3] = {xrg, c(mw.gate_w1), tg1, R_GATE, 1};
        a.seg[4] = {xwa, c(mw.time_decay_w1), tw1, R_DECAY, 1};
        a.seg[5] = {xk, c(mw.time_kkk_w1), kk1, R_KKK, 0};
        a.seg[6] = {xk, c(mw.mk_w1), mk1, R_MK, 0};
        a.seg[7] = {xwa, c(mw.time_aaa_w1), a1, R_AAA, 0};
        a.seg[8] = {xwa, c(mw.ma_w1), ma1, R_MA, 0};
        a.nseg = 9;
        a.C = C;
        a.rows = Bp;
        const int nblk = (3 * C + R_GATE + R_DECAY + R_KKK + R_MK + R_AAA + R_MA) / 16;
        hipLaunchKernelGGL(decode_linear_kernel, dim3(nblk, Bp / TOK), dim3(256), 0, stream, a);
    }
    {
        const ExpandArgs a{Bp, C, k, tg1, tw1, kk1, mk1, a1, ma1,
                           c(mw.gate_w2), c(mw.time_decay_w2), c(mw.time_kkk_w2), c(mw.time_aaa_w2), c(mw.ma_w2), c(mw.mk_w2),
                           c(mw.time_decay), c(mw.time_aaaaa), c(mw.time_misc_a), c(mw.time_misc_k), w, k2, kk, b, g};
        hipLaunchKernelGGL(decode_expand_kernel, dim3(H, Bp / TOK), dim3(64), 0, stream, a);
    }
    launch_decode(B, H, state_f32, w, r, k2, v, kk, b, state, ya, stream, g, mw.ln_params);
    {
        LinArgs a{};
        a.seg[0] = {ya, c(mw.Wo), static_cast<__bf16*>(y), C, 0};
        a.nseg = 1;
        a.C = C;
        a.rows = B;
        hipLaunchKernelGGL(decode_linear_kernel, dim3(C / 16, Bp / TOK), dim3(256), 0, stream, a);
    }
}

}  // namespace wkv
