// expand_loras: second halves of the four rank-D LoRAs of the RWKV-7 time mixer and the elementwise
// tail that turns them into the WKV7 operands, forward and backward, for gfx950.
//
// Replaces the Triton kernels of the reference (rwkv7_expand_loras.py: fw_triton_ :33-70, bw_triton_
// :92-189, host glue :72-79, :192-211).  Spec (tests/test_expand_loras.py:6-19), per token:
//     w   = -softplus(-(w_bias + w_in)) - 0.5
//     z   = tanh(z_in) Wz^T + k_in ;   kk = z / sqrt(max(sum_head z^2, 1e-12))       (per head)
//     a   = sigmoid(a_in Wa^T + a_bias) ;  ma, mk likewise
//     k   = k_in (ma + a - ma a) exp(w mk) ;   b = -kk a
// Shapes: w_in, k_in and the four outputs [M, C]; z_in, a_in, ma_in, mk_in [M, D]; W* [C, D]; biases [C].
// One wavefront owns a tile of 16 tokens x 64 channels - one head at head size 64: the head norm is a 16-term
// register sum plus two cross-lane adds - and each rank-D product is one 16x16x16 (or 16x16x32) MFMA per 16
// channels.  Other head sizes: expand_loras_head_kernel below.
#include "frag.hpp"
#include "device_info.hpp"
#include "expand_loras_kernels.hpp"

namespace wkv {

namespace {

constexpr int TOK = 16;

struct LoraIn {   // the four [M, D] activations
    const __bf16* p[4];   // z, a, ma, mk
};
struct LoraW {    // the four [C, D] matrices and four [C] biases
    const __bf16* W[4];   // Wz, Wa, Wma, Wmk
    const __bf16* bias[4];  // w_bias, a_bias, ma_bias, mk_bias
};

// v_rcp_f32 (1 ulp) instead of an IEEE division: the division expands to ten instructions per element
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

template <int ND>
struct Frags {
    bf16x4 f[ND];
};
// F(in[16 tokens, D])  lane = token, reg = rank index
template <int ND>
__device__ __forceinline__ Frags<ND> load_act(const __bf16* __restrict__ p, long m0, const Lane& L) {
    Frags<ND> r;
    const __bf16* row = p + (m0 + L.n) * (16 * ND) + 4 * L.g;
#pragma unroll
    for (int j = 0; j < ND; j++) r.f[j] = *reinterpret_cast<const bf16x4*>(row + 16 * j);
    return r;
}
// F(W[c0+16cb .. , D])  lane = channel, reg = rank index
template <int ND>
__device__ __forceinline__ Frags<ND> load_w(const __bf16* __restrict__ W, int c, const Lane& L) {
    Frags<ND> r;
    const __bf16* row = W + (long)(c + L.n) * (16 * ND) + 4 * L.g;
#pragma unroll
    for (int j = 0; j < ND; j++) r.f[j] = *reinterpret_cast<const bf16x4*>(row + 16 * j);
    return r;
}
// acc + F(in W^T) for one block of 16 channels  (lane = token, reg = channel)
template <int ND>
__device__ __forceinline__ f32x4 lora_block(f32x4 acc, const Frags<ND>& w, const Frags<ND>& in) {
    if constexpr (ND == 1) {
        acc = mma(acc, w.f[0], in.f[0]);
    } else {
#pragma unroll
        for (int j = 0; j < ND; j += 2) acc = mma2(acc, w.f[j], w.f[j + 1], in.f[j], in.f[j + 1]);
    }
    return acc;
}
__device__ __forceinline__ f32x4 load_bias(const __bf16* __restrict__ b, int c, const Lane& L) {
    return to_f32(*reinterpret_cast<const bf16x4*>(b + c + 4 * L.g));
}

// everything the forward computes for one tile, in fp32 (lane = token, 16 channels per lane)
struct Fwd {
    TileF w, k, kk, b;          // the four outputs
    TileF z, a, ma, mk, e, u;   // z before normalisation, the three gates, exp(w*mk), u = w_bias + w_in
    float inorm[NBLK];          // 1 / sqrt(max(sum z^2, 1e-12)) of the head each block of 16 channels lies in
    float proj[NBLK];           // with STATS: the projection term of the normalisation's backward (see HeadStat)
};
// What the normalisation needs of a (token, head) when the head is not the 64 channels a wavefront holds: written
// by expand_loras_head_kernel, read by the backward kernels in place of their own sums.
struct HeadStat {
    float inorm;   // 1 / sqrt(max(sum_head z^2, 1e-12))
    float proj;    // (sum_head dkk z) inorm^3, or 0 where the norm is clamped
};
// STATS: st is this lane's token row of the statistics, [C / HS] entries.
template <int ND, bool STATS = false>
__device__ __forceinline__ Fwd forward_tile(const TileB& w_in, const TileB& k_in, const Frags<ND> act[4], const LoraW& lw,
                                            int c0, const Lane& L, const HeadStat* __restrict__ st = nullptr, int HS = HEAD) {
    Fwd r;
    Frags<ND> tz;
#pragma unroll
    for (int j = 0; j < ND; j++) {
        const f32x4 zi = to_f32(act[0].f[j]);
        f32x4 t;
#pragma unroll
        for (int q = 0; q < 4; q++) t[q] = tanhf_(zi[q]);
        tz.f[j] = to_bf16(t);
    }
    float ss = 0.f;
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) {
        const int c = c0 + 16 * cb;
        const f32x4 kin = to_f32(k_in.f[cb]);
        r.z.f[cb] = lora_block<ND>(kin, load_w<ND>(lw.W[0], c, L), tz);
        const f32x4 pa = lora_block<ND>(load_bias(lw.bias[1], c, L), load_w<ND>(lw.W[1], c, L), act[1]);
        const f32x4 pma = lora_block<ND>(load_bias(lw.bias[2], c, L), load_w<ND>(lw.W[2], c, L), act[2]);
        const f32x4 pmk = lora_block<ND>(load_bias(lw.bias[3], c, L), load_w<ND>(lw.W[3], c, L), act[3]);
        r.u.f[cb] = load_bias(lw.bias[0], c, L) + to_f32(w_in.f[cb]);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            r.a.f[cb][q] = sigmoidf_(pa[q]);
            r.ma.f[cb][q] = sigmoidf_(pma[q]);
            r.mk.f[cb][q] = sigmoidf_(pmk[q]);
            // -softplus(-u) - 0.5 = log(sigmoid(u)) - 0.5, evaluated without overflow
            const float u = r.u.f[cb][q];
            r.w.f[cb][q] = -(fmaxf(-u, 0.f) + log1pexp_(u)) - 0.5f;
            r.e.f[cb][q] = __expf(r.w.f[cb][q] * r.mk.f[cb][q]);
            ss += r.z.f[cb][q] * r.z.f[cb][q];
        }
        r.k.f[cb] = kin * (r.ma.f[cb] + r.a.f[cb] - r.ma.f[cb] * r.a.f[cb]) * r.e.f[cb];
    }
    if constexpr (STATS) {
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            const HeadStat hs = st[(c0 + 16 * cb) / HS];
            r.inorm[cb] = hs.inorm;
            r.proj[cb] = hs.proj;
        }
    } else {
        const float inorm = rsqrtf(fmaxf(group_sum(ss), 1e-12f));
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) r.inorm[cb] = inorm;
    }
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) {
        r.kk.f[cb] = r.z.f[cb] * r.inorm[cb];
        r.b.f[cb] = -r.kk.f[cb] * r.a.f[cb];
    }
    return r;
}

}  // namespace

// ------------------------------------------------------------------------------------------------
// forward: one wavefront per (16 tokens, head)
// ------------------------------------------------------------------------------------------------
template <int ND>
__global__ __launch_bounds__(256) void expand_loras_fwd_kernel(long M, int C, const __bf16* __restrict__ w_in,
                                                               const __bf16* __restrict__ k_in, LoraIn in, LoraW lw,
                                                               __bf16* __restrict__ w_out, __bf16* __restrict__ k_out,
                                                               __bf16* __restrict__ kk_out, __bf16* __restrict__ b_out) {
    const Lane L;
    const int H = C / HEAD;
    const long tile = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tile >= (M / TOK) * H) return;
    const long m0 = (tile / H) * TOK;
    const int c0 = (int)(tile % H) * HEAD;
    const long off = m0 * C + c0;
    const TileB wi = load_rows(w_in + off, C, L), ki = load_rows(k_in + off, C, L);
    Frags<ND> act[4];
#pragma unroll
    for (int i = 0; i < 4; i++) act[i] = load_act<ND>(in.p[i], m0, L);
    const Fwd f = forward_tile<ND>(wi, ki, act, lw, c0, L);
    store_rows(w_out + off, C, L, to_bf16(f.w));
    store_rows(k_out + off, C, L, to_bf16(f.k));
    store_rows(kk_out + off, C, L, to_bf16(f.kk));
    store_rows(b_out + off, C, L, to_bf16(f.b));
}

// ------------------------------------------------------------------------------------------------
// forward for rank 16: block = (head, range of token tiles).  The head's weights and biases are staged in
// LDS once and each wavefront walks its tiles with the next tile's inputs already in flight - the generic
// kernel above fetches forty weight fragments per tile from memory in the middle of dependent arithmetic
// and spends most of its time waiting for them.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void expand_loras_fwd16_kernel(long M, int C, int tiles_per_split,
                                                                 const __bf16* __restrict__ w_in,
                                                                 const __bf16* __restrict__ k_in, LoraIn in, LoraW lw,
                                                                 __bf16* __restrict__ w_out, __bf16* __restrict__ k_out,
                                                                 __bf16* __restrict__ kk_out, __bf16* __restrict__ b_out) {
    __shared__ bf16x4 sW[4 * NBLK][WAVE];    // F(W_i[c0 + 16cb .., :])    lane = channel, reg = rank index
    __shared__ float sBias[4][HEAD];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    const int h = blockIdx.x, split = blockIdx.y;
    const int c0 = h * HEAD;
    const long ntiles = M / TOK;
    const long tile_begin = (long)split * tiles_per_split;
    const long tile_end = tile_begin + tiles_per_split < ntiles ? tile_begin + tiles_per_split : ntiles;
    // Channel order inside the head: nothing here depends on which 16 channels form a block (the norm sums all
    // 64, the rest is elementwise), so blocks 2p and 2p+1 interleave in groups of four - register r of block cb
    // in column group g is channel 32p + 8g + 4(cb & 1) + r - and a lane's pieces of the two blocks are 8
    // contiguous channels: one 16-byte access instead of two of 8.
    auto chan = [](int cb, int j) { return 32 * (cb >> 1) + 8 * (j >> 2) + 4 * (cb & 1) + (j & 3); };   // j = 4g + r
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++)
        sW[wave * NBLK + cb][lane] = *reinterpret_cast<const bf16x4*>(lw.W[wave] + (long)(c0 + chan(cb, L.n)) * 16 + 4 * L.g);
    sBias[wave][lane] = (float)lw.bias[wave][c0 + lane];
    __syncthreads();
    auto bias4 = [&](int i, int cb) { return *reinterpret_cast<const f32x4*>(&sBias[i][chan(cb, 4 * L.g)]); };
    auto load_tile = [&](const __bf16* p) {   // p: this lane's row, channel c0
        TileB t;
#pragma unroll
        for (int pr = 0; pr < 2; pr++) {
            const bf16x8 v = *reinterpret_cast<const bf16x8*>(p + 32 * pr + 8 * L.g);
            t.f[2 * pr] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
            t.f[2 * pr + 1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
        }
        return t;
    };
    auto store_tile = [&](__bf16* p, const TileB& t) {
#pragma unroll
        for (int pr = 0; pr < 2; pr++)
            *reinterpret_cast<bf16x8*>(p + 32 * pr + 8 * L.g) =
                __builtin_shufflevector(t.f[2 * pr], t.f[2 * pr + 1], 0, 1, 2, 3, 4, 5, 6, 7);
    };

    struct TileIn {
        TileB wi, ki;
        bf16x4 act[4];
    };
    auto fetch = [&](long tile) {
        TileIn t;
        const long m0 = tile * TOK;
        t.wi = load_tile(w_in + (m0 + L.n) * C + c0);
        t.ki = load_tile(k_in + (m0 + L.n) * C + c0);
#pragma unroll
        for (int i = 0; i < 4; i++) t.act[i] = load_act<1>(in.p[i], m0, L).f[0];
        return t;
    };
    long tile = tile_begin + wave;
    TileIn nxt;
    if (tile < tile_end) nxt = fetch(tile);
    for (; tile < tile_end; tile += 4) {
        const TileIn cur = nxt;
        nxt = fetch(tile + 4 < tile_end ? tile + 4 : tile);   // past the end: the current tile again (never used)
        const long off = (tile * TOK + L.n) * C + c0;
        bf16x4 tz;
        {
            f32x4 t = to_f32(cur.act[0]);
#pragma unroll
            for (int q = 0; q < 4; q++) t[q] = tanhf_(t[q]);
            tz = to_bf16(t);
        }
        TileF z, a;
        TileB wo, ko;
        float ss = 0.f;
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            const f32x4 kin = to_f32(cur.ki.f[cb]);
            z.f[cb] = mma(kin, sW[0 * NBLK + cb][lane], tz);
            const f32x4 pa = mma(bias4(1, cb), sW[1 * NBLK + cb][lane], cur.act[1]);
            const f32x4 pma = mma(bias4(2, cb), sW[2 * NBLK + cb][lane], cur.act[2]);
            const f32x4 pmk = mma(bias4(3, cb), sW[3 * NBLK + cb][lane], cur.act[3]);
            const f32x4 u = bias4(0, cb) + to_f32(cur.wi.f[cb]);
            f32x4 w, k;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float av = sigmoidf_(pa[q]), mav = sigmoidf_(pma[q]), mkv = sigmoidf_(pmk[q]);
                // -softplus(-u) - 0.5 = log(sigmoid(u)) - 0.5, evaluated without overflow
                w[q] = -(fmaxf(-u[q], 0.f) + log1pexp_(u[q])) - 0.5f;
                k[q] = kin[q] * (mav + av - mav * av) * __expf(w[q] * mkv);
                a.f[cb][q] = av;
                ss += z.f[cb][q] * z.f[cb][q];
            }
            wo.f[cb] = to_bf16(w);
            ko.f[cb] = to_bf16(k);
        }
        store_tile(w_out + off, wo);
        store_tile(k_out + off, ko);
        const float inorm = rsqrtf(fmaxf(group_sum(ss), 1e-12f));
        TileB kko, bo;
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            const f32x4 kk = z.f[cb] * inorm;
            kko.f[cb] = to_bf16(kk);
            bo.f[cb] = to_bf16(-kk * a.f[cb]);
        }
        store_tile(kk_out + off, kko);
        store_tile(b_out + off, bo);
    }
}

// ------------------------------------------------------------------------------------------------
// Head sizes other than 64 (any multiple of 16 that divides C; the reference takes the head size as an
// argument, rwkv7_expand_loras.py:72-79).  Only the norm of kk knows about heads.  One wavefront per
// (16 tokens, head) walks the head's blocks of 16 channels twice: once for z and its norm, once more for the
// outputs (z is recomputed: one more matrix instruction per block instead of the head's z in registers).
// STAT_ONLY stops after the first pass, which then also forms sum_head dkk z (dkk = dkk_out - db_out a), and
// leaves the two scalars of every (token, head) for the backward kernels, which keep working on blocks of 64
// channels and read them instead of summing over their own 64.
// ------------------------------------------------------------------------------------------------
template <int ND, bool STAT_ONLY>
__global__ __launch_bounds__(256) void expand_loras_head_kernel(long M, int C, int HS, const __bf16* __restrict__ w_in,
                                                                const __bf16* __restrict__ k_in, LoraIn in, LoraW lw,
                                                                __bf16* __restrict__ w_out, __bf16* __restrict__ k_out,
                                                                __bf16* __restrict__ kk_out, __bf16* __restrict__ b_out,
                                                                const __bf16* __restrict__ g_kk,
                                                                const __bf16* __restrict__ g_b,
                                                                HeadStat* __restrict__ stats) {
    const Lane L;
    const int NH = C / HS, nb = HS / 16;
    const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= (M / TOK) * NH) return;
    const long m0 = (item / NH) * TOK;
    const int h = (int)(item % NH), c0 = h * HS;
    const long row = (m0 + L.n) * C + c0 + 4 * L.g;   // this lane's piece of the head's first block
    Frags<ND> act[4];
#pragma unroll
    for (int i = 0; i < 4; i++) act[i] = load_act<ND>(in.p[i], m0, L);
    Frags<ND> tz;
#pragma unroll
    for (int j = 0; j < ND; j++) {
        f32x4 t = to_f32(act[0].f[j]);
#pragma unroll
        for (int q = 0; q < 4; q++) t[q] = tanhf_(t[q]);
        tz.f[j] = to_bf16(t);
    }
    auto piece = [&](const __bf16* p, int cb) { return to_f32(*reinterpret_cast<const bf16x4*>(p + row + 16 * cb)); };
    auto gate = [&](int i, int c) {
        f32x4 v = lora_block<ND>(load_bias(lw.bias[i], c, L), load_w<ND>(lw.W[i], c, L), act[i]);
#pragma unroll
        for (int q = 0; q < 4; q++) v[q] = sigmoidf_(v[q]);
        return v;
    };
    float ss = 0.f, dot = 0.f;
    for (int cb = 0; cb < nb; cb++) {
        const int c = c0 + 16 * cb;
        const f32x4 z = lora_block<ND>(piece(k_in, cb), load_w<ND>(lw.W[0], c, L), tz);
        f32x4 dkk = zero4();
        if constexpr (STAT_ONLY) dkk = piece(g_kk, cb) - piece(g_b, cb) * gate(1, c);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            ss += z[q] * z[q];
            dot += dkk[q] * z[q];
        }
    }
    const float inorm = rsqrtf(fmaxf(group_sum(ss), 1e-12f));
    if constexpr (STAT_ONLY) {
        dot = group_sum(dot);
        // z below the clamp has a constant norm: no gradient through it
        if (L.g == 0) stats[(m0 + L.n) * NH + h] = HeadStat{inorm, (inorm < 1e6f) ? dot * inorm * inorm * inorm : 0.f};
    } else {
        for (int cb = 0; cb < nb; cb++) {
            const int c = c0 + 16 * cb;
            const f32x4 kin = piece(k_in, cb);
            const f32x4 z = lora_block<ND>(kin, load_w<ND>(lw.W[0], c, L), tz);
            const f32x4 a = gate(1, c), ma = gate(2, c), mk = gate(3, c);
            const f32x4 u = load_bias(lw.bias[0], c, L) + piece(w_in, cb);
            f32x4 w, k;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                // -softplus(-u) - 0.5 = log(sigmoid(u)) - 0.5, evaluated without overflow
                w[q] = -(fmaxf(-u[q], 0.f) + log1pexp_(u[q])) - 0.5f;
                k[q] = kin[q] * (ma[q] + a[q] - ma[q] * a[q]) * __expf(w[q] * mk[q]);
            }
            const f32x4 kk = z * inorm;
            *reinterpret_cast<bf16x4*>(w_out + row + 16 * cb) = to_bf16(w);
            *reinterpret_cast<bf16x4*>(k_out + row + 16 * cb) = to_bf16(k);
            *reinterpret_cast<bf16x4*>(kk_out + row + 16 * cb) = to_bf16(kk);
            *reinterpret_cast<bf16x4*>(b_out + row + 16 * cb) = to_bf16(-kk * a);
        }
    }
}

// The same forward for rank 16 and heads of up to 128 channels (NB blocks of 16), organised like
// expand_loras_fwd16_kernel: block = (head, range of token tiles), the head's four weight matrices and biases
// staged in LDS once, every wavefront walking its tiles with z of the whole head in registers (no second pass over
// the inputs).  With an even NB the blocks 2p and 2p+1 interleave as in chan16 and the tiles move in 16-byte pieces.
// (The kernel above fetches its weight fragments from memory per block, in the middle of dependent arithmetic:
// 49 us at [8192 tokens, 6 heads of 128] against 20 us for the head-64 kernel.)
template <int NB>
__global__ __launch_bounds__(256) void expand_loras_head_fwd16_kernel(long M, int C, int tiles_per_split,
                                                                      const __bf16* __restrict__ w_in,
                                                                      const __bf16* __restrict__ k_in, LoraIn in, LoraW lw,
                                                                      __bf16* __restrict__ w_out, __bf16* __restrict__ k_out,
                                                                      __bf16* __restrict__ kk_out, __bf16* __restrict__ b_out) {
    constexpr int HS = 16 * NB;
    constexpr bool PAIRS = NB % 2 == 0;
    __shared__ bf16x4 sW[4][NB][WAVE];   // F(W_i[c0 + chan(cb, .), :])  lane = channel, reg = rank index
    __shared__ __attribute__((aligned(16))) float sBias[4][HS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    const int c0 = blockIdx.x * HS, split = blockIdx.y;
    const long ntiles = M / TOK;
    const long tile_begin = (long)split * tiles_per_split;
    const long tile_end = tile_begin + tiles_per_split < ntiles ? tile_begin + tiles_per_split : ntiles;
    // channel (inside the head) of index j = 4g + r of block cb
    auto chan = [](int cb, int j) { return PAIRS ? chan16(cb, j) : 16 * cb + j; };
#pragma unroll
    for (int cb = 0; cb < NB; cb++)
        sW[wave][cb][lane] = *reinterpret_cast<const bf16x4*>(lw.W[wave] + (long)(c0 + chan(cb, L.n)) * 16 + 4 * L.g);
    for (int c = lane; c < HS; c += WAVE) sBias[wave][c] = (float)lw.bias[wave][c0 + c];
    __syncthreads();
    auto bias4 = [&](int i, int cb) { return *reinterpret_cast<const f32x4*>(&sBias[i][chan(cb, 4 * L.g)]); };
    auto load_head = [&](bf16x4 (&t)[NB], const __bf16* p) {   // p: the head's first channel in this lane's row
        if constexpr (PAIRS) {
#pragma unroll
            for (int pr = 0; pr < NB / 2; pr++) {
                const bf16x8 v = *reinterpret_cast<const bf16x8*>(p + 32 * pr + 8 * L.g);
                t[2 * pr] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
                t[2 * pr + 1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
            }
        } else {
#pragma unroll
            for (int cb = 0; cb < NB; cb++) t[cb] = *reinterpret_cast<const bf16x4*>(p + 16 * cb + 4 * L.g);
        }
    };
    auto store_head = [&](__bf16* p, const bf16x4 (&t)[NB]) {
        if constexpr (PAIRS) {
#pragma unroll
            for (int pr = 0; pr < NB / 2; pr++)
                *reinterpret_cast<bf16x8*>(p + 32 * pr + 8 * L.g) = __builtin_shufflevector(t[2 * pr], t[2 * pr + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
#pragma unroll
            for (int cb = 0; cb < NB; cb++) *reinterpret_cast<bf16x4*>(p + 16 * cb + 4 * L.g) = t[cb];
        }
    };
    for (long tile = tile_begin + wave; tile < tile_end; tile += 4) {
        const long m0 = tile * TOK;
        const long off = (m0 + L.n) * C + c0;
        bf16x4 wi[NB], ki[NB], act[4];
        load_head(wi, w_in + off);
        load_head(ki, k_in + off);
#pragma unroll
        for (int i = 0; i < 4; i++) act[i] = load_act<1>(in.p[i], m0, L).f[0];
        bf16x4 tz;
        {
            f32x4 t = to_f32(act[0]);
#pragma unroll
            for (int q = 0; q < 4; q++) t[q] = tanhf_(t[q]);
            tz = to_bf16(t);
        }
        f32x4 z[NB], a[NB];
        bf16x4 wo[NB], ko[NB];
        float ss = 0.f;
#pragma unroll
        for (int cb = 0; cb < NB; cb++) {
            const f32x4 kin = to_f32(ki[cb]);
            z[cb] = mma(kin, sW[0][cb][lane], tz);
            const f32x4 pa = mma(bias4(1, cb), sW[1][cb][lane], act[1]);
            const f32x4 pma = mma(bias4(2, cb), sW[2][cb][lane], act[2]);
            const f32x4 pmk = mma(bias4(3, cb), sW[3][cb][lane], act[3]);
            const f32x4 u = bias4(0, cb) + to_f32(wi[cb]);
            f32x4 w, k;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float av = sigmoidf_(pa[q]), mav = sigmoidf_(pma[q]), mkv = sigmoidf_(pmk[q]);
                // -softplus(-u) - 0.5 = log(sigmoid(u)) - 0.5, evaluated without overflow
                w[q] = -(fmaxf(-u[q], 0.f) + log1pexp_(u[q])) - 0.5f;
                k[q] = kin[q] * (mav + av - mav * av) * __expf(w[q] * mkv);
                a[cb][q] = av;
                ss += z[cb][q] * z[cb][q];
            }
            wo[cb] = to_bf16(w);
            ko[cb] = to_bf16(k);
        }
        store_head(w_out + off, wo);
        store_head(k_out + off, ko);
        const float inorm = rsqrtf(fmaxf(group_sum(ss), 1e-12f));
        bf16x4 kko[NB], bo[NB];
#pragma unroll
        for (int cb = 0; cb < NB; cb++) {
            const f32x4 kk = z[cb] * inorm;
            kko[cb] = to_bf16(kk);
            bo[cb] = to_bf16(-kk * a[cb]);
        }
        store_head(kk_out + off, kko);
        store_head(b_out + off, bo);
    }
}

// ------------------------------------------------------------------------------------------------
// backward: block = (head, range of token tiles); its four wavefronts take every fourth tile.
// Per tile: recompute the forward, write dw_in, dk_in and this head's share of the four d*_in
// ([M, H, D], summed over heads afterwards: each head contributes to every rank channel), and
// accumulate the head's weight and bias gradients in registers; these are combined across the four
// wavefronts through LDS and written as one partial record per block.
//   record: dW [4][64][D] floats, then dbias [4][64] floats
// ------------------------------------------------------------------------------------------------
struct LoraDy {
    const __bf16* p[4];   // dw_out, dk_out, dkk_out, db_out
};
struct LoraDIn {
    __bf16* p[4];         // per-head partials of dz_in, da_in, dma_in, dmk_in: [M, H, D]
};

template <int ND, bool STATS>
__global__ __launch_bounds__(256) void expand_loras_bwd_kernel(long M, int C, int tiles_per_split,
                                                               const __bf16* __restrict__ w_in,
                                                               const __bf16* __restrict__ k_in, LoraIn in, LoraW lw,
                                                               LoraDy dy, __bf16* __restrict__ dw_in,
                                                               __bf16* __restrict__ dk_in, LoraDIn din,
                                                               float* __restrict__ partial,
                                                               const HeadStat* __restrict__ stats, int HS) {
    constexpr int D = 16 * ND;
    constexpr int REC = 4 * HEAD * D + 4 * HEAD;
    __shared__ __attribute__((aligned(16))) float comb[REC];
    const int wave = threadIdx.x >> 6;
    const Lane L;
    const int H = C / HEAD;
    const int h = blockIdx.x, split = blockIdx.y;
    const int c0 = h * HEAD;
    const long ntiles = M / TOK;
    const long tile_begin = (long)split * tiles_per_split;
    const long tile_end = tile_begin + tiles_per_split < ntiles ? tile_begin + tiles_per_split : ntiles;
    const bf16x4 eye = identity_bf16(L);

    f32x4 dW[4][NBLK][ND];   // F(dW_i[c0+16cb.., 16j..])  lane = channel, reg = rank index
    TileF dbias[4];          // per-token partial sums (lane = token)
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            dbias[i].f[cb] = zero4();
#pragma unroll
            for (int j = 0; j < ND; j++) dW[i][cb][j] = zero4();
        }

    for (long tile = tile_begin + wave; tile < tile_end; tile += 4) {
        const long m0 = tile * TOK;
        const long off = m0 * C + c0;
        const TileB wi = load_rows(w_in + off, C, L), ki = load_rows(k_in + off, C, L);
        Frags<ND> act[4];
#pragma unroll
        for (int i = 0; i < 4; i++) act[i] = load_act<ND>(in.p[i], m0, L);
        const Fwd f = forward_tile<ND, STATS>(wi, ki, act, lw, c0, L, STATS ? stats + (m0 + L.n) * (C / HS) : nullptr, HS);
        const TileB g_w = load_rows(dy.p[0] + off, C, L), g_k = load_rows(dy.p[1] + off, C, L);
        const TileB g_kk = load_rows(dy.p[2] + off, C, L), g_b = load_rows(dy.p[3] + off, C, L);

        // elementwise chain; pre[i] = gradient w.r.t. the pre-activation of LoRA i (i = 0: z, 1: a, 2: ma, 3: mk)
        TileF pre[4], dkin, dkk;
        float dot = 0.f;   // sum_c dkk * z  (for the normalisation)
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            const f32x4 kin = to_f32(ki.f[cb]);
            const f32x4 gb = to_f32(g_b.f[cb]);
            const f32x4 a = f.a.f[cb], ma = f.ma.f[cb], mk = f.mk.f[cb];
            dkk.f[cb] = to_f32(g_kk.f[cb]) - gb * a;
            f32x4 da = -gb * f.kk.f[cb];
            const f32x4 dk = to_f32(g_k.f[cb]) * f.e.f[cb];            // d/d(k_in * mix)
            const f32x4 de = dk * kin * (ma + a - ma * a);             // d/d(w*mk), already times e
            const f32x4 dw = to_f32(g_w.f[cb]) + de * mk;
            const f32x4 dmk = de * f.w.f[cb];
            f32x4 du;
#pragma unroll
            for (int q = 0; q < 4; q++) du[q] = dw[q] * sigmoidf_(-f.u.f[cb][q]);
            *reinterpret_cast<bf16x4*>(dw_in + off + (long)L.n * C + 16 * cb + 4 * L.g) = to_bf16(du);
            dbias[0].f[cb] += du;
            dkin.f[cb] = dk * (ma + a - ma * a);
            const f32x4 dma = dk * kin * (1.f - a);
            da += dk * kin * (1.f - ma);
            pre[1].f[cb] = da * a * (1.f - a);
            pre[2].f[cb] = dma * ma * (1.f - ma);
            pre[3].f[cb] = dmk * mk * (1.f - mk);
            if constexpr (!STATS) {
#pragma unroll
                for (int q = 0; q < 4; q++) dot += dkk.f[cb][q] * f.z.f[cb][q];
            }
        }
        float proj[NBLK];
        if constexpr (STATS) {
#pragma unroll
            for (int cb = 0; cb < NBLK; cb++) proj[cb] = f.proj[cb];
        } else {
            dot = group_sum(dot);
            // z below the clamp has a constant norm: no gradient through it
            const float pj = (f.inorm[0] < 1e6f) ? dot * f.inorm[0] * f.inorm[0] * f.inorm[0] : 0.f;
#pragma unroll
            for (int cb = 0; cb < NBLK; cb++) proj[cb] = pj;
        }
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            pre[0].f[cb] = dkk.f[cb] * f.inorm[cb] - proj[cb] * f.z.f[cb];
            dkin.f[cb] += pre[0].f[cb];
            *reinterpret_cast<bf16x4*>(dk_in + off + (long)L.n * C + 16 * cb + 4 * L.g) = to_bf16(dkin.f[cb]);
        }

        // rank-space gradients: d_in_i[t, d] = sum_c pre_i[t, c] W_i[c, d]  (this head's 64 channels only),
        // weight gradients: dW_i[c, d] += sum_t pre_i[t, c] in_i[t, d]
#pragma unroll
        for (int i = 0; i < 4; i++) {
            TileB pb = to_bf16(pre[i]);
            if (i > 0) {
#pragma unroll
                for (int cb = 0; cb < NBLK; cb++) dbias[i].f[cb] += pre[i].f[cb];
            }
            Frags<ND> inT;   // F(in_i^T)  lane = rank index, reg = token   (tanh(z_in) for i = 0)
            f32x4 dact[ND];  // F(d in_i)  lane = token, reg = rank index
#pragma unroll
            for (int j = 0; j < ND; j++) {
                bf16x4 v = act[i].f[j];
                if (i == 0) {
                    f32x4 t = to_f32(v);
#pragma unroll
                    for (int q = 0; q < 4; q++) t[q] = tanhf_(t[q]);
                    v = to_bf16(t);
                }
                inT.f[j] = transpose(v, eye);
                dact[j] = zero4();
            }
#pragma unroll
            for (int cb = 0; cb < NBLK; cb++) {
                const bf16x4 pT = transpose(pb.f[cb], eye);   // F(pre_i[:, 16cb..]^T)  lane = channel, reg = token
#pragma unroll
                for (int j = 0; j < ND; j++) dW[i][cb][j] = mma(dW[i][cb][j], inT.f[j], pT);   // + F(pre^T in)
                // W^T fragments for the contraction over channels: lane = rank index, reg = channel
                const Frags<ND> wf = load_w<ND>(lw.W[i], c0 + 16 * cb, L);
#pragma unroll
                for (int j = 0; j < ND; j++) dact[j] = mma(dact[j], transpose(wf.f[j], eye), pb.f[cb]);   // + F(pre W)
            }
            __bf16* dst = din.p[i] + ((m0 + L.n) * H + h) * D + 4 * L.g;
#pragma unroll
            for (int j = 0; j < ND; j++) {
                f32x4 v = dact[j];
                if (i == 0) {   // through tanh
                    const f32x4 t = to_f32(transpose(inT.f[j], eye));   // tanh(z_in) back in token-major order
                    v = v * (1.f - t * t);
                }
                *reinterpret_cast<bf16x4*>(dst + 16 * j) = to_bf16(v);
            }
        }
    }

    // bias partials: sum over the tile's 16 token lanes (total in lane n = 15)
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++)
#pragma unroll
            for (int q = 0; q < 4; q++) dbias[i].f[cb][q] = row_prefix_sum(dbias[i].f[cb][q]);

    for (int w = 0; w < 4; w++) {
        if (wave == w) {
            auto put = [&](float* p, f32x4 v) {
                if (w > 0) v += *reinterpret_cast<f32x4*>(p);
                *reinterpret_cast<f32x4*>(p) = v;
            };
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int cb = 0; cb < NBLK; cb++) {
#pragma unroll
                    for (int j = 0; j < ND; j++) put(comb + ((i * HEAD + 16 * cb + L.n) * D) + 16 * j + 4 * L.g, dW[i][cb][j]);
                    if (L.n == 15) put(comb + 4 * HEAD * D + i * HEAD + 16 * cb + 4 * L.g, dbias[i].f[cb]);
                }
        }
        __syncthreads();
    }
    float* out = partial + ((long)split * gridDim.x + h) * REC;
    for (int i = threadIdx.x; i < REC / 4; i += 256)
        *reinterpret_cast<f32x4*>(out + 4 * i) = *reinterpret_cast<const f32x4*>(comb + 4 * i);
}

// ------------------------------------------------------------------------------------------------
// backward for rank 16 (the rank of the time mixer's four LoRAs), the same mathematics as above reorganised
// around what bounds it: the head's weights are loop-invariant, so they sit in LDS (as fragments, in both
// orientations) instead of being fetched from memory forty times per tile in the middle of dependent
// arithmetic; the next tile's streamed inputs are loaded while the current tile is computed; and the tile is
// walked one 16-channel block at a time (three short passes) so that the live state stays in registers.
// ------------------------------------------------------------------------------------------------
template <bool STATS>
__global__ __launch_bounds__(256) void expand_loras_bwd16_kernel(long M, int C, int tiles_per_split,
                                                                 const __bf16* __restrict__ w_in,
                                                                 const __bf16* __restrict__ k_in, LoraIn in, LoraW lw,
                                                                 LoraDy dy, __bf16* __restrict__ dw_in,
                                                                 __bf16* __restrict__ dk_in, LoraDIn din,
                                                                 float* __restrict__ partial,
                                                                 const HeadStat* __restrict__ stats, int HS) {
    constexpr int D = 16;
    constexpr int REC = 4 * HEAD * D + 4 * HEAD;
    __shared__ __attribute__((aligned(16))) float comb[REC];
    __shared__ bf16x4 sW[4 * NBLK][WAVE];    // F(W_i[c0 + 16cb .., :])    lane = channel, reg = rank index
    __shared__ bf16x4 sWT[4 * NBLK][WAVE];   // F(W_i[c0 + 16cb .., :]^T)  lane = rank index, reg = channel
    __shared__ float sBias[4][HEAD];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    const int H = C / HEAD;
    const int h = blockIdx.x, split = blockIdx.y;
    const int c0 = h * HEAD;
    const long ntiles = M / TOK;
    const long tile_begin = (long)split * tiles_per_split;
    const long tile_end = tile_begin + tiles_per_split < ntiles ? tile_begin + tiles_per_split : ntiles;
    const bf16x4 eye = identity_bf16(L);

    // wavefront i stages LoRA i
    // channel blocks follow the interleaved order of chan16 (frag.hpp) so that tiles move with 16-byte accesses
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) {
        const bf16x4 f = *reinterpret_cast<const bf16x4*>(lw.W[wave] + (long)(c0 + chan16(cb, L.n)) * D + 4 * L.g);
        sW[wave * NBLK + cb][lane] = f;
        sWT[wave * NBLK + cb][lane] = transpose(f, eye);
    }
    sBias[wave][lane] = (float)lw.bias[wave][c0 + lane];
    __syncthreads();
    auto bias4 = [&](int i, int cb) { return *reinterpret_cast<const f32x4*>(&sBias[i][chan16(cb, 4 * L.g)]); };

    f32x4 dW[4][NBLK];   // F(dW_i[c0+16cb.., :])  lane = channel, reg = rank index
    // The four bias gradients of a channel block are token sums of du, pre_1, pre_2, pre_3.  One accumulator
    // holds all four: contract the transposed tiles, laid side by side along the token axis, with selector
    // fragments sel_i[col][t] = (col == i); column i of the result is sum_t x_i[t][c].
    f32x4 dB[NBLK];      // lane = channel, columns 0..3 (the lanes with g = 0) = the four bias gradients
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) {
        dB[cb] = zero4();
#pragma unroll
        for (int i = 0; i < 4; i++) dW[i][cb] = zero4();
    }
    bf16x4 sel[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float v = (L.n == i) ? 1.f : 0.f;
        sel[i] = to_bf16(f32x4{v, v, v, v});
    }

    struct TileIn {
        TileB wi, ki, g[4];
        bf16x4 act[4];
    };
    auto fetch = [&](long tile) {
        TileIn t;
        const long m0 = tile * TOK;
        const long off = m0 * C + c0;
        t.wi = load_rows16(w_in + off, C, L);
        t.ki = load_rows16(k_in + off, C, L);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            t.g[i] = load_rows16(dy.p[i] + off, C, L);
            t.act[i] = load_act<1>(in.p[i], m0, L).f[0];
        }
        return t;
    };

    // The streamed inputs are prefetched IN PLACE: as soon as pass 2 is done with channel block cb of the current
    // tile, the same registers receive block cb of this wavefront's next tile (one tile's worth of registers
    // instead of two; the loads have the rest of the tile to arrive).
    long tile = tile_begin + wave;
    TileIn cur;
    if (tile < tile_end) cur = fetch(tile);
    for (; tile < tile_end; tile += 4) {
        const long m0 = tile * TOK;
        const long off = m0 * C + c0;
        // the next tile of this wavefront; past the end, the current one again (never used)
        const long m0n = (tile + 4 < tile_end ? tile + 4 : tile) * TOK;
        const long offn = m0n * C + c0 + (long)L.n * C + 8 * L.g;
        const long offs = off + (long)L.n * C + 8 * L.g;   // this lane's 16-byte pieces of the current tile
        // rank-space operands: tanh(z_in) and the transposed inputs (lane = rank index, reg = token)
        bf16x4 tz;
        {
            f32x4 t = to_f32(cur.act[0]);
#pragma unroll
            for (int q = 0; q < 4; q++) t[q] = tanhf_(t[q]);
            tz = to_bf16(t);
        }
        bf16x4 inT[4];
        inT[0] = transpose(tz, eye);
#pragma unroll
        for (int i = 1; i < 4; i++) inT[i] = transpose(cur.act[i], eye);

        // pass 1: z and the head norm.  inormp / projp: per pair of channel blocks (a lane's 8 contiguous channels
        // of blocks 2p and 2p+1 lie in one head whatever its size; with a head of 64 both pairs share the values)
        float inormp[NBLK / 2], projp[NBLK / 2];
        if constexpr (STATS) {
            const HeadStat* st = stats + (m0 + L.n) * (C / HS);
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; pr++) {
                const HeadStat hs = st[(c0 + 32 * pr + 8 * L.g) / HS];
                inormp[pr] = hs.inorm;
                projp[pr] = hs.proj;
            }
        }
        TileF z;
        float ss = 0.f;
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            z.f[cb] = mma(to_f32(cur.ki.f[cb]), sW[0 * NBLK + cb][lane], tz);
            if constexpr (!STATS) {
#pragma unroll
                for (int q = 0; q < 4; q++) ss += z.f[cb][q] * z.f[cb][q];
            }
        }
        if constexpr (!STATS) {
            const float inorm = rsqrtf(fmaxf(group_sum(ss), 1e-12f));
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; pr++) inormp[pr] = inorm;
        }

        // pass 2: everything that does not need the projection of dkk on z
        TileF dkk, dkin;
        bf16x4 du_prev = {};
        f32x4 dact[4] = {zero4(), zero4(), zero4(), zero4()};   // F(d in_i)  lane = token, reg = rank index
        float dot = 0.f;
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            const f32x4 kin = to_f32(cur.ki.f[cb]);
            const f32x4 pa = mma(bias4(1, cb), sW[1 * NBLK + cb][lane], cur.act[1]);
            const f32x4 pma = mma(bias4(2, cb), sW[2 * NBLK + cb][lane], cur.act[2]);
            const f32x4 pmk = mma(bias4(3, cb), sW[3 * NBLK + cb][lane], cur.act[3]);
            const f32x4 u = bias4(0, cb) + to_f32(cur.wi.f[cb]);
            f32x4 a, ma, mk, w, e, su;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                a[q] = sigmoidf_(pa[q]);
                ma[q] = sigmoidf_(pma[q]);
                mk[q] = sigmoidf_(pmk[q]);
                w[q] = -(fmaxf(-u[q], 0.f) + log1pexp_(u[q])) - 0.5f;
                e[q] = __expf(w[q] * mk[q]);
                su[q] = sigmoidf_(-u[q]);
            }
            const f32x4 kk = z.f[cb] * inormp[cb >> 1];
            const f32x4 gb = to_f32(cur.g[3].f[cb]);
            dkk.f[cb] = to_f32(cur.g[2].f[cb]) - gb * a;
            f32x4 da = -gb * kk;
            const f32x4 mix = ma + a - ma * a;
            const f32x4 dk = to_f32(cur.g[1].f[cb]) * e;          // d/d(k_in * mix)
            const f32x4 de = dk * kin * mix;                      // d/d(w*mk), already times e
            const f32x4 dw = to_f32(cur.g[0].f[cb]) + de * mk;
            const f32x4 dmk = de * w;
            const f32x4 du = dw * su;
            const bf16x4 du_b = to_bf16(du);
            if (cb & 1) *reinterpret_cast<bf16x8*>(dw_in + offs + 32 * (cb >> 1)) = __builtin_shufflevector(du_prev, du_b, 0, 1, 2, 3, 4, 5, 6, 7);
            du_prev = du_b;
            bf16x4 pT[4];
            pT[0] = transpose(du_b, eye);
            dkin.f[cb] = dk * mix;
            const f32x4 dma = dk * kin * (1.f - a);
            da += dk * kin * (1.f - ma);
            f32x4 pre[4];
            pre[1] = da * a * (1.f - a);
            pre[2] = dma * ma * (1.f - ma);
            pre[3] = dmk * mk * (1.f - mk);
            if constexpr (!STATS) {
#pragma unroll
                for (int q = 0; q < 4; q++) dot += dkk.f[cb][q] * z.f[cb][q];
            }
#pragma unroll
            for (int i = 1; i < 4; i++) {
                const bf16x4 pb = to_bf16(pre[i]);
                pT[i] = transpose(pb, eye);
                dW[i][cb] = mma(dW[i][cb], inT[i], pT[i]);                // + F(pre^T in)
                dact[i] = mma(dact[i], sWT[i * NBLK + cb][lane], pb);     // + F(pre W)
            }
            dB[cb] = mma2(dB[cb], sel[0], sel[1], pT[0], pT[1]);
            dB[cb] = mma2(dB[cb], sel[2], sel[3], pT[2], pT[3]);
            if (cb & 1) {   // blocks cb-1 and cb of the next tile: one 16-byte piece per tensor
                auto reload = [&](TileB& t, const __bf16* p) {
                    const bf16x8 v = *reinterpret_cast<const bf16x8*>(p + offn + 32 * (cb >> 1));
                    t.f[cb - 1] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
                    t.f[cb] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
                };
                reload(cur.wi, w_in);
                reload(cur.ki, k_in);
#pragma unroll
                for (int i = 0; i < 4; i++) reload(cur.g[i], dy.p[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++) cur.act[i] = load_act<1>(in.p[i], m0n, L).f[0];
        if constexpr (!STATS) {
            dot = group_sum(dot);
            // z below the clamp has a constant norm: no gradient through it
            const float inorm = inormp[0];
            const float proj = (inorm < 1e6f) ? dot * inorm * inorm * inorm : 0.f;
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; pr++) projp[pr] = proj;
        }

        // pass 3: the z LoRA and dk_in
        bf16x4 dk_prev = {};
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            const f32x4 pre0 = dkk.f[cb] * inormp[cb >> 1] - projp[cb >> 1] * z.f[cb];
            const bf16x4 dk_b = to_bf16(dkin.f[cb] + pre0);
            if (cb & 1) *reinterpret_cast<bf16x8*>(dk_in + offs + 32 * (cb >> 1)) = __builtin_shufflevector(dk_prev, dk_b, 0, 1, 2, 3, 4, 5, 6, 7);
            dk_prev = dk_b;
            const bf16x4 pb = to_bf16(pre0);
            dW[0][cb] = mma(dW[0][cb], inT[0], transpose(pb, eye));
            dact[0] = mma(dact[0], sWT[0 * NBLK + cb][lane], pb);
        }
        {   // through tanh
            const f32x4 t = to_f32(tz);
            dact[0] = dact[0] * (1.f - t * t);
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
            *reinterpret_cast<bf16x4*>(din.p[i] + ((m0 + L.n) * H + h) * D + 4 * L.g) = to_bf16(dact[i]);
    }

    for (int w = 0; w < 4; w++) {
        if (wave == w) {
            auto put = [&](float* p, f32x4 v) {
                if (w > 0) v += *reinterpret_cast<f32x4*>(p);
                *reinterpret_cast<f32x4*>(p) = v;
            };
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int cb = 0; cb < NBLK; cb++) {
                    put(comb + ((i * HEAD + chan16(cb, L.n)) * D) + 4 * L.g, dW[i][cb]);
                }
            if (L.g == 0) {   // this lane's channel, bias gradients 0..3 in the four registers
#pragma unroll
                for (int cb = 0; cb < NBLK; cb++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        float* p = comb + 4 * HEAD * D + i * HEAD + chan16(cb, L.n);
                        *p = (w > 0 ? *p : 0.f) + dB[cb][i];
                    }
            }
        }
        __syncthreads();
    }
    float* out = partial + ((long)split * gridDim.x + h) * REC;
    for (int i = threadIdx.x; i < REC / 4; i += 256)
        *reinterpret_cast<f32x4*>(out + 4 * i) = *reinterpret_cast<const f32x4*>(comb + 4 * i);
}

// d_in[i][m][d] = sum over heads of the per-head partials (bf16 in, fp32 sum, bf16 out); one thread per
// 8 consecutive rank channels
__global__ __launch_bounds__(256) void expand_loras_din_reduce_kernel(long M, int H, int D, LoraDIn part, LoraDIn out) {
    const long n8 = M * D / 8;
    const long e = blockIdx.x * 256L + threadIdx.x;
    if (e >= 4 * n8) return;
    const int i = (int)(e / n8);
    const long r = (e % n8) * 8;          // element offset in [M][D]
    const long m = r / D;
    const int d = (int)(r % D);
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const __bf16* src = part.p[i] + m * H * D + d;
    for (int h = 0; h < H; h++) {
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(src + (long)h * D);
#pragma unroll
        for (int q = 0; q < 8; q++) acc[q] += (float)v[q];
    }
    bf16x8 o;
#pragma unroll
    for (int q = 0; q < 8; q++) o[q] = (__bf16)acc[q];
    *reinterpret_cast<bf16x8*>(out.p[i] + r) = o;
}

// dW_i [C][D] and dbias_i [C]: sum of the block records over the token splits, in order; one thread per element
struct LoraParamOut {
    float* dW[4];
    float* db[4];
};
__global__ __launch_bounds__(256) void expand_loras_param_reduce_kernel(int C, int D, int nsplit,
                                                                        const float* __restrict__ partial,
                                                                        LoraParamOut out) {
    const int H = C / HEAD;
    const int h = blockIdx.y;
    const int REC = 4 * HEAD * D + 4 * HEAD;
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= REC) return;
    float s = 0.f;
    for (int sp = 0; sp < nsplit; sp++) s += partial[((long)sp * H + h) * REC + e];
    if (e < 4 * HEAD * D) {
        const int i = e / (HEAD * D), r = e % (HEAD * D);
        out.dW[i][(long)h * HEAD * D + r] = s;
    } else {
        const int f = e - 4 * HEAD * D;
        out.db[f / HEAD][h * HEAD + f % HEAD] = s;
    }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
namespace {
constexpr size_t A256(size_t x) { return (x + 255) / 256 * 256; }
// Blocks of the backward kernel per head.  The kernel holds one block per compute unit (one wavefront per SIMD),
// so the grid must fit ONE round of the MI355X's 256 compute units: rounding 256 / H up gave 264 blocks at 12
// heads, a second round of 8 blocks and twice the run time.  At least four token tiles (one per wavefront) each.
int loras_splits(long M, int H) {
    const long ntiles = M / TOK;
    long s = compute_units() / H;
    if (s > ntiles / 4) s = ntiles / 4;
    if (s < 1) s = 1;
    return (int)s;
}
}  // namespace

bool expand_loras_rank_supported(int D) { return D == 16 || D == 32 || D == 64; }
bool expand_loras_head_size_supported(int C, int HS) { return HS >= 16 && HS % 16 == 0 && C % HS == 0; }

// (the statistics of the smallest head size are always included: the size does not depend on the head size)
size_t expand_loras_bwd_workspace_bytes(long M, int C, int D) {
    const int H = C / HEAD;
    const size_t din = A256((size_t)M * H * D * 2) * 4;
    const size_t partial = A256((size_t)loras_splits(M, H) * H * (4 * HEAD * D + 4 * HEAD) * 4);
    const size_t stats = A256((size_t)M * (C / 16) * sizeof(HeadStat));
    return din + partial + stats;
}

void launch_expand_loras_forward(long M, int C, int D, int HS, const void* w_in, const void* k_in, const void* const acts[4],
                                 const void* const Ws[4], const void* const biases[4], void* const outs[4],
                                 hipStream_t stream) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    auto m = [](void* p) { return static_cast<__bf16*>(p); };
    const LoraIn in{{c(acts[0]), c(acts[1]), c(acts[2]), c(acts[3])}};
    const LoraW lw{{c(Ws[0]), c(Ws[1]), c(Ws[2]), c(Ws[3])}, {c(biases[0]), c(biases[1]), c(biases[2]), c(biases[3])}};
    const dim3 block(256);
    if (HS != HEAD && D == 16 && HS <= 128) {
        // two blocks fit a compute unit: two full rounds, at least four token tiles (one per wavefront) each
        const int NH = C / HS;
        const long ntiles = M / TOK;
        long nsplit = 4 * compute_units() / NH;
        if (nsplit > ntiles / 4) nsplit = ntiles / 4;
        if (nsplit < 1) nsplit = 1;
        const int tiles_per_split = (int)((ntiles + nsplit - 1) / nsplit);
        const dim3 hgrid(NH, (unsigned)nsplit);
#define WKV_LAUNCH_HEAD16(NB)                                                                                          \
    case NB:                                                                                                           \
        hipLaunchKernelGGL(expand_loras_head_fwd16_kernel<NB>, hgrid, block, 0, stream, M, C, tiles_per_split, c(w_in),  \
                           c(k_in), in, lw, m(outs[0]), m(outs[1]), m(outs[2]), m(outs[3]));                           \
        break
        switch (HS / 16) {
            WKV_LAUNCH_HEAD16(1);
            WKV_LAUNCH_HEAD16(2);
            WKV_LAUNCH_HEAD16(3);
            WKV_LAUNCH_HEAD16(5);
            WKV_LAUNCH_HEAD16(6);
            WKV_LAUNCH_HEAD16(7);
            default: WKV_LAUNCH_HEAD16(8);
        }
#undef WKV_LAUNCH_HEAD16
        return;
    }
    if (HS != HEAD) {
        const long items = (M / TOK) * (C / HS);
        const dim3 hgrid((unsigned)((items + 3) / 4));
#define WKV_LAUNCH_HEAD(ND)                                                                                             \
    hipLaunchKernelGGL((expand_loras_head_kernel<ND, false>), hgrid, block, 0, stream, M, C, HS, c(w_in), c(k_in), in, lw, \
                       m(outs[0]), m(outs[1]), m(outs[2]), m(outs[3]), nullptr, nullptr, nullptr)
        if (D == 16) WKV_LAUNCH_HEAD(1);
        else if (D == 32) WKV_LAUNCH_HEAD(2);
        else WKV_LAUNCH_HEAD(4);
#undef WKV_LAUNCH_HEAD
        return;
    }
    const long tiles = (M / TOK) * (C / HEAD);
    const dim3 grid((unsigned)((tiles + 3) / 4));
#define WKV_LAUNCH_FWD(ND)                                                                                            \
    hipLaunchKernelGGL(expand_loras_fwd_kernel<ND>, grid, block, 0, stream, M, C, c(w_in), c(k_in), in, lw, m(outs[0]), \
                       m(outs[1]), m(outs[2]), m(outs[3]))
    if (D == 16) {
        // two blocks fit a compute unit: two full rounds of 512, at least four token tiles (one per wavefront) each
        const int H = C / HEAD;
        const long ntiles = M / TOK;
        long nsplit = 4 * compute_units() / H;
        if (nsplit > ntiles / 4) nsplit = ntiles / 4;
        if (nsplit < 1) nsplit = 1;
        const int tiles_per_split = (int)((ntiles + nsplit - 1) / nsplit);
        hipLaunchKernelGGL(expand_loras_fwd16_kernel, dim3(H, (unsigned)nsplit), block, 0, stream, M, C, tiles_per_split,
                           c(w_in), c(k_in), in, lw, m(outs[0]), m(outs[1]), m(outs[2]), m(outs[3]));
    } else if (D == 32) WKV_LAUNCH_FWD(2);
    else WKV_LAUNCH_FWD(4);
#undef WKV_LAUNCH_FWD
}

void launch_expand_loras_backward(long M, int C, int D, int HS, const void* w_in, const void* k_in, const void* const acts[4],
                                  const void* const Ws[4], const void* const biases[4], const void* const dys[4],
                                  void* dw_in, void* dk_in, void* const dacts[4], void* const dWs[4],
                                  void* const dbiases[4], void* workspace, hipStream_t stream) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    auto m = [](void* p) { return static_cast<__bf16*>(p); };
    auto f = [](void* p) { return static_cast<float*>(p); };
    const int H = C / HEAD;
    const LoraIn in{{c(acts[0]), c(acts[1]), c(acts[2]), c(acts[3])}};
    const LoraW lw{{c(Ws[0]), c(Ws[1]), c(Ws[2]), c(Ws[3])}, {c(biases[0]), c(biases[1]), c(biases[2]), c(biases[3])}};
    const LoraDy dy{{c(dys[0]), c(dys[1]), c(dys[2]), c(dys[3])}};
    char* p = static_cast<char*>(workspace);
    LoraDIn part;
    for (int i = 0; i < 4; i++) {
        part.p[i] = reinterpret_cast<__bf16*>(p);
        p += A256((size_t)M * H * D * 2);
    }
    float* partial = reinterpret_cast<float*>(p);
    const int nsplit = loras_splits(M, H);
    p += A256((size_t)nsplit * H * (4 * HEAD * D + 4 * HEAD) * 4);
    HeadStat* stats = reinterpret_cast<HeadStat*>(p);
    const LoraDIn dout{{m(dacts[0]), m(dacts[1]), m(dacts[2]), m(dacts[3])}};
    const int tiles_per_split = (int)((M / TOK + nsplit - 1) / nsplit);
    const dim3 grid(H, nsplit), block(256);
#define WKV_LAUNCH_BWD(ND, STATS)                                                                                       \
    hipLaunchKernelGGL((expand_loras_bwd_kernel<ND, STATS>), grid, block, 0, stream, M, C, tiles_per_split, c(w_in),    \
                       c(k_in), in, lw, dy, m(dw_in), m(dk_in), part, partial, stats, HS)
#define WKV_LAUNCH_BWD16(STATS)                                                                                         \
    hipLaunchKernelGGL(expand_loras_bwd16_kernel<STATS>, grid, block, 0, stream, M, C, tiles_per_split, c(w_in), c(k_in), \
                       in, lw, dy, m(dw_in), m(dk_in), part, partial, stats, HS)
    if (HS != HEAD) {
        const long items = (M / TOK) * (C / HS);
        const dim3 hgrid((unsigned)((items + 3) / 4));
#define WKV_LAUNCH_STAT(ND)                                                                                            \
    hipLaunchKernelGGL((expand_loras_head_kernel<ND, true>), hgrid, block, 0, stream, M, C, HS, c(w_in), c(k_in), in, lw, \
                       nullptr, nullptr, nullptr, nullptr, dy.p[2], dy.p[3], stats)
        if (D == 16) {
            WKV_LAUNCH_STAT(1);
            WKV_LAUNCH_BWD16(true);
        } else if (D == 32) {
            WKV_LAUNCH_STAT(2);
            WKV_LAUNCH_BWD(2, true);
        } else {
            WKV_LAUNCH_STAT(4);
            WKV_LAUNCH_BWD(4, true);
        }
#undef WKV_LAUNCH_STAT
    } else if (D == 16) WKV_LAUNCH_BWD16(false);
    else if (D == 32) WKV_LAUNCH_BWD(2, false);
    else WKV_LAUNCH_BWD(4, false);
#undef WKV_LAUNCH_BWD
#undef WKV_LAUNCH_BWD16
    hipLaunchKernelGGL(expand_loras_din_reduce_kernel, dim3((unsigned)((4 * M * D / 8 + 255) / 256)), dim3(256), 0, stream,
                       M, H, D, part, dout);
    const LoraParamOut pout{{f(dWs[0]), f(dWs[1]), f(dWs[2]), f(dWs[3])},
                            {f(dbiases[0]), f(dbiases[1]), f(dbiases[2]), f(dbiases[3])}};
    const int rec = 4 * HEAD * D + 4 * HEAD;
    hipLaunchKernelGGL(expand_loras_param_reduce_kernel, dim3((rec + 255) / 256, H), dim3(256), 0, stream, C, D, nsplit,
                       partial, pout);
}

}  // namespace wkv
