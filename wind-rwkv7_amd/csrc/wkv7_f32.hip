// WKV7 in fp32: sequences, state, arithmetic and saved states all fp32 (no matrix cores), head sizes 16 .. 128.
//
// The accuracy mode of the path - what the reference's Triton kernels provide with dot_prec='fp32'
// (rwkv7_attn_triton.py:27-156, :182-190) - and what its large-head variant runs by default
// (rwkv7_attn_triton_bighead.py:31-322, any multiple of 16).  Results are within 1e-4 of the fp64 recurrence, where
// the bf16 kernels are within 1e-2.  It is the token-by-token recurrence itself,
//     sa = S a_t;   S <- S diag(exp(-exp(w_t))) + sa b_t^T + v_t k_t^T;   y_t = S q_t,
// with the state in registers, spread thin so that a token costs few instructions per wavefront and little LDS
// traffic: a thread holds R rows x 4 columns.  A block works at a width C of 64 or 128 channels (a smaller head is
// padded: channels and rows past the head size read as zero and are never written); the C / 4 lanes that share a
// state row are one DPP row (C = 64) or two neighbouring ones (C = 128), so a row sum (S a, S q, dS k, dS b) is four
// DPP adds (and one lane swap); a wavefront holds 4 or 2 such row groups, and a column sum over them (S^T dy, dS^T v,
// ...) is three (one) of gfx950's lane swaps (col_sum4, store_col_sums), then LDS across the wavefronts.  The vectors
// of a token are read as one 16-byte LDS access each, one token ahead of their use.
// The value rows of a state never mix, so a head can be cut over blocks by rows.  Forward: eight wavefronts per block
// (two per SIMD cover each other's waits), four or two blocks per head (a quarter or half of the rows each) while every
// block still gets a compute unit of its own, else one block with all rows.  Backward: always two blocks of four wavefronts per head (all
// rows in one block need more registers than a wavefront has); the gradients that sum over value rows (dq, dk, da, db,
// dw) are the sum of the two blocks' parts, added with floating-point atomics onto zeroed tensors - with exactly two
// addends per element the result does not depend on their order, so results are reproducible.
// The forward keeps the state every CHUNK tokens and S a of every token; the backward walks the chunks in reverse,
// recomputes a window of states of a chunk into registers (three multiply-adds per element, no row sums to wait for)
// and runs the adjoint recurrence through them.
#include "wkv7_f32_kernels.hpp"

#include <hip/hip_runtime.h>

namespace wkv {
namespace {

typedef float f4 __attribute__((ext_vector_type(4)));

// gfx950's lane-swap instructions, one swap and one add for two values at once: v_permlane32_swap exchanges lanes
// 32-63 of its first register with lanes 0-31 of its second, so with X and Y two values to be summed over the lane
// pairs (l, l + 32), X' + Y' is X summed over the pair in lanes 0-31 and Y summed over the pair in lanes 32-63;
// v_permlane16_swap does the same between neighbouring rows of 16 lanes (even rows keep X, odd rows Y).
__device__ __forceinline__ float swap_add32(float x, float y) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float swap_add16(float x, float y) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// index of element (token t, head h, channel c) of a [B,T,H,C] tensor, b folded into t
__device__ __forceinline__ long seq_index(long bt, int H, int h, int c, int C) { return (bt * H + h) * C + c; }

enum { V_DEC = 0, V_Q, V_K, V_V, V_A, V_B, FWD_VECS };
enum { W_DEC = 0, W_Q, W_K, W_V, W_A, W_B, W_DY, W_DDEC, BWD_VECS };   // W_DDEC: d(decay)/dw = -exp(w) decay
enum { R_DQ = 0, R_DK, R_DB, R_DA, R_DW, RED_VECS };

constexpr int CH64 = WKV7_F32_CHUNK;   // tokens between saved states

template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
// sum over the 16 lanes of a DPP row, result in all of them (every step adds two values that both lanes hold, so the
// 16 results are the same bits)
__device__ __forceinline__ float row_sum16(float x) {
    x += dpp<0xB1>(x);     // quad_perm [1,0,3,2]
    x += dpp<0x4E>(x);     // quad_perm [2,3,0,1]
    x += dpp<0x141>(x);    // row_half_mirror
    x += dpp<0x140>(x);    // row_mirror
    return x;
}
__device__ __forceinline__ float dot4(f4 x, f4 y) { return ((x[0] * y[0] + x[1] * y[1]) + x[2] * y[2]) + x[3] * y[3]; }
// p: this thread's terms for columns 4 jb .. 4 jb + 3.  Returns the sum over the wavefront's four row groups of column
// 4 jb + ib: lanes 0-31 keep columns 0 and 1, lanes 32-63 columns 2 and 3; then even rows of 16 lanes keep the lower
// of their two, odd rows the upper.
__device__ __forceinline__ float col_sum4(f4 p) {
    const float lo = swap_add32(p[0], p[2]), hi = swap_add32(p[1], p[3]);
    return swap_add16(lo, hi);
}
template <int R>
struct RowVals {
    float x[R];
};
template <int R>
__device__ __forceinline__ RowVals<R> lds_rows(const float* p) {
    RowVals<R> r;
    if constexpr (R % 4 == 0) {
#pragma unroll
        for (int i = 0; i < R / 4; i++) {
            const f4 v = *reinterpret_cast<const f4*>(p + 4 * i);
            r.x[4 * i] = v[0], r.x[4 * i + 1] = v[1], r.x[4 * i + 2] = v[2], r.x[4 * i + 3] = v[3];
        }
    } else if constexpr (R == 2) {
        typedef float f2 __attribute__((ext_vector_type(2)));
        const f2 v = *reinterpret_cast<const f2*>(p);
        r.x[0] = v[0], r.x[1] = v[1];
    } else {
        r.x[0] = *p;
    }
    return r;
}

// sum over the LPR lanes that share a state row (16: a DPP row; 32: two neighbouring DPP rows), result in all of them
template <int LPR>
__device__ __forceinline__ float row_sum(float x) {
    x = row_sum16(x);
    if constexpr (LPR == 32) x = swap_add16(x, x);   // both operands the same: every lane gets this row plus its neighbour
    return x;
}
// Column sums over the row groups of a wavefront, stored for the cross-wavefront sum.  p: this thread's terms for
// columns col0 .. col0 + 3; to: the 4 LPR columns of one token and gradient in LDS.  16 lanes per row (four row groups):
// the lane of group ib ends up with column col0 + ib; 32 lanes per row (two groups): with columns col0 + 2 ib, + 1.
template <int LPR>
__device__ __forceinline__ void store_col_sums(float* to, f4 p, int col0, int ib) {
    if constexpr (LPR == 16) {
        to[col0 + ib] = col_sum4(p);
    } else {
        typedef float f2 __attribute__((ext_vector_type(2)));
        *reinterpret_cast<f2*>(to + col0 + 2 * ib) = f2{swap_add32(p[0], p[2]), swap_add32(p[1], p[3])};
    }
}

// sum over the 64 lanes of a wavefront, result in all of them
__device__ __forceinline__ float wave_sum(float x) {
    x = row_sum16(x);
    x += __shfl_xor(x, 16, 64);
    x += __shfl_xor(x, 32, 64);
    return x;
}

// What the forward keeps for the backward, in one buffer: the state entering every CH64 tokens ([B,H,T/CH64,C,C]) and
// then S a of every token ([B,T,H,C]; the backward's recomputation of the states inside a chunk then needs no row sums).
__host__ __device__ inline long saved_states(long BH, int T, int C) { return BH * (T / CH64) * C * C; }

template <int C, int R, int NW, bool FULL>
__global__ __launch_bounds__(64 * NW) void wkv7_f32_fwd_thin_kernel(int T, int H, int CR, const float* __restrict__ w,
                                                             const float* __restrict__ q, const float* __restrict__ k,
                                                             const float* __restrict__ v, const float* __restrict__ a,
                                                             const float* __restrict__ b, const float* __restrict__ s0,
                                                             float* __restrict__ y, float* __restrict__ ckpt,
                                                             float* __restrict__ sT) {
    typedef float f2 __attribute__((ext_vector_type(2)));
    constexpr int CH = CH64, LPR = C / 4, GPW = 64 / LPR, THREADS = 64 * NW, ROWS = NW * GPW * R, NSPLIT = C / ROWS;
    constexpr int PER = CH * C / THREADS, TPJ = THREADS / C, NH = C / 64;
    static_assert(C % ROWS == 0 && (CH * C) % THREADS == 0 && (CH * ROWS) % THREADS == 0, "whole tokens and rows per thread");
    __shared__ __attribute__((aligned(16))) float in[FWD_VECS][CH][C];    // the slot of q holds decay * q
    __shared__ f2 bkq[CH][NH];                                            // (b . q, k . q) of every token, per 64 channels
    __shared__ __attribute__((aligned(16))) float yout[CH][ROWS], saout[CH][ROWS];
    const int bh = blockIdx.x / NSPLIT, part = blockIdx.x % NSPLIT, h = bh % H;
    const long bt0 = (long)(bh / H) * T;
    const int tid = threadIdx.x, lane = tid & 63, jb = lane % LPR, rl = ((tid >> 6) * GPW + lane / LPR) * R;
    const int row0 = part * ROWS + rl, col0 = 4 * jb;
    const float* const src[FWD_VECS] = {w, q, k, v, a, b};
    float* const sav = ckpt == nullptr ? nullptr : ckpt + saved_states(gridDim.x / NSPLIT, T, CR);
    // Addresses are a base per chunk that is the same in every lane (scalar registers) plus a small 32-bit offset per
    // thread, instead of a 64-bit address per thread and access.
    // CR: the head size itself; C: the width the block works at (channels and rows past CR read as zero, are never
    // written, and stay zero in the state).  FULL: CR == C, no access needs a bound.
    const unsigned ld = (unsigned)H * CR;                                    // floats between consecutive tokens
    const bool col_ok = FULL || col0 < CR, stage_ok = FULL || (int)(tid % C) < CR;
    const unsigned state_off = (unsigned)(row0 * CR + (col_ok ? col0 : 0));  // this thread's first row in a CR x CR state
    const unsigned tok_off = (unsigned)(tid / C) * ld + (stage_ok ? tid % C : 0);   // (token, channel) this thread stages
    auto chunk_base = [&](int c0) { return seq_index(bt0 + c0, H, h, 0, CR); };
    auto row_ok = [&](int r) { return FULL || (col_ok && row0 + r < CR); };
    const f4 zero = {0.f, 0.f, 0.f, 0.f};

    f4 S[R];
#pragma unroll
    for (int r = 0; r < R; r++)
        S[r] = row_ok(r) ? *reinterpret_cast<const f4*>(s0 + (long)bh * CR * CR + (state_off + r * CR)) : zero;
    float pre[FWD_VECS][PER];
    auto fetch = [&](int c0) {
        const long base = chunk_base(c0);
#pragma unroll
        for (int vec = 0; vec < FWD_VECS; vec++) {
#pragma unroll
            for (int j = 0; j < PER; j++) {
                const float x = (src[vec] + base)[tok_off + (unsigned)(TPJ * j) * ld];
                pre[vec][j] = stage_ok ? x : 0.f;
            }
        }
    };
    fetch(0);
    for (int c0 = 0; c0 < T; c0 += CH) {
        // stage the chunk: the decay instead of w, decay * q instead of q.  With them
        //   y_t = S_t q = S_{t-1} (decay * q) + (S_{t-1} a) (b . q) + v (k . q),
        // so that both row sums of a token work on the state BEFORE its update and neither waits for the other.
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const int tok = TPJ * j + tid / C, ch = tid % C;
            const float d = expf(-expf(pre[V_DEC][j]));
            in[V_DEC][tok][ch] = d;
            in[V_Q][tok][ch] = d * pre[V_Q][j];
            in[V_K][tok][ch] = pre[V_K][j];
            in[V_V][tok][ch] = pre[V_V][j];
            in[V_A][tok][ch] = pre[V_A][j];
            in[V_B][tok][ch] = pre[V_B][j];
            const float bq = wave_sum(pre[V_B][j] * pre[V_Q][j]), kq = wave_sum(pre[V_K][j] * pre[V_Q][j]);
            if (lane == 0) bkq[tok][ch >> 6] = f2{bq, kq};
        }
        if (ckpt != nullptr) {
            float* const to = ckpt + ((long)bh * (T / CH) + c0 / CH) * CR * CR;
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (row_ok(r)) *reinterpret_cast<f4*>(to + (state_off + r * CR)) = S[r];
            }
        }
        __syncthreads();
        fetch(c0 + CH < T ? c0 + CH : c0);   // (after the last chunk: the same one again, not used)
        // a token's operands are requested from LDS one token ahead (the stores of the results in between keep the
        // compiler from moving the reads up by itself)
        struct Ops {
            f4 dec, av, bv, kv, dqv;
            RowVals<R> vr;
            f2 sc;
        };
        auto read_ops = [&](int t) {
            Ops o;
            o.dec = *reinterpret_cast<const f4*>(&in[V_DEC][t][col0]), o.av = *reinterpret_cast<const f4*>(&in[V_A][t][col0]);
            o.bv = *reinterpret_cast<const f4*>(&in[V_B][t][col0]), o.kv = *reinterpret_cast<const f4*>(&in[V_K][t][col0]);
            o.dqv = *reinterpret_cast<const f4*>(&in[V_Q][t][col0]);
            o.vr = lds_rows<R>(&in[V_V][t][row0]);
            o.sc = bkq[t][0];
            if constexpr (NH == 2) o.sc += bkq[t][1];
            return o;
        };
        Ops ahead = read_ops(0);
#pragma unroll
        for (int t = 0; t < CH; t++) {
            const Ops o = ahead;
            if (t + 1 < CH) ahead = read_ops(t + 1);
            const f4 dec = o.dec, av = o.av, bv = o.bv, kv = o.kv, dqv = o.dqv;
            const RowVals<R> vr = o.vr;
            const f2 sc = o.sc;
            RowVals<R> yr, sar;
#pragma unroll
            for (int r = 0; r < R; r++) {
                sar.x[r] = row_sum<LPR>(dot4(S[r], av));
                yr.x[r] = row_sum<LPR>(dot4(S[r], dqv)) + sar.x[r] * sc[0] + vr.x[r] * sc[1];
                S[r] = S[r] * dec + sar.x[r] * bv + vr.x[r] * kv;
            }
            if (jb == 0) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    yout[t][rl + r] = yr.x[r];
                    saout[t][rl + r] = sar.x[r];
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < CH * ROWS / THREADS; m++) {
            const int e = tid + THREADS * m;
            const int tok = e / ROWS, ch = e % ROWS;
            const unsigned at = (unsigned)tok * ld + (unsigned)(part * ROWS + ch);
            if (FULL || part * ROWS + ch < CR) {
                (y + chunk_base(c0))[at] = yout[tok][ch];
                if (sav != nullptr) (sav + chunk_base(c0))[at] = saout[tok][ch];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (row_ok(r)) *reinterpret_cast<f4*>(sT + (long)bh * CR * CR + (state_off + r * CR)) = S[r];
    }
}

template <int C, int R, int NW, int WIN, bool FULL>
__global__ __launch_bounds__(64 * NW) void wkv7_f32_bwd_thin_kernel(int T, int H, int CR, const float* __restrict__ w,
                                                             const float* __restrict__ q, const float* __restrict__ k,
                                                             const float* __restrict__ v, const float* __restrict__ a,
                                                             const float* __restrict__ b, const float* __restrict__ dy,
                                                             const float* __restrict__ ckpt, const float* __restrict__ dsT,
                                                             float* __restrict__ dw, float* __restrict__ dq,
                                                             float* __restrict__ dk, float* __restrict__ dv,
                                                             float* __restrict__ da, float* __restrict__ db,
                                                             float* __restrict__ ds0) {
    constexpr int CH = CH64, LPR = C / 4, GPW = 64 / LPR, THREADS = 64 * NW, ROWS = NW * GPW * R, NSPLIT = C / ROWS;
    constexpr int PER = CH * C / THREADS, TPJ = THREADS / C;
    static_assert(C == 2 * ROWS && CH % WIN == 0 && (CH * C) % THREADS == 0 && (WIN * C) % THREADS == 0,
                  "two blocks per head (two addends per gradient element), whole windows, whole tokens per thread");
    constexpr int NSRC = 8, W_SA = BWD_VECS;     // the eighth vector per token: the forward's S a
    __shared__ __attribute__((aligned(16))) float in[BWD_VECS + 1][CH][C];
    __shared__ float red[NW][RED_VECS][WIN][C];   // per wavefront: column sums over its 4 R rows, a window of tokens
    __shared__ __attribute__((aligned(16))) float dvout[WIN][ROWS];
    const int bh = blockIdx.x / NSPLIT, part = blockIdx.x % NSPLIT, h = bh % H;
    const long bt0 = (long)(bh / H) * T;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, jb = lane % LPR, ib = lane / LPR, rl = (wv * GPW + ib) * R;
    const int row0 = part * ROWS + rl, col0 = 4 * jb;
    const float* const src[NSRC] = {w, q, k, v, a, b, dy, ckpt + saved_states(gridDim.x / NSPLIT, T, CR)};
    float* const dst[RED_VECS] = {dq, dk, db, da, dw};

    const unsigned ld = (unsigned)H * CR;                                    // (addresses and bounds: as in the forward kernel)
    const bool col_ok = FULL || col0 < CR, stage_ok = FULL || (int)(tid % C) < CR;
    const unsigned state_off = (unsigned)(row0 * CR + (col_ok ? col0 : 0));
    const unsigned tok_off = (unsigned)(tid / C) * ld + (stage_ok ? tid % C : 0);
    auto chunk_base = [&](int c0) { return seq_index(bt0 + c0, H, h, 0, CR); };
    auto row_ok = [&](int r) { return FULL || (col_ok && row0 + r < CR); };
    const f4 zero = {0.f, 0.f, 0.f, 0.f};

    f4 dS[R];
#pragma unroll
    for (int r = 0; r < R; r++)
        dS[r] = row_ok(r) ? *reinterpret_cast<const f4*>(dsT + (long)bh * CR * CR + (state_off + r * CR)) : zero;
    // the eight vectors per token and the saved state of the NEXT chunk (the one before in time) are fetched while the
    // current one runs
    float pre[NSRC][PER];
    f4 pre_s[R];
    auto fetch = [&](int c0) {
        const long base = chunk_base(c0);
#pragma unroll
        for (int vec = 0; vec < NSRC; vec++) {
#pragma unroll
            for (int j = 0; j < PER; j++) {
                const float x = (src[vec] + base)[tok_off + (unsigned)(TPJ * j) * ld];
                pre[vec][j] = stage_ok ? x : 0.f;
            }
        }
        const float* const from = ckpt + ((long)bh * (T / CH) + c0 / CH) * CR * CR;
#pragma unroll
        for (int r = 0; r < R; r++) pre_s[r] = row_ok(r) ? *reinterpret_cast<const f4*>(from + (state_off + r * CR)) : zero;
    };
    fetch(T - CH);
    for (int c0 = T - CH; c0 >= 0; c0 -= CH) {
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const int tok = TPJ * j + tid / C, ch = tid % C;
            const float ew = expf(pre[W_DEC][j]), d = expf(-ew);
            in[W_DEC][tok][ch] = d;
            in[W_DDEC][tok][ch] = -ew * d;
#pragma unroll
            for (int vec = 1; vec < NSRC; vec++) in[vec == NSRC - 1 ? W_SA : vec][tok][ch] = pre[vec][j];
        }
        f4 Sx[R];             // the state entering the chunk
#pragma unroll
        for (int r = 0; r < R; r++) Sx[r] = pre_s[r];
        __syncthreads();
        fetch(c0 >= CH ? c0 - CH : c0);   // (after the first chunk in time: the same one again)
        // S_{t+1} = S_t diag(decay_t) + (S a)_t b_t^T + v_t k_t^T, with S a as the forward saved it.  Operands are read
        // from LDS one token ahead; the compiler barrier after each request keeps it from requesting a whole window's
        // operands at once (and from keeping them for the adjoint: 14 registers per token and row group).
        struct AdvOps {
            f4 dec, bv, kv;
            RowVals<R> vr, sar;
        };
        auto read_adv = [&](int t) {
            AdvOps o;
            o.dec = *reinterpret_cast<const f4*>(&in[W_DEC][t][col0]);
            o.bv = *reinterpret_cast<const f4*>(&in[W_B][t][col0]), o.kv = *reinterpret_cast<const f4*>(&in[W_K][t][col0]);
            o.vr = lds_rows<R>(&in[W_V][t][row0]), o.sar = lds_rows<R>(&in[W_SA][t][row0]);
            return o;
        };
        auto advance = [&](const f4 (&from)[R], f4 (&to)[R], const AdvOps& o) {
#pragma unroll
            for (int r = 0; r < R; r++) to[r] = from[r] * o.dec + o.sar.x[r] * o.bv + o.vr.x[r] * o.kv;
        };
        // a token's operands for the adjoint are requested from LDS one token ahead (the stores of the results in
        // between keep the compiler from moving the reads up by itself)
        struct AdjOps {
            f4 dec, av, bv, kv, qv;
            RowVals<R> vr, dyr, sar;
        };
        auto read_adj = [&](int t) {
            AdjOps o;
            o.dec = *reinterpret_cast<const f4*>(&in[W_DEC][t][col0]), o.av = *reinterpret_cast<const f4*>(&in[W_A][t][col0]);
            o.bv = *reinterpret_cast<const f4*>(&in[W_B][t][col0]), o.kv = *reinterpret_cast<const f4*>(&in[W_K][t][col0]);
            o.qv = *reinterpret_cast<const f4*>(&in[W_Q][t][col0]);
            o.vr = lds_rows<R>(&in[W_V][t][row0]), o.dyr = lds_rows<R>(&in[W_DY][t][row0]), o.sar = lds_rows<R>(&in[W_SA][t][row0]);
            return o;
        };
        // the chunk in windows of WIN tokens, last window first: the states of a window are recomputed into registers
        // (from the chunk's first state: the windows before it are run through once more, a running state only), then
        // the adjoint recurrence walks back through them
#pragma unroll 1
        for (int win = CH / WIN - 1; win >= 0; win--) {
            const int t0 = win * WIN;
            f4 St[WIN + 1][R];     // St[t] enters token t0 + t
#pragma unroll
            for (int r = 0; r < R; r++) St[0][r] = Sx[r];
            AdvOps adv = read_adv(0);
#pragma unroll 1
            for (int t = 0; t < t0; t++) {
                const AdvOps o = adv;
                adv = read_adv(t + 1);
                asm volatile("" ::: "memory");
                advance(St[0], St[0], o);
            }
#pragma unroll
            for (int tw = 0; tw < WIN; tw++) {
                const AdvOps o = adv;
                if (tw + 1 < WIN) adv = read_adv(t0 + tw + 1);
                asm volatile("" ::: "memory");
                advance(St[tw], St[tw + 1], o);
            }
            AdjOps ahead = read_adj(t0 + WIN - 1);
#pragma unroll
            for (int tw = WIN - 1; tw >= 0; tw--) {
                const int t = t0 + tw;
                const AdjOps o = ahead;
                if (tw > 0) ahead = read_adj(t - 1);
                asm volatile("" ::: "memory");
                const f4 dec = o.dec, av = o.av, bv = o.bv, kv = o.kv, qv = o.qv;
                const RowVals<R> vr = o.vr, dyr = o.dyr, sar = o.sar;
                // dq = S_t^T dy;  dS_t += dy q^T;  dv = dS k;  dsa = dS b
                f4 pq = St[tw + 1][0] * dyr.x[0];
#pragma unroll
                for (int r = 1; r < R; r++) pq += St[tw + 1][r] * dyr.x[r];
                float dsa[R];
                RowVals<R> dvr;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    dS[r] += dyr.x[r] * qv;
                    dvr.x[r] = row_sum<LPR>(dot4(dS[r], kv));
                    dsa[r] = row_sum<LPR>(dot4(dS[r], bv));
                }
                if (jb == 0) {
#pragma unroll
                    for (int r = 0; r < R; r++) dvout[tw][rl + r] = dvr.x[r];
                }
                // dk = dS^T v;  db = dS^T sa;  da = S_{t-1}^T dsa;  ddecay = sum over rows of dS * S_{t-1}
                f4 pk = dS[0] * vr.x[0], pb = dS[0] * sar.x[0], pa = St[tw][0] * dsa[0], pw = dS[0] * St[tw][0];
#pragma unroll
                for (int r = 1; r < R; r++) {
                    pk += dS[r] * vr.x[r];
                    pb += dS[r] * sar.x[r];
                    pa += St[tw][r] * dsa[r];
                    pw += dS[r] * St[tw][r];
                }
                store_col_sums<LPR>(red[wv][R_DQ][tw], pq, col0, ib);
                store_col_sums<LPR>(red[wv][R_DK][tw], pk, col0, ib);
                store_col_sums<LPR>(red[wv][R_DB][tw], pb, col0, ib);
                store_col_sums<LPR>(red[wv][R_DA][tw], pa, col0, ib);
                store_col_sums<LPR>(red[wv][R_DW][tw], pw, col0, ib);
                // dS_{t-1} = dS_t diag(decay) + dsa a^T
#pragma unroll
                for (int r = 0; r < R; r++) dS[r] = dS[r] * dec + dsa[r] * av;
            }
            __syncthreads();
            // the wavefronts' sums of this window, in a fixed order, and out
#pragma unroll
            for (int vec = 0; vec < RED_VECS; vec++) {
#pragma unroll
                for (int j = 0; j < WIN * C / THREADS; j++) {
                    const int tw = TPJ * j + tid / C, tok = win * WIN + tw, ch = tid % C;
                    float s = red[0][vec][tw][ch];
#pragma unroll
                    for (int g = 1; g < NW; g++) s += red[g][vec][tw][ch];
                    if (vec == R_DW) s *= in[W_DDEC][tok][ch];
                    float* const p = dst[vec] + chunk_base(c0) + (tok_off + (unsigned)(win * WIN + TPJ * j) * ld);
                    if (FULL || ch < CR) unsafeAtomicAdd(p, s);   // (onto zeros; the other block of the head adds its part)
                }
            }
#pragma unroll
            for (int m = 0; m < (WIN * ROWS + THREADS - 1) / THREADS; m++) {
                const int e = tid + THREADS * m;
                const int tw = e / ROWS, ch = e % ROWS;
                if (((WIN * ROWS) % THREADS == 0 || e < WIN * ROWS) && (FULL || part * ROWS + ch < CR))
                    (dv + chunk_base(c0))[(unsigned)(win * WIN + tw) * ld + (unsigned)(part * ROWS + ch)] = dvout[tw][ch];
            }
            __syncthreads();
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (row_ok(r)) *reinterpret_cast<f4*>(ds0 + (long)bh * CR * CR + (state_off + r * CR)) = dS[r];
    }
}

// five tensors of n floats each to zero (what the two-blocks-per-head backward adds its parts onto)
__global__ __launch_bounds__(256) void zero5_kernel(long n4, f4* __restrict__ p0, f4* __restrict__ p1, f4* __restrict__ p2,
                                                    f4* __restrict__ p3, f4* __restrict__ p4) {
    f4* const p[5] = {p0, p1, p2, p3, p4};
    const f4 z = {0.f, 0.f, 0.f, 0.f};
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n4; i += (long)gridDim.x * 256) {
#pragma unroll
        for (int t = 0; t < 5; t++) p[t][i] = z;
    }
}


// blocks per head in the forward kernel: as many of 4, 2, 1 as still leave every block a compute unit of its own
int forward_split(int BH) {
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 256;
        return n;
    }();
    return 4 * BH <= cus ? 4 : 2 * BH <= cus ? 2 : 1;
}

}  // namespace

size_t wkv7_f32_saved_bytes(int B, int T, int H, int C) {
    return ((size_t)saved_states((long)B * H, T, C) + (size_t)B * T * H * C) * sizeof(float);
}

// (head sizes up to 64 run at a width of 64 channels, larger ones at 128; FULL: the head fills the width)
void launch_wkv7_f32_forward(int B, int T, int H, int C, const float* w, const float* q, const float* k, const float* v,
                             const float* a, const float* b, const float* s0, float* y, float* ckpt, float* sT,
                             hipStream_t stream) {
    const int split = forward_split(B * H);
    auto go = [&](auto k4, auto k2, auto k1, int threads4) {
        auto launch = [&](auto kernel, int threads) {
            hipLaunchKernelGGL(kernel, dim3(split * B * H), dim3(threads), 0, stream, T, H, C, w, q, k, v, a, b, s0, y, ckpt, sT);
        };
        if (split == 4) launch(k4, threads4);
        else if (split == 2) launch(k2, 512);
        else launch(k1, 512);
    };
    // (width, rows per thread, wavefronts): rows per block = wavefronts x row groups per wavefront x rows per thread
    if (C == 64) go(wkv7_f32_fwd_thin_kernel<64, 1, 4, true>, wkv7_f32_fwd_thin_kernel<64, 1, 8, true>, wkv7_f32_fwd_thin_kernel<64, 2, 8, true>, 256);
    else if (C < 64) go(wkv7_f32_fwd_thin_kernel<64, 1, 4, false>, wkv7_f32_fwd_thin_kernel<64, 1, 8, false>, wkv7_f32_fwd_thin_kernel<64, 2, 8, false>, 256);
    else if (C == 128) go(wkv7_f32_fwd_thin_kernel<128, 2, 8, true>, wkv7_f32_fwd_thin_kernel<128, 4, 8, true>, wkv7_f32_fwd_thin_kernel<128, 8, 8, true>, 512);
    else go(wkv7_f32_fwd_thin_kernel<128, 2, 8, false>, wkv7_f32_fwd_thin_kernel<128, 4, 8, false>, wkv7_f32_fwd_thin_kernel<128, 8, 8, false>, 512);
}

void launch_wkv7_f32_backward(int B, int T, int H, int C, const float* w, const float* q, const float* k, const float* v,
                              const float* a, const float* b, const float* dy, const float* ckpt, const float* dsT,
                              float* dw, float* dq, float* dk, float* dv, float* da, float* db, float* ds0,
                              hipStream_t stream) {
    const long n4 = (long)B * T * H * C / 4;
    auto z = [](float* p) { return reinterpret_cast<f4*>(p); };
    hipLaunchKernelGGL(zero5_kernel, dim3((unsigned)((n4 + 255) / 256 < 2048 ? (n4 + 255) / 256 : 2048)), dim3(256), 0, stream, n4,
                       z(dq), z(dk), z(db), z(da), z(dw));
    auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(2 * B * H), dim3(256), 0, stream, T, H, C, w, q, k, v, a, b, dy, ckpt, dsT, dw, dq, dk, dv,
                           da, db, ds0);
    };
    if (C == 64) go(wkv7_f32_bwd_thin_kernel<64, 2, 4, 16, true>);
    else if (C < 64) go(wkv7_f32_bwd_thin_kernel<64, 2, 4, 16, false>);
    else if (C == 128) go(wkv7_f32_bwd_thin_kernel<128, 8, 4, 4, true>);
    else go(wkv7_f32_bwd_thin_kernel<128, 8, 4, 4, false>);
}

}  // namespace wkv
