// WKV7 in fp32: sequences, state, arithmetic and checkpoints all fp32 (no matrix cores), head sizes 16 .. 128.
//
// The accuracy mode of the path - what the reference's Triton kernels provide with dot_prec='fp32'
// (rwkv7_attn_triton.py:27-156, :182-190) - and the kernels behind head sizes other than 64, which the
// reference serves with rwkv7_attn_triton_bighead.py:31-322 (any multiple of 16).  Results are within 1e-4 of
// the fp64 recurrence, where the bf16 kernels are within 1e-2.  It is the token-by-token recurrence itself,
//     sa = S a_t;   S <- S diag(exp(-exp(w_t))) + sa b_t^T + v_t k_t^T;   y_t = S q_t,
// one block per (batch, head) with the state in registers.  The head is padded to CP = 64 NCG channels (NCG =
// 1 or 2 column groups; channels past the head size read as zero and are never written).  A block has 256 NCG
// threads: thread (cg, i, jb) holds columns 64 cg + 16 jb .. + 15 of rows i, i + 64, ... (NCG rows).  Row sums
// (S a, S q, dS k, dS b) are two lane exchanges within the 64 columns of a wavefront; with two column groups
// the halves meet through LDS (one barrier per token for S a and for dS b, none for the outputs).  Column sums
// (S^T dy, dS^T v, ...) use a halving butterfly over the 16 rows of a wavefront (15 exchanges for 16 columns)
// and LDS across the four row groups.  The forward kernel saves the state every CH tokens (8 with one column
// group, 2 with two: the backward kernel keeps CH + 1 states of NCG rows in registers); the backward kernel
// walks those chunks in reverse, recomputes the CH states of a chunk into registers and runs the adjoint
// recurrence through them.  Summation orders are fixed, so results are reproducible.
#include "wkv7_f32_kernels.hpp"

#include <hip/hip_runtime.h>

namespace wkv {
namespace {

constexpr int COLS = 16;       // state columns per thread

typedef float f4 __attribute__((ext_vector_type(4)));

struct Vec16 {
    float x[COLS];
};

// 16 consecutive floats from LDS (all rows read the same addresses: broadcast)
__device__ __forceinline__ Vec16 lds16(const float* p) {
    Vec16 r;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const f4 v = *reinterpret_cast<const f4*>(p + 4 * q);
        r.x[4 * q] = v[0];
        r.x[4 * q + 1] = v[1];
        r.x[4 * q + 2] = v[2];
        r.x[4 * q + 3] = v[3];
    }
    return r;
}

// sum over the four threads that share a row (lanes differing in bits 0..1), result in all four
__device__ __forceinline__ float row_sum4(float x) {
    x += __shfl_xor(x, 1, 64);
    x += __shfl_xor(x, 2, 64);
    return x;
}

// Column sums over the 16 rows of a wavefront.  In: p[c] = this row's term for column 16 jb + c.  Out: the
// sum over the wavefront's rows of ONE column, c = 8 b5 + 4 b4 + 2 b3 + b2 with b2..b5 bits 2..5 of the lane.
// A halving butterfly: at each level a lane keeps one half of its columns and hands the other half to the lane
// that keeps it.  The two wide levels (8 and 4 column pairs) use gfx950's lane-swap instructions, one swap and
// one add per pair: v_permlane32_swap exchanges lanes 32-63 of its first register with lanes 0-31 of its
// second, so with X = the lower column and Y = the upper one, X' + Y' is X summed over the pair in lanes 0-31
// and Y summed over the pair in lanes 32-63; v_permlane16_swap does the same between neighbouring rows of 16
// lanes.  (Selects and ds_bpermute for these levels were 60 of the 75 cross-lane operations of a column sum.)
__device__ __forceinline__ float swap_add32(float x, float y) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float swap_add16(float x, float y) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float col_sum16(const Vec16& p, int lane) {
    float a8[8], a4[4], a2[2];
    const bool b2 = lane & 4, b3 = lane & 8;
#pragma unroll
    for (int c = 0; c < 8; c++) a8[c] = swap_add32(p.x[c], p.x[c + 8]);       // lanes 32-63 keep columns 8-15
#pragma unroll
    for (int c = 0; c < 4; c++) a4[c] = swap_add16(a8[c], a8[c + 4]);          // odd rows keep the upper four
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const float keep = b3 ? a4[c + 2] : a4[c], send = b3 ? a4[c] : a4[c + 2];
        a2[c] = keep + __shfl_xor(send, 8, 64);
    }
    const float keep = b2 ? a2[1] : a2[0], send = b2 ? a2[0] : a2[1];
    return keep + __shfl_xor(send, 4, 64);
}
__device__ __forceinline__ int col_of_lane(int lane) {
    return 16 * (lane & 3) + 8 * ((lane >> 5) & 1) + 4 * ((lane >> 4) & 1) + 2 * ((lane >> 3) & 1) + ((lane >> 2) & 1);
}

// index of element (token t, head h, channel c) of a [B,T,H,C] tensor, b folded into t
__device__ __forceinline__ long seq_index(long bt, int H, int h, int c, int C) { return (bt * H + h) * C + c; }

// Sum of a per-row value over the column groups of the block: the threads with jb == 0 post their wavefront's
// sum, one barrier, everyone reads all groups in a fixed order.  buf: [NCG][CP], alternating between two
// buffers from one call to the next (a thread can be one barrier ahead of another, not two).
template <int NCG>
__device__ __forceinline__ void across_groups(float (&x)[NCG], float* buf, int cg, int i, int jb) {
    if constexpr (NCG > 1) {
        constexpr int CP = 64 * NCG;
        if (jb == 0) {
#pragma unroll
            for (int s = 0; s < NCG; s++) buf[cg * CP + i + 64 * s] = x[s];
        }
        __syncthreads();
#pragma unroll
        for (int s = 0; s < NCG; s++) {
            float sum = buf[i + 64 * s];
#pragma unroll
            for (int g = 1; g < NCG; g++) sum += buf[g * CP + i + 64 * s];
            x[s] = sum;
        }
    }
}

// ---- forward -------------------------------------------------------------------------------------------------
enum { V_DEC = 0, V_Q, V_K, V_V, V_A, V_B, FWD_VECS };

template <int NCG, bool FULL>
__global__ __launch_bounds__(256 * NCG) void wkv7_f32_fwd_kernel(int T, int H, int C, const float* __restrict__ w,
                                                                 const float* __restrict__ q, const float* __restrict__ k,
                                                                 const float* __restrict__ v, const float* __restrict__ a,
                                                                 const float* __restrict__ b, const float* __restrict__ s0,
                                                                 float* __restrict__ y, float* __restrict__ ckpt,
                                                                 float* __restrict__ sT) {
    constexpr int THREADS = 256 * NCG, CP = 64 * NCG, CH = NCG == 1 ? 8 : 2;
    __shared__ __attribute__((aligned(16))) float in[FWD_VECS][CH][CP];
    __shared__ float ypart[NCG][CH][CP];          // per column group: its share of y
    __shared__ float xch[2][NCG * CP];
    const int bh = blockIdx.x, h = bh % H;
    const long bt0 = (long)(bh / H) * T;
    const int tid = threadIdx.x, cg = tid >> 8, i = (tid & 255) >> 2, jb = tid & 3;
    const int col0 = 64 * cg + COLS * jb;
    const float* const src[FWD_VECS] = {w, q, k, v, a, b};
    bool ok[NCG];     // this thread's piece of row i + 64 s lies inside the head
#pragma unroll
    for (int s = 0; s < NCG; s++) ok[s] = FULL || (col0 < C && i + 64 * s < C);

    float S[NCG][COLS];
#pragma unroll
    for (int s = 0; s < NCG; s++) {
        const float* p = s0 + ((long)bh * C + i + 64 * s) * C + col0;
#pragma unroll
        for (int c = 0; c < COLS; c++) S[s][c] = ok[s] ? p[c] : 0.f;
    }
    // the six vectors per token of the NEXT chunk are fetched (into registers, unconditionally: a channel past the
    // head reads channel 0 and is zeroed when staged) while the current chunk runs
    constexpr int NLD = (FWD_VECS * CH * CP + THREADS - 1) / THREADS;
    float pre[NLD];
    auto fetch = [&](int c0) {
#pragma unroll
        for (int m = 0; m < NLD; m++) {
            const int e = tid + THREADS * m;
            if ((FWD_VECS * CH * CP) % THREADS != 0 && e >= FWD_VECS * CH * CP) break;
            const int vec = e / (CH * CP), tok = (e / CP) % CH, ch = e % CP;
            pre[m] = src[vec][seq_index(bt0 + c0 + tok, H, h, (FULL || ch < C) ? ch : 0, C)];
        }
    };
    fetch(0);
    for (int c0 = 0; c0 < T; c0 += CH) {
        // stage the chunk (the decay instead of w)
#pragma unroll
        for (int m = 0; m < NLD; m++) {
            const int e = tid + THREADS * m;
            if ((FWD_VECS * CH * CP) % THREADS != 0 && e >= FWD_VECS * CH * CP) break;
            const int vec = e / (CH * CP), tok = (e / CP) % CH, ch = e % CP;
            float x = pre[m];
            if (vec == V_DEC) x = expf(-expf(x));
            in[vec][tok][ch] = (FULL || ch < C) ? x : 0.f;
        }
        // the state entering the chunk (kept for the backward pass; a forward nothing differentiates passes no buffer)
#pragma unroll
        for (int s = 0; s < NCG; s++) {
            if (ckpt != nullptr && ok[s]) {
                float* p = ckpt + (((long)bh * (T / CH) + c0 / CH) * C + i + 64 * s) * C + col0;
#pragma unroll
                for (int c = 0; c < COLS; c += 4) *reinterpret_cast<f4*>(p + c) = f4{S[s][c], S[s][c + 1], S[s][c + 2], S[s][c + 3]};
            }
        }
        __syncthreads();
        fetch(c0 + CH < T ? c0 + CH : c0);   // (after the last chunk: the same one again, not used)
#pragma unroll
        for (int t = 0; t < CH; t++) {
            const Vec16 dec = lds16(&in[V_DEC][t][col0]), av = lds16(&in[V_A][t][col0]);
            const Vec16 bv = lds16(&in[V_B][t][col0]), kv = lds16(&in[V_K][t][col0]);
            const Vec16 qv = lds16(&in[V_Q][t][col0]);
            float sa[NCG];
#pragma unroll
            for (int s = 0; s < NCG; s++) {
                float x = 0.f;
#pragma unroll
                for (int c = 0; c < COLS; c++) x += S[s][c] * av.x[c];
                sa[s] = row_sum4(x);
            }
            across_groups<NCG>(sa, xch[t & 1], cg, i, jb);
#pragma unroll
            for (int s = 0; s < NCG; s++) {
                const float vi = in[V_V][t][i + 64 * s];
                float yi = 0.f;
#pragma unroll
                for (int c = 0; c < COLS; c++) {
                    S[s][c] = S[s][c] * dec.x[c] + sa[s] * bv.x[c] + vi * kv.x[c];
                    yi += S[s][c] * qv.x[c];
                }
                yi = row_sum4(yi);
                if (jb == 0) ypart[cg][t][i + 64 * s] = yi;
            }
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < (CH * CP + THREADS - 1) / THREADS; m++) {
            const int e = tid + THREADS * m;
            if ((CH * CP) % THREADS != 0 && e >= CH * CP) break;
            const int tok = e / CP, ch = e % CP;
            float sum = ypart[0][tok][ch];
#pragma unroll
            for (int g = 1; g < NCG; g++) sum += ypart[g][tok][ch];
            if (FULL || ch < C) y[seq_index(bt0 + c0 + tok, H, h, ch, C)] = sum;
        }
    }
#pragma unroll
    for (int s = 0; s < NCG; s++) {
        if (ok[s]) {
            float* p = sT + ((long)bh * C + i + 64 * s) * C + col0;
#pragma unroll
            for (int c = 0; c < COLS; c++) p[c] = S[s][c];
        }
    }
}

// ---- backward ------------------------------------------------------------------------------------------------
enum { W_DEC = 0, W_Q, W_K, W_V, W_A, W_B, W_DY, W_DDEC, BWD_VECS };   // W_DDEC: d(decay)/dw = -exp(w) decay
enum { R_DQ = 0, R_DK, R_DB, R_DA, R_DW, RED_VECS };

template <int NCG, bool FULL>
__global__ __launch_bounds__(256 * NCG) void wkv7_f32_bwd_kernel(int T, int H, int C, const float* __restrict__ w,
                                                                 const float* __restrict__ q, const float* __restrict__ k,
                                                                 const float* __restrict__ v, const float* __restrict__ a,
                                                                 const float* __restrict__ b, const float* __restrict__ dy,
                                                                 const float* __restrict__ ckpt, const float* __restrict__ dsT,
                                                                 float* __restrict__ dw, float* __restrict__ dq,
                                                                 float* __restrict__ dk, float* __restrict__ dv,
                                                                 float* __restrict__ da, float* __restrict__ db,
                                                                 float* __restrict__ ds0) {
    constexpr int THREADS = 256 * NCG, CP = 64 * NCG, CH = NCG == 1 ? 8 : 2;
    __shared__ __attribute__((aligned(16))) float in[BWD_VECS][CH][CP];
    __shared__ float red[4][RED_VECS][CH][CP];    // per row group (wavefront): partial column sums
    __shared__ float dvpart[NCG][CH][CP];         // per column group: its share of dv
    __shared__ float xch[4][NCG * CP];            // 0, 1: the recomputation's S a;  2, 3: the adjoint's dS b
    const int bh = blockIdx.x, h = bh % H;
    const long bt0 = (long)(bh / H) * T;
    const int tid = threadIdx.x, cg = tid >> 8, i = (tid & 255) >> 2, jb = tid & 3, lane = tid & 63, rg = (tid & 255) >> 6;
    const int col0 = 64 * cg + COLS * jb;
    const int mycol = 64 * cg + col_of_lane(lane);
    const float* const src[7] = {w, q, k, v, a, b, dy};
    float* const dst[RED_VECS] = {dq, dk, db, da, dw};
    bool ok[NCG];
#pragma unroll
    for (int s = 0; s < NCG; s++) ok[s] = FULL || (col0 < C && i + 64 * s < C);

    float dS[NCG][COLS];
#pragma unroll
    for (int s = 0; s < NCG; s++) {
        const float* p = dsT + ((long)bh * C + i + 64 * s) * C + col0;
#pragma unroll
        for (int c = 0; c < COLS; c++) dS[s][c] = ok[s] ? p[c] : 0.f;
    }
    // With one column group there are registers to spare: the seven vectors per token and the checkpoint of the
    // NEXT chunk (the one before in time) are fetched while the current one runs, unconditionally (a channel or
    // row past the head reads element 0 and is zeroed when used).  With two groups the loads stay where they
    // are needed.
    constexpr bool AHEAD = NCG == 1;
    constexpr int NLD = (7 * CH * CP + THREADS - 1) / THREADS;
    float pre[AHEAD ? NLD : 1];
    f4 pre_s[AHEAD ? NCG : 1][COLS / 4];
    auto fetch = [&](int c0) {
#pragma unroll
        for (int m = 0; m < NLD; m++) {
            const int e = tid + THREADS * m;
            if ((7 * CH * CP) % THREADS != 0 && e >= 7 * CH * CP) break;
            const int vec = e / (CH * CP), tok = (e / CP) % CH, ch = e % CP;
            pre[m] = src[vec][seq_index(bt0 + c0 + tok, H, h, (FULL || ch < C) ? ch : 0, C)];
        }
#pragma unroll
        for (int s = 0; s < NCG; s++) {
            const float* p = ckpt + (((long)bh * (T / CH) + c0 / CH) * C + (ok[s] ? i + 64 * s : 0)) * C + (ok[s] ? col0 : 0);
#pragma unroll
            for (int c = 0; c < COLS; c += 4) pre_s[s][c / 4] = *reinterpret_cast<const f4*>(p + c);
        }
    };
    if constexpr (AHEAD) fetch(T - CH);
    for (int c0 = T - CH; c0 >= 0; c0 -= CH) {
#pragma unroll
        for (int m = 0; m < NLD; m++) {
            const int e = tid + THREADS * m;
            if ((7 * CH * CP) % THREADS != 0 && e >= 7 * CH * CP) break;
            const int vec = e / (CH * CP), tok = (e / CP) % CH, ch = e % CP;
            float x;
            if constexpr (AHEAD) x = (FULL || ch < C) ? pre[m] : 0.f;
            else x = (FULL || ch < C) ? src[vec][seq_index(bt0 + c0 + tok, H, h, ch, C)] : 0.f;
            if (vec == W_DEC) {
                const float ew = expf(x), d = expf(-ew);
                in[W_DEC][tok][ch] = d;
                in[W_DDEC][tok][ch] = -ew * d;
            } else {
                in[vec][tok][ch] = x;
            }
        }
        // the chunk's states: St[t] enters token t
        float St[CH + 1][NCG][COLS], sa[CH][NCG];
#pragma unroll
        for (int s = 0; s < NCG; s++) {
            const float* p = ckpt + (((long)bh * (T / CH) + c0 / CH) * C + i + 64 * s) * C + col0;
#pragma unroll
            for (int c = 0; c < COLS; c += 4) {
                f4 x = {0.f, 0.f, 0.f, 0.f};
                if constexpr (AHEAD) {
                    if (ok[s]) x = pre_s[s][c / 4];
                } else {
                    if (ok[s]) x = *reinterpret_cast<const f4*>(p + c);
                }
                St[0][s][c] = x[0];
                St[0][s][c + 1] = x[1];
                St[0][s][c + 2] = x[2];
                St[0][s][c + 3] = x[3];
            }
        }
        __syncthreads();
        if constexpr (AHEAD) fetch(c0 >= CH ? c0 - CH : c0);   // (after the first chunk in time: the same one again)
#pragma unroll
        for (int t = 0; t < CH; t++) {
            const Vec16 dec = lds16(&in[W_DEC][t][col0]), av = lds16(&in[W_A][t][col0]);
            const Vec16 bv = lds16(&in[W_B][t][col0]), kv = lds16(&in[W_K][t][col0]);
#pragma unroll
            for (int s = 0; s < NCG; s++) {
                float x = 0.f;
#pragma unroll
                for (int c = 0; c < COLS; c++) x += St[t][s][c] * av.x[c];
                sa[t][s] = row_sum4(x);
            }
            across_groups<NCG>(sa[t], xch[t & 1], cg, i, jb);
#pragma unroll
            for (int s = 0; s < NCG; s++) {
                const float vi = in[W_V][t][i + 64 * s];
#pragma unroll
                for (int c = 0; c < COLS; c++) St[t + 1][s][c] = St[t][s][c] * dec.x[c] + sa[t][s] * bv.x[c] + vi * kv.x[c];
            }
        }
#pragma unroll
        for (int t = CH - 1; t >= 0; t--) {
            const Vec16 dec = lds16(&in[W_DEC][t][col0]), av = lds16(&in[W_A][t][col0]);
            const Vec16 bv = lds16(&in[W_B][t][col0]), kv = lds16(&in[W_K][t][col0]);
            const Vec16 qv = lds16(&in[W_Q][t][col0]);
            float vi[NCG], dyi[NCG];
#pragma unroll
            for (int s = 0; s < NCG; s++) {
                vi[s] = in[W_V][t][i + 64 * s];
                dyi[s] = in[W_DY][t][i + 64 * s];
            }
            Vec16 p;
            // dq = S_t^T dy
#pragma unroll
            for (int c = 0; c < COLS; c++) {
                float x = St[t + 1][0][c] * dyi[0];
#pragma unroll
                for (int s = 1; s < NCG; s++) x += St[t + 1][s][c] * dyi[s];
                p.x[c] = x;
            }
            red[rg][R_DQ][t][mycol] = col_sum16(p, lane);
            // dS_t += dy q^T;  dv = dS k;  dsa = dS b
            float dsa[NCG];
#pragma unroll
            for (int s = 0; s < NCG; s++) {
                float dvi = 0.f, x = 0.f;
#pragma unroll
                for (int c = 0; c < COLS; c++) {
                    dS[s][c] += dyi[s] * qv.x[c];
                    dvi += dS[s][c] * kv.x[c];
                    x += dS[s][c] * bv.x[c];
                }
                dvi = row_sum4(dvi);
                dsa[s] = row_sum4(x);
                if (jb == 0) dvpart[cg][t][i + 64 * s] = dvi;
            }
            across_groups<NCG>(dsa, xch[2 + (t & 1)], cg, i, jb);
            // dk = dS^T v;  db = dS^T sa;  da = S_{t-1}^T dsa;  ddecay = sum_i dS * S_{t-1}
#pragma unroll
            for (int c = 0; c < COLS; c++) {
                float x = dS[0][c] * vi[0];
#pragma unroll
                for (int s = 1; s < NCG; s++) x += dS[s][c] * vi[s];
                p.x[c] = x;
            }
            red[rg][R_DK][t][mycol] = col_sum16(p, lane);
#pragma unroll
            for (int c = 0; c < COLS; c++) {
                float x = dS[0][c] * sa[t][0];
#pragma unroll
                for (int s = 1; s < NCG; s++) x += dS[s][c] * sa[t][s];
                p.x[c] = x;
            }
            red[rg][R_DB][t][mycol] = col_sum16(p, lane);
#pragma unroll
            for (int c = 0; c < COLS; c++) {
                float x = St[t][0][c] * dsa[0];
#pragma unroll
                for (int s = 1; s < NCG; s++) x += St[t][s][c] * dsa[s];
                p.x[c] = x;
            }
            red[rg][R_DA][t][mycol] = col_sum16(p, lane);
#pragma unroll
            for (int c = 0; c < COLS; c++) {
                float x = dS[0][c] * St[t][0][c];
#pragma unroll
                for (int s = 1; s < NCG; s++) x += dS[s][c] * St[t][s][c];
                p.x[c] = x;
            }
            red[rg][R_DW][t][mycol] = col_sum16(p, lane);
            // dS_{t-1} = dS_t diag(decay) + dsa a^T
#pragma unroll
            for (int s = 0; s < NCG; s++) {
#pragma unroll
                for (int c = 0; c < COLS; c++) dS[s][c] = dS[s][c] * dec.x[c] + dsa[s] * av.x[c];
            }
        }
        __syncthreads();
        // the four row groups' partial sums, in a fixed order, and out
#pragma unroll
        for (int m = 0; m < (RED_VECS * CH * CP + THREADS - 1) / THREADS; m++) {
            const int e = tid + THREADS * m;
            if ((RED_VECS * CH * CP) % THREADS != 0 && e >= RED_VECS * CH * CP) break;
            const int vec = e / (CH * CP), tok = (e / CP) % CH, ch = e % CP;
            float s = ((red[0][vec][tok][ch] + red[1][vec][tok][ch]) + red[2][vec][tok][ch]) + red[3][vec][tok][ch];
            if (vec == R_DW) s *= in[W_DDEC][tok][ch];
            if (FULL || ch < C) dst[vec][seq_index(bt0 + c0 + tok, H, h, ch, C)] = s;
        }
#pragma unroll
        for (int m = 0; m < (CH * CP + THREADS - 1) / THREADS; m++) {
            const int e = tid + THREADS * m;
            if ((CH * CP) % THREADS != 0 && e >= CH * CP) break;
            const int tok = e / CP, ch = e % CP;
            float sum = dvpart[0][tok][ch];
#pragma unroll
            for (int g = 1; g < NCG; g++) sum += dvpart[g][tok][ch];
            if (FULL || ch < C) dv[seq_index(bt0 + c0 + tok, H, h, ch, C)] = sum;
        }
        __syncthreads();
    }
#pragma unroll
    for (int s = 0; s < NCG; s++) {
        if (ok[s]) {
            float* p = ds0 + ((long)bh * C + i + 64 * s) * C + col0;
#pragma unroll
            for (int c = 0; c < COLS; c++) p[c] = dS[s][c];
        }
    }
}

}  // namespace

int wkv7_f32_chunk(int C) { return C <= 64 ? 8 : 2; }

// FULL: the head fills the padded width (64 or 128 channels) and no access needs a bound
void launch_wkv7_f32_forward(int B, int T, int H, int C, const float* w, const float* q, const float* k, const float* v,
                             const float* a, const float* b, const float* s0, float* y, float* ckpt, float* sT,
                             hipStream_t stream) {
    auto go = [&](auto kernel, int threads) {
        hipLaunchKernelGGL(kernel, dim3(B * H), dim3(threads), 0, stream, T, H, C, w, q, k, v, a, b, s0, y, ckpt, sT);
    };
    if (C == 64) go(wkv7_f32_fwd_kernel<1, true>, 256);
    else if (C < 64) go(wkv7_f32_fwd_kernel<1, false>, 256);
    else if (C == 128) go(wkv7_f32_fwd_kernel<2, true>, 512);
    else go(wkv7_f32_fwd_kernel<2, false>, 512);
}

void launch_wkv7_f32_backward(int B, int T, int H, int C, const float* w, const float* q, const float* k, const float* v,
                              const float* a, const float* b, const float* dy, const float* ckpt, const float* dsT,
                              float* dw, float* dq, float* dk, float* dv, float* da, float* db, float* ds0,
                              hipStream_t stream) {
    auto go = [&](auto kernel, int threads) {
        hipLaunchKernelGGL(kernel, dim3(B * H), dim3(threads), 0, stream, T, H, C, w, q, k, v, a, b, dy, ckpt, dsT, dw, dq,
                           dk, dv, da, db, ds0);
    };
    if (C == 64) go(wkv7_f32_bwd_kernel<1, true>, 256);
    else if (C < 64) go(wkv7_f32_bwd_kernel<1, false>, 256);
    else if (C == 128) go(wkv7_f32_bwd_kernel<2, true>, 512);
    else go(wkv7_f32_bwd_kernel<2, false>, 512);
}

}  // namespace wkv
