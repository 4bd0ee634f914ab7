// WKV7 in fp32: sequences, state, arithmetic and checkpoints all fp32 (no matrix cores).
//
// The accuracy mode of the path - what the reference's Triton kernels provide with dot_prec='fp32'
// (rwkv7_attn_triton.py:27-156, :182-190): results within 1e-4 of the fp64 recurrence, where the bf16 kernels
// are within 1e-2.  It is the token-by-token recurrence itself,
//     sa = S a_t;   S <- S diag(exp(-exp(w_t))) + sa b_t^T + v_t k_t^T;   y_t = S q_t,
// one block of 256 threads per (batch, head) with the 64 x 64 state in registers: thread (i, jb) holds row i,
// columns 16 jb .. 16 jb + 15.  Row sums (S a, S q, dS k, dS b) are two lane exchanges; column sums
// (S^T dy, dS^T v, ...) use a halving butterfly over the 16 rows of a wavefront (15 exchanges for 16 columns)
// and LDS across the four wavefronts.  The forward kernel saves the state every 8 tokens; the backward kernel
// walks the chunks in reverse, recomputes the 8 states of a chunk into registers and runs the adjoint
// recurrence through them.  Summation orders are fixed, so results are reproducible.
#include "wkv7_f32_kernels.hpp"

#include <hip/hip_runtime.h>

namespace wkv {
namespace {

constexpr int N = 64;          // head size
constexpr int CH = F32_CHUNK;  // tokens per checkpoint
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
// sum over the wavefront's rows of ONE column, c = 8 b2 + 4 b3 + 2 b4 + b5 with b2..b5 bits 2..5 of the lane.
__device__ __forceinline__ float col_sum16(const Vec16& p, int lane) {
    float a8[8], a4[4], a2[2];
    const bool b2 = lane & 4, b3 = lane & 8, b4 = lane & 16, b5 = lane & 32;
#pragma unroll
    for (int c = 0; c < 8; c++) {
        const float keep = b2 ? p.x[c + 8] : p.x[c], send = b2 ? p.x[c] : p.x[c + 8];
        a8[c] = keep + __shfl_xor(send, 4, 64);
    }
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const float keep = b3 ? a8[c + 4] : a8[c], send = b3 ? a8[c] : a8[c + 4];
        a4[c] = keep + __shfl_xor(send, 8, 64);
    }
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const float keep = b4 ? a4[c + 2] : a4[c], send = b4 ? a4[c] : a4[c + 2];
        a2[c] = keep + __shfl_xor(send, 16, 64);
    }
    const float keep = b5 ? a2[1] : a2[0], send = b5 ? a2[0] : a2[1];
    return keep + __shfl_xor(send, 32, 64);
}
__device__ __forceinline__ int col_of_lane(int lane) {
    return 16 * (lane & 3) + 8 * ((lane >> 2) & 1) + 4 * ((lane >> 3) & 1) + 2 * ((lane >> 4) & 1) + ((lane >> 5) & 1);
}

// index of element (token t, head h, channel c) of a [B,T,H,N] tensor, b folded into t
__device__ __forceinline__ long seq_index(long bt, int H, int h, int c) { return (bt * H + h) * N + c; }

// ---- forward -------------------------------------------------------------------------------------------------
enum { V_DEC = 0, V_Q, V_K, V_V, V_A, V_B, FWD_VECS };

__global__ __launch_bounds__(256) void wkv7_f32_fwd_kernel(int T, int H, const float* __restrict__ w,
                                                           const float* __restrict__ q, const float* __restrict__ k,
                                                           const float* __restrict__ v, const float* __restrict__ a,
                                                           const float* __restrict__ b, const float* __restrict__ s0,
                                                           float* __restrict__ y, float* __restrict__ ckpt,
                                                           float* __restrict__ sT) {
    __shared__ __attribute__((aligned(16))) float in[FWD_VECS][CH][N];
    __shared__ __attribute__((aligned(16))) float yout[CH][N];
    const int bh = blockIdx.x, h = bh % H;
    const long bt0 = (long)(bh / H) * T;
    const int tid = threadIdx.x, i = tid >> 2, jb = tid & 3;
    const float* const src[FWD_VECS] = {w, q, k, v, a, b};

    float S[COLS];
    {
        const float* p = s0 + ((long)bh * N + i) * N + COLS * jb;
#pragma unroll
        for (int c = 0; c < COLS; c++) S[c] = p[c];
    }
    for (int c0 = 0; c0 < T; c0 += CH) {
        // stage the chunk's six vectors per token (the decay instead of w)
#pragma unroll
        for (int m = 0; m < FWD_VECS * CH * N / 256; m++) {
            const int e = tid + 256 * m, vec = e / (CH * N), tok = (e / N) % CH, ch = e % N;
            float x = src[vec][seq_index(bt0 + c0 + tok, H, h, ch)];
            if (vec == V_DEC) x = expf(-expf(x));
            in[vec][tok][ch] = x;
        }
        // the state entering the chunk
        {
            float* p = ckpt + (((long)bh * (T / CH) + c0 / CH) * N + i) * N + COLS * jb;
#pragma unroll
            for (int c = 0; c < COLS; c += 4) *reinterpret_cast<f4*>(p + c) = f4{S[c], S[c + 1], S[c + 2], S[c + 3]};
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < CH; t++) {
            const Vec16 dec = lds16(&in[V_DEC][t][COLS * jb]), av = lds16(&in[V_A][t][COLS * jb]);
            const Vec16 bv = lds16(&in[V_B][t][COLS * jb]), kv = lds16(&in[V_K][t][COLS * jb]);
            const Vec16 qv = lds16(&in[V_Q][t][COLS * jb]);
            const float vi = in[V_V][t][i];
            float sa = 0.f;
#pragma unroll
            for (int c = 0; c < COLS; c++) sa += S[c] * av.x[c];
            sa = row_sum4(sa);
            float yi = 0.f;
#pragma unroll
            for (int c = 0; c < COLS; c++) {
                S[c] = S[c] * dec.x[c] + sa * bv.x[c] + vi * kv.x[c];
                yi += S[c] * qv.x[c];
            }
            yi = row_sum4(yi);
            if (jb == 0) yout[t][i] = yi;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < CH * N / 256; m++) {
            const int e = tid + 256 * m;
            y[seq_index(bt0 + c0 + e / N, H, h, e % N)] = yout[e / N][e % N];
        }
    }
    float* p = sT + ((long)bh * N + i) * N + COLS * jb;
#pragma unroll
    for (int c = 0; c < COLS; c++) p[c] = S[c];
}

// ---- backward ------------------------------------------------------------------------------------------------
enum { W_DEC = 0, W_Q, W_K, W_V, W_A, W_B, W_DY, W_DDEC, BWD_VECS };   // W_DDEC: d(decay)/dw = -exp(w) decay
enum { R_DQ = 0, R_DK, R_DB, R_DA, R_DW, RED_VECS };

__global__ __launch_bounds__(256) void wkv7_f32_bwd_kernel(int T, int H, const float* __restrict__ w,
                                                           const float* __restrict__ q, const float* __restrict__ k,
                                                           const float* __restrict__ v, const float* __restrict__ a,
                                                           const float* __restrict__ b, const float* __restrict__ dy,
                                                           const float* __restrict__ ckpt, const float* __restrict__ dsT,
                                                           float* __restrict__ dw, float* __restrict__ dq,
                                                           float* __restrict__ dk, float* __restrict__ dv,
                                                           float* __restrict__ da, float* __restrict__ db,
                                                           float* __restrict__ ds0) {
    __shared__ __attribute__((aligned(16))) float in[BWD_VECS][CH][N];
    __shared__ float red[4][RED_VECS][CH][N];   // per wavefront partial column sums
    __shared__ float dvout[CH][N];
    const int bh = blockIdx.x, h = bh % H;
    const long bt0 = (long)(bh / H) * T;
    const int tid = threadIdx.x, i = tid >> 2, jb = tid & 3, lane = tid & 63, wave = tid >> 6;
    const int mycol = col_of_lane(lane);
    const float* const src[7] = {w, q, k, v, a, b, dy};
    float* const dst[RED_VECS] = {dq, dk, db, da, dw};

    float dS[COLS];
    {
        const float* p = dsT + ((long)bh * N + i) * N + COLS * jb;
#pragma unroll
        for (int c = 0; c < COLS; c++) dS[c] = p[c];
    }
    for (int c0 = T - CH; c0 >= 0; c0 -= CH) {
#pragma unroll
        for (int m = 0; m < 7 * CH * N / 256; m++) {
            const int e = tid + 256 * m, vec = e / (CH * N), tok = (e / N) % CH, ch = e % N;
            const float x = src[vec][seq_index(bt0 + c0 + tok, H, h, ch)];
            if (vec == W_DEC) {
                const float ew = expf(x), d = expf(-ew);
                in[W_DEC][tok][ch] = d;
                in[W_DDEC][tok][ch] = -ew * d;
            } else {
                in[vec][tok][ch] = x;
            }
        }
        // the chunk's states: St[t] enters token t
        float St[CH + 1][COLS], sa[CH];
        {
            const float* p = ckpt + (((long)bh * (T / CH) + c0 / CH) * N + i) * N + COLS * jb;
#pragma unroll
            for (int c = 0; c < COLS; c += 4) {
                const f4 x = *reinterpret_cast<const f4*>(p + c);
                St[0][c] = x[0];
                St[0][c + 1] = x[1];
                St[0][c + 2] = x[2];
                St[0][c + 3] = x[3];
            }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < CH; t++) {
            const Vec16 dec = lds16(&in[W_DEC][t][COLS * jb]), av = lds16(&in[W_A][t][COLS * jb]);
            const Vec16 bv = lds16(&in[W_B][t][COLS * jb]), kv = lds16(&in[W_K][t][COLS * jb]);
            const float vi = in[W_V][t][i];
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < COLS; c++) s += St[t][c] * av.x[c];
            sa[t] = row_sum4(s);
#pragma unroll
            for (int c = 0; c < COLS; c++) St[t + 1][c] = St[t][c] * dec.x[c] + sa[t] * bv.x[c] + vi * kv.x[c];
        }
#pragma unroll
        for (int t = CH - 1; t >= 0; t--) {
            const Vec16 dec = lds16(&in[W_DEC][t][COLS * jb]), av = lds16(&in[W_A][t][COLS * jb]);
            const Vec16 bv = lds16(&in[W_B][t][COLS * jb]), kv = lds16(&in[W_K][t][COLS * jb]);
            const Vec16 qv = lds16(&in[W_Q][t][COLS * jb]);
            const float vi = in[W_V][t][i], dyi = in[W_DY][t][i];
            Vec16 p;
            // dq = S_t^T dy
#pragma unroll
            for (int c = 0; c < COLS; c++) p.x[c] = St[t + 1][c] * dyi;
            red[wave][R_DQ][t][mycol] = col_sum16(p, lane);
            // dS_t += dy q^T;  dv = dS k;  dsa = dS b
            float dvi = 0.f, dsa = 0.f;
#pragma unroll
            for (int c = 0; c < COLS; c++) {
                dS[c] += dyi * qv.x[c];
                dvi += dS[c] * kv.x[c];
                dsa += dS[c] * bv.x[c];
            }
            dvi = row_sum4(dvi);
            dsa = row_sum4(dsa);
            if (jb == 0) dvout[t][i] = dvi;
            // dk = dS^T v;  db = dS^T sa;  da = S_{t-1}^T dsa;  ddecay = sum_i dS * S_{t-1}
#pragma unroll
            for (int c = 0; c < COLS; c++) p.x[c] = dS[c] * vi;
            red[wave][R_DK][t][mycol] = col_sum16(p, lane);
#pragma unroll
            for (int c = 0; c < COLS; c++) p.x[c] = dS[c] * sa[t];
            red[wave][R_DB][t][mycol] = col_sum16(p, lane);
#pragma unroll
            for (int c = 0; c < COLS; c++) p.x[c] = St[t][c] * dsa;
            red[wave][R_DA][t][mycol] = col_sum16(p, lane);
#pragma unroll
            for (int c = 0; c < COLS; c++) p.x[c] = dS[c] * St[t][c];
            red[wave][R_DW][t][mycol] = col_sum16(p, lane);
            // dS_{t-1} = dS_t diag(decay) + dsa a^T
#pragma unroll
            for (int c = 0; c < COLS; c++) dS[c] = dS[c] * dec.x[c] + dsa * av.x[c];
        }
        __syncthreads();
        // the four wavefronts' partial sums, in a fixed order, and out
#pragma unroll
        for (int m = 0; m < RED_VECS * CH * N / 256; m++) {
            const int e = tid + 256 * m, vec = e / (CH * N), tok = (e / N) % CH, ch = e % N;
            float s = ((red[0][vec][tok][ch] + red[1][vec][tok][ch]) + red[2][vec][tok][ch]) + red[3][vec][tok][ch];
            if (vec == R_DW) s *= in[W_DDEC][tok][ch];
            dst[vec][seq_index(bt0 + c0 + tok, H, h, ch)] = s;
        }
#pragma unroll
        for (int m = 0; m < CH * N / 256; m++) {
            const int e = tid + 256 * m;
            dv[seq_index(bt0 + c0 + e / N, H, h, e % N)] = dvout[e / N][e % N];
        }
        __syncthreads();
    }
    float* p = ds0 + ((long)bh * N + i) * N + COLS * jb;
#pragma unroll
    for (int c = 0; c < COLS; c++) p[c] = dS[c];
}

}  // namespace

void launch_wkv7_f32_forward(int B, int T, int H, const float* w, const float* q, const float* k, const float* v,
                             const float* a, const float* b, const float* s0, float* y, float* ckpt, float* sT,
                             hipStream_t stream) {
    hipLaunchKernelGGL(wkv7_f32_fwd_kernel, dim3(B * H), dim3(256), 0, stream, T, H, w, q, k, v, a, b, s0, y, ckpt, sT);
}

void launch_wkv7_f32_backward(int B, int T, int H, const float* w, const float* q, const float* k, const float* v,
                              const float* a, const float* b, const float* dy, const float* ckpt, const float* dsT,
                              float* dw, float* dq, float* dk, float* dv, float* da, float* db, float* ds0,
                              hipStream_t stream) {
    hipLaunchKernelGGL(wkv7_f32_bwd_kernel, dim3(B * H), dim3(256), 0, stream, T, H, w, q, k, v, a, b, dy, ckpt, dsT, dw,
                       dq, dk, dv, da, db, ds0);
}

}  // namespace wkv
