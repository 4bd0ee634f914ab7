// WKV7 for gfx950, what runs beside the one-kernel organisation of wkv7_fused.hip in the forward direction:
//   * the composition of the segments' affine maps for long sequences on few heads (the states entering the segments),
//   * the attn_ln epilogue as a kernel of its own (GroupNorm + bonus + gate on the kept WKV7 output; attn_ln.cu:11-37),
//     used where the plain forward kernel runs two blocks per (batch, head) and cannot host it,
//   * the rule that says when a sequence is cut into segments.
#include "ln_epilogue.hpp"
#include "device_info.hpp"
#include "wkv7_common.hpp"
#include "wkv7_kernels.hpp"

namespace wkv {

// ------------------------------------------------------------------------------------------------
// Composes the segment maps in processing order: S_in(0) = s0, S_in(g+1) = S_in(g) M_g + N_g, all in fp32 (fp32
// matrix instructions).  maps: as written by the MAP form of wkv7_fused_kernel; s_seg: [pair][segment][64][64]
// floats, the state entering each segment.
// The value rows of a state go through the maps independently, so a block takes 16 of them (four blocks per (batch,
// head)) and its four wavefronts a block of 16 key columns each: 16 matrix instructions per wavefront and segment,
// then the row block's four fragments change hands through LDS.  All maps a wavefront needs (NSEG <= 8: seven times
// 20 registers) are requested before the first product.  (One block per (batch, head), a wavefront per 16 rows doing
// all four column blocks: 64 dependent-by-fours matrix instructions per segment, 2.8 us each, 23 us at 8 segments.)
// ------------------------------------------------------------------------------------------------
constexpr int CARRY_MAX_SEG = 8;
__global__ __launch_bounds__(256) void segment_carry_kernel(int NSEG, int s0_f32, const void* __restrict__ s0,
                                                            const float* __restrict__ maps, float* __restrict__ s_seg) {
    __shared__ f32x4 xch[2][NBLK][WAVE];
    const int jb = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int bh = blockIdx.x >> 2, ib = blockIdx.x & 3;
    const Lane L;
    f32x4 S[NBLK];
#pragma unroll
    for (int kb = 0; kb < NBLK; kb++) S[kb] = load_state_frag(s0, s0_f32, bh, ib, kb, L);
    f32x4 n[CARRY_MAX_SEG - 1], mt[CARRY_MAX_SEG - 1][NBLK];
#pragma unroll
    for (int g = 0; g < CARRY_MAX_SEG - 1; g++) {
        const long e = (long)bh * NSEG + (g < NSEG - 1 ? g : NSEG - 2);   // (past the end: a valid map, not used)
        const float* N = maps + (e * 2 + 0) * HEAD * HEAD;
        const float* MT = maps + (e * 2 + 1) * HEAD * HEAD;
        n[g] = *reinterpret_cast<const f32x4*>(N + (16 * ib + L.n) * HEAD + 16 * jb + 4 * L.g);
#pragma unroll
        for (int kb = 0; kb < NBLK; kb++)   // A operand of S[ib][kb] M[kb][jb]: F(M[kb][jb]^T) = the (jb, kb) block of MT
            mt[g][kb] = *reinterpret_cast<const f32x4*>(MT + (16 * jb + L.n) * HEAD + 16 * kb + 4 * L.g);
    }
    store_state_frag(s_seg, 1, bh * NSEG, ib, jb, L, jb == 0 ? S[0] : jb == 1 ? S[1] : jb == 2 ? S[2] : S[3]);
#pragma unroll
    for (int g = 0; g < CARRY_MAX_SEG - 1; g++) {
        if (g < NSEG - 1) {   // (uniform; no load inside)
            f32x4 a0 = mma_f32(n[g], mt[g][0], S[0]), a1 = mma_f32(zero4(), mt[g][1], S[1]);
            a0 = mma_f32(a0, mt[g][2], S[2]);
            a1 = mma_f32(a1, mt[g][3], S[3]);
            const f32x4 T = a0 + a1;
            store_state_frag(s_seg, 1, bh * NSEG + g + 1, ib, jb, L, T);
            xch[g & 1][jb][lane] = T;
            __syncthreads();
#pragma unroll
            for (int kb = 0; kb < NBLK; kb++) S[kb] = xch[g & 1][kb][lane];
        }
    }
}


// ------------------------------------------------------------------------------------------------
// attn_ln epilogue: one wavefront per chunk applies GroupNorm + bonus + gate to the WKV7 output the scan
// left in y_wkv (kept, bf16, for the backward pass; centred per block when `centers` is given, see ln_epilogue.hpp).
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ln_epilogue_kernel(int T, int H, int nchunks, const __bf16* __restrict__ y_wkv,
                                                          const float* __restrict__ centers, const __bf16* __restrict__ q_, const __bf16* __restrict__ k_,
                                                          const __bf16* __restrict__ v_, const __bf16* __restrict__ g_,
                                                          const float* __restrict__ params, __bf16* __restrict__ y_) {
    const int wid = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wid >= nchunks) return;
    const int cid = H >= 16 ? head_major_chunk(wid, nchunks, T) : wid;   // (long rows: see head_major_chunk)
    const Lane L;
    const ChunkAddr ca(cid, T, H);
    const TileB yw = load_rows16(y_wkv + ca.row0, ca.ld, L);
    const TileB q = load_rows16(q_ + ca.row0, ca.ld, L);
    const TileB k = load_rows16(k_ + ca.row0, ca.ld, L);
    const TileB v = load_rows16(v_ + ca.row0, ca.ld, L);
    const TileB g = load_rows16(g_ + ca.row0, ca.ld, L);
    const LnParams p = load_ln_params(params, ca.bh % H, H, L);
    const TileF yf = uncentre(yw, centers, ca.row0 / HEAD + (long)L.n * H);   // (row0 / 64 = token * H + head of the chunk's first token)
    store_rows16(y_ + ca.row0, ca.ld, L, ln_forward(yf, q, k, v, g, p));
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
// Segments per (batch, head) for long sequences on few heads: a power of two, at most 8, that spreads the (batch, head)s
// over an MI355X's 256 compute units, with at least 32 chunks per segment; 1 = the whole sequence in one block (or two).
// A segmented pass is two launches of the one-kernel organisation (wkv7_fused.hip: every segment's affine map, then
// the scan proper from the composed entering states) with the carry between them, so it costs twice a launch's fixed
// 11-14 us, the carry's 3 us per segment, and 1.2 us per chunk and segment instead of 0.55: below four segments
// it does not pay (measured forward+backward, 12 heads: 1024 tokens 133 us in two segments against 103 in one block).
// Four segments fit up to a quarter of the compute units' worth of (batch, head) pairs (64: 8192 tokens 876 -> 768 us,
// 60 pairs: 4096 tokens 459 -> 425 us, 2048 tokens 242 -> 246 us against the unsegmented kernel).
int scan_segments(int B, int T, int H) {
    const int BH = B * H, NC = T / CHUNK;
    int g = 1;
    while (g < 8 && BH * g * 2 <= compute_units() && NC % (g * 2) == 0 && NC / (g * 2) >= 32) g *= 2;
    return g >= 4 ? g : 1;
}
size_t scan_segment_workspace_bytes(int B, int T, int H) {
    const int g = scan_segments(B, T, H);
    return g == 1 ? 0 : (size_t)B * H * g * 3 * HEAD * HEAD * sizeof(float);   // N, M^T and the entering state per segment
}

void launch_segment_carry(int BH, int nseg, int state_f32, const void* s_in, const float* maps, float* s_seg,
                          hipStream_t stream) {
    hipLaunchKernelGGL(segment_carry_kernel, dim3(4 * BH), dim3(256), 0, stream, nseg, state_f32, s_in, maps, s_seg);
}

void launch_ln_epilogue(int B, int T, int H, const void* y_wkv, const float* centers, const void* q, const void* k,
                        const void* v, const void* g, const void* params, void* y, hipStream_t stream) {
    const int nchunks = B * H * (T / CHUNK);
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    hipLaunchKernelGGL(ln_epilogue_kernel, dim3((nchunks + 3) / 4), dim3(256), 0, stream, T, H, nchunks, c(y_wkv), centers, c(q),
                       c(k), c(v), c(g), static_cast<const float*>(params), static_cast<__bf16*>(y));
}

}  // namespace wkv
