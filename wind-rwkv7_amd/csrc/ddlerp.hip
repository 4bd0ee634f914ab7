// ddlerp: data-dependent token-shift interpolation of RWKV-7, forward and backward, for gfx950.
//
// Replaces the six Triton kernels of the reference (rwkv7_ddlerp.py: fw1 :20-49, fw2 :53-84, bw1 :93-139,
// bw2 :143-167, bw3 :189-265, bw4 :269-303).  Spec (tests/test_ddlerp.py:5-13), per token m = (b, t):
//     xx   = x[t-1] - x[t]                       (zero row before t = 0)
//     a    = x + xx * alpha                       [C]
//     bmid = tanh(a L^T)                          [4D]      L: [4D, C]
//     c_k  = bmid_k R_k^T + beta_k                [C]       R: [4, C, D], k = 0..3
//     y_k  = x + xx * c_k
// The work is bandwidth-bound (x in, four streams out), but its inner products (C x 4D and 4D x C per
// token) only stay off the critical path on the matrix cores, so every contraction is a 16x16x32 MFMA on
// fragments (see frag.hpp): token tiles of 16 rows, channel blocks of 64.
#include "frag.hpp"
#include "device_info.hpp"
#include "ddlerp_kernels.hpp"
#include <type_traits>

namespace wkv {

namespace {

constexpr int TOK = 16;  // tokens per tile

struct Dy4 {  // the four upstream gradients, each [M, C]
    const __bf16* p[4];
};

// x tile and its token-shifted difference for 16 tokens x 64 channels starting at channel c0.
struct XTile {
    TileF x, xx;
};
__device__ __forceinline__ XTile load_x_tile(const __bf16* __restrict__ x, long m0, int T, int C, int c0, const Lane& L) {
    XTile r;
    const long m = m0 + L.n;
    const bool has_prev = (m % T) != 0;
    // 16-byte accesses: blocks 2p and 2p+1 of the tile are the interleaved channels of chan16 (frag.hpp); every
    // per-channel operand of these kernels is indexed through the same map
    const __bf16* row = x + m * C + c0 + 8 * L.g;
#pragma unroll
    for (int pr = 0; pr < NBLK / 2; pr++) {
        const bf16x8 cur = *reinterpret_cast<const bf16x8*>(row + 32 * pr);
        bf16x8 prev = {};
        if (has_prev) prev = *reinterpret_cast<const bf16x8*>(row - C + 32 * pr);
#pragma unroll
        for (int hlf = 0; hlf < 2; hlf++) {
            const f32x4 c = to_f32(hlf ? __builtin_shufflevector(cur, cur, 4, 5, 6, 7) : __builtin_shufflevector(cur, cur, 0, 1, 2, 3));
            const f32x4 q = to_f32(hlf ? __builtin_shufflevector(prev, prev, 4, 5, 6, 7) : __builtin_shufflevector(prev, prev, 0, 1, 2, 3));
            r.x.f[2 * pr + hlf] = c;
            r.xx.f[2 * pr + hlf] = q - c;
        }
    }
    return r;
}
}  // namespace

// ------------------------------------------------------------------------------------------------
// The two contractions over all C channels (forward 1 and backward 1) give a block TPB token tiles (16 tokens
// each) and walk the channel blocks: the weight fragments of a channel block (16 KiB) are loaded once per block,
// passed through a double-buffered LDS image in matrix-instruction order (one barrier per channel block), and
// each tile is finished by 4 / TPB wavefronts, which split the output blocks.  A tile per block with the channel
// contraction split over its wavefronts, as a first version had it, fetched the whole 196 KiB of weights from
// L2 for every 16 tokens (1.6x the streamed bytes at C = 768) and needed a cross-wavefront reduction.
// ------------------------------------------------------------------------------------------------
template <int NB>
struct MidWeights {   // LDS image of the weights of one 64-channel block: [output block][channel pair][lane]
    bf16x8 f[2][NB][2][WAVE];
};
// wavefront w loads output blocks 2w, 2w+1 of W[16 db .., c0 ..] (row stride C) as fragment pairs
template <int NB>
__device__ __forceinline__ void load_mid_weights(bf16x8 (&r)[NB / 4][2], const __bf16* __restrict__ W, int C, int c0,
                                                 int wave, const Lane& L) {
#pragma unroll
    for (int i = 0; i < NB / 4; i++) {
        const TileB t = load_rows16(W + (long)(16 * (wave * (NB / 4) + i)) * C + c0, C, L);
        r[i][0] = __builtin_shufflevector(t.f[0], t.f[1], 0, 1, 2, 3, 4, 5, 6, 7);
        r[i][1] = __builtin_shufflevector(t.f[2], t.f[3], 0, 1, 2, 3, 4, 5, 6, 7);
    }
}

// The same fragments of R^T ([4D, C], row kD+d) taken from R ([4, C, D]) itself: F(R_k[c.., 16j..]) is loaded with the
// channels on the lanes (8 contiguous bytes each, raw registers) and transposed on the matrix cores when it is used.
template <int NB, int D>
__device__ __forceinline__ void load_r_fragments(bf16x4 (&raw)[NB / 4][NBLK], const __bf16* __restrict__ R, int C, int c0,
                                                 int wave, const Lane& L) {
#pragma unroll
    for (int i = 0; i < NB / 4; i++) {
        const int ob = wave * (NB / 4) + i, k = ob / (D / 16), j = ob % (D / 16);
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++)
            raw[i][cb] = *reinterpret_cast<const bf16x4*>(R + ((long)k * C + c0 + chan16(cb, L.n)) * D + 16 * j + 4 * L.g);
    }
}

// forward 1: bmid = tanh((x + xx*alpha) L^T), bder = 1 - bmid^2
template <int D, int TPB>
__global__ __launch_bounds__(256) void ddlerp_fwd_mid_kernel(long M, int T, int C, const __bf16* __restrict__ x,
                                                             const __bf16* __restrict__ alpha,
                                                             const __bf16* __restrict__ Lw, __bf16* __restrict__ bmid,
                                                             __bf16* __restrict__ bder) {
    constexpr int NB = 4 * D / 16;       // output blocks of 16
    constexpr int WPT = 4 / TPB;         // wavefronts per tile
    constexpr int NBW = NB / WPT;        // output blocks per wavefront
    __shared__ MidWeights<NB> w;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    const long ntiles = M / TOK;
    const long tile_raw = (long)blockIdx.x * TPB + wave / WPT;
    const bool live = tile_raw < ntiles;
    const long m0 = (live ? tile_raw : ntiles - 1) * TOK;   // a spare wavefront repeats the last tile and stores nothing
    const int db0 = (wave % WPT) * NBW;

    f32x4 acc[NBW];
#pragma unroll
    for (int i = 0; i < NBW; i++) acc[i] = zero4();
    // Blocks start at different channel blocks: all of them asking for the same 16 KiB of weights at the same
    // moment queue on the few L2 channels that hold it.
    const int ncb = C / 64;
    auto advance = [&](int c) { return c + 1 < ncb ? c + 1 : 0; };
    // Two sets of streamed operands (weights, x rows, alpha), each refilled right after the round that used it, so
    // a load has two rounds to arrive.  The operands stay raw registers until the round that uses them: a
    // conversion at the point of the load, or a load under a condition, makes the compiler wait for the data
    // right there (8192 tokens: 24 -> 18 us with raw operands one round ahead, 17 us two rounds ahead; with every
    // operand cache-resident the same instructions take 13.5 us, so what is left is the rounds themselves).
    struct Set {
        bf16x8 wr[NB / 4][2];
        bf16x8 xc[NBLK / 2], xp[NBLK / 2];
        bf16x4 al[NBLK];
    };
    const bool has_prev = ((m0 + L.n) % T) != 0;
    auto fetch = [&](Set& st, int cbk) {
        const int c0 = 64 * cbk;
        load_mid_weights<NB>(st.wr, Lw, C, c0, wave, L);
        const __bf16* row = x + (m0 + L.n) * C + c0 + 8 * L.g;
        const __bf16* prow = has_prev ? row - C : row;
#pragma unroll
        for (int pr = 0; pr < NBLK / 2; pr++) {
            st.xc[pr] = *reinterpret_cast<const bf16x8*>(row + 32 * pr);
            st.xp[pr] = *reinterpret_cast<const bf16x8*>(prow + 32 * pr);
        }
#pragma unroll
        for (int i = 0; i < NBLK; i++) st.al[i] = *reinterpret_cast<const bf16x4*>(alpha + c0 + chan16(i, 4 * L.g));
    };
    int next_cb = blockIdx.x % ncb;
    Set sa, sb;
    fetch(sa, next_cb);
    next_cb = advance(next_cb);
    fetch(sb, next_cb);
    next_cb = advance(next_cb);
    auto round = [&](Set& st, int buf) {
#pragma unroll
        for (int i = 0; i < NB / 4; i++) {
            w.f[buf][wave * (NB / 4) + i][0][lane] = st.wr[i][0];
            w.f[buf][wave * (NB / 4) + i][1][lane] = st.wr[i][1];
        }
        __syncthreads();
        // a = x + xx*alpha as a bf16 pair (hi + lo): the pre-activation feeds tanh', which is steep, so the
        // interpolated input must not be rounded to 8 bits before the 768-term sum (L itself is bf16)
        bf16x8 a[2], alo[2];
#pragma unroll
        for (int pr = 0; pr < NBLK / 2; pr++) {
            const bf16x8 zero = {};
            const bf16x8 prev = has_prev ? st.xp[pr] : zero;
            f32x4 av[2];
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) {
                const f32x4 c = to_f32(hlf ? __builtin_shufflevector(st.xc[pr], st.xc[pr], 4, 5, 6, 7)
                                           : __builtin_shufflevector(st.xc[pr], st.xc[pr], 0, 1, 2, 3));
                const f32x4 q = to_f32(hlf ? __builtin_shufflevector(prev, prev, 4, 5, 6, 7) : __builtin_shufflevector(prev, prev, 0, 1, 2, 3));
                av[hlf] = c + (q - c) * to_f32(st.al[2 * pr + hlf]);
            }
            const bf16x4 h0 = to_bf16(av[0]), h1 = to_bf16(av[1]);
            a[pr] = __builtin_shufflevector(h0, h1, 0, 1, 2, 3, 4, 5, 6, 7);
            alo[pr] = __builtin_shufflevector(to_bf16(av[0] - to_f32(h0)), to_bf16(av[1] - to_f32(h1)), 0, 1, 2, 3, 4, 5, 6, 7);
        }
        fetch(st, next_cb);   // (the last two rounds fetch blocks that are not used)
        next_cb = advance(next_cb);
#pragma unroll
        for (int i = 0; i < NBW; i++) {
            const bf16x8 l0 = w.f[buf][db0 + i][0][lane], l1 = w.f[buf][db0 + i][1][lane];   // F(L[16db.., c0..]) lane = output
            acc[i] = mma8(acc[i], l0, a[0]);                                                     // + F(a L^T) lane = token
            acc[i] = mma8(acc[i], l1, a[1]);
            acc[i] = mma8(acc[i], l0, alo[0]);
            acc[i] = mma8(acc[i], l1, alo[1]);
        }
    };
    int it = 0;
    for (; it + 2 <= ncb; it += 2) {
        round(sa, 0);
        round(sb, 1);
    }
    if (it < ncb) round(sa, 0);
    if (!live) return;
#pragma unroll
    for (int i = 0; i < NBW; i++) {
        // tanh and its derivative 1 - tanh^2 = 4e/(e+1)^2, e = exp(2s).  The derivative is stored on its own:
        // recovering it from a bf16-rounded tanh loses all precision where the unit saturates.
        f32x4 t, dt;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float e = __expf(2.f * fminf(acc[i][r], 40.f));
            const float inv = __builtin_amdgcn_rcpf(e + 1.f);   // 1 ulp; an IEEE division is ten instructions
            t[r] = 1.f - 2.f * inv;
            dt[r] = 4.f * e * inv * inv;
        }
        const long off = (m0 + L.n) * (4 * D) + 16 * (db0 + i) + 4 * L.g;
        *reinterpret_cast<bf16x4*>(bmid + off) = to_bf16(t);
        *reinterpret_cast<bf16x4*>(bder + off) = to_bf16(dt);
    }
}

// ------------------------------------------------------------------------------------------------
// backward 1: dpre = ((dy_k * xx) R_k) * (1 - bmid^2)        [M, 4D]   (the factor 1 - bmid^2 was saved by forward)
// Same structure as forward 1; the weights are R^T ([4D, C], output block k*D/16 + j), transposed from R on the way
// into LDS.
// ------------------------------------------------------------------------------------------------
template <int D, int TPB>
__global__ __launch_bounds__(256) void ddlerp_bwd_mid_kernel(long M, int T, int C, const __bf16* __restrict__ x,
                                                             Dy4 dy,
                                                             const __bf16* __restrict__ R,
                                                             const __bf16* __restrict__ bder,
                                                             __bf16* __restrict__ dpre) {
    constexpr int ND = D / 16, NB = 4 * ND;
    constexpr int WPT = 4 / TPB, NBW = NB / WPT;
    static_assert(NBW % ND == 0, "a wavefront owns whole interpolations k");
    __shared__ MidWeights<NB> w;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    const long ntiles = M / TOK;
    const long tile_raw = (long)blockIdx.x * TPB + wave / WPT;
    const bool live = tile_raw < ntiles;
    const long m0 = (live ? tile_raw : ntiles - 1) * TOK;
    const int db0 = (wave % WPT) * NBW, k0 = db0 / ND;

    f32x4 acc[NBW];
#pragma unroll
    for (int i = 0; i < NBW; i++) acc[i] = zero4();
    struct Loads {
        bf16x8 xc[NBLK / 2], xp[NBLK / 2], dy[NBW / ND][NBLK / 2];
    };
    auto issue = [&](int c0) {
        Loads ld;
        const long m = m0 + L.n;
        const __bf16* row = x + m * C + c0 + 8 * L.g;
        const __bf16* prow = (m % T) != 0 ? row - C : row;
#pragma unroll
        for (int pr = 0; pr < NBLK / 2; pr++) {
            ld.xc[pr] = *reinterpret_cast<const bf16x8*>(row + 32 * pr);
            ld.xp[pr] = *reinterpret_cast<const bf16x8*>(prow + 32 * pr);
        }
#pragma unroll
        for (int k = 0; k < NBW / ND; k++)
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; pr++)
                ld.dy[k][pr] = *reinterpret_cast<const bf16x8*>(dy.p[k0 + k] + m * C + c0 + 8 * L.g + 32 * pr);
        return ld;
    };
    const bool has_prev = ((m0 + L.n) % T) != 0;
    const bf16x4 eye = identity_bf16(L);
    bf16x4 wr[NB / 4][NBLK];
    load_r_fragments<NB, D>(wr, R, C, 0, wave, L);
    Loads cur = issue(0);
    for (int c0 = 0, it = 0; c0 < C; c0 += 64, it++) {
        const int buf = it & 1;
#pragma unroll
        for (int i = 0; i < NB / 4; i++) {
            bf16x4 t[NBLK];
#pragma unroll
            for (int cb = 0; cb < NBLK; cb++) t[cb] = transpose(wr[i][cb], eye);
            w.f[buf][wave * (NB / 4) + i][0][lane] = __builtin_shufflevector(t[0], t[1], 0, 1, 2, 3, 4, 5, 6, 7);
            w.f[buf][wave * (NB / 4) + i][1][lane] = __builtin_shufflevector(t[2], t[3], 0, 1, 2, 3, 4, 5, 6, 7);
        }
        const int cn = c0 + 64 < C ? c0 + 64 : c0;
        load_r_fragments<NB, D>(wr, R, C, cn, wave, L);
        const Loads nxt = issue(cn);
        __syncthreads();
        f32x4 xx[NBLK];
#pragma unroll
        for (int pr = 0; pr < NBLK / 2; pr++) {
            const bf16x8 zero = {};
            const bf16x8 prev = has_prev ? cur.xp[pr] : zero;
            xx[2 * pr] = to_f32(__builtin_shufflevector(prev, prev, 0, 1, 2, 3)) -
                         to_f32(__builtin_shufflevector(cur.xc[pr], cur.xc[pr], 0, 1, 2, 3));
            xx[2 * pr + 1] = to_f32(__builtin_shufflevector(prev, prev, 4, 5, 6, 7)) -
                             to_f32(__builtin_shufflevector(cur.xc[pr], cur.xc[pr], 4, 5, 6, 7));
        }
#pragma unroll
        for (int k = 0; k < NBW / ND; k++) {
            bf16x8 dc[2];
#pragma unroll
            for (int pr = 0; pr < 2; pr++) {
                const bf16x8 d = cur.dy[k][pr];
                dc[pr] = __builtin_shufflevector(to_bf16(to_f32(__builtin_shufflevector(d, d, 0, 1, 2, 3)) * xx[2 * pr]),
                                                 to_bf16(to_f32(__builtin_shufflevector(d, d, 4, 5, 6, 7)) * xx[2 * pr + 1]),
                                                 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int j = 0; j < ND; j++) {
                const int i = k * ND + j;
                acc[i] = mma8(acc[i], w.f[buf][db0 + i][0][lane], dc[0]);   // + F(dc R_k) lane = token
                acc[i] = mma8(acc[i], w.f[buf][db0 + i][1][lane], dc[1]);
            }
        }
        cur = nxt;
    }
    if (!live) return;
#pragma unroll
    for (int i = 0; i < NBW; i++) {
        const long off = (m0 + L.n) * (4 * D) + 16 * (db0 + i) + 4 * L.g;
        *reinterpret_cast<bf16x4*>(dpre + off) = to_bf16(acc[i] * to_f32(*reinterpret_cast<const bf16x4*>(bder + off)));
    }
}

// ------------------------------------------------------------------------------------------------
// Forward 2 gives a block one 64-channel block and a range of token tiles: the block's 16 KiB of weight
// fragments (R) are staged in LDS once, in the order the matrix instructions take them (16 bytes per lane per
// pair), and every wavefront walks its tiles.  Fetching the fragments per tile from memory in the middle of
// dependent arithmetic, as a tile-per-wavefront kernel must, left the kernel waiting for loads most of the time.
// ------------------------------------------------------------------------------------------------
template <int D>
struct LerpWeights {   // LDS image for one 64-channel block
    static constexpr int ND = D / 16;
    bf16x8 R[4][NBLK][ND / 2][WAVE];   // (F(R_k[c.., 16j..]), F(R_k[c.., 16j+16..]))  lane = channel, reg = d
    float beta[4][64];
};
template <int D>
__device__ __forceinline__ void stage_lerp_weights(LerpWeights<D>& w, const __bf16* __restrict__ R,
                                                   const __bf16* __restrict__ beta, int C, int c0) {
    constexpr int ND = D / 16;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    // wavefront k stages R_k
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) {
        const long ch = c0 + chan16(cb, L.n);
#pragma unroll
        for (int j = 0; j < ND / 2; j++) {
            const __bf16* rrow = R + ((long)wave * C + ch) * D + 32 * j + 4 * L.g;
            w.R[wave][cb][j][lane] = __builtin_shufflevector(*reinterpret_cast<const bf16x4*>(rrow),
                                                             *reinterpret_cast<const bf16x4*>(rrow + 16), 0, 1, 2, 3, 4, 5, 6, 7);
        }
    }
    w.beta[wave][lane] = (float)beta[(long)wave * C + c0 + lane];
}
// this lane's mid-index fragments of one token row (bmid or dpre), as pairs
template <int NPAIR>
__device__ __forceinline__ void load_mid_pairs(bf16x8 (&out)[NPAIR], const __bf16* __restrict__ row, const Lane& L) {
#pragma unroll
    for (int j = 0; j < NPAIR; j++)
        out[j] = __builtin_shufflevector(*reinterpret_cast<const bf16x4*>(row + 32 * j + 4 * L.g),
                                         *reinterpret_cast<const bf16x4*>(row + 32 * j + 16 + 4 * L.g), 0, 1, 2, 3, 4, 5, 6, 7);
}

// forward 2: y_k = x + xx * (bmid_k R_k^T + beta_k).  Block = (64 channels, range of token tiles).
template <int D>
__global__ __launch_bounds__(256) void ddlerp_fwd_out2_kernel(long M, int T, int C, int tiles_per_split,
                                                              const __bf16* __restrict__ x, const __bf16* __restrict__ R,
                                                              const __bf16* __restrict__ beta,
                                                              const __bf16* __restrict__ bmid, __bf16* __restrict__ y) {
    constexpr int ND = D / 16;
    __shared__ LerpWeights<D> w;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    const int c0 = blockIdx.x * 64;
    const long ntiles = M / TOK;
    const long tile_begin = (long)blockIdx.y * tiles_per_split;
    const long tile_end = tile_begin + tiles_per_split < ntiles ? tile_begin + tiles_per_split : ntiles;
    stage_lerp_weights<D>(w, R, beta, C, c0);
    __syncthreads();
    for (long tile = tile_begin + wave; tile < tile_end; tile += 4) {
        const long m0 = tile * TOK;
        const XTile xt = load_x_tile(x, m0, T, C, c0, L);
        bf16x8 bm[4 * ND / 2];
        load_mid_pairs(bm, bmid + (m0 + L.n) * (4 * D), L);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            TileB out;
#pragma unroll
            for (int cb = 0; cb < NBLK; cb++) {
                f32x4 c = *reinterpret_cast<const f32x4*>(&w.beta[k][chan16(cb, 4 * L.g)]);
#pragma unroll
                for (int j = 0; j < ND / 2; j++) c = mma8(c, w.R[k][cb][j][lane], bm[k * (ND / 2) + j]);
                out.f[cb] = to_bf16(xt.x.f[cb] + xt.xx.f[cb] * c);
            }
            store_rows16(y + ((long)k * M + m0) * C + c0, C, L, out);
        }
    }
}

// backward 2: everything that walks the tokens a second time, in one pass: dx and the parameter gradients.
//   da  = dpre L ;  dxx = da*alpha + sum_k dy_k*c_k ;  dx[t] = da + sum_k dy_k - dxx[t] + dxx[t+1]
//   dR_k = (dy_k*xx)^T bmid_k,  dbeta_k = sum_t dy_k*xx,  dL = dpre^T a,  dalpha = sum_t da*xx
// Block = (64 channels, a contiguous range of token tiles); each of its four wavefronts owns 16 of the channels for
// the whole range and never meets the others: it reads its 8-byte pieces of x, x[t-1] and the four dy rows, the full
// 256-byte rows of bmid and dpre (16 bytes per lane), and keeps dR[:, its channels, :], dL[:, its channels] and the
// two vectors in registers.  The tiles are walked from the last one down, so the shifted term of the tile above is
// the carry; only the first tile a wavefront touches has none, and when the token after the range continues the
// sequence the wavefront evaluates that tile first without storing or accumulating anything.
// The contraction index of a 32-wide product may be permuted at will as long as both operands agree, so a lane
// group g holds mid indices 8g .. 8g+7 of each interpolation (one 16-byte load); as two 16-wide fragments that is
// index dmap(jj, 4g + r), and the transposed fragments and the accumulators built from them carry the same map.
// (Separate kernels for dx, for dR/dbeta and for dL/dalpha read x three times and dy twice at one wavefront per
// SIMD, 98 us together at 8192 tokens x 768 channels.  One wavefront per interpolation k instead of per channel
// group repeated the x arithmetic four times and added four partial dx tiles through LDS: 47 us.  This
// organisation with every wavefront loading its own pieces from memory: 58 us, bound by the L2-to-CU traffic of
// quarter-used lines; with the shared LDS images: 35 us, of which about 30 are the arithmetic.)
template <int D>
struct ParamPartial {   // per (split, 64-channel block); element counts
    static constexpr int DR = 4 * 64 * D, DL = 4 * D * 64, DBETA = 4 * 64, DALPHA = 64;
    static constexpr int TOTAL = DR + DL + DBETA + DALPHA;
};
__host__ __device__ constexpr int dmap(int jj, int j) { return 8 * (j >> 2) + 4 * jj + (j & 3); }

template <int D>
__global__ __launch_bounds__(256, D == 32 ? 2 : 1) void ddlerp_bwd_main_kernel(long M, int T, int C, int tiles_per_split,
                                                                 const __bf16* __restrict__ x, Dy4 dy,
                                                                 const __bf16* __restrict__ alpha,
                                                                 const __bf16* __restrict__ Lw,
                                                                 const __bf16* __restrict__ R,
                                                                 const __bf16* __restrict__ beta,
                                                                 const __bf16* __restrict__ bmid,
                                                                 const __bf16* __restrict__ dpre,
                                                                 __bf16* __restrict__ dx, float* __restrict__ partial) {
    static_assert(D % 32 == 0 && D <= 64, "32-wide contractions, HH of them per interpolation");
    using P = ParamPartial<D>;
    constexpr int HH = D / 32;
    // Each wavefront's own weight fragments, [k][32-wide half]: 8 KiB in LDS at rank 32 ([wavefront][k][lane]); at
    // rank 64 the streamed images below leave no room for 16 KiB per wavefront and they stay in registers.
    constexpr bool W_LDS = HH == 1;
    __shared__ bf16x8 s_R[W_LDS ? 4 : 1][W_LDS ? 4 : 1][W_LDS ? WAVE : 1], s_L[W_LDS ? 4 : 1][W_LDS ? 4 : 1][W_LDS ? WAVE : 1];
    bf16x8 r_R[W_LDS ? 1 : 4][HH], r_L[W_LDS ? 1 : 4][HH];
    // LDS images of a tile's streamed rows (elements; row pitches padded by 16 bytes against bank conflicts)
    constexpr int ROW_LD = 64 + 8, MID_LD = 4 * D + 8;
    __shared__ __attribute__((aligned(16))) __bf16 s_x[2][17 * ROW_LD], s_row[2][4][16 * ROW_LD], s_mid[2][2][16 * MID_LD];
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const Lane L;
    const int cw = blockIdx.x * 64 + 16 * w;   // this wavefront's channel j is cw + j
    const long ntiles = M / TOK;
    const long lo = (long)blockIdx.y * tiles_per_split;
    const long hi = lo + tiles_per_split < ntiles ? lo + tiles_per_split : ntiles;
    const bf16x4 eye = identity_bf16(L);
    const int cl = cw + 4 * L.g;          // the four contiguous channels of this lane in token layout

    f32x4 al, be[4];
    al = to_f32(*reinterpret_cast<const bf16x4*>(alpha + cl));
#pragma unroll
    for (int k = 0; k < 4; k++) {
        be[k] = to_f32(*reinterpret_cast<const bf16x4*>(beta + (long)k * C + cl));
#pragma unroll
        for (int hh = 0; hh < HH; hh++) {
            // F(R_k[c.., 32hh ..]) lane = channel, mid indices 32hh + 8g .. 8g+7
            const bf16x8 fr = *reinterpret_cast<const bf16x8*>(R + ((long)k * C + cw + L.n) * D + 32 * hh + 8 * L.g);
            // L is [4D, C]: rows kD + 32hh + dmap(jj, n), four contiguous channels per lane, transposed on the matrix cores
            const bf16x8 fl = __builtin_shufflevector(
                transpose(*reinterpret_cast<const bf16x4*>(Lw + (long)(k * D + 32 * hh + dmap(0, L.n)) * C + cl), eye),
                transpose(*reinterpret_cast<const bf16x4*>(Lw + (long)(k * D + 32 * hh + dmap(1, L.n)) * C + cl), eye), 0, 1, 2, 3, 4, 5, 6, 7);
            if constexpr (W_LDS) {
                s_R[w][k][lane] = fr;
                s_L[w][k][lane] = fl;
            } else {
                r_R[k][hh] = fr;
                r_L[k][hh] = fl;
            }
        }
    }
    // F(dR_k[c.., 32hh + dmap(jj, .)]) lane = channel;  F(dL[kD + 32hh + dmap(jj, .), c..]) lane = mid index; [k][2hh + jj]
    f32x4 accR[4][2 * HH], accL[4][2 * HH];
    f32x4 vbeta[4], valpha = zero4();   // per-token partial sums, lane = token
    f32x4 carry = zero4();              // lane 15: the shifted term of the first token of the tile above
#pragma unroll
    for (int k = 0; k < 4; k++) {
        vbeta[k] = zero4();
#pragma unroll
        for (int j = 0; j < 2 * HH; j++) accR[k][j] = accL[k][j] = zero4();
    }
    if (lo >= hi) return;   // (cannot happen with the launcher's ranges)

    // The streamed operands of a tile - 17 rows of x (one above the tile), 16 rows of each dy, of bmid and of dpre,
    // 18 KiB - are fetched ONCE per block with full 128-byte lines (16 bytes per thread, five loads each), parked in
    // registers for a tile, and written to one of two LDS images from which the wavefronts take their pieces.
    // (Each wavefront fetching its own 32-byte pieces of the rows, and all four the same rows of bmid and dpre,
    // moved four times the bytes between L2 and the compute units and ran at the rate of that link.)
    const int t = threadIdx.x;
    auto stage_tile = [&](long tile) { return tile < lo ? lo : tile; };   // (past the range: loaded and never used)
    // bmid / dpre: 16 rows of 4D elements, 8 per thread and pass, HH passes
    auto mid_row = [&](int ps) { return (8 * t + 2048 * ps) / (4 * D); };
    auto mid_col = [&](int ps) { return (8 * t + 2048 * ps) % (4 * D); };
    const int row_thread = ((t & 127) >> 3) * C + blockIdx.x * 64 + 8 * (t & 7);   // dy: 8 threads per row, two arrays per pass
    const __bf16* __restrict__ dya = t < 128 ? dy.p[0] : dy.p[1];
    const __bf16* __restrict__ dyb = t < 128 ? dy.p[2] : dy.p[3];
    const int xrow = (t >> 3) - 1;                                       // x: rows -1 .. 15, threads 0 .. 135
    bf16x8 g_bm[HH], g_dp[HH], g_dya, g_dyb, g_x;
    auto fetch = [&](long tile) {
        tile = stage_tile(tile);
        const long m0 = tile * TOK;
#pragma unroll
        for (int ps = 0; ps < HH; ps++) {
            g_bm[ps] = *reinterpret_cast<const bf16x8*>(bmid + m0 * (4 * D) + 8 * t + 2048 * ps);
            g_dp[ps] = *reinterpret_cast<const bf16x8*>(dpre + m0 * (4 * D) + 8 * t + 2048 * ps);
        }
        g_dya = *reinterpret_cast<const bf16x8*>(dya + m0 * C + row_thread);
        g_dyb = *reinterpret_cast<const bf16x8*>(dyb + m0 * C + row_thread);
        if (t < 17 * 8) {
            const long m = m0 + xrow > 0 ? m0 + xrow : 0;   // (the row above token 0 is masked at the use)
            g_x = *reinterpret_cast<const bf16x8*>(x + m * C + blockIdx.x * 64 + 8 * (t & 7));
        }
    };
    auto park = [&](int buf) {
#pragma unroll
        for (int ps = 0; ps < HH; ps++) {
            *reinterpret_cast<bf16x8*>(&s_mid[buf][0][mid_row(ps) * MID_LD + mid_col(ps)]) = g_bm[ps];
            *reinterpret_cast<bf16x8*>(&s_mid[buf][1][mid_row(ps) * MID_LD + mid_col(ps)]) = g_dp[ps];
        }
        *reinterpret_cast<bf16x8*>(&s_row[buf][t < 128 ? 0 : 1][((t & 127) >> 3) * ROW_LD + 8 * (t & 7)]) = g_dya;
        *reinterpret_cast<bf16x8*>(&s_row[buf][t < 128 ? 2 : 3][((t & 127) >> 3) * ROW_LD + 8 * (t & 7)]) = g_dyb;
        if (t < 17 * 8) *reinterpret_cast<bf16x8*>(&s_x[buf][(t >> 3) * ROW_LD + 8 * (t & 7)]) = g_x;
    };
    // One tile, out of LDS image buf.  tpos: position of its first token in the sequence.  KEEP = false is the
    // warm-up tile, which only produces the carry.
    auto body = [&](long tile, int tpos, int buf, auto keep_c) {
        constexpr bool KEEP = decltype(keep_c)::value;
        const bool has_prev = (tpos + L.n) != 0;
        const bool chain = tpos != 0;   // the tile below is followed by this tile's first token in the same sequence
        const int piece = 16 * w + 4 * L.g;
        const bf16x4 zero = {};
        const f32x4 xv = to_f32(*reinterpret_cast<const bf16x4*>(&s_x[buf][(L.n + 1) * ROW_LD + piece]));
        const bf16x4 xp = *reinterpret_cast<const bf16x4*>(&s_x[buf][L.n * ROW_LD + piece]);
        const f32x4 xxv = to_f32(has_prev ? xp : zero) - xv;
        bf16x4 aT;
        if constexpr (KEEP) aT = transpose(to_bf16(xv + xxv * al), eye);   // F(a^T) lane = channel
        f32x4 da = zero4(), dxx = zero4(), dxd = zero4();
#pragma unroll
        for (int k = 0; k < 4; k++) {
            bf16x8 bm[HH], dp[HH];
            f32x4 c = be[k];
#pragma unroll
            for (int hh = 0; hh < HH; hh++) {
                bm[hh] = *reinterpret_cast<const bf16x8*>(&s_mid[buf][0][L.n * MID_LD + k * D + 32 * hh + 8 * L.g]);
                dp[hh] = *reinterpret_cast<const bf16x8*>(&s_mid[buf][1][L.n * MID_LD + k * D + 32 * hh + 8 * L.g]);
                bf16x8 fr, fl;
                if constexpr (W_LDS) {
                    fr = s_R[w][k][lane];
                    fl = s_L[w][k][lane];
                } else {
                    fr = r_R[k][hh];
                    fl = r_L[k][hh];
                }
                c = mma8(c, fr, bm[hh]);     // F(c_k) lane = token, reg = channel
                da = mma8(da, fl, dp[hh]);   // F(dpre L)
            }
            const f32x4 d = to_f32(*reinterpret_cast<const bf16x4*>(&s_row[buf][k][L.n * ROW_LD + piece]));
            dxx += d * c;
            dxd += d;
            if constexpr (KEEP) {
                const f32x4 dc = d * xxv;
                vbeta[k] += dc;
                const bf16x4 dcT = transpose(to_bf16(dc), eye);   // F(dc^T) lane = channel, reg = token
                // F(bmid_k^T), F(dpre_k^T) halves: lane = mid index 32hh + dmap(jj, n), reg = token
#pragma unroll
                for (int hh = 0; hh < HH; hh++) {
                    accR[k][2 * hh] = mma(accR[k][2 * hh], transpose(__builtin_shufflevector(bm[hh], bm[hh], 0, 1, 2, 3), eye), dcT);   // + F(dc^T bmid_k)
                    accR[k][2 * hh + 1] = mma(accR[k][2 * hh + 1], transpose(__builtin_shufflevector(bm[hh], bm[hh], 4, 5, 6, 7), eye), dcT);
                    accL[k][2 * hh] = mma(accL[k][2 * hh], aT, transpose(__builtin_shufflevector(dp[hh], dp[hh], 0, 1, 2, 3), eye));    // + F(dpre_k^T a)
                    accL[k][2 * hh + 1] = mma(accL[k][2 * hh + 1], aT, transpose(__builtin_shufflevector(dp[hh], dp[hh], 4, 5, 6, 7), eye));
                }
            }
        }
        dxx += da * al;
        dxd += da;
        f32x4 o;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float rot = row_rot<1>(dxx[r]);   // token n+1's term; lane 15 gets the tile's first token
            o[r] = dxd[r] - dxx[r] + (L.n < TOK - 1 ? rot : carry[r]);
            carry[r] = chain ? rot : 0.f;
        }
        if constexpr (KEEP) {
            *reinterpret_cast<bf16x4*>(dx + (tile * TOK + L.n) * C + cl) = to_bf16(o);
            valpha += da * xxv;
        }
    };
    int tpos = (int)(((hi - 1) * TOK) % T);
    const bool warm = hi < ntiles && tpos + TOK != T;   // the token after the range continues the sequence
    // Iteration i works on image i&1 while the registers hold the tile after it, fetched during iteration i-1; they
    // are written to the other image (last read before the previous barrier) and refilled for the tile after that.
    long next = warm ? hi : hi - 1;   // the tile the registers are fetched for
    fetch(next);
    park(0);
    fetch(--next);
    __syncthreads();
    int it = 0;
    if (warm) {
        park(1);
        fetch(--next);
        body(hi, tpos + TOK, 0, std::false_type{});
        __syncthreads();
        it = 1;
    }
    for (long tile = hi - 1; tile >= lo; tile--, it++) {
        park((it + 1) & 1);
        fetch(--next);
        body(tile, tpos, it & 1, std::true_type{});
        __syncthreads();
        tpos = tpos >= TOK ? tpos - TOK : T - TOK;
    }
    // this block's partial record: dR [4][64][D], dL [4D][64], dbeta [4][64], dalpha [64]
    float* out = partial + ((long)blockIdx.y * gridDim.x + blockIdx.x) * P::TOTAL;
    const int jw = 16 * w;   // first channel of this wavefront inside the block
#pragma unroll
    for (int k = 0; k < 4; k++) {
#pragma unroll
        for (int j = 0; j < 2 * HH; j++) {
            const int hh = j / 2, jj = j % 2;
            *reinterpret_cast<f32x4*>(out + (k * 64 + jw + L.n) * D + 32 * hh + dmap(jj, 4 * L.g)) = accR[k][j];
            *reinterpret_cast<f32x4*>(out + P::DR + (k * D + 32 * hh + dmap(jj, L.n)) * 64 + jw + 4 * L.g) = accL[k][j];
        }
        f32x4 sb;
#pragma unroll
        for (int r = 0; r < 4; r++) sb[r] = row_sum(vbeta[k][r]);
        if (L.n == 0) *reinterpret_cast<f32x4*>(out + P::DR + P::DL + k * 64 + jw + 4 * L.g) = sb;
    }
    f32x4 sa;
#pragma unroll
    for (int r = 0; r < 4; r++) sa[r] = row_sum(valpha[r]);
    if (L.n == 0) *reinterpret_cast<f32x4*>(out + P::DR + P::DL + P::DBETA + jw + 4 * L.g) = sa;
}

// sums the partial records over the token splits and scatters them to dR [4][C][D], dL [4D][C],
// dbeta [4][C], dalpha [C] (all fp32)
template <int D>
__global__ __launch_bounds__(256) void ddlerp_param_reduce_kernel(int C, int nsplit, const float* __restrict__ partial,
                                                                  float* __restrict__ dR, float* __restrict__ dL,
                                                                  float* __restrict__ dbeta,
                                                                  float* __restrict__ dalpha) {
    using P = ParamPartial<D>;
    const int ncb = C / 64;
    const int cblk = blockIdx.y;
    const int c0 = cblk * 64;
    const int e = 4 * (blockIdx.x * 256 + threadIdx.x);   // one thread per four elements of the record
    if (e >= P::TOTAL) return;
    // four running sums, so that four loads are in flight at a time; the order of the additions is fixed
    f32x4 s4[4] = {zero4(), zero4(), zero4(), zero4()};
    const float* src = partial + (long)cblk * P::TOTAL + e;
    const long pitch = (long)ncb * P::TOTAL;
    int sp = 0;
    for (; sp + 4 <= nsplit; sp += 4) {
#pragma unroll
        for (int u = 0; u < 4; u++) s4[u] += *reinterpret_cast<const f32x4*>(src + (sp + u) * pitch);
    }
    for (; sp < nsplit; sp++) s4[0] += *reinterpret_cast<const f32x4*>(src + sp * pitch);
    const f32x4 s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
    float* dst;
    if (e < P::DR) {
        const int d = e % D, c = (e / D) % 64, k = e / (64 * D);
        dst = dR + ((long)k * C + c0 + c) * D + d;
    } else if (e < P::DR + P::DL) {
        const int f = e - P::DR;
        const int c = f % 64, j = f / 64;
        dst = dL + (long)j * C + c0 + c;
    } else if (e < P::DR + P::DL + P::DBETA) {
        const int f = e - P::DR - P::DL;
        dst = dbeta + (long)(f / 64) * C + c0 + f % 64;
    } else {
        dst = dalpha + c0 + e - P::DR - P::DL - P::DBETA;
    }
    *reinterpret_cast<f32x4*>(dst) = s;
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
namespace {
constexpr size_t A256(size_t x) { return (x + 255) / 256 * 256; }
// Token ranges of the second backward pass: two blocks per compute unit of an MI355X (256) over the channel
// blocks, at least eight tiles each (every block spends one more tile on its carry and writes a 66 KiB record
// that the reduction reads back).
int param_splits(long M, int ncb) {
    const long ntiles = M / TOK;
    long s = ntiles / 8;
    const long cap = 2 * compute_units() / ncb > 0 ? 2 * compute_units() / ncb : 1;
    if (s > cap) s = cap;
    if (s < 1) s = 1;
    return (int)s;
}
// token-tile ranges of forward 2: a few blocks per compute unit of an MI355X (256) over the channel blocks, at
// least four tiles (one per wavefront) each
struct StreamSplit {
    int nsplit, tiles_per_split;
};
StreamSplit stream_splits(long M, int ncb, int slots) {   // slots: blocks the machine holds at once, times rounds
    const long ntiles = M / TOK;
    long s = slots / ncb > 0 ? slots / ncb : 1;
    if (s > ntiles / 4) s = ntiles / 4;
    if (s < 1) s = 1;
    return {(int)s, (int)((ntiles + s - 1) / s)};
}
}  // namespace

bool ddlerp_rank_supported(int D) { return D == 32 || D == 64; }

size_t ddlerp_bwd_workspace_bytes(long M, int C, int D) {
    const int ncb = C / 64;
    const size_t dpre = A256((size_t)M * 4 * D * 2);
    const size_t record = D == 64 ? ParamPartial<64>::TOTAL : ParamPartial<32>::TOTAL;
    const size_t partial = A256((size_t)param_splits(M, ncb) * ncb * record * 4);
    return dpre + partial;
}

namespace {
template <int D>
void forward_rank(long M, int T, int C, const void* x, const void* alpha, const void* Lw, const void* R, const void* beta,
                  void* bmid, void* bder, void* y, hipStream_t stream) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    // four tiles per block when that still gives every compute unit a block, else two
    const long ntiles = M / TOK;
    if (ntiles >= 4 * 256)
        hipLaunchKernelGGL((ddlerp_fwd_mid_kernel<D, 4>), dim3((unsigned)((ntiles + 3) / 4)), dim3(256), 0, stream, M, T, C,
                           c(x), c(alpha), c(Lw), static_cast<__bf16*>(bmid), static_cast<__bf16*>(bder));
    else
        hipLaunchKernelGGL((ddlerp_fwd_mid_kernel<D, 2>), dim3((unsigned)((ntiles + 1) / 2)), dim3(256), 0, stream, M, T, C,
                           c(x), c(alpha), c(Lw), static_cast<__bf16*>(bmid), static_cast<__bf16*>(bder));
    const StreamSplit sp = stream_splits(M, C / 64, 4 * compute_units());   // two blocks per compute unit, two rounds
    hipLaunchKernelGGL(ddlerp_fwd_out2_kernel<D>, dim3(C / 64, sp.nsplit), dim3(256), 0, stream, M, T, C, sp.tiles_per_split,
                       c(x), c(R), c(beta), c(bmid), static_cast<__bf16*>(y));
}

template <int D>
void backward_rank(long M, int T, int C, const void* x, const void* alpha, const void* Lw, const void* R, const void* beta,
                   const void* bmid, const void* bder, const void* const dy4[4], void* dx, void* dalpha, void* dL, void* dR,
                   void* dbeta, void* workspace, hipStream_t stream) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    const Dy4 dy{{c(dy4[0]), c(dy4[1]), c(dy4[2]), c(dy4[3])}};
    const int ncb = C / 64;
    char* p = static_cast<char*>(workspace);
    __bf16* dpre = reinterpret_cast<__bf16*>(p); p += A256((size_t)M * 4 * D * 2);
    float* partial = reinterpret_cast<float*>(p);
    const int tiles_per_split = (int)((M / TOK + param_splits(M, ncb) - 1) / param_splits(M, ncb));
    const int nsplit = (int)((M / TOK + tiles_per_split - 1) / tiles_per_split);   // no empty range: every block writes a record

    if (M / TOK >= 4 * 256)
        hipLaunchKernelGGL((ddlerp_bwd_mid_kernel<D, 4>), dim3((unsigned)((M / TOK + 3) / 4)), dim3(256), 0, stream, M, T, C,
                           c(x), dy, c(R), c(bder), dpre);
    else
        hipLaunchKernelGGL((ddlerp_bwd_mid_kernel<D, 2>), dim3((unsigned)((M / TOK + 1) / 2)), dim3(256), 0, stream, M, T, C,
                           c(x), dy, c(R), c(bder), dpre);
    hipLaunchKernelGGL(ddlerp_bwd_main_kernel<D>, dim3(ncb, nsplit), dim3(256), 0, stream, M, T, C, tiles_per_split, c(x), dy,
                       c(alpha), c(Lw), c(R), c(beta), c(bmid), dpre, static_cast<__bf16*>(dx), partial);
    hipLaunchKernelGGL(ddlerp_param_reduce_kernel<D>, dim3((ParamPartial<D>::TOTAL / 4 + 255) / 256, ncb), dim3(256), 0,
                       stream, C, nsplit, partial,
                       static_cast<float*>(dR), static_cast<float*>(dL), static_cast<float*>(dbeta),
                       static_cast<float*>(dalpha));
}
}  // namespace

// (the callers have checked ddlerp_rank_supported(D))
void launch_ddlerp_forward(long M, int T, int C, int D, const void* x, const void* alpha, const void* Lw, const void* R,
                           const void* beta, void* bmid, void* bder, void* y, hipStream_t stream) {
    if (D == 64) forward_rank<64>(M, T, C, x, alpha, Lw, R, beta, bmid, bder, y, stream);
    else forward_rank<32>(M, T, C, x, alpha, Lw, R, beta, bmid, bder, y, stream);
}

void launch_ddlerp_backward(long M, int T, int C, int D, const void* x, const void* alpha, const void* Lw, const void* R,
                            const void* beta, const void* bmid, const void* bder, const void* const dy4[4], void* dx,
                            void* dalpha,
                            void* dL, void* dR, void* dbeta, void* workspace, hipStream_t stream) {
    if (D == 64) backward_rank<64>(M, T, C, x, alpha, Lw, R, beta, bmid, bder, dy4, dx, dalpha, dL, dR, dbeta, workspace, stream);
    else backward_rank<32>(M, T, C, x, alpha, Lw, R, beta, bmid, bder, dy4, dx, dalpha, dL, dR, dbeta, workspace, stream);
}

}  // namespace wkv
