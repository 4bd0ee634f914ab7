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
#include "ddlerp_kernels.hpp"

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
// this lane's 16 channels (of the 64 starting at c0) of a per-channel bf16 vector
__device__ __forceinline__ TileF load_chan_vec(const __bf16* __restrict__ v, int c0, const Lane& L) {
    TileF r;
#pragma unroll
    for (int i = 0; i < NBLK; i++) r.f[i] = to_f32(*reinterpret_cast<const bf16x4*>(v + c0 + chan16(i, 4 * L.g)));
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
// transposed copies of the two weight matrices (tiny): RT[k][d][c] = R[k][c][d], LT[c][j] = L[j][c].
// ------------------------------------------------------------------------------------------------
__global__ void ddlerp_transpose_kernel(int C, int D, const __bf16* __restrict__ R, const __bf16* __restrict__ Lw,
                                        __bf16* __restrict__ RT, __bf16* __restrict__ LT) {
    const long n = 4L * C * D;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int d = i % D;
        const long kc = i / D;
        const int c = kc % C, k = kc / C;
        RT[((long)k * D + d) * C + c] = R[i];
        // L: [4D][C]; element i of L (row j = i / C, column cc = i % C)
        const int cc = i % C;
        const long j = i / C;
        LT[(long)cc * 4 * D + j] = Lw[i];
    }
}

// ------------------------------------------------------------------------------------------------
// backward 1: dpre = ((dy_k * xx) R_k) * (1 - bmid^2)        [M, 4D]   (the factor 1 - bmid^2 was saved by forward)
// Same structure as forward 1; the weights are R^T ([4D, C], output block k*D/16 + j).
// ------------------------------------------------------------------------------------------------
template <int D, int TPB>
__global__ __launch_bounds__(256) void ddlerp_bwd_mid_kernel(long M, int T, int C, const __bf16* __restrict__ x,
                                                             Dy4 dy,
                                                             const __bf16* __restrict__ RT,
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
    bf16x8 wr[NB / 4][2];
    load_mid_weights<NB>(wr, RT, C, 0, wave, L);
    Loads cur = issue(0);
    for (int c0 = 0, it = 0; c0 < C; c0 += 64, it++) {
        const int buf = it & 1;
#pragma unroll
        for (int i = 0; i < NB / 4; i++) {
            w.f[buf][wave * (NB / 4) + i][0][lane] = wr[i][0];
            w.f[buf][wave * (NB / 4) + i][1][lane] = wr[i][1];
        }
        const int cn = c0 + 64 < C ? c0 + 64 : c0;
        load_mid_weights<NB>(wr, RT, C, cn, wave, L);
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

// da tile for 16 tokens x 64 channels: dpre L      (lane = token, reg = channel)
template <int D>
__device__ __forceinline__ TileF lerp_grad(const __bf16* __restrict__ dpre_row, const __bf16* __restrict__ LT, int c0,
                                           const Lane& L) {
    constexpr int NB = 4 * D / 16;
    bf16x4 dp[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) dp[j] = *reinterpret_cast<const bf16x4*>(dpre_row + 16 * j + 4 * L.g);
    TileF da;
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) {
        const __bf16* lrow = LT + (long)(c0 + chan16(cb, L.n)) * (4 * D) + 4 * L.g;   // F(L^T[c.., :]) lane = channel
        f32x4 acc = zero4();
#pragma unroll
        for (int j = 0; j < NB; j += 2)
            acc = mma2(acc, *reinterpret_cast<const bf16x4*>(lrow + 16 * j), *reinterpret_cast<const bf16x4*>(lrow + 16 * j + 16),
                       dp[j], dp[j + 1]);
        da.f[cb] = acc;
    }
    return da;
}

// ------------------------------------------------------------------------------------------------
// The two streaming kernels (forward 2 and backward 2) give a block one 64-channel block and a range of token
// tiles: the block's 32 KiB of weight fragments (R, L^T) are staged in LDS once, in the order the matrix
// instructions take them (16 bytes per lane per pair), and every wavefront walks its tiles.  Fetching the
// seventy fragments per tile from memory in the middle of dependent arithmetic, as a tile-per-wavefront kernel
// must, left the kernels waiting for loads most of the time.
// ------------------------------------------------------------------------------------------------
template <int D>
struct LerpWeights {   // LDS image for one 64-channel block
    static constexpr int ND = D / 16, NB = 4 * ND;
    bf16x8 R[4][NBLK][ND / 2][WAVE];   // (F(R_k[c.., 16j..]), F(R_k[c.., 16j+16..]))  lane = channel, reg = d
    bf16x8 LT[NBLK][NB / 2][WAVE];     // (F(L^T[c.., 16j..]), F(L^T[c.., 16j+16..]))  lane = channel, reg = mid index
    float beta[4][64];
    float alpha[64];
};
template <int D>
__device__ __forceinline__ void stage_lerp_weights(LerpWeights<D>& w, const __bf16* __restrict__ R, const __bf16* __restrict__ LT,
                                                   const __bf16* __restrict__ beta, const __bf16* __restrict__ alpha, int C,
                                                   int c0, bool with_lt) {
    constexpr int ND = D / 16, NB = 4 * ND;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    // wavefront k stages R_k; all share L^T by channel block
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
    if (with_lt) {
        const int cb = wave;
        const __bf16* lrow = LT + (long)(c0 + chan16(cb, L.n)) * (4 * D) + 4 * L.g;
#pragma unroll
        for (int j = 0; j < NB / 2; j++)
            w.LT[cb][j][lane] = __builtin_shufflevector(*reinterpret_cast<const bf16x4*>(lrow + 32 * j),
                                                        *reinterpret_cast<const bf16x4*>(lrow + 32 * j + 16), 0, 1, 2, 3, 4, 5, 6, 7);
    }
    w.beta[wave][lane] = (float)beta[(long)wave * C + c0 + lane];
    if (wave == 0) w.alpha[lane] = (float)alpha[c0 + lane];
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
    stage_lerp_weights<D>(w, R, nullptr, beta, beta, C, c0, false);   // alpha is not used here
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

// backward 2: dx, written in one pass.
//   da  = dpre L ;  dxx = da*alpha + sum_k dy_k*c_k ;  dx[t] = da + sum_k dy_k - dxx[t] + dxx[t+1]
// The dxx[t+1] of the tile's last token belongs to the next tile; instead of a second pass over an fp32 copy of
// dx, the wavefront evaluates dxx for that one token itself: the same products with the token's row broadcast to
// all sixteen rows of the operand (the weight fragments are already in registers).
template <int D>
__global__ __launch_bounds__(256) void ddlerp_bwd_dx2_kernel(long M, int T, int C, int tiles_per_split,
                                                             const __bf16* __restrict__ x, Dy4 dy,
                                                             const __bf16* __restrict__ alpha,
                                                             const __bf16* __restrict__ R, const __bf16* __restrict__ beta,
                                                             const __bf16* __restrict__ LT,
                                                             const __bf16* __restrict__ bmid,
                                                             const __bf16* __restrict__ dpre, __bf16* __restrict__ dx) {
    constexpr int ND = D / 16, NB = 4 * ND;
    __shared__ LerpWeights<D> w;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Lane L;
    const int c0 = blockIdx.x * 64;
    const long ntiles = M / TOK;
    const long tile_begin = (long)blockIdx.y * tiles_per_split;
    const long tile_end = tile_begin + tiles_per_split < ntiles ? tile_begin + tiles_per_split : ntiles;
    stage_lerp_weights<D>(w, R, LT, beta, alpha, C, c0, true);
    __syncthreads();
    // dx of token t needs the shifted term of token t + 1.  Inside a tile that is a lane shift; across tiles each
    // wavefront walks a CONTIGUOUS part of the block's range from its last tile down, carrying the first token's
    // term of the tile it has just finished.  Only the first tile it touches has no carry: when the token after
    // its part belongs to the same sequence, the wavefront first evaluates that next tile without storing it.
    // (Evaluating the following token in place for every tile, as a first version did, doubled the matrix work
    // and the loads.)  The loads of the tile below are issued before the current one is worked on.
    const long per = (tile_end - tile_begin + 3) / 4;
    const long lo = tile_begin + wave * per;
    const long hi = lo + per < tile_end ? lo + per : tile_end;
    if (lo >= hi) return;
    const bool warm = hi < ntiles && ((hi * TOK) % T) != 0;
    struct Loads {
        bf16x8 bm[NB / 2], dp[NB / 2], dy[4][NBLK / 2];
    };
    auto issue = [&](long tile) {
        Loads ld;
        const long m = tile * TOK + L.n;
        load_mid_pairs(ld.bm, bmid + m * (4 * D), L);
        load_mid_pairs(ld.dp, dpre + m * (4 * D), L);
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; pr++)
                ld.dy[k][pr] = *reinterpret_cast<const bf16x8*>(dy.p[k] + m * C + c0 + 8 * L.g + 32 * pr);
        return ld;
    };
    f32x4 carry[NBLK];   // the shifted term of the first token of the tile above, the same in every lane n
#pragma unroll
    for (int cb = 0; cb < NBLK; cb++) carry[cb] = zero4();
    const long start = warm ? hi : hi - 1;
    Loads cur = issue(start);
    for (long tile = start; tile >= lo; tile--) {
        const Loads nxt = issue(tile > lo ? tile - 1 : lo);
        const bool same_seq = (((tile + 1) * TOK) % T) != 0;   // the token after this tile continues the sequence
        TileB out;
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) {
            const f32x4 al = *reinterpret_cast<const f32x4*>(&w.alpha[chan16(cb, 4 * L.g)]);
            f32x4 da = zero4();
#pragma unroll
            for (int j = 0; j < NB / 2; j++) da = mma8(da, w.LT[cb][j][lane], cur.dp[j]);
            f32x4 dxx = da * al, dxd = da;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                f32x4 c = *reinterpret_cast<const f32x4*>(&w.beta[k][chan16(cb, 4 * L.g)]);
#pragma unroll
                for (int j = 0; j < ND / 2; j++) c = mma8(c, w.R[k][cb][j][lane], cur.bm[k * (ND / 2) + j]);
                const bf16x8 pair = cur.dy[k][cb / 2];
                const f32x4 d = to_f32((cb & 1) ? __builtin_shufflevector(pair, pair, 4, 5, 6, 7)
                                                : __builtin_shufflevector(pair, pair, 0, 1, 2, 3));
                dxx += d * c;
                dxd += d;
            }
            f32x4 o, first;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                // the lane shift runs for all lanes (under a lane condition its source lane could be switched off)
                const float shifted = row_shl<1>(dxx[r]);
                const float above = L.n < TOK - 1 ? shifted : (same_seq ? carry[cb][r] : 0.f);
                o[r] = dxd[r] - dxx[r] + above;
                first[r] = row_bcast(dxx[r], 0);
            }
            carry[cb] = first;
            out.f[cb] = to_bf16(o);
        }
        if (tile < hi) store_rows16(dx + tile * TOK * C + c0, C, L, out);
        cur = nxt;
    }
}

// ------------------------------------------------------------------------------------------------
// backward 3: parameter gradients (sums over tokens).  Block = (64 channels, a range of token tiles);
// its four wavefronts take every fourth tile of the range, partial sums meet in LDS, and the block writes
// one partial per output element:  dR_k = (dy_k*xx)^T bmid_k,  dL = dpre^T a,  dbeta_k = sum dy_k*xx,
// dalpha = sum (dpre L)*xx.  A last kernel adds the partials over the token ranges in a fixed order.
// ------------------------------------------------------------------------------------------------
template <int D>
struct ParamPartial {   // per (split, 64-channel block); element counts
    static constexpr int DR = 4 * 64 * D, DL = 4 * D * 64, DBETA = 4 * 64, DALPHA = 64;
    static constexpr int TOTAL = DR + DL + DBETA + DALPHA;
};

template <int D, int PART>   // PART 0: dR and dbeta (reads dy, bmid);  PART 1: dL and dalpha (reads dpre)
__global__ __launch_bounds__(256) void ddlerp_bwd_param_kernel(long M, int T, int C, int tiles_per_split,
                                                               const __bf16* __restrict__ x,
                                                               Dy4 dy,
                                                               const __bf16* __restrict__ alpha,
                                                               const __bf16* __restrict__ LT,
                                                               const __bf16* __restrict__ bmid,
                                                               const __bf16* __restrict__ dpre,
                                                               float* __restrict__ partial) {
    constexpr int ND = D / 16, NB = 4 * ND;
    using P = ParamPartial<D>;
    constexpr int COMB = PART == 0 ? P::DR : P::DL;
    __shared__ __attribute__((aligned(16))) float comb[COMB];
    __shared__ __attribute__((aligned(16))) float comb_vec[5 * 64];   // dbeta [4][64] then dalpha [64]
    const int wave = threadIdx.x >> 6;
    const Lane L;
    const int c0 = blockIdx.x * 64;
    const int split = blockIdx.y;
    const long ntiles = M / TOK;
    const long tile_begin = (long)split * tiles_per_split;
    const long tile_end = tile_begin + tiles_per_split < ntiles ? tile_begin + tiles_per_split : ntiles;
    const bf16x4 eye = identity_bf16(L);
    const TileF al = load_chan_vec(alpha, c0, L);

    // PART 0: acc[k*NBLK*ND + cb*ND + j] = F(dR_k[c0+16cb.., 16j..])  lane = channel, reg = d
    // PART 1: acc[db*NBLK + cb]          = F(dL[16db.., c0+16cb..])   lane = d, reg = channel
    constexpr int NACC = PART == 0 ? 4 * NBLK * ND : NB * NBLK;
    f32x4 acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; i++) acc[i] = zero4();
    constexpr int NVEC = PART == 0 ? 4 : 1;
    TileF vec[NVEC];   // per-token partial sums of dbeta_k (PART 0) or dalpha (PART 1), lane = token
#pragma unroll
    for (int k = 0; k < NVEC; k++)
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++) vec[k].f[cb] = zero4();

    if constexpr (PART == 0) {
        // One wavefront per SIMD and ~0.4 k instructions per tile: the loads of the NEXT tile are issued before the
        // current one is worked on (raw registers, nothing consumes them early), otherwise every tile waits out a
        // full memory latency.
        struct Loads {
            bf16x8 xc[NBLK / 2], xp[NBLK / 2], dy[4][NBLK / 2];
            bf16x4 bm[NB];
        };
        auto issue = [&](long tile) {
            Loads ld;
            const long m = tile * TOK + L.n;
            const __bf16* row = x + m * C + c0 + 8 * L.g;
            const __bf16* prow = (m % T) != 0 ? row - C : row;   // the masked case never leaves the tensor
            const __bf16* bm_row = bmid + m * (4 * D) + 4 * L.g;
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; pr++) {
                ld.xc[pr] = *reinterpret_cast<const bf16x8*>(row + 32 * pr);
                ld.xp[pr] = *reinterpret_cast<const bf16x8*>(prow + 32 * pr);
            }
#pragma unroll
            for (int j = 0; j < NB; j++) ld.bm[j] = *reinterpret_cast<const bf16x4*>(bm_row + 16 * j);
#pragma unroll
            for (int k = 0; k < 4; k++)
#pragma unroll
                for (int pr = 0; pr < NBLK / 2; pr++)
                    ld.dy[k][pr] = *reinterpret_cast<const bf16x8*>(dy.p[k] + m * C + c0 + 8 * L.g + 32 * pr);
            return ld;
        };
        const long first = tile_begin + wave;
        Loads cur = issue(first < tile_end ? first : tile_end - 1);
        for (long tile = first; tile < tile_end; tile += 4) {
            const Loads nxt = issue(tile + 4 < tile_end ? tile + 4 : tile_end - 1);
            const bool has_prev = ((tile * TOK + L.n) % T) != 0;
            TileF xx;
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; pr++) {
                const bf16x8 zero = {};
                const bf16x8 prev = has_prev ? cur.xp[pr] : zero;
                xx.f[2 * pr] = to_f32(__builtin_shufflevector(prev, prev, 0, 1, 2, 3)) -
                               to_f32(__builtin_shufflevector(cur.xc[pr], cur.xc[pr], 0, 1, 2, 3));
                xx.f[2 * pr + 1] = to_f32(__builtin_shufflevector(prev, prev, 4, 5, 6, 7)) -
                                   to_f32(__builtin_shufflevector(cur.xc[pr], cur.xc[pr], 4, 5, 6, 7));
            }
            bf16x4 bmT[NB];   // F(bmid[:,16j..]^T)  lane = d, reg = token
#pragma unroll
            for (int j = 0; j < NB; j++) bmT[j] = transpose(cur.bm[j], eye);
#pragma unroll
            for (int k = 0; k < 4; k++) {
#pragma unroll
                for (int cb = 0; cb < NBLK; cb++) {
                    const bf16x8 pair = cur.dy[k][cb / 2];
                    const bf16x4 dyk = (cb & 1) ? __builtin_shufflevector(pair, pair, 4, 5, 6, 7)
                                                : __builtin_shufflevector(pair, pair, 0, 1, 2, 3);
                    const f32x4 dc = to_f32(dyk) * xx.f[cb];
                    vec[k].f[cb] += dc;
                    const bf16x4 dcT = transpose(to_bf16(dc), eye);   // F(dc^T) lane = channel, reg = token
#pragma unroll
                    for (int j = 0; j < ND; j++) {
                        f32x4& a = acc[(k * NBLK + cb) * ND + j];
                        a = mma(a, bmT[k * ND + j], dcT);             // + F(dc^T bmid_k)
                    }
                }
            }
            cur = nxt;
        }
    } else {
        // the same one-tile-ahead loads; the block's L^T fragments are staged in LDS once, in matrix-instruction
        // order (fetching them from memory inside every tile left the wavefront waiting for 32 loads per tile)
        __shared__ bf16x8 ltw[NBLK][NB / 2][WAVE];
        {
            const int lane = threadIdx.x & 63;
            const __bf16* lrow = LT + (long)(c0 + chan16(wave, L.n)) * (4 * D) + 4 * L.g;
#pragma unroll
            for (int j = 0; j < NB / 2; j++)
                ltw[wave][j][lane] = __builtin_shufflevector(*reinterpret_cast<const bf16x4*>(lrow + 32 * j),
                                                             *reinterpret_cast<const bf16x4*>(lrow + 32 * j + 16), 0, 1, 2, 3, 4, 5, 6, 7);
        }
        __syncthreads();
        struct Loads {
            bf16x8 xc[NBLK / 2], xp[NBLK / 2];
            bf16x4 dp[NB];
        };
        auto issue = [&](long tile) {
            Loads ld;
            const long m = tile * TOK + L.n;
            const __bf16* row = x + m * C + c0 + 8 * L.g;
            const __bf16* prow = (m % T) != 0 ? row - C : row;
            const __bf16* dp_row = dpre + m * (4 * D) + 4 * L.g;
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; pr++) {
                ld.xc[pr] = *reinterpret_cast<const bf16x8*>(row + 32 * pr);
                ld.xp[pr] = *reinterpret_cast<const bf16x8*>(prow + 32 * pr);
            }
#pragma unroll
            for (int j = 0; j < NB; j++) ld.dp[j] = *reinterpret_cast<const bf16x4*>(dp_row + 16 * j);
            return ld;
        };
        const long first = tile_begin + wave;
        Loads cur = issue(first < tile_end ? first : tile_end - 1);
        for (long tile = first; tile < tile_end; tile += 4) {
            const Loads nxt = issue(tile + 4 < tile_end ? tile + 4 : tile_end - 1);
            const bool has_prev = ((tile * TOK + L.n) % T) != 0;
            bf16x4 dpT[NB];   // F(dpre[:,16j..]^T)  lane = d, reg = token
#pragma unroll
            for (int j = 0; j < NB; j++) dpT[j] = transpose(cur.dp[j], eye);
#pragma unroll
            for (int cb = 0; cb < NBLK; cb++) {
                const bf16x8 zero = {};
                const bf16x8 prev8 = has_prev ? cur.xp[cb / 2] : zero, cur8 = cur.xc[cb / 2];
                const f32x4 xv = to_f32((cb & 1) ? __builtin_shufflevector(cur8, cur8, 4, 5, 6, 7)
                                                 : __builtin_shufflevector(cur8, cur8, 0, 1, 2, 3));
                const f32x4 xxv = to_f32((cb & 1) ? __builtin_shufflevector(prev8, prev8, 4, 5, 6, 7)
                                                  : __builtin_shufflevector(prev8, prev8, 0, 1, 2, 3)) - xv;
                // da = dpre L for this channel block (lane = token, reg = channel)
                f32x4 da = zero4();
#pragma unroll
                for (int j = 0; j < NB / 2; j++)
                    da = mma8(da, ltw[cb][j][threadIdx.x & 63],
                              __builtin_shufflevector(cur.dp[2 * j], cur.dp[2 * j + 1], 0, 1, 2, 3, 4, 5, 6, 7));
                vec[0].f[cb] += da * xxv;
                const bf16x4 aT = transpose(to_bf16(xv + xxv * al.f[cb]), eye);   // F(a^T) lane = channel
#pragma unroll
                for (int db = 0; db < NB; db++) acc[db * NBLK + cb] = mma(acc[db * NBLK + cb], aT, dpT[db]);   // + F(dpre^T a)
            }
            cur = nxt;
        }
    }
    // per-token partials -> sums over the 16 token lanes (total lands in lane n = 15)
#pragma unroll
    for (int k = 0; k < NVEC; k++)
#pragma unroll
        for (int cb = 0; cb < NBLK; cb++)
#pragma unroll
            for (int r = 0; r < 4; r++) vec[k].f[cb][r] = row_prefix_sum(vec[k].f[cb][r]);

    // combine the four wavefronts in a fixed order through LDS, then write this block's partial record
    // (record layout: dR [4][64][D], dL [4D][64], dbeta [4][64], dalpha [64])
    for (int w = 0; w < 4; w++) {
        if (wave == w) {
            auto put = [&](float* p, f32x4 v) {
                if (w > 0) v += *reinterpret_cast<f32x4*>(p);
                *reinterpret_cast<f32x4*>(p) = v;
            };
            if constexpr (PART == 0) {
#pragma unroll
                for (int k = 0; k < 4; k++)
#pragma unroll
                    for (int cb = 0; cb < NBLK; cb++)
#pragma unroll
                        for (int j = 0; j < ND; j++)
                            put(comb + (k * 64 + chan16(cb, L.n)) * D + 16 * j + 4 * L.g, acc[(k * NBLK + cb) * ND + j]);
            } else {
#pragma unroll
                for (int db = 0; db < NB; db++)
#pragma unroll
                    for (int cb = 0; cb < NBLK; cb++) put(comb + (16 * db + L.n) * 64 + chan16(cb, 4 * L.g), acc[db * NBLK + cb]);
            }
            if (L.n == 15) {
#pragma unroll
                for (int cb = 0; cb < NBLK; cb++) {
                    if constexpr (PART == 0) {
#pragma unroll
                        for (int k = 0; k < 4; k++) put(comb_vec + k * 64 + chan16(cb, 4 * L.g), vec[k].f[cb]);
                    } else {
                        put(comb_vec + 4 * 64 + chan16(cb, 4 * L.g), vec[0].f[cb]);
                    }
                }
            }
        }
        __syncthreads();
    }
    float* out = partial + ((long)split * gridDim.x + blockIdx.x) * P::TOTAL;
    float* dst = out + (PART == 0 ? 0 : P::DR);
    for (int i = threadIdx.x; i < COMB / 4; i += 256)
        *reinterpret_cast<f32x4*>(dst + 4 * i) = *reinterpret_cast<const f32x4*>(comb + 4 * i);
    float* vdst = out + P::DR + P::DL;
    if (PART == 0) {
        for (int i = threadIdx.x; i < 4 * 64; i += 256) vdst[i] = comb_vec[i];
    } else {
        for (int i = threadIdx.x; i < 64; i += 256) vdst[4 * 64 + i] = comb_vec[4 * 64 + i];
    }
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
    const int e = blockIdx.x * 256 + threadIdx.x;   // one thread per element of the record
    if (e >= P::TOTAL) return;
    float s = 0.f;
    for (int sp = 0; sp < nsplit; sp++) s += partial[((long)sp * ncb + cblk) * P::TOTAL + e];
    if (e < P::DR) {
        const int d = e % D, c = (e / D) % 64, k = e / (64 * D);
        dR[((long)k * C + c0 + c) * D + d] = s;
    } else if (e < P::DR + P::DL) {
        const int f = e - P::DR;
        const int c = f % 64, j = f / 64;
        dL[(long)j * C + c0 + c] = s;
    } else if (e < P::DR + P::DL + P::DBETA) {
        const int f = e - P::DR - P::DL;
        dbeta[(long)(f / 64) * C + c0 + f % 64] = s;
    } else {
        dalpha[c0 + e - P::DR - P::DL - P::DBETA] = s;
    }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
namespace {
constexpr size_t A256(size_t x) { return (x + 255) / 256 * 256; }
// The parameter kernels keep one block per compute unit (one wavefront per SIMD), so the grid should be ONE round
// of at most 256 blocks over the channel blocks: 384 blocks, as an earlier cap of 32 ranges gave at 12 channel
// blocks, run as two rounds with the second half empty.  At least 32 token tiles per block (8 per wavefront).
int param_splits(long M, int ncb) {
    const long ntiles = M / TOK;
    long s = ntiles / 32;
    const long cap = 256 / ncb > 0 ? 256 / ncb : 1;
    if (s > cap) s = cap;
    if (s < 1) s = 1;
    return (int)s;
}
// token-tile ranges of the streaming kernels: about three blocks per compute unit of an MI355X (256) over the
// channel blocks, at least four tiles (one per wavefront) each
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

bool ddlerp_rank_supported(int D) { return D == 32; }

size_t ddlerp_bwd_workspace_bytes(long M, int C, int D) {
    const int ncb = C / 64;
    const size_t transposed = A256((size_t)4 * C * D * 2) * 2;
    const size_t dpre = A256((size_t)M * 4 * D * 2);
    const size_t partial = A256((size_t)param_splits(M, ncb) * ncb * ParamPartial<32>::TOTAL * 4);
    return transposed + dpre + partial;
}

void launch_ddlerp_forward(long M, int T, int C, int D, const void* x, const void* alpha, const void* Lw, const void* R,
                           const void* beta, void* bmid, void* bder, void* y, hipStream_t stream) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    // four tiles per block when that still gives every compute unit a block, else two
    const long ntiles = M / TOK;
    if (ntiles >= 4 * 256)
        hipLaunchKernelGGL((ddlerp_fwd_mid_kernel<32, 4>), dim3((unsigned)((ntiles + 3) / 4)), dim3(256), 0, stream, M, T, C,
                           c(x), c(alpha), c(Lw), static_cast<__bf16*>(bmid), static_cast<__bf16*>(bder));
    else
        hipLaunchKernelGGL((ddlerp_fwd_mid_kernel<32, 2>), dim3((unsigned)((ntiles + 1) / 2)), dim3(256), 0, stream, M, T, C,
                           c(x), c(alpha), c(Lw), static_cast<__bf16*>(bmid), static_cast<__bf16*>(bder));
    const StreamSplit sp = stream_splits(M, C / 64, 2 * 512);   // two blocks per compute unit, two rounds
    hipLaunchKernelGGL(ddlerp_fwd_out2_kernel<32>, dim3(C / 64, sp.nsplit), dim3(256), 0, stream, M, T, C, sp.tiles_per_split,
                       c(x), c(R), c(beta), c(bmid), static_cast<__bf16*>(y));
    (void)D;
}

void launch_ddlerp_backward(long M, int T, int C, int D, const void* x, const void* alpha, const void* Lw, const void* R,
                            const void* beta, const void* bmid, const void* bder, const void* const dy4[4], void* dx,
                            void* dalpha,
                            void* dL, void* dR, void* dbeta, void* workspace, hipStream_t stream) {
    auto c = [](const void* p) { return static_cast<const __bf16*>(p); };
    const Dy4 dy{{c(dy4[0]), c(dy4[1]), c(dy4[2]), c(dy4[3])}};
    const int ncb = C / 64;
    char* p = static_cast<char*>(workspace);
    __bf16* RT = reinterpret_cast<__bf16*>(p); p += A256((size_t)4 * C * D * 2);
    __bf16* LT = reinterpret_cast<__bf16*>(p); p += A256((size_t)4 * C * D * 2);
    __bf16* dpre = reinterpret_cast<__bf16*>(p); p += A256((size_t)M * 4 * D * 2);
    float* partial = reinterpret_cast<float*>(p);
    const int nsplit = param_splits(M, ncb);
    const int tiles_per_split = (int)((M / TOK + nsplit - 1) / nsplit);

    hipLaunchKernelGGL(ddlerp_transpose_kernel, dim3(96), dim3(256), 0, stream, C, D, c(R), c(Lw), RT, LT);
    if (M / TOK >= 4 * 256)
        hipLaunchKernelGGL((ddlerp_bwd_mid_kernel<32, 4>), dim3((unsigned)((M / TOK + 3) / 4)), dim3(256), 0, stream, M, T, C,
                           c(x), dy, RT, c(bder), dpre);
    else
        hipLaunchKernelGGL((ddlerp_bwd_mid_kernel<32, 2>), dim3((unsigned)((M / TOK + 1) / 2)), dim3(256), 0, stream, M, T, C,
                           c(x), dy, RT, c(bder), dpre);
    {
        const StreamSplit sp = stream_splits(M, ncb, 3 * 256);    // one block per compute unit, three rounds
        hipLaunchKernelGGL(ddlerp_bwd_dx2_kernel<32>, dim3(ncb, sp.nsplit), dim3(256), 0, stream, M, T, C, sp.tiles_per_split,
                           c(x), dy, c(alpha), c(R), c(beta), LT, c(bmid), dpre, static_cast<__bf16*>(dx));
    }
    hipLaunchKernelGGL((ddlerp_bwd_param_kernel<32, 0>), dim3(ncb, nsplit), dim3(256), 0, stream, M, T, C,
                       tiles_per_split, c(x), dy, c(alpha), LT, c(bmid), dpre, partial);
    hipLaunchKernelGGL((ddlerp_bwd_param_kernel<32, 1>), dim3(ncb, nsplit), dim3(256), 0, stream, M, T, C,
                       tiles_per_split, c(x), dy, c(alpha), LT, c(bmid), dpre, partial);
    hipLaunchKernelGGL(ddlerp_param_reduce_kernel<32>, dim3((ParamPartial<32>::TOTAL + 255) / 256, ncb), dim3(256), 0,
                       stream, C, nsplit, partial,
                       static_cast<float*>(dR), static_cast<float*>(dL), static_cast<float*>(dbeta),
                       static_cast<float*>(dalpha));
}

}  // namespace wkv
