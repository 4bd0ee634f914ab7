// Weight gradient of a bias-free projection y = x W^T:  dW[o][i] = sum_t dy[t][o] * x[t][i].
//
// Both operands are token-major ([tokens, channels] bf16), so the contraction runs over the SLOW index of
// both: the matrix instruction wants, per lane, eight consecutive tokens of one channel, while memory offers
// eight consecutive channels of one token.  gfx950 has an LDS read that does exactly this transposition
// (ds_read_b64_tr_b16): tiles are copied token-major into LDS with plain 16-byte accesses and read back
// channel-major, four tokens per lane and instruction; two reads make one operand of the 32x32x16 MFMA (the
// instruction shape this chip sustains best: 1.85-1.9 PFLOP/s in a loop of nothing else, against 1.15 for
// the 16x16x32 shape).
//
// D[i][j] = sum_t A[t][i] * B[t][j] with A the wider operand.  A block of four wavefronts (WM x WN) owns a
// tile of D and one contiguous range of tokens (split-K: tiles x splits ~ one block per compute unit, a
// multiple of eight splits so that every split's operands are read by one XCD's L2 only); a wavefront owns
// TMB x TNB blocks of 32 x 32.  Per step of 32 tokens the pipeline is: global -> registers four steps ahead,
// registers -> LDS two steps ahead, LDS -> operand registers one step ahead, one barrier; the LDS reads and
// writes of a step are issued BETWEEN its matrix instructions, in a pinned order (a wavefront issues in order,
// and an LDS read occupies the compute unit's LDS pipe for about 8 cycles, a 16-byte write for 13: issued as
// a group they would stall the wavefront for as long as its matrix work takes).  With one wavefront per SIMD
// every instruction of the loop costs issue time, so the per-step address and mask work is scalar: a uniform
// pointer per step plus a fixed 32-bit offset per thread, and one precomputed bit per piece for the tail.  The fp32 partial tiles go to the
// workspace in register order and linear_wgrad_reduce_kernel sums them over the splits in a fixed order,
// applies the output strides (either orientation of dW) and the output type.
#include "linear_kernels.hpp"
#include "device_info.hpp"

#include "frag.hpp"

namespace wkv {
namespace {

constexpr int STEP = 32;         // tokens per step (the K of one matrix instruction)
constexpr int LDS_PAD = 16;      // elements; makes every row pitch an odd multiple of 32 bytes modulo 256
constexpr int DEPTH = 4;         // steps of global loads in flight

typedef __bf16 __attribute__((address_space(3))) lds_bf16;
typedef s16x4 __attribute__((address_space(3))) lds_s16x4;
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Lane (kg, p) of each 16-lane group points at token row 4kg + p/4, channels 4(p%4)..+3; the instruction
// hands lane (kg, i) the four tokens 4kg..4kg+3 of channel i.
__device__ __forceinline__ bf16x4 read_tr(const __bf16* p) {
    return __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(lds_bf16*)p));
}

// Tile shapes, in blocks of 32.  Wide outputs: 192 x 192 per block, 96 x 96 per wavefront (18 matrix
// instructions for 24 transposed reads per step); narrow ones (one side <= 128): the block spans the narrow side.
template <int TMB_, int TNB_, int WM_, int WN_>
struct Shape {
    static constexpr int TMB = TMB_, TNB = TNB_, WM = WM_, WN = WN_;
    static constexpr int WG_M = 32 * TMB * WM, WG_N = 32 * TNB * WN;
    static constexpr int PA = WG_M + LDS_PAD, PB = WG_N + LDS_PAD;
    static constexpr int QA = WG_M / 64;                       // 16-byte pieces of A per thread and step
    static constexpr int B_PIECES = STEP * WG_N / 8;
    static constexpr int QB = (B_PIECES + 255) / 256;
    static_assert(WM * WN == 4 && WG_M % 64 == 0, "four wavefronts; A pieces divide evenly");
};

template <class S>
struct WgradLds {
    __bf16 a[2][STEP][S::PA];
    __bf16 b[2][STEP][S::PB];
};

struct WgradArgs {
    long tokens;
    int M, N;
    const __bf16* A;
    long lda;
    const __bf16* B;
    long ldb;
    float* partial;
    int ksplit, ntn, ntiles;
};

// One block's work: tile `tile` of problem g, token range `split` of g.ksplit.
template <class S>
__device__ __forceinline__ void wgrad_block(WgradLds<S>& lds, const WgradArgs& g, const int split, const int tile) {
    constexpr int TMB = S::TMB, TNB = S::TNB, QA = S::QA, QB = S::QB;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave / S::WN, wn = wave % S::WN;
    const int m0 = (tile / g.ntn) * S::WG_M, n0 = (tile % g.ntn) * S::WG_N;
    // this block's steps (units of 32 tokens) u0 .. u0 + nsteps - 1, as scalars
    const long nunits = (g.tokens + STEP - 1) / STEP;
    const int u0 = __builtin_amdgcn_readfirstlane((int)(split * nunits / g.ksplit));
    const int nsteps = __builtin_amdgcn_readfirstlane((int)((split + 1) * nunits / g.ksplit)) - u0;
    // Steps 0 .. nfull - 1 lie wholly inside the tensor.  At most one more step exists, the tensor's last, partial
    // unit: its 32-row window is pulled back to end at the last token and the rows it shares with the unit before
    // are masked out (with fewer than 32 tokens in all, rows are clamped instead).  Where a token lands in LDS
    // is irrelevant as long as both operands put it in the same row, which they do.
    const int nfull = __builtin_amdgcn_readfirstlane(max(0, min(nsteps, (int)(g.tokens / STEP) - u0)));
    const long tail_w0 = max(0L, g.tokens - STEP);
    const int tail_lo = (int)((long)(u0 + nfull) * STEP - tail_w0), tail_hi = (int)min((long)STEP, g.tokens - tail_w0);
    const int last_row = (int)min((long)STEP - 1, g.tokens - 1);

    // Addresses are (uniform pointer of the step) + (a 32-bit offset fixed per thread): the per-step address work is
    // a few scalar instructions.  A thread without a B piece of its own repeats one (same data to the same place:
    // no branch in the loop).
    int a_row[QA], b_row[QB];
    unsigned a_off[QA], b_off[QB];
    unsigned tail_rows = 0;   // bit q: this thread's row of piece q belongs to the partial unit
    __bf16* a_dst[QA];
    __bf16* b_dst[QB];
#pragma unroll
    for (int q = 0; q < QA; q++) {
        const int p = tid + 256 * q;
        a_row[q] = p / (S::WG_M / 8);
        const int c = 8 * (p % (S::WG_M / 8));
        a_off[q] = (unsigned)(min(a_row[q], last_row) * g.lda + min(m0 + c, g.M - 8));
        tail_rows |= (unsigned)(a_row[q] >= tail_lo && a_row[q] < tail_hi) << q;
        a_dst[q] = &lds.a[0][a_row[q]][c];
    }
#pragma unroll
    for (int q = 0; q < QB; q++) {
        const int p = tid + 256 * q;
        const int pc = p < S::B_PIECES ? p : tid % S::B_PIECES;
        b_row[q] = pc / (S::WG_N / 8);
        const int c = 8 * (pc % (S::WG_N / 8));
        b_off[q] = (unsigned)(min(b_row[q], last_row) * g.ldb + min(n0 + c, g.N - 8));
        tail_rows |= (unsigned)(b_row[q] >= tail_lo && b_row[q] < tail_hi) << (QA + q);
        b_dst[q] = &lds.b[0][b_row[q]][c];
    }
    const bf16x8 zero8 = {};
    const __bf16* const a_first = g.A + (long)u0 * STEP * g.lda;
    const __bf16* const b_first = g.B + (long)u0 * STEP * g.ldb;
    const __bf16* const a_tail = g.A + tail_w0 * g.lda;
    const __bf16* const b_tail = g.B + tail_w0 * g.ldb;
    // Register sets: r?[j] holds the tokens of a step = j (mod DEPTH), fetched DEPTH steps before its turn.
    // Loads only: the mask is applied when a set is handed to LDS, so that nothing consumes a load before its
    // turn.  Steps past the end of the range read the tail window (always inside the tensor) and multiply zeros.
    bf16x8 ra[DEPTH][QA], rb[DEPTH][QB];
    constexpr int PIECES = QA + QB;   // this thread's 16-byte pieces per step: A first, then B
    auto fetch_one = [&](int set, int step, int piece) {
        const bool full = step < nfull;
        if (piece < QA)
            ra[set][piece] = *reinterpret_cast<const bf16x8*>((full ? a_first + (long)step * STEP * g.lda : a_tail) + a_off[piece]);
        else
            rb[set][piece - QA] =
                *reinterpret_cast<const bf16x8*>((full ? b_first + (long)step * STEP * g.ldb : b_tail) + b_off[piece - QA]);
    };
    auto stage_one = [&](int set, int buf, int step, int piece) {
        // does this row hold one of the step's own tokens: always in a full step, per the precomputed bit in the
        // partial unit, never past the end
        const bool keep = step < nfull || (step < nsteps && ((tail_rows >> piece) & 1));
        if (piece < QA)
            *reinterpret_cast<bf16x8*>(a_dst[piece] + buf * (STEP * S::PA)) = keep ? ra[set][piece] : zero8;
        else
            *reinterpret_cast<bf16x8*>(b_dst[piece - QA] + buf * (STEP * S::PB)) = keep ? rb[set][piece - QA] : zero8;
    };
    auto fetch = [&](int set, int step) {
#pragma unroll
        for (int q = 0; q < PIECES; q++) fetch_one(set, step, q);
    };
    auto stage = [&](int set, int buf, int step) {
#pragma unroll
        for (int q = 0; q < PIECES; q++) stage_one(set, buf, step, q);
    };

    f32x16 acc[TMB][TNB];
#pragma unroll
    for (int mb = 0; mb < TMB; mb++)
#pragma unroll
        for (int nb = 0; nb < TNB; nb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[mb][nb][r] = 0.f;

    // Operand of a 32-row block for one half (16 tokens) of a step: lane (g, p) of 16-lane group g covers rows
    // 16 (g % 2) .. + 15 and the contraction slots of group g / 2.  Which token sits in which slot is free as long
    // as both operands agree: read e hands slot 4e + r of group g / 2 the token 8e + 4 (g / 2) + r, so that one
    // instruction reads eight consecutive token rows.
    const int grp = lane >> 4, p16 = lane & 15;
    const int rd_row = 4 * (grp >> 1) + (p16 >> 2), rd_col = 16 * (grp & 1) + 4 * (p16 & 3);
    const __bf16* a_rd = &lds.a[0][rd_row][32 * TMB * wm + rd_col];
    const __bf16* b_rd = &lds.b[0][rd_row][32 * TNB * wn + rd_col];
    // operand sets: op?[s & 1] holds step s, read from LDS while the matrix work of step s - 1 runs.  A set is
    // READS transposed reads of four tokens: per half, two per A block, then two per B block.
    constexpr int READS = 4 * (TMB + TNB), MFMAS = 2 * TMB * TNB;
    bf16x4 opa[2][2][TMB][2], opb[2][2][TNB][2];   // [set][half][block][low / high four slots]
    auto read_one = [&](int set, int buf, int n) {
        const int half = n / (2 * (TMB + TNB)), m = n % (2 * (TMB + TNB));
        if (m < 2 * TMB)
            opa[set][half][m / 2][m % 2] = read_tr(a_rd + buf * (STEP * S::PA) + (16 * half + 8 * (m % 2)) * S::PA + 32 * (m / 2));
        else
            opb[set][half][(m - 2 * TMB) / 2][m % 2] =
                read_tr(b_rd + buf * (STEP * S::PB) + (16 * half + 8 * (m % 2)) * S::PB + 32 * ((m - 2 * TMB) / 2));
    };
    auto multiply_one = [&](int set, int n) {   // matrix instruction n of a step: half-major, then A block, then B block
        const int half = n / (TMB * TNB), mb = (n / TNB) % TMB, nb = n % TNB;
        const bf16x8 a = __builtin_shufflevector(opa[set][half][mb][0], opa[set][half][mb][1], 0, 1, 2, 3, 4, 5, 6, 7);
        const bf16x8 b = __builtin_shufflevector(opb[set][half][nb][0], opb[set][half][nb][1], 0, 1, 2, 3, 4, 5, 6, 7);
        acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[mb][nb], 0, 0, 0);
    };

    // Step s, after its barrier: buffer s & 1 (whose tokens sit in op[s & 1] since step s - 1) takes step s + 2,
    // buffer (s + 1) & 1 (written during step s - 1) is read into op[(s + 1) & 1], and op[s & 1] multiplies.
    // Reads and writes touch different buffers, so one barrier per step is enough and all LDS traffic can be
    // issued between the matrix instructions.
    if (nsteps > 0) {
        fetch(0, 0);
        fetch(1, 1);
        stage(0, 0, 0);
        stage(1, 1, 1);
#pragma unroll
        for (int j = 2; j < 2 + DEPTH; j++) fetch(j % DEPTH, j);
        __syncthreads();
#pragma unroll
        for (int n = 0; n < READS; n++) read_one(0, 0, n);
        for (int base = 0; base < nsteps; base += DEPTH) {
#pragma unroll
            for (int k = 0; k < DEPTH; k++) {
                __syncthreads();
                // Issue order, pinned: before matrix instruction i its share of the step's transposed reads (for
                // step s + 1), of the 16-byte LDS writes (step s + 2) and of the global loads (step s + 2 + DEPTH).
                // An even spread measured best; bunching the LDS traffic early in the step costs 9 %.
#pragma unroll
                for (int i = 0; i < MFMAS; i++) {
#pragma unroll
                    for (int n = READS * i / MFMAS; n < READS * (i + 1) / MFMAS; n++) read_one((k + 1) & 1, (k + 1) & 1, n);
#pragma unroll
                    for (int q = PIECES * i / MFMAS; q < PIECES * (i + 1) / MFMAS; q++) {
                        stage_one((k + 2) % DEPTH, k & 1, base + k + 2, q);
                        fetch_one((k + 2) % DEPTH, base + k + 2 + DEPTH, q);
                    }
                    multiply_one(k & 1, i);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }

    // register order: register r of lane l of block (mb, nb) is
    // D[m0 + 32 TMB wm + 32 mb + 8 (r / 4) + 4 (l / 32) + r % 4][n0 + 32 TNB wn + 32 nb + l % 32]
    float* out = g.partial + ((((long)split * g.ntiles + tile) * 4 + wave) * (TMB * TNB)) * 1024 + 4 * lane;
#pragma unroll
    for (int mb = 0; mb < TMB; mb++)
#pragma unroll
        for (int nb = 0; nb < TNB; nb++)
#pragma unroll
            for (int qd = 0; qd < 4; qd++)
                *reinterpret_cast<f32x4*>(out + ((mb * TNB + nb) * 4 + qd) * 256) =
                    f32x4{acc[mb][nb][4 * qd], acc[mb][nb][4 * qd + 1], acc[mb][nb][4 * qd + 2], acc[mb][nb][4 * qd + 3]};
}

template <class S>
__global__ __launch_bounds__(256) void linear_wgrad_kernel(WgradArgs g) {
    __shared__ WgradLds<S> lds;
    wgrad_block<S>(lds, g, blockIdx.x % g.ksplit, blockIdx.x / g.ksplit);
}

// shape table: index = WgradPlan::shape
using Wide = Shape<3, 3, 2, 2>;      // 192 x 192
using Thin1 = Shape<2, 1, 4, 1>;     // 256 x 32
using Thin2 = Shape<2, 2, 4, 1>;     // 256 x 64
using Thin3 = Shape<2, 3, 4, 1>;     // 256 x 96
using Thin4 = Shape<2, 4, 4, 1>;     // 256 x 128
struct ShapeInfo { int TMB, TNB, WM, WN; };
constexpr ShapeInfo kShapes[5] = {{3, 3, 2, 2}, {2, 1, 4, 1}, {2, 2, 4, 1}, {2, 3, 4, 1}, {2, 4, 4, 1}};


// Several problems in one launch (the weight gradients of projections whose upstream gradients arrive together),
// each with the tile shape that suits it: with the tiles of all of them in one grid a compute unit's block covers
// a longer token range, so there are fewer fp32 partial tiles to write and to sum (three 768 x 768 problems at
// 8192 tokens: 48 tiles x 5 ranges instead of 3 x (16 x 16), 35 MB of partials instead of 113 MB), and problems
// too small to fill the machine on their own share one launch.
constexpr int WGRAD_MAX_JOBS = 8;
struct WgradGroup {
    WgradArgs job[WGRAD_MAX_JOBS];
    int first_tile[WGRAD_MAX_JOBS + 1];   // job j owns the grid's tiles first_tile[j] .. first_tile[j+1]-1
    int shape[WGRAD_MAX_JOBS];            // index into the shape table
    int njobs, ksplit;
};
template <class A, class B>
constexpr size_t max_lds() { return sizeof(WgradLds<A>) > sizeof(WgradLds<B>) ? sizeof(WgradLds<A>) : sizeof(WgradLds<B>); }
constexpr size_t GROUP_LDS = max_lds<Wide, Thin4>();
static_assert(sizeof(WgradLds<Thin1>) <= GROUP_LDS && sizeof(WgradLds<Thin2>) <= GROUP_LDS && sizeof(WgradLds<Thin3>) <= GROUP_LDS);

__global__ __launch_bounds__(256) void linear_wgrad_group_kernel(WgradGroup G) {
    __shared__ __attribute__((aligned(16))) char raw[GROUP_LDS];
    const int split = blockIdx.x % G.ksplit, t = blockIdx.x / G.ksplit;
    int j = 0;
#pragma unroll
    for (int i = 1; i < WGRAD_MAX_JOBS; i++) j += (i < G.njobs && t >= G.first_tile[i]) ? 1 : 0;
    // (j is the same in every lane: the job is read from the argument block with scalar loads)
    const WgradArgs g = G.job[j];
    const int tile = t - G.first_tile[j];
    switch (G.shape[j]) {
        case 0: wgrad_block<Wide>(*reinterpret_cast<WgradLds<Wide>*>(raw), g, split, tile); break;
        case 1: wgrad_block<Thin1>(*reinterpret_cast<WgradLds<Thin1>*>(raw), g, split, tile); break;
        case 2: wgrad_block<Thin2>(*reinterpret_cast<WgradLds<Thin2>*>(raw), g, split, tile); break;
        case 3: wgrad_block<Thin3>(*reinterpret_cast<WgradLds<Thin3>*>(raw), g, split, tile); break;
        default: wgrad_block<Thin4>(*reinterpret_cast<WgradLds<Thin4>*>(raw), g, split, tile); break;
    }
}

struct ReduceArgs {
    int M, N, TMB, TNB, WN, WG_M, WG_N, ntn, ntiles, ksplit;
    const float* partial;
    long si, sj;
};

// One block = 64 register quads x 4 groups of splits (group k sums splits k, k+4, ...; the four sums are then
// added in a fixed order), so that narrow outputs with many splits still fill the machine.
template <typename OUT>
__device__ __forceinline__ void reduce_block(const ReduceArgs& g, OUT* __restrict__ out, const long block) {
    __shared__ f32x4 part[3][64];
    const long quads = (long)g.ntiles * 4 * g.TMB * g.TNB * 4 * 64;
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const long q = block * 64 + lane;
    const float* src = g.partial + (q < quads ? q : quads - 1) * 4;
    f32x4 s = zero4();
#pragma unroll 4
    for (int k = grp; k < g.ksplit; k += 4) s += *reinterpret_cast<const f32x4*>(src + (long)k * quads * 4);
    if (grp > 0) part[grp - 1][lane] = s;
    __syncthreads();
    if (grp > 0 || q >= quads) return;
    s = ((s + part[0][lane]) + part[1][lane]) + part[2][lane];
    long t = q >> 6;
    const int qd = (int)(t & 3);
    t >>= 2;
    const int blk = (int)(t % (g.TMB * g.TNB));
    t /= g.TMB * g.TNB;
    const int wave = (int)(t & 3), tile = (int)(t >> 2);
    const int mb = blk / g.TNB, nb = blk % g.TNB;
    const int m = (tile / g.ntn) * g.WG_M + 32 * g.TMB * (wave / g.WN) + 32 * mb + 8 * qd + 4 * (lane >> 5);
    const int j = (tile % g.ntn) * g.WG_N + 32 * g.TNB * (wave % g.WN) + 32 * nb + (lane & 31);
    if (j >= g.N) return;
#pragma unroll
    for (int r = 0; r < 4; r++)
        if (m + r < g.M) out[(m + r) * g.si + j * g.sj] = (OUT)s[r];
}
template <typename OUT>
__global__ __launch_bounds__(256) void linear_wgrad_reduce_kernel(ReduceArgs g, OUT* __restrict__ out) {
    reduce_block<OUT>(g, out, blockIdx.x);
}
// the reductions of a grouped launch, one grid over all of its problems
struct ReduceGroup {
    ReduceArgs job[WGRAD_MAX_JOBS];
    void* out[WGRAD_MAX_JOBS];
    long first_block[WGRAD_MAX_JOBS + 1];
    int njobs;
};
template <typename OUT>
__global__ __launch_bounds__(256) void linear_wgrad_reduce_group_kernel(ReduceGroup R) {
    const long b = blockIdx.x;
    int j = 0;
#pragma unroll
    for (int i = 1; i < WGRAD_MAX_JOBS; i++) j += (i < R.njobs && b >= R.first_block[i]) ? 1 : 0;
    const ReduceArgs& g = R.job[j];
    OUT* out = static_cast<OUT*>(R.out[j]);
    reduce_block<OUT>(g, out, b - R.first_block[j]);
}

}  // namespace

WgradPlan linear_wgrad_plan(long tokens, int O, int I) {
    WgradPlan best{};
    const int M = O >= I ? O : I, N = O >= I ? I : O;
    const long nunits = (tokens + STEP - 1) / STEP;
    double best_score = -1.0;
    for (int sh = 0; sh < 5; sh++) {
        if (sh == 0 && N <= 128) continue;   // the wide tile is for two large sides
        if (sh != 0 && N > 128 && sh != 3 && sh != 4) continue;
        const ShapeInfo s = kShapes[sh];
        const int wg_m = 32 * s.TMB * s.WM, wg_n = 32 * s.TNB * s.WN;
        const int ntm = (M + wg_m - 1) / wg_m, ntn = (N + wg_n - 1) / wg_n;
        const long tiles = (long)ntm * ntn;
        const int cus = compute_units();
        long k = cus / tiles;
        if (k >= 8) k -= k % 8;
        if (k > nunits) k = nunits;
        if (k < 1) k = 1;
        const long wgs = tiles * k;
        const double used = (double)M * N / ((double)ntm * wg_m * ntn * wg_n);
        const double fill = (double)wgs / ((double)cus * ((wgs + cus - 1) / cus));
        // the wide tile does the most matrix work per LDS read
        const double score = used * fill * (sh == 0 ? 1.4 : 1.0);
        if (score > best_score + 1e-9) {
            best_score = score;
            best.shape = sh;
            best.ntn = ntn;
            best.ntiles = (int)tiles;
            best.ksplit = (int)k;
        }
    }
    best.swap = O < I;
    const ShapeInfo s = kShapes[best.shape];
    best.partial_bytes = (size_t)best.ksplit * best.ntiles * 4 * s.TMB * s.TNB * 1024 * sizeof(float);
    return best;
}

void launch_linear_wgrad(long tokens, int O, int I, const void* dy, long ld_dy, const void* x, long ld_x, void* dW,
                         bool out_f32, void* workspace, hipStream_t stream) {
    const WgradPlan plan = linear_wgrad_plan(tokens, O, I);
    WgradArgs g;
    g.tokens = tokens;
    g.M = plan.swap ? I : O;
    g.N = plan.swap ? O : I;
    g.A = static_cast<const __bf16*>(plan.swap ? x : dy);
    g.lda = plan.swap ? ld_x : ld_dy;
    g.B = static_cast<const __bf16*>(plan.swap ? dy : x);
    g.ldb = plan.swap ? ld_dy : ld_x;
    g.partial = static_cast<float*>(workspace);
    g.ksplit = plan.ksplit;
    g.ntn = plan.ntn;
    g.ntiles = plan.ntiles;
    const dim3 grid(plan.ntiles * plan.ksplit), block(256);
    switch (plan.shape) {
        case 0: hipLaunchKernelGGL(linear_wgrad_kernel<Wide>, grid, block, 0, stream, g); break;
        case 1: hipLaunchKernelGGL(linear_wgrad_kernel<Thin1>, grid, block, 0, stream, g); break;
        case 2: hipLaunchKernelGGL(linear_wgrad_kernel<Thin2>, grid, block, 0, stream, g); break;
        case 3: hipLaunchKernelGGL(linear_wgrad_kernel<Thin3>, grid, block, 0, stream, g); break;
        default: hipLaunchKernelGGL(linear_wgrad_kernel<Thin4>, grid, block, 0, stream, g); break;
    }
    const ShapeInfo s = kShapes[plan.shape];
    ReduceArgs r;
    r.M = g.M;
    r.N = g.N;
    r.TMB = s.TMB;
    r.TNB = s.TNB;
    r.WN = s.WN;
    r.WG_M = 32 * s.TMB * s.WM;
    r.WG_N = 32 * s.TNB * s.WN;
    r.ntn = plan.ntn;
    r.ntiles = plan.ntiles;
    r.ksplit = plan.ksplit;
    r.partial = g.partial;
    // D[i][j] -> dW[o][i']: row-major [O, I] when A = dy, transposed walk when the operands were swapped
    r.si = plan.swap ? 1 : I;
    r.sj = plan.swap ? I : 1;
    const long quads = (long)plan.ntiles * 4 * s.TMB * s.TNB * 4 * 64;
    const dim3 rgrid((unsigned)((quads + 63) / 64));
    if (out_f32)
        hipLaunchKernelGGL(linear_wgrad_reduce_kernel<float>, rgrid, block, 0, stream, r, static_cast<float*>(dW));
    else
        hipLaunchKernelGGL(linear_wgrad_reduce_kernel<__bf16>, rgrid, block, 0, stream, r, static_cast<__bf16*>(dW));
}

// ---- several problems in one launch ----
namespace {
struct GroupPlan {
    int n, ksplit, shape[WGRAD_MAX_JOBS], ntn[WGRAD_MAX_JOBS], ntiles[WGRAD_MAX_JOBS], first_tile[WGRAD_MAX_JOBS + 1];
    bool swap[WGRAD_MAX_JOBS];
    size_t partial_off[WGRAD_MAX_JOBS + 1];   // bytes
};
bool group_plan(int n, long tokens, const int* O, const int* I, GroupPlan& p) {
    if (n < 1 || n > WGRAD_MAX_JOBS || tokens < 1) return false;
    p.n = n;
    p.first_tile[0] = 0;
    for (int j = 0; j < n; j++) {
        const int M = O[j] >= I[j] ? O[j] : I[j], N = O[j] >= I[j] ? I[j] : O[j];
        if (N < 1) return false;
        // the wide tile for two large sides, else the block spans the narrow side
        p.shape[j] = N > 128 ? 0 : (N + 31) / 32;
        const ShapeInfo s = kShapes[p.shape[j]];
        const int wg_m = 32 * s.TMB * s.WM, wg_n = 32 * s.TNB * s.WN;
        p.swap[j] = O[j] < I[j];
        p.ntn[j] = (N + wg_n - 1) / wg_n;
        p.ntiles[j] = ((M + wg_m - 1) / wg_m) * p.ntn[j];
        p.first_tile[j + 1] = p.first_tile[j] + p.ntiles[j];
    }
    const long nunits = (tokens + STEP - 1) / STEP;
    long k = compute_units() / p.first_tile[n];
    if (k >= 8) k -= k % 8;
    if (k > nunits) k = nunits;
    if (k < 1) k = 1;
    p.ksplit = (int)k;
    p.partial_off[0] = 0;
    for (int j = 0; j < n; j++) {
        const ShapeInfo s = kShapes[p.shape[j]];
        p.partial_off[j + 1] = p.partial_off[j] + (size_t)k * p.ntiles[j] * 4 * s.TMB * s.TNB * 1024 * sizeof(float);
    }
    return true;
}
}  // namespace

size_t linear_wgrad_group_workspace_bytes(int n, long tokens, const int* O, const int* I) {
    GroupPlan p;
    return group_plan(n, tokens, O, I, p) ? p.partial_off[n] : 0;
}

bool launch_linear_wgrad_group(int n, long tokens, const int* O, const int* I, const void* const* dy, const long* ld_dy,
                               const void* const* x, const long* ld_x, void* const* dW, bool out_f32, void* workspace,
                               hipStream_t stream) {
    GroupPlan p;
    if (!group_plan(n, tokens, O, I, p)) return false;
    WgradGroup G{};
    ReduceGroup R{};
    G.njobs = R.njobs = n;
    G.ksplit = p.ksplit;
    R.first_block[0] = 0;
    for (int j = 0; j < n; j++) {
        const ShapeInfo s = kShapes[p.shape[j]];
        G.shape[j] = p.shape[j];
        WgradArgs& g = G.job[j];
        g.tokens = tokens;
        g.M = p.swap[j] ? I[j] : O[j];
        g.N = p.swap[j] ? O[j] : I[j];
        g.A = static_cast<const __bf16*>(p.swap[j] ? x[j] : dy[j]);
        g.lda = p.swap[j] ? ld_x[j] : ld_dy[j];
        g.B = static_cast<const __bf16*>(p.swap[j] ? dy[j] : x[j]);
        g.ldb = p.swap[j] ? ld_dy[j] : ld_x[j];
        g.partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + p.partial_off[j]);
        g.ksplit = p.ksplit;
        g.ntn = p.ntn[j];
        g.ntiles = p.ntiles[j];
        G.first_tile[j] = p.first_tile[j];
        ReduceArgs& r = R.job[j];
        r.M = g.M;
        r.N = g.N;
        r.TMB = s.TMB;
        r.TNB = s.TNB;
        r.WN = s.WN;
        r.WG_M = 32 * s.TMB * s.WM;
        r.WG_N = 32 * s.TNB * s.WN;
        r.ntn = p.ntn[j];
        r.ntiles = p.ntiles[j];
        r.ksplit = p.ksplit;
        r.partial = g.partial;
        r.si = p.swap[j] ? 1 : I[j];
        r.sj = p.swap[j] ? I[j] : 1;
        R.out[j] = dW[j];
        const long quads = (long)p.ntiles[j] * 4 * s.TMB * s.TNB * 4 * 64;
        R.first_block[j + 1] = R.first_block[j] + (quads + 63) / 64;
    }
    G.first_tile[n] = p.first_tile[n];
    hipLaunchKernelGGL(linear_wgrad_group_kernel, dim3((unsigned)(p.first_tile[n] * p.ksplit)), dim3(256), 0, stream, G);
    const dim3 rgrid((unsigned)R.first_block[n]);
    if (out_f32) hipLaunchKernelGGL(linear_wgrad_reduce_group_kernel<float>, rgrid, dim3(256), 0, stream, R);
    else hipLaunchKernelGGL(linear_wgrad_reduce_group_kernel<__bf16>, rgrid, dim3(256), 0, stream, R);
    return true;
}

}  // namespace wkv
