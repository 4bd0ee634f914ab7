// Weight gradient of a bias-free projection y = x W^T:  dW[o][i] = sum_t dy[t][o] * x[t][i].
//
// Both operands are token-major ([tokens, channels] bf16), so the contraction runs over the SLOW index of
// both: the matrix instruction wants, per lane, eight consecutive tokens of one channel, while memory offers
// eight consecutive channels of one token.  gfx950 has an LDS read that does exactly this transposition
// (ds_read_b64_tr_b16): tiles are copied token-major into LDS with plain 16-byte accesses and read back
// channel-major, four tokens per lane and instruction; two reads make one operand of the 16x16x32 MFMA.
//
// D[i][j] = sum_t A[t][i] * B[t][j] with A the wider operand.  A block of four wavefronts (WM x WN) owns a
// tile of D and one contiguous range of tokens (split-K: tiles x splits ~ one block per compute unit, a
// multiple of eight splits so that every split's operands are read by one XCD's L2 only); a wavefront owns
// TMB x TNB blocks of 16 x 16.  Per step of 32 tokens the pipeline is: global -> registers four steps ahead,
// registers -> LDS two steps ahead, LDS -> operand registers one step ahead, one barrier; the LDS reads and
// writes of a step are issued BETWEEN its matrix instructions (a wavefront issues in order, and an LDS read
// occupies the compute unit's LDS pipe for about 8 cycles, a 16-byte write for 13: issued as a group they
// would stall the wavefront for as long as its matrix work takes).  The fp32 partial tiles go to the
// workspace in register order and linear_wgrad_reduce_kernel sums them over the splits in a fixed order,
// applies the output strides (either orientation of dW) and the output type.
#include "linear_kernels.hpp"

#include "frag.hpp"

namespace wkv {
namespace {

constexpr int STEP = 32;         // tokens per step (the K of one matrix instruction)
constexpr int LDS_PAD = 16;      // elements; makes every row pitch an odd multiple of 32 bytes modulo 256
constexpr int DEPTH = 4;         // steps of global loads in flight

typedef __bf16 __attribute__((address_space(3))) lds_bf16;
typedef s16x4 __attribute__((address_space(3))) lds_s16x4;

// Lane (kg, p) of each 16-lane group points at token row 4kg + p/4, channels 4(p%4)..+3; the instruction
// hands lane (kg, i) the four tokens 4kg..4kg+3 of channel i.
__device__ __forceinline__ bf16x4 read_tr(const __bf16* p) {
    return __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(lds_bf16*)p));
}

// Tile shapes.  Wide outputs: 192 x 192 per block, 96 x 96 per wavefront (36 matrix instructions for 24
// transposed reads per step); narrow ones (one side <= 128): the block spans the narrow side.
template <int TMB_, int TNB_, int WM_, int WN_>
struct Shape {
    static constexpr int TMB = TMB_, TNB = TNB_, WM = WM_, WN = WN_;
    static constexpr int WG_M = 16 * TMB * WM, WG_N = 16 * TNB * WN;
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

template <class S>
__global__ __launch_bounds__(256) void linear_wgrad_kernel(WgradArgs g) {
    constexpr int TMB = S::TMB, TNB = S::TNB, QA = S::QA, QB = S::QB;
    __shared__ WgradLds<S> lds;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave / S::WN, wn = wave % S::WN;
    const int split = blockIdx.x % g.ksplit, tile = blockIdx.x / g.ksplit;
    const int m0 = (tile / g.ntn) * S::WG_M, n0 = (tile % g.ntn) * S::WG_N;
    const long nunits = (g.tokens + STEP - 1) / STEP;
    const long u0 = split * nunits / g.ksplit, u1 = (split + 1) * nunits / g.ksplit;
    const long nsteps = u1 - u0;
    const long t_end = min(g.tokens, u1 * STEP);

    // this thread's pieces of a step: row (token within the step) and channel, clamped into the operand;
    // a thread without a B piece of its own repeats one (same data to the same place: no branch in the loop)
    int a_row[QA], b_row[QB];
    const __bf16* a_src[QA];
    const __bf16* b_src[QB];
    __bf16* a_dst[QA];
    __bf16* b_dst[QB];
#pragma unroll
    for (int q = 0; q < QA; q++) {
        const int p = tid + 256 * q;
        a_row[q] = p / (S::WG_M / 8);
        const int c = 8 * (p % (S::WG_M / 8));
        a_src[q] = g.A + min(m0 + c, g.M - 8);
        a_dst[q] = &lds.a[0][a_row[q]][c];
    }
#pragma unroll
    for (int q = 0; q < QB; q++) {
        const int p = tid + 256 * q;
        const int pc = p < S::B_PIECES ? p : tid % S::B_PIECES;
        b_row[q] = pc / (S::WG_N / 8);
        const int c = 8 * (pc % (S::WG_N / 8));
        b_src[q] = g.B + min(n0 + c, g.N - 8);
        b_dst[q] = &lds.b[0][b_row[q]][c];
    }
    const bf16x8 zero8 = {};
    // Register sets: r?[j] holds the tokens of a step = j (mod DEPTH), fetched DEPTH steps before its turn.
    // Loads only: the tail mask is applied when a set is handed to LDS, so that nothing consumes a load before
    // its turn.  Steps past the end of the range re-read the last step and multiply zeros.
    bf16x8 ra[DEPTH][QA], rb[DEPTH][QB];
    auto fetch = [&](int set, long step) {
        const long t0 = (u0 + (step < nsteps ? step : nsteps - 1)) * STEP;
#pragma unroll
        for (int q = 0; q < QA; q++)
            ra[set][q] = *reinterpret_cast<const bf16x8*>(a_src[q] + min(t0 + a_row[q], g.tokens - 1) * g.lda);
#pragma unroll
        for (int q = 0; q < QB; q++)
            rb[set][q] = *reinterpret_cast<const bf16x8*>(b_src[q] + min(t0 + b_row[q], g.tokens - 1) * g.ldb);
    };
    auto stage = [&](int set, int buf, long step) {
        const long t0 = (u0 + step) * STEP;
#pragma unroll
        for (int q = 0; q < QA; q++)
            *reinterpret_cast<bf16x8*>(a_dst[q] + buf * (STEP * S::PA)) = t0 + a_row[q] < t_end ? ra[set][q] : zero8;
#pragma unroll
        for (int q = 0; q < QB; q++)
            *reinterpret_cast<bf16x8*>(b_dst[q] + buf * (STEP * S::PB)) = t0 + b_row[q] < t_end ? rb[set][q] : zero8;
    };

    f32x4 acc[TMB][TNB];
#pragma unroll
    for (int mb = 0; mb < TMB; mb++)
#pragma unroll
        for (int nb = 0; nb < TNB; nb++) acc[mb][nb] = zero4();

    const int kg = lane >> 4, p16 = lane & 15;
    const __bf16* a_rd = &lds.a[0][4 * kg + (p16 >> 2)][16 * TMB * wm + 4 * (p16 & 3)];
    const __bf16* b_rd = &lds.b[0][4 * kg + (p16 >> 2)][16 * TNB * wn + 4 * (p16 & 3)];
    // operand sets: op?[s & 1] holds step s, read from LDS while the matrix work of step s - 1 runs
    bf16x8 opa[2][TMB], opb[2][TNB];
    auto read_ops = [&](int set, int buf) {
        const __bf16* ar = a_rd + buf * (STEP * S::PA);
        const __bf16* br = b_rd + buf * (STEP * S::PB);
#pragma unroll
        for (int mb = 0; mb < TMB; mb++) {
            const bf16x4 lo = read_tr(ar + 16 * mb), hi = read_tr(ar + 16 * S::PA + 16 * mb);
            opa[set][mb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int nb = 0; nb < TNB; nb++) {
            const bf16x4 lo = read_tr(br + 16 * nb), hi = read_tr(br + 16 * S::PB + 16 * nb);
            opb[set][nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
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
        read_ops(0, 0);
        constexpr int READS = 2 * (TMB + TNB), MFMAS = TMB * TNB, WRITES = QA + QB;
        constexpr int PAIRED = READS < MFMAS ? READS : MFMAS;
        constexpr int PER_WRITE = (MFMAS - PAIRED) / WRITES;
        for (long base = 0; base < nsteps; base += DEPTH) {
#pragma unroll
            for (int k = 0; k < DEPTH; k++) {
                __syncthreads();
                read_ops((k + 1) & 1, (k + 1) & 1);
                stage((k + 2) % DEPTH, k & 1, base + k + 2);
                fetch((k + 2) % DEPTH, base + k + 2 + DEPTH);
#pragma unroll
                for (int mb = 0; mb < TMB; mb++)
#pragma unroll
                    for (int nb = 0; nb < TNB; nb++)
                        acc[mb][nb] = mma8(acc[mb][nb], opa[k & 1][mb], opb[k & 1][nb]);
                // issue order: (transposed read, matrix instruction) pairs, then each 16-byte write and each
                // global load with its share of the remaining matrix instructions
#pragma unroll
                for (int i = 0; i < PAIRED; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
                if (READS > PAIRED) __builtin_amdgcn_sched_group_barrier(0x100, READS - PAIRED, 0);
#pragma unroll
                for (int i = 0; i < WRITES; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    if (PER_WRITE > 0) __builtin_amdgcn_sched_group_barrier(0x008, PER_WRITE, 0);
                }
            }
        }
    }

    // register order: lane (n, g) register r of block (mb, nb) is
    // D[m0 + 16 TMB wm + 16 mb + 4g + r][n0 + 16 TNB wn + 16 nb + n]
    float* out = g.partial + ((((long)split * g.ntiles + tile) * 4 + wave) * (TMB * TNB)) * 256 + 4 * lane;
#pragma unroll
    for (int mb = 0; mb < TMB; mb++)
#pragma unroll
        for (int nb = 0; nb < TNB; nb++) *reinterpret_cast<f32x4*>(out + (mb * TNB + nb) * 256) = acc[mb][nb];
}

struct ReduceArgs {
    int M, N, TMB, TNB, WN, WG_M, WG_N, ntn, ntiles, ksplit;
    const float* partial;
    long si, sj;
};

// One block = 64 register quads x 4 groups of splits (group k sums splits k, k+4, ...; the four sums are then
// added in a fixed order), so that narrow outputs with many splits still fill the machine.
template <typename OUT>
__global__ __launch_bounds__(256) void linear_wgrad_reduce_kernel(ReduceArgs g, OUT* __restrict__ out) {
    __shared__ f32x4 part[3][64];
    const long quads = (long)g.ntiles * 4 * g.TMB * g.TNB * 64;
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const long q = (long)blockIdx.x * 64 + lane;
    const float* src = g.partial + (q < quads ? q : quads - 1) * 4;
    f32x4 s = zero4();
#pragma unroll 4
    for (int k = grp; k < g.ksplit; k += 4) s += *reinterpret_cast<const f32x4*>(src + (long)k * quads * 4);
    if (grp > 0) part[grp - 1][lane] = s;
    __syncthreads();
    if (grp > 0 || q >= quads) return;
    s = ((s + part[0][lane]) + part[1][lane]) + part[2][lane];
    long t = q >> 6;
    const int blk = (int)(t % (g.TMB * g.TNB));
    t /= g.TMB * g.TNB;
    const int wave = (int)(t & 3), tile = (int)(t >> 2);
    const int mb = blk / g.TNB, nb = blk % g.TNB;
    const int m = (tile / g.ntn) * g.WG_M + 16 * g.TMB * (wave / g.WN) + 16 * mb + 4 * (lane >> 4);
    const int j = (tile % g.ntn) * g.WG_N + 16 * g.TNB * (wave % g.WN) + 16 * nb + (lane & 15);
    if (j >= g.N) return;
#pragma unroll
    for (int r = 0; r < 4; r++)
        if (m + r < g.M) out[(m + r) * g.si + j * g.sj] = (OUT)s[r];
}

// shape table: index = WgradPlan::shape
using Wide = Shape<6, 6, 2, 2>;      // 192 x 192
using Thin2 = Shape<3, 2, 4, 1>;     // 192 x 32
using Thin4 = Shape<3, 4, 4, 1>;     // 192 x 64
using Thin6 = Shape<3, 6, 4, 1>;     // 192 x 96
using Thin8 = Shape<3, 8, 4, 1>;     // 192 x 128
struct ShapeInfo { int TMB, TNB, WM, WN; };
constexpr ShapeInfo kShapes[5] = {{6, 6, 2, 2}, {3, 2, 4, 1}, {3, 4, 4, 1}, {3, 6, 4, 1}, {3, 8, 4, 1}};

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
        const int wg_m = 16 * s.TMB * s.WM, wg_n = 16 * s.TNB * s.WN;
        const int ntm = (M + wg_m - 1) / wg_m, ntn = (N + wg_n - 1) / wg_n;
        const long tiles = (long)ntm * ntn;
        long k = 256 / tiles;
        if (k >= 8) k -= k % 8;
        if (k > nunits) k = nunits;
        if (k < 1) k = 1;
        const long wgs = tiles * k;
        const double used = (double)M * N / ((double)ntm * wg_m * ntn * wg_n);
        const double fill = (double)wgs / (256.0 * ((wgs + 255) / 256));
        // the wide tile does 1.5 matrix instructions per LDS read, the narrow ones 1 or fewer
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
    best.partial_bytes = (size_t)best.ksplit * best.ntiles * 4 * s.TMB * s.TNB * 256 * sizeof(float);
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
        case 1: hipLaunchKernelGGL(linear_wgrad_kernel<Thin2>, grid, block, 0, stream, g); break;
        case 2: hipLaunchKernelGGL(linear_wgrad_kernel<Thin4>, grid, block, 0, stream, g); break;
        case 3: hipLaunchKernelGGL(linear_wgrad_kernel<Thin6>, grid, block, 0, stream, g); break;
        default: hipLaunchKernelGGL(linear_wgrad_kernel<Thin8>, grid, block, 0, stream, g); break;
    }
    const ShapeInfo s = kShapes[plan.shape];
    ReduceArgs r;
    r.M = g.M;
    r.N = g.N;
    r.TMB = s.TMB;
    r.TNB = s.TNB;
    r.WN = s.WN;
    r.WG_M = 16 * s.TMB * s.WM;
    r.WG_N = 16 * s.TNB * s.WN;
    r.ntn = plan.ntn;
    r.ntiles = plan.ntiles;
    r.ksplit = plan.ksplit;
    r.partial = g.partial;
    // D[i][j] -> dW[o][i']: row-major [O, I] when A = dy, transposed walk when the operands were swapped
    r.si = plan.swap ? 1 : I;
    r.sj = plan.swap ? I : 1;
    const long quads = (long)plan.ntiles * 4 * s.TMB * s.TNB * 64;
    const dim3 rgrid((unsigned)((quads + 63) / 64));
    if (out_f32)
        hipLaunchKernelGGL(linear_wgrad_reduce_kernel<float>, rgrid, block, 0, stream, r, static_cast<float*>(dW));
    else
        hipLaunchKernelGGL(linear_wgrad_reduce_kernel<__bf16>, rgrid, block, 0, stream, r, static_cast<__bf16*>(dW));
}

}  // namespace wkv
