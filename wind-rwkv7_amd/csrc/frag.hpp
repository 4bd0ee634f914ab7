// Wave64 fragment algebra for gfx950 (CDNA4) matrix cores.
//
// Everything in the WKV7 kernels is expressed with one register layout, the "fragment":
//
//     F(M) for a 16x16 matrix M:  lane l = 16*g + n  (n = 0..15, g = 0..3) holds
//                                 M[n][4*g + r], r = 0..3          (4 values per lane)
//
// i.e. the lane's low four bits pick a row of M, and (g, r) picks the column.  All 16x16
// MFMA instructions read their A and B operands in exactly this layout (row/column index
// on lane%16, contraction index on (lane/16, register)) and write D with
// D[4*g + r][n] in lane (n, g) register r.  Consequence (used everywhere below):
//
//     mma(acc, F(MA), F(MB))  ==  acc + F(MB * MA^T)
//
// so an MFMA result is again a fragment and can feed the next MFMA after a type conversion,
// with no shuffles and no LDS.  A transpose is a product with the identity:
//     F(M^T) = mma(0, F(M), F(I)).
//
// A 16 x 64 tile (16 tokens x 64 channels of one head) is four fragments, one per block of
// 16 channels: tile.f[blk] = F(X[:, 16*blk : 16*blk+16]).  In memory order that means lane
// (n, g) owns channels 16*blk + 4*g + r of token row n: an 8-byte piece of a 128-byte row.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace wkv {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;
constexpr int CHUNK = 16;   // tokens per chunk
constexpr int HEAD = 64;    // channels per head handled by these kernels
constexpr int NBLK = HEAD / 16;

struct Lane {
    int n;  // lane % 16 : row index of every fragment this lane holds
    int g;  // lane / 16 : column group (columns 4g .. 4g+3)
    __device__ Lane() {
        int l = threadIdx.x & (WAVE - 1);
        n = l & 15;
        g = l >> 4;
    }
};

// fp32 -> bf16, round to nearest even, as two packed conversions whose results are handled as 32-bit words.  (A plain
// four-wide conversion that feeds a matrix instruction is done element by element by this compiler and re-packed with
// permutes: three instructions per pair instead of one.)
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ bf16x4 pack_bf16(float a, float b, float c, float d) {
    const bf16x2 lo = __builtin_convertvector((f32x2){a, b}, bf16x2);
    const bf16x2 hi = __builtin_convertvector((f32x2){c, d}, bf16x2);
    const u32x2 r = {__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi)};
    return __builtin_bit_cast(bf16x4, r);
}
__device__ __forceinline__ bf16x4 to_bf16(f32x4 x) { return pack_bf16(x[0], x[1], x[2], x[3]); }
__device__ __forceinline__ f32x4 to_f32(bf16x4 x) { return __builtin_convertvector(x, f32x4); }
__device__ __forceinline__ f32x4 zero4() { return f32x4{0.f, 0.f, 0.f, 0.f}; }

// acc + F(MB * MA^T), bf16 operands, fp32 accumulate (one v_mfma_f32_16x16x16_bf16).
__device__ __forceinline__ f32x4 mma(f32x4 acc, bf16x4 A, bf16x4 B) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, A), __builtin_bit_cast(s16x4, B), acc, 0, 0, 0);
}
// Same with two fragment pairs contracted at once (one v_mfma_f32_16x16x32_bf16):
// acc + F(MB0*MA0^T + MB1*MA1^T).
__device__ __forceinline__ f32x4 mma2(f32x4 acc, bf16x4 A0, bf16x4 A1, bf16x4 B0, bf16x4 B1) {
    bf16x8 a = __builtin_shufflevector(A0, A1, 0, 1, 2, 3, 4, 5, 6, 7);
    bf16x8 b = __builtin_shufflevector(B0, B1, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
}
// the same with each operand's two fragments already side by side in one register quad
__device__ __forceinline__ f32x4 mma8(f32x4 acc, bf16x8 a, bf16x8 b) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
}
// fp32 operands (four v_mfma_f32_16x16x4_f32): used where bf16 operand rounding is not acceptable.
__device__ __forceinline__ f32x4 mma_f32(f32x4 acc, f32x4 A, f32x4 B) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(A[0], B[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(A[1], B[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(A[2], B[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(A[3], B[3], acc, 0, 0, 0);
    return acc;
}

// F(I)
__device__ __forceinline__ bf16x4 identity_bf16(const Lane& L) {
    f32x4 e;
#pragma unroll
    for (int r = 0; r < 4; r++) e[r] = (L.n == 4 * L.g + r) ? 1.f : 0.f;
    return to_bf16(e);
}
__device__ __forceinline__ f32x4 identity_f32(const Lane& L) {
    f32x4 e;
#pragma unroll
    for (int r = 0; r < 4; r++) e[r] = (L.n == 4 * L.g + r) ? 1.f : 0.f;
    return e;
}

// F(M^T) from F(M); exact for bf16 data.
__device__ __forceinline__ bf16x4 transpose(bf16x4 M, bf16x4 eye) { return to_bf16(mma(zero4(), M, eye)); }

// Keep M[row][col] where the predicate holds.  For a fragment F(M): row = n, col = 4g+r.
// lower_strict: col < row;  lower_incl: col <= row;  upper_*: the transposed patterns.
__device__ __forceinline__ f32x4 mask_lower_strict(f32x4 x, const Lane& L) {
#pragma unroll
    for (int r = 0; r < 4; r++) x[r] = (4 * L.g + r < L.n) ? x[r] : 0.f;
    return x;
}
__device__ __forceinline__ f32x4 mask_lower_incl(f32x4 x, const Lane& L) {
#pragma unroll
    for (int r = 0; r < 4; r++) x[r] = (4 * L.g + r <= L.n) ? x[r] : 0.f;
    return x;
}
__device__ __forceinline__ f32x4 mask_upper_strict(f32x4 x, const Lane& L) {
#pragma unroll
    for (int r = 0; r < 4; r++) x[r] = (4 * L.g + r > L.n) ? x[r] : 0.f;
    return x;
}
__device__ __forceinline__ f32x4 mask_upper_incl(f32x4 x, const Lane& L) {
#pragma unroll
    for (int r = 0; r < 4; r++) x[r] = (4 * L.g + r >= L.n) ? x[r] : 0.f;
    return x;
}

// ---- cross-lane helpers inside a row of 16 lanes (the token axis of a tile) ----
// value of lane (n - d) of the same row, 0 for n < d
template <int d>
__device__ __forceinline__ float row_shr(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x110 + d, 0xf, 0xf, true));
}
// value of lane (n + d) of the same row, 0 for n + d > 15
template <int d>
__device__ __forceinline__ float row_shl(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x100 + d, 0xf, 0xf, true));
}
// inclusive prefix sum over n (tokens 0..n)
__device__ __forceinline__ float row_prefix_sum(float x) {
    x += row_shr<1>(x);
    x += row_shr<2>(x);
    x += row_shr<4>(x);
    x += row_shr<8>(x);
    return x;
}
// inclusive suffix sum over n (tokens n..15)
__device__ __forceinline__ float row_suffix_sum(float x) {
    x += row_shl<1>(x);
    x += row_shl<2>(x);
    x += row_shl<4>(x);
    x += row_shl<8>(x);
    return x;
}
// value held by lane `src` (0..15) of the same row
__device__ __forceinline__ float row_bcast(float x, int src) { return __shfl(x, src, 16); }
// the row's lane 15 in every lane of the row, in four lane-crossing moves on the vector ALU (the general broadcast
// above goes through the LDS crossbar, a pipe the whole compute unit shares): mirror the row (lane 0 <- lane 15),
// spread lane 0 over its quad, then copy the quad to lanes 4-7 and lanes 0-7 to lanes 8-15.
__device__ __forceinline__ float row_bcast_last(float x) {
    int v = __builtin_bit_cast(int, x);
    v = __builtin_amdgcn_update_dpp(v, v, 0x140, 0xf, 0xf, false);    // row_mirror
    v = __builtin_amdgcn_update_dpp(v, v, 0x00, 0xf, 0xf, false);     // quad_perm [0,0,0,0]
    v = __builtin_amdgcn_update_dpp(v, v, 0x114, 0xf, 0xe, false);    // row_shr:4 into lanes 4-15
    v = __builtin_amdgcn_update_dpp(v, v, 0x118, 0xf, 0xc, false);    // row_shr:8 into lanes 8-15
    return __builtin_bit_cast(float, v);
}
// value of lane (n + d) mod 16 of the same row
template <int d>
__device__ __forceinline__ float row_rot(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + (16 - d), 0xf, 0xf, false));
}
// sum over the 16 lanes of a row, result in every lane of the row: four rotations on the vector ALU (lane shuffles
// through __shfl go through the LDS crossbar, ~100 cycles each in a dependent chain)
__device__ __forceinline__ float row_sum(float x) {
    x += row_rot<8>(x);
    x += row_rot<4>(x);
    x += row_rot<2>(x);
    x += row_rot<1>(x);
    return x;
}
// sum over the four lanes (n, 0..3) that together hold one token row; result in all four
__device__ __forceinline__ float group_sum(float x) {
    x += __shfl_xor(x, 16, 64);
    x += __shfl_xor(x, 32, 64);
    return x;
}

// Sum over ALL sixteen columns of each row of a fragment (register and column group are the contraction index of a
// matrix instruction): F(M 1 1^T), i.e. the row sum in every register of the row's four lanes, from one matrix
// instruction on the bf16-rounded values - for uses where that rounding does not matter.  (The cross-lane route costs
// two trips through the LDS crossbar; gfx950's lane-swap instructions, fed the same value twice, were compiled into
// a sum of one result with itself.)
__device__ __forceinline__ float row_sum16_bf16(f32x4 x) {
    const bf16x4 ones = pack_bf16(1.f, 1.f, 1.f, 1.f);
    return mma(zero4(), ones, to_bf16(x))[0];
}

// Block barrier that orders LDS traffic only.  __syncthreads() also waits for every global load and store the
// wavefront has in flight, which serialises a prefetch with the work it is meant to overlap; use this one where
// the wavefronts of a block exchange data through LDS alone.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---- tiles ----
struct TileF {  // 16 x 64 tile, fp32 registers
    f32x4 f[NBLK];
};
struct TileB {  // 16 x 64 tile, bf16 registers
    bf16x4 f[NBLK];
};
__device__ __forceinline__ TileB to_bf16(const TileF& x) {
    TileB r;
#pragma unroll
    for (int i = 0; i < NBLK; i++) r.f[i] = to_bf16(x.f[i]);
    return r;
}
__device__ __forceinline__ TileF to_f32(const TileB& x) {
    TileF r;
#pragma unroll
    for (int i = 0; i < NBLK; i++) r.f[i] = to_f32(x.f[i]);
    return r;
}

// Load a [16 tokens x 64 channels] tile whose row n starts at p + n*ld (elements).
__device__ __forceinline__ TileB load_rows(const __bf16* __restrict__ p, long ld, const Lane& L) {
    TileB t;
    const __bf16* row = p + (long)L.n * ld + 4 * L.g;
#pragma unroll
    for (int i = 0; i < NBLK; i++) t.f[i] = *reinterpret_cast<const bf16x4*>(row + 16 * i);
    return t;
}
// The same tile with 16-byte accesses (half the memory instructions, 64 contiguous bytes per row and column
// group).  A kernel whose blocks of 16 channels are only ever contracted over, or combined elementwise with
// tiles loaded the same way, does not care WHICH 16 channels form a block; so blocks 2p and 2p+1 interleave in
// groups of four - register r of block cb in column group g is channel chan16(cb, 4g + r) - and a lane's pieces
// of the two blocks are 8 contiguous channels.  Row index j of a transposed fragment maps the same way.
__host__ __device__ constexpr int chan16(int cb, int j) { return 32 * (cb >> 1) + 8 * (j >> 2) + 4 * (cb & 1) + (j & 3); }
__device__ __forceinline__ TileB load_rows16(const __bf16* __restrict__ p, long ld, const Lane& L) {
    TileB t;
    const __bf16* row = p + (long)L.n * ld + 8 * L.g;
#pragma unroll
    for (int pr = 0; pr < NBLK / 2; pr++) {
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(row + 32 * pr);
        t.f[2 * pr] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
        t.f[2 * pr + 1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
    }
    return t;
}
__device__ __forceinline__ void store_rows16(__bf16* __restrict__ p, long ld, const Lane& L, const TileB& t) {
    __bf16* row = p + (long)L.n * ld + 8 * L.g;
#pragma unroll
    for (int pr = 0; pr < NBLK / 2; pr++)
        *reinterpret_cast<bf16x8*>(row + 32 * pr) = __builtin_shufflevector(t.f[2 * pr], t.f[2 * pr + 1], 0, 1, 2, 3, 4, 5, 6, 7);
}
__device__ __forceinline__ void store_rows(__bf16* __restrict__ p, long ld, const Lane& L, const TileB& t) {
    __bf16* row = p + (long)L.n * ld + 4 * L.g;
#pragma unroll
    for (int i = 0; i < NBLK; i++) *reinterpret_cast<bf16x4*>(row + 16 * i) = t.f[i];
}

// Fragment-order storage used by the workspace arrays: a fragment is 64 lanes x 4 bf16 = 512 bytes,
// lane-major (a wave reads or writes it as one contiguous 512-byte run, 8 bytes per lane); a tile is
// four consecutive fragments (2 KiB).
constexpr int FRAG_ELEMS = 256;
constexpr int TILE_ELEMS = 4 * FRAG_ELEMS;
__device__ __forceinline__ bf16x4 load_frag(const __bf16* __restrict__ p, int lane) {
    return *reinterpret_cast<const bf16x4*>(p + 4 * lane);
}
__device__ __forceinline__ void store_frag(__bf16* __restrict__ p, int lane, bf16x4 v) {
    *reinterpret_cast<bf16x4*>(p + 4 * lane) = v;
}
__device__ __forceinline__ TileB load_frags(const __bf16* __restrict__ p, int lane) {
    TileB t;
#pragma unroll
    for (int i = 0; i < NBLK; i++) t.f[i] = load_frag(p + i * FRAG_ELEMS, lane);
    return t;
}
__device__ __forceinline__ void store_frags(__bf16* __restrict__ p, int lane, const TileB& t) {
#pragma unroll
    for (int i = 0; i < NBLK; i++) store_frag(p + i * FRAG_ELEMS, lane, t.f[i]);
}

// sum over the four channel blocks: F(X * Y^T) for 16x64 tiles X (rows -> result rows) and Y.
// Note the operand order of mma(): result rows come from the B operand.
__device__ __forceinline__ f32x4 tile_xyT(const TileB& X, const TileB& Y) {
    f32x4 acc = zero4();
    acc = mma2(acc, Y.f[0], Y.f[1], X.f[0], X.f[1]);
    acc = mma2(acc, Y.f[2], Y.f[3], X.f[2], X.f[3]);
    return acc;
}

// inv(I - X) for a strictly lower-triangular 16x16 X, by recursive block inversion:
// with M the inverse of the block-diagonal part at block size s, the inverse at block size 2s is
// M + M * Xs * M, where Xs keeps the s x s sub-diagonal blocks of X.  The products carry ~16 bits per operand
// (bf16 hi + lo, see tri_inverse_level) and accumulate in fp32 (a Neumann product (I+X)(I+X^2)... loses digits when
// the entries of X are close to -1).
// In: F(X) and F(X^T) (both already masked).  Out: F(inv) and F(inv^T).
// The levels are also available one by one (a caller that interleaves them with other work): tri_inverse_begin does
// block size 1 -> 2, tri_inverse_level<s> takes block size s -> 2s for s = 2, 4, 8.
__device__ __forceinline__ void tri_inverse_begin(f32x4 X, f32x4 XT, const Lane& L, f32x4& M, f32x4& MT) {
    const f32x4 eye = identity_f32(L);
    // level s = 1: inverse of [[1,0],[-x,1]] is [[1,0],[x,1]]
    M = eye;
    MT = eye;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        int row = L.n, col = 4 * L.g + r;             // entry of X (row > col)
        bool keep = (row >> 1) == (col >> 1) && (row & 1) == 1 && (col & 1) == 0;
        M[r] += keep ? X[r] : 0.f;
        int rowT = 4 * L.g + r, colT = L.n;           // XT[n][4g+r] = X[4g+r][n]
        bool keepT = (rowT >> 1) == (colT >> 1) && (rowT & 1) == 1 && (colT & 1) == 0;
        MT[r] += keepT ? XT[r] : 0.f;
    }
}
template <int s>
__device__ __forceinline__ void tri_inverse_level(f32x4 X, const Lane& L, f32x4& M, f32x4& MT) {
    f32x4 Xs;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        int row = L.n, col = 4 * L.g + r;
        bool keep = (row / (2 * s)) == (col / (2 * s)) && ((row / s) & 1) == 1 && ((col / s) & 1) == 0;
        Xs[r] = keep ? X[r] : 0.f;
    }
    // Every product on the bf16 matrix instruction with each operand split into a bf16 value and the bf16 of what that
    // leaves (x = hi + lo to ~16 bits; the lo * lo term is dropped): three instructions of 16 cycles per product where
    // the fp32 instruction needs four of 32, and these products are one long dependent chain.
    auto lo = [](f32x4 x, bf16x4 h) { return to_bf16(x - to_f32(h)); };
    const bf16x4 Mh = to_bf16(M), MTh = to_bf16(MT), Xh = to_bf16(Xs);
    const bf16x4 Ml = lo(M, Mh), MTl = lo(MT, MTh), Xl = lo(Xs, Xh);
    // P = Xs * M.   F(P^T) = F(M^T * Xs^T) = mma(A = F(Xs), B = F(M^T))
    const f32x4 PT = mma(mma(mma(zero4(), Xl, MTh), Xh, MTl), Xh, MTh);
    const bf16x4 PTh = to_bf16(PT), PTl = lo(PT, PTh);
    // F(M * P) = F(M * (P^T)^T) = mma(A = F(P^T), B = F(M));  F((M*P)^T) = F(P^T * M^T) = mma(A = F(M), B = F(P^T))
    const f32x4 Mn = mma(mma(mma(M, PTl, Mh), PTh, Ml), PTh, Mh);
    const f32x4 MTn = mma(mma(mma(MT, Ml, PTh), Mh, PTl), Mh, PTh);
    M = Mn;
    MT = MTn;
}
__device__ __forceinline__ void tri_inverse(f32x4 X, f32x4 XT, const Lane& L, f32x4& M, f32x4& MT) {
    tri_inverse_begin(X, XT, L, M, MT);
    tri_inverse_level<2>(X, L, M, MT);
    tri_inverse_level<4>(X, L, M, MT);
    tri_inverse_level<8>(X, L, M, MT);
}

// One wavefront per chunk, handed out head-major: wavefronts that run side by side take the same 16 tokens of
// consecutive (batch, head) pairs, whose rows are neighbours in memory (128 bytes each of a token's row), instead of
// consecutive chunks of one head.  i: the wavefront's index in the grid; returns the chunk id (batch*H + head)*NC + c.
__device__ __forceinline__ int head_major_chunk(int i, int nchunks, int T) {
    const int NC = T / CHUNK, BH = nchunks / NC;
    const int c = i / BH, bh = i - c * BH;
    return bh * NC + c;
}

}  // namespace wkv
