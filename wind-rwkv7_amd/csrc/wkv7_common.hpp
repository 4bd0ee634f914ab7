// Shared pieces of the WKV7 kernels: chunk addressing, decay factors, workspace layout.
//
// Semantics follow the reference's chunked algebra (rwkv7_attn_triton.py:27-69 forward,
// :72-156 backward; attn.cu:48-101, 177-321) but the work is organised differently: per direction one kernel
// whose producer wavefronts prepare the 16-token chunks while its chain wavefronts carry the 64x64 state from
// chunk to chunk (wkv7_fused.hip), then a chunk-parallel gradient kernel in which a wavefront handles pairs of
// chunks on its own (wkv7_bwd.hip).
#pragma once
#include "frag.hpp"

namespace wkv {

// One chunk = 16 tokens of one (batch, head).  cid = (b*H + h)*NC + c.
struct ChunkAddr {
    int cid, bh, c;
    long row0;  // element offset of token 0 of the chunk, channel 0 of the head, in a [B,T,H,64] tensor
    long ld;    // elements between consecutive tokens
    __device__ ChunkAddr(int cid_, int T, int H) {
        int NC = T / CHUNK;
        cid = cid_;
        bh = cid / NC;
        c = cid - bh * NC;
        int b = bh / H, h = bh - b * H;
        ld = (long)H * HEAD;
        row0 = ((long)b * T + (long)c * CHUNK) * ld + (long)h * HEAD;
    }
};

// Per-chunk decay factors for the 16 channels this lane holds of token row n.
// lw = -exp(w) is the log of the per-step decay; Lc its inclusive prefix sum over the chunk's tokens, kept in
// fp32 so that every product below comes from one accurately summed exponent:
//   P  = exp(Lc)        decay from the chunk start up to and including token n
//   Pi = exp(-Lc)       its reciprocal (its own exponential, not a division)
//   Px = P of token n-1 (1 at the first token): the decay up to but excluding token n - a lane shift of P
//   fw = P of token 15  the whole chunk's decay - a lane broadcast of P
//   E  = fw * Pi        decay from token n (exclusive) to the chunk end
// Transcendentals cost four issue slots each on this hardware, so only lw, P and Pi use one.
struct Decay {
    TileF lw, P, Pi, Px, fw;
};
__device__ __forceinline__ Decay chunk_decay(const TileB& w) {
    Decay d;
    constexpr float LOG2E = 1.4426950408889634f;
#pragma unroll
    for (int i = 0; i < NBLK; i++) {
        const f32x4 wf = to_f32(w.f[i]);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float lw = -__expf(wf[r]);
            const float lc2 = row_prefix_sum(lw) * LOG2E;
            const float P = __builtin_amdgcn_exp2f(lc2);
            d.lw.f[i][r] = lw;
            d.P.f[i][r] = P;
            d.Pi.f[i][r] = __builtin_amdgcn_exp2f(-lc2);
            d.Px.f[i][r] = __builtin_bit_cast(
                float, __builtin_amdgcn_update_dpp(0x3f800000, __builtin_bit_cast(int, P), 0x111, 0xf, 0xf, false));
            d.fw.f[i][r] = row_bcast_last(P);
        }
    }
    return d;
}

// x * f, elementwise over a tile (x bf16, f fp32)
__device__ __forceinline__ TileF mul(const TileB& x, const TileF& f) {
    TileF r;
#pragma unroll
    for (int i = 0; i < NBLK; i++) r.f[i] = to_f32(x.f[i]) * f.f[i];
    return r;
}
__device__ __forceinline__ TileF mul(const TileF& x, const TileF& f) {
    TileF r;
#pragma unroll
    for (int i = 0; i < NBLK; i++) r.f[i] = x.f[i] * f.f[i];
    return r;
}

// State tensors [B,H,64,64] (value row i, key column j) in the caller's layout, fp32 or bf16.
// Fragment (ib, jb) of a state: lane (n,g) holds S[chan16(ib, n)][chan16(jb, 4g) + r] - the kernels' tiles are
// loaded with load_rows16, so block indices follow its interleaved channel order.
// A null state reads as zero (a sequence that starts from nothing, a final state nobody differentiates) and a null
// destination is not written; the pointer is the same in every lane, so the test is a scalar branch.
__device__ __forceinline__ f32x4 load_state_frag(const void* s, int state_f32, int bh, int ib, int jb, const Lane& L) {
    if (s == nullptr) return zero4();
    long off = ((long)bh * HEAD + chan16(ib, L.n)) * HEAD + chan16(jb, 4 * L.g);
    if (state_f32) return *reinterpret_cast<const f32x4*>(static_cast<const float*>(s) + off);
    return to_f32(*reinterpret_cast<const bf16x4*>(static_cast<const __bf16*>(s) + off));
}
__device__ __forceinline__ void store_state_frag(void* s, int state_f32, int bh, int ib, int jb, const Lane& L, f32x4 v) {
    if (s == nullptr) return;
    long off = ((long)bh * HEAD + chan16(ib, L.n)) * HEAD + chan16(jb, 4 * L.g);
    if (state_f32) *reinterpret_cast<f32x4*>(static_cast<float*>(s) + off) = v;
    else *reinterpret_cast<bf16x4*>(static_cast<__bf16*>(s) + off) = to_bf16(v);
}

// What a direction's scan leaves in memory for bwd_grads_kernel, per chunk: the state entering the chunk (backward:
// the dstate arriving at its end) as 16 bf16 fragments - per value block ib 2048 B, per lane 16 bf16 = fragments
// F(S[16ib.., 16jb..]) for jb = 0..3 (lane = value row, reg = key column) - then F(U_ib^T), ib = 0..3 (backward
// dab_u^T; lane = value ch, reg = token).
struct Saved {   // offsets in bf16 elements
    static constexpr long CKPT = 0;
    static constexpr long UT = 16 * FRAG_ELEMS;
    static constexpr long ELEMS = UT + TILE_ELEMS;
    static constexpr size_t BYTES = ELEMS * sizeof(__bf16);   // 10240
    __host__ __device__ static long ckpt(long cid, int ib) { return cid * ELEMS + CKPT + (long)ib * TILE_ELEMS; }
    __host__ __device__ static long ut(long cid) { return cid * ELEMS + UT; }
};

// The backward direction keeps the dstate only every SECOND chunk (32 tokens): the gradient kernel handles the two chunks
// of a pair one after the other and carries the dstate across the boundary between them itself (one more 64x64 update
// from operands it has anyway).  Per pair of chunks (2p, 2p+1) of a (batch, head): the dstate arriving at the END of
// the pair's last chunk, 16 bf16 fragments as in Saved, then dab_u^T of chunk 2p and of chunk 2p+1.
struct SavedPair {   // offsets in bf16 elements
    static constexpr long DS = 0;
    static constexpr long UT = 16 * FRAG_ELEMS;
    static constexpr long ELEMS = UT + 2 * TILE_ELEMS;
    static constexpr size_t BYTES = ELEMS * sizeof(__bf16);   // 12288
    __host__ __device__ static int pairs(int NC) { return (NC + 1) / 2; }
    // pid = (batch, head) * pairs(NC) + p;  c = chunk within the sequence
    __host__ __device__ static long ds(long pid, int ib) { return pid * ELEMS + DS + (long)ib * TILE_ELEMS; }
    __host__ __device__ static long ut(long pid, int c) { return pid * ELEMS + UT + (long)(c & 1) * TILE_ELEMS; }
    // whether the dstate arriving at the end of chunk c is kept: the second chunk of a pair, or a last chunk without partner
    __host__ __device__ static bool keeps(int c, int NC) { return (c & 1) || c == NC - 1; }
    // The gradient kernel's wavefronts take RUNS of `run` consecutive pairs (pair ids run*r .. run*r + run - 1, from
    // the last one down) and carry the dstate from a pair to the one before it themselves, as they do inside a pair.
    // So the reverse scan keeps the dstate only where a run starts: at the end of the last pair of every run, and of
    // the last pair of every (batch, head), since a run does not carry across heads.  pid = (batch, head) * NP + p.
    // run > 0: runs cut the flattened pair ids (every wavefront gets the same number of pairs whatever NP is);
    // run < 0: runs of -run pairs cut each (batch, head)'s pairs on their own, and wavefronts that run side by side take
    // the same run of consecutive heads (see bwd_grads_kernel).
    __host__ __device__ static bool ds_kept(long pid, int p, int NP, int run) {
        const int r = run < 0 ? -run : run;
        return r == 1 || (run < 0 ? p : pid) % r == r - 1 || p == NP - 1;
    }
};

// 16 bf16 per lane, contiguous (two 16-byte accesses)
__device__ __forceinline__ TileB load_lane16(const __bf16* __restrict__ p, int lane) {
    TileB t;
    const bf16x8* q = reinterpret_cast<const bf16x8*>(p + (long)lane * 16);
    const bf16x8 lo = q[0], hi = q[1];
    t.f[0] = __builtin_shufflevector(lo, lo, 0, 1, 2, 3);
    t.f[1] = __builtin_shufflevector(lo, lo, 4, 5, 6, 7);
    t.f[2] = __builtin_shufflevector(hi, hi, 0, 1, 2, 3);
    t.f[3] = __builtin_shufflevector(hi, hi, 4, 5, 6, 7);
    return t;
}
__device__ __forceinline__ void store_lane16(__bf16* __restrict__ p, int lane, const TileB& t) {
    bf16x8* q = reinterpret_cast<bf16x8*>(p + (long)lane * 16);
    q[0] = __builtin_shufflevector(t.f[0], t.f[1], 0, 1, 2, 3, 4, 5, 6, 7);
    q[1] = __builtin_shufflevector(t.f[2], t.f[3], 0, 1, 2, 3, 4, 5, 6, 7);
}
// the (U0^T, V^T) pair of one value block: 8 bf16 per lane
__device__ __forceinline__ void store_pair(__bf16* __restrict__ p, int lane, bf16x4 u, bf16x4 v) {
    *reinterpret_cast<bf16x8*>(p + (long)lane * 8) = __builtin_shufflevector(u, v, 0, 1, 2, 3, 4, 5, 6, 7);
}

// attn_ln: dparams[p][h*64 + ch] = sum over batches and chunks of the per-chunk partials ([chunk][3][64] floats), in a
// fixed order (the reference accumulates these with atomicAdd, attn_ln.cu:450-463, so its sums are order-dependent).
// The work of one block for one (head, parameter): 64 channels x `groups` strided partial sums (one wavefront each),
// combined through `red` ([groups][64] floats of LDS).
__device__ __forceinline__ void dparams_reduce_block(int B, int H, int NC, const float* __restrict__ part,
                                                     float* __restrict__ dparams, int h, int p, float* red, int groups) {
    const int ch = threadIdx.x & 63, grp = threadIdx.x >> 6;
    float acc = 0.f;
    for (int bi = 0; bi < B; bi++) {
        const long cid0 = ((long)bi * H + h) * NC;
#pragma unroll 4
        for (int c = grp; c < NC; c += groups) acc += part[((cid0 + c) * 3 + p) * HEAD + ch];
    }
    red[grp * HEAD + ch] = acc;
    __syncthreads();
    if (grp == 0) {
        float s = 0.f;
        for (int g = 0; g < groups; g++) s += red[g * HEAD + ch];
        dparams[(long)p * H * HEAD + (long)h * HEAD + ch] = s;
    }
}

}  // namespace wkv
