// Shared pieces of the WKV7 kernels: chunk addressing, decay factors, workspace layout.
//
// Semantics follow the reference's chunked algebra (rwkv7_attn_triton.py:27-69 forward,
// :72-156 backward; attn.cu:48-101, 177-321) but the work is organised differently: every chunk
// of 16 tokens is handled by ONE autonomous wavefront (no block barriers, no LDS), and the only
// sequential part - carrying the 64x64 state from chunk to chunk - is a separate light scan.
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
// lw = -exp(w) is the log of the per-step decay; Lc its inclusive prefix sum over the chunk's tokens
// (fp32, so the products P = exp(Lc), 1/P = exp(-Lc) are formed from one accurately summed exponent).
struct Decay {
    TileF lw, Lc, Ltot;
};
__device__ __forceinline__ Decay chunk_decay(const TileB& w) {
    Decay d;
#pragma unroll
    for (int i = 0; i < NBLK; i++) {
        f32x4 wf = to_f32(w.f[i]);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float lw = -__expf(wf[r]);
            float lc = row_prefix_sum(lw);
            d.lw.f[i][r] = lw;
            d.Lc.f[i][r] = lc;
            d.Ltot.f[i][r] = row_bcast(lc, 15);
        }
    }
    return d;
}

// x * exp(e), elementwise over a tile
__device__ __forceinline__ TileF mul_exp(const TileB& x, const TileF& e) {
    TileF r;
#pragma unroll
    for (int i = 0; i < NBLK; i++) {
        f32x4 xf = to_f32(x.f[i]);
#pragma unroll
        for (int j = 0; j < 4; j++) r.f[i][j] = xf[j] * __expf(e.f[i][j]);
    }
    return r;
}
__device__ __forceinline__ TileF sub(const TileF& a, const TileF& b) {
    TileF r;
#pragma unroll
    for (int i = 0; i < NBLK; i++) r.f[i] = a.f[i] - b.f[i];
    return r;
}
__device__ __forceinline__ TileF neg(const TileF& a) {
    TileF r;
#pragma unroll
    for (int i = 0; i < NBLK; i++) r.f[i] = -a.f[i];
    return r;
}

// State tensors [B,H,64,64] (value row i, key column j) in the caller's layout, fp32 or bf16.
// Fragment F(S[16*ib.., 16*jb..]) : lane (n,g) holds S[16*ib+n][16*jb+4g+r].
__device__ __forceinline__ f32x4 load_state_frag(const void* s, int state_f32, int bh, int ib, int jb, const Lane& L) {
    long off = ((long)bh * HEAD + 16 * ib + L.n) * HEAD + 16 * jb + 4 * L.g;
    if (state_f32) return *reinterpret_cast<const f32x4*>(static_cast<const float*>(s) + off);
    return to_f32(*reinterpret_cast<const bf16x4*>(static_cast<const __bf16*>(s) + off));
}
__device__ __forceinline__ void store_state_frag(void* s, int state_f32, int bh, int ib, int jb, const Lane& L, f32x4 v) {
    long off = ((long)bh * HEAD + 16 * ib + L.n) * HEAD + 16 * jb + 4 * L.g;
    if (state_f32) *reinterpret_cast<f32x4*>(static_cast<float*>(s) + off) = v;
    else *reinterpret_cast<bf16x4*>(static_cast<__bf16*>(s) + off) = to_bf16(v);
}

// ---- workspace for one direction of the scan (sizes in bf16 elements per chunk) ----
// Five tiles per chunk in fragment order plus 64 floats:
//   A   F(A[:,16jb..])    lane = token, reg = key channel   (forward: Wm = Tinv*wa ; backward: Bm = Tinv^T*bf)
//   KT  F(K[:,16jb..]^T)  lane = key channel, reg = token   (forward: kf = k*E      ; backward: wq)
//   BT  F(B[:,16jb..]^T)  lane = key channel, reg = token   (forward: bf = b*E      ; backward: wa)
//   UT  F(U0[:,16ib..]^T) lane = value channel, reg = token (forward: Tinv*AK*V     ; backward: Tinv^T*QB^T*dY)
//   VT  F(V[:,16ib..]^T)  lane = value channel, reg = token (forward: v             ; backward: dy)
//   FW  fw[j] = exp(sum of the chunk's log decays), fp32
struct ScanWs {
    __bf16 *A, *KT, *BT, *UT, *VT;
    float* FW;
};
constexpr size_t SCAN_WS_BYTES_PER_CHUNK = 5 * TILE_ELEMS * sizeof(__bf16) + HEAD * sizeof(float);

__host__ __device__ inline ScanWs carve_scan_ws(void* base, long nchunks) {
    ScanWs w;
    __bf16* p = static_cast<__bf16*>(base);
    w.A = p;  p += nchunks * TILE_ELEMS;
    w.KT = p; p += nchunks * TILE_ELEMS;
    w.BT = p; p += nchunks * TILE_ELEMS;
    w.UT = p; p += nchunks * TILE_ELEMS;
    w.VT = p; p += nchunks * TILE_ELEMS;
    w.FW = reinterpret_cast<float*>(p);
    return w;
}

// The tensor saved for backward ("s" in the reference's Function, rwkv7_attn.py:9,33) holds per chunk
// the chunk-start state as bf16 fragments [ib][jb] (16 fragments = 8 KiB) and U^T as 4 fragments (2 KiB).
constexpr long CKPT_ELEMS = 16 * FRAG_ELEMS;
constexpr long SAVED_ELEMS_PER_CHUNK = CKPT_ELEMS + TILE_ELEMS;

}  // namespace wkv
