// Host-side launchers of the WKV7 device kernels (internal to the library; the public surface is
// include/wind_rwkv7.h).  All pointers are device pointers; nothing here allocates or synchronises.
#pragma once
#include <hip/hip_runtime.h>

namespace wkv {

// Long sequences on few (batch, head) pairs run as segments (scan_segments > 1), which needs
// scan_segment_workspace_bytes of scratch (seg_ws, 256-byte aligned; unused and may be null otherwise).
int scan_segments(int B, int T, int H);
size_t scan_segment_workspace_bytes(int B, int T, int H);
// One launch for chunk preparation + state scan (wkv7_fused.hip).  `saved`: B*H*(T/16) records of Saved::BYTES, or with
// `paired` (an even number of chunks) one SavedPair per 32 tokens: the state entering the pair and U^T of both chunks
// (forward: may be null, then nothing is kept for a backward pass).  params != nullptr: attn_ln - y receives
// (group_norm(y_wkv) * ln_w + ln_b + (q.k.bonus) v) * g and, if saved, y_wkv the plain output for the backward pass,
// centred per token and block of 16 channels, with the centres in `centers` ([B*T*H][4] floats; see ln_epilogue.hpp).
// params == nullptr with centers != nullptr: the plain forward whose y is that kept output (the epilogue follows as
// a kernel of its own): y is written centred.
void launch_fused_forward(int B, int T, int H, int state_f32, const void* w, const void* q, const void* k, const void* v,
                          const void* a, const void* b, const void* s_in, void* s_out, void* y, void* saved,
                          int paired, hipStream_t stream, const void* g = nullptr, const void* params = nullptr,
                          void* y_wkv = nullptr, float* centers = nullptr, void* seg_ws = nullptr);
// Long sequences on few heads (scan_segments(B, T, H) > 1; not with params): the two launchers above and below run the
// sequence as that many segments per (batch, head) - a first launch of the same kernel leaves each segment's affine
// map, segment_carry composes them, then the kernel proper starts every segment from the state entering it.  seg_ws:
// scan_segment_workspace_bytes(B, T, H) of scratch.
void launch_segment_carry(int BH, int nseg, int state_f32, const void* s_in, const float* maps, float* s_seg,
                          hipStream_t stream);
// dparams != nullptr (attn_ln; only where fused_backward_scan_takes_dparams: the scan leaves that many compute units
// idle): the launch also carries the blocks of launch_dparams_reduce, which then is not called.
bool fused_backward_scan_takes_dparams(int B, int T, int H);
// How many consecutive pairs of chunks a wavefront of the gradient kernel takes as one run after the fused reverse scan
// with a state per pair (SavedPair::ds_kept): 6, 3 or 1, whichever leaves the wavefronts the least uneven; negative
// for runs that are cut per (batch, head) and handed out head-major (16 heads or more: their rows are long).
int dstate_run(int B, int T, int H);
void launch_fused_backward_scan(int B, int T, int H, int state_f32, const void* w, const void* q, const void* a,
                                const void* b, const void* dy, const void* ds_in, void* ds_out, void* saved,
                                int paired, hipStream_t stream, const float* dparams_part = nullptr,
                                float* dparams = nullptr, void* seg_ws = nullptr);
// attn_ln: y = (group_norm(y_wkv) * ln_w + ln_b + (q.k.bonus) v) * g; centers: the centres y_wkv was kept with, or null
void launch_ln_epilogue(int B, int T, int H, const void* y_wkv, const float* centers, const void* q, const void* k,
                        const void* v, const void* g, const void* params, void* y, hipStream_t stream);

// Buffers of the attn_ln epilogue's backward (see LnBwdArgs in wkv7_bwd.hip).
struct LnBackwardBuffers {
    const void *k, *v, *g, *y_wkv, *params;
    const float* centers;   // of y_wkv, or null
    void *dg, *dY, *dv;
    float *ddot, *dparams_part;
};
// attn_ln: backward of the epilogue; dy is the gradient of the attn_ln output, ln.dY receives the gradient of the
// plain WKV7 output, which the two launches below then take as their dy.
void launch_ln_epilogue_bwd(int B, int T, int H, const void* q, const void* dy, const LnBackwardBuffers& ln,
                            hipStream_t stream);
// ln_params != nullptr: add the bonus term's gradients (dv must already hold its bonus part).
// fused: 1 = the scans left a state per chunk (Saved) in both directions; 3 = a state per pair of chunks in both
// (SavedPair both; an even number of chunks).
void launch_bwd_grads(int B, int T, int H, const void* w, const void* q, const void* k, const void* v, const void* a,
                      const void* b, const void* dy, const void* rec_fwd, const void* rec_bwd,
                      void* dw, void* dq, void* dk, void* dv, void* da, void* db, int fused, hipStream_t stream,
                      const float* ln_params = nullptr, const float* ln_ddot = nullptr);
// One token per sequence on a resident state (updated in place); params != nullptr adds the attn_ln epilogue.
void launch_decode(int B, int H, int state_f32, const void* w, const void* q, const void* k, const void* v, const void* a,
                   const void* b, void* state, void* y, hipStream_t stream, const void* g = nullptr,
                   const void* params = nullptr);
void launch_dparams_reduce(int B, int T, int H, const float* part, float* dparams, hipStream_t stream);

}  // namespace wkv
