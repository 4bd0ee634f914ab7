// C ABI of the library (declared in include/wind_rwkv7.h): host-side validation and kernel sequencing.
#include "../../include/wind_rwkv7.h"

#include <stdint.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "device_info.hpp"
#include "wkv7_common.hpp"
#include "wkv7_kernels.hpp"
#include "wkv7_wide_kernels.hpp"
#include "ddlerp_kernels.hpp"
#include "expand_loras_kernels.hpp"
#include "ln_epilogue_heads_kernels.hpp"
#include "linear_kernels.hpp"
#include "wkv7_f32_kernels.hpp"
#include "mixer_decode_kernels.hpp"

// ---- device-resident scratch for the entry point that allocates nothing (wind_rwkv7_attn_prefill_static) ----
// One array per GPU, part of the code object: each device that loads the library holds its own copy at its own
// address until the process ends.  In host code the array's NAME is only a handle for hipGetSymbolAddress - the
// device address is looked up once per device (with that device current) and only that pointer is ever handed to a
// kernel, a copy or a memset.
static __device__ __align__(256) unsigned char scratch[WIND_RWKV7_STATIC_SCRATCH_BYTES];

namespace {

constexpr size_t ALIGN = 256;
inline size_t align_up(size_t x) { return (x + ALIGN - 1) / ALIGN * ALIGN; }

int check_shape(int B, int T, int H, int C, bool any_head = false) {
    if (B <= 0 || T <= 0 || H <= 0 || C <= 0) return WIND_RWKV7_ERR_BAD_SHAPE;
    // any_head: the plain WKV7 entry points, which have kernels for other head sizes as well
    if (!(any_head ? wind_rwkv7_attn_head_size_supported(C) : wind_rwkv7_head_size_supported(C))) return WIND_RWKV7_ERR_HEAD_SIZE;
    if (T % wkv::CHUNK != 0) return WIND_RWKV7_ERR_SEQ_MULTIPLE;
    // element counts must fit the 32-bit chunk index used on the device
    const long long nchunks = (long long)B * H * (T / wkv::CHUNK);
    if (nchunks > (1LL << 30)) return WIND_RWKV7_ERR_BAD_SHAPE;
    // the one-kernel organisation addresses a batch element's rows of a tensor with 32-bit byte offsets
    if (C == wkv::HEAD && (long long)T * H * C * 2 >= (1LL << 31)) return WIND_RWKV7_ERR_BAD_SHAPE;
    return WIND_RWKV7_OK;
}

int check_dtypes(int io_dtype, int state_dtype) {
    if (io_dtype != WIND_RWKV7_BF16) return WIND_RWKV7_ERR_DTYPE;
    if (state_dtype != WIND_RWKV7_BF16 && state_dtype != WIND_RWKV7_F32) return WIND_RWKV7_ERR_DTYPE;
    return WIND_RWKV7_OK;
}

int check_workspace(const void* ws, size_t have, size_t need) {
    if (ws == nullptr) return WIND_RWKV7_ERR_WORKSPACE;
    if (have < need) return WIND_RWKV7_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(ws) % ALIGN != 0) return WIND_RWKV7_ERR_WORKSPACE;
    return WIND_RWKV7_OK;
}

inline long long chunks(int B, int T, int H) { return (long long)B * H * (T / wkv::CHUNK); }
// One organisation for head size 64: blocks that prepare and scan in one launch (operands through LDS), one or two per
// (batch, head), or for long sequences on few heads one or two per segment of a (batch, head)'s sequence.  What one
// direction leaves in memory per chunk: a state + U^T.
// With an even number of chunks the kernels keep a state only per pair of chunks, in both directions: the
// forward the state entering the pair (the gradient kernel advances it across the pair's first chunk itself), the
// backward the dstate arriving at its end.
std::atomic<int> g_checkpoint_tokens{2 * wkv::CHUNK};   // wind_rwkv7_set_checkpoint_interval
inline bool pair_states(int B, int T, int H) {
    (void)B, (void)H;
    return g_checkpoint_tokens.load(std::memory_order_relaxed) == 2 * wkv::CHUNK && (T / wkv::CHUNK) % 2 == 0;
}
// (the forward's is the tensor saved for backward; callers size it per chunk - linear in B, H and T / 16, also for
// shapes they only know symbolically - so it has ONE per-chunk size, that of the larger layout, 10 KiB per chunk; with
// a state per pair the kernels use the first 12 KiB per pair of chunks of it)
inline size_t rec_fwd_bytes(int B, int T, int H) { return align_up((size_t)chunks(B, T, H) * wkv::Saved::BYTES); }
inline size_t rec_bwd_bytes(int B, int T, int H, bool ln = false) {
    (void)ln;
    if (pair_states(B, T, H)) return align_up((size_t)B * H * wkv::SavedPair::pairs(T / wkv::CHUNK) * wkv::SavedPair::BYTES);
    return align_up((size_t)chunks(B, T, H) * wkv::Saved::BYTES);
}
// the forward needs scratch only when the scan runs in segments; the argument is always checked
inline size_t seg_bytes(int B, int T, int H) { return align_up(wkv::scan_segment_workspace_bytes(B, T, H)); }
inline size_t fwd_ws_bytes(int B, int T, int H) { const size_t s = seg_bytes(B, T, H); return s ? s : 256; }

// ---- optional per-kernel timing (process-global, measurement only) ----
struct Profile {
    bool on = false;
    hipEvent_t ev[2][WIND_RWKV7_PROFILE_SLOTS + 1];
    const char* name[2][WIND_RWKV7_PROFILE_SLOTS] = {};   // what ran between events i and i+1 in the last call
    int count[2] = {0, 0};
};
Profile g_prof;

struct Stamp {
    int dir, i = 0;
    hipStream_t stream;
    Stamp(int d, hipStream_t s) : dir(d), stream(s) { mark(nullptr); }
    // `what`: the kernel(s) launched since the previous mark
    void mark(const char* what) {
        if (g_prof.on && i <= WIND_RWKV7_PROFILE_SLOTS) {
            (void)hipEventRecord(g_prof.ev[dir][i], stream);
            if (i > 0) g_prof.name[dir][i - 1] = what;
            g_prof.count[dir] = i;
            i++;
        }
    }
};

inline size_t seq_bytes(int B, int T, int H) { return align_up((size_t)B * T * H * wkv::HEAD * 2); }
// attn_ln keeps the plain WKV7 output centred per token and block of 16 channels: four floats per token and head
inline size_t centers_bytes(int B, int T, int H) { return align_up((size_t)B * T * H * 4 * sizeof(float)); }
inline size_t ddot_bytes(int B, int T, int H) { return align_up((size_t)chunks(B, T, H) * wkv::CHUNK * sizeof(float)); }
inline size_t dpart_bytes(int B, int T, int H) { return align_up((size_t)chunks(B, T, H) * 3 * wkv::HEAD * sizeof(float)); }

int launch_status() { return hipGetLastError() == hipSuccess ? WIND_RWKV7_OK : WIND_RWKV7_ERR_LAUNCH; }


constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[MAX_DEVICES] = {};

// The current device's copy of `scratch`; nullptr if the runtime cannot name it.
void* static_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}

}  // namespace

extern "C" {

int wind_rwkv7_abi_version(void) { return WIND_RWKV7_ABI_VERSION; }

const char* wind_rwkv7_strerror(int code) {
    switch (code) {
        case WIND_RWKV7_OK: return "success";
        case WIND_RWKV7_ERR_NULL_POINTER: return "a required pointer is NULL";
        case WIND_RWKV7_ERR_BAD_SHAPE: return "B, T, H and C must be positive and the problem must fit the index range";
        case WIND_RWKV7_ERR_HEAD_SIZE: return "unsupported head size (64; the plain WKV7 entry points: multiples of 16 up to 128)";
        case WIND_RWKV7_ERR_SEQ_MULTIPLE: return "T must be a multiple of the chunk length (16)";
        case WIND_RWKV7_ERR_DTYPE: return "unsupported element type";
        case WIND_RWKV7_ERR_WORKSPACE: return "workspace is NULL, too small or not 256-byte aligned";
        case WIND_RWKV7_ERR_LAUNCH: return "HIP kernel launch failed";
        case WIND_RWKV7_ERR_RANK: return "unsupported LoRA rank";
        case WIND_RWKV7_ERR_CHANNELS: return "channel count must be a multiple of 64 and of the head size";
        case WIND_RWKV7_ERR_STATIC_LIMIT: return "the problem needs more scratch than the library's built-in device buffer holds";
        default: return "unknown error code";
    }
}

int wind_rwkv7_head_size_supported(int C) { return C == wkv::HEAD ? 1 : 0; }

int wind_rwkv7_attn_head_size_supported(int C) { return C == wkv::HEAD || wkv::wide::head_size_supported(C) ? 1 : 0; }

int wind_rwkv7_chunk_len(void) { return wkv::CHUNK; }

int wind_rwkv7_checkpoint_interval(void) { return g_checkpoint_tokens.load(std::memory_order_relaxed); }

int wind_rwkv7_set_checkpoint_interval(int tokens) {
    if (tokens != wkv::CHUNK && tokens != 2 * wkv::CHUNK) return WIND_RWKV7_ERR_BAD_SHAPE;
    g_checkpoint_tokens.store(tokens, std::memory_order_relaxed);
    return WIND_RWKV7_OK;
}

size_t wind_rwkv7_attn_saved_bytes(int B, int T, int H, int C) {
    if (check_shape(B, T, H, C, true) != WIND_RWKV7_OK) return 0;
    if (C != wkv::HEAD) return wkv::wide::kept_bytes(B, T, H, C);
    return rec_fwd_bytes(B, T, H);
}

size_t wind_rwkv7_attn_fwd_workspace_bytes(int B, int T, int H, int C) {
    if (check_shape(B, T, H, C, true) != WIND_RWKV7_OK) return 0;
    if (C != wkv::HEAD) return wkv::wide::record_bytes(B, T, H, C, true);
    return fwd_ws_bytes(B, T, H);
}

size_t wind_rwkv7_attn_bwd_workspace_bytes(int B, int T, int H, int C) {
    if (check_shape(B, T, H, C, true) != WIND_RWKV7_OK) return 0;
    if (C != wkv::HEAD) return wkv::wide::record_bytes(B, T, H, C, false) + wkv::wide::kept_bytes(B, T, H, C);
    return rec_bwd_bytes(B, T, H) + seg_bytes(B, T, H);
}

// wide_centers (head sizes other than 64 only): y is attn_ln's kept output and is written centred, the centres there
static int attn_forward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                        const void* w, const void* q, const void* k, const void* v,
                        const void* a, const void* b, const void* s0,
                        void* y, void* s, void* sT,
                        void* workspace, size_t workspace_bytes, int save, void* stream_, float* wide_centers = nullptr) {
    int rc = check_shape(B, T, H, C, true);
    if (rc) return rc;
    rc = check_dtypes(io_dtype, state_dtype);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !y || !s || !sT) return WIND_RWKV7_ERR_NULL_POINTER;   // (s0 may be null: a zero state)
    rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_attn_fwd_workspace_bytes(B, T, H, C));
    if (rc) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    Stamp st(0, stream);
    if (C != wkv::HEAD) {   // other head sizes: chunk records in the workspace, what backward needs in s
        wkv::wide::launch_forward(B, T, H, C, state_dtype == WIND_RWKV7_F32, w, q, k, v, a, b, s0, sT, y, workspace,
                                  save ? s : nullptr, stream, wide_centers);
        st.mark("wide::fwd_prepare_kernel + wide::scan_kernel[fwd]");
        return launch_status();
    }
    wkv::launch_fused_forward(B, T, H, state_dtype == WIND_RWKV7_F32, w, q, k, v, a, b, s0, sT, y, save ? s : nullptr,
                              pair_states(B, T, H), stream, nullptr, nullptr, nullptr, nullptr, workspace);
    st.mark("wkv7_fused_kernel[fwd]");
    return launch_status();
}

int wind_rwkv7_attn_forward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                            const void* w, const void* q, const void* k, const void* v,
                            const void* a, const void* b, const void* s0,
                            void* y, void* s, void* sT,
                            void* workspace, size_t workspace_bytes, void* stream) {
    return attn_forward(B, T, H, C, io_dtype, state_dtype, w, q, k, v, a, b, s0, y, s, sT, workspace, workspace_bytes, 1,
                        stream);
}

int wind_rwkv7_attn_prefill(int B, int T, int H, int C, int io_dtype, int state_dtype,
                            const void* w, const void* q, const void* k, const void* v,
                            const void* a, const void* b, const void* s0,
                            void* y, void* scratch, void* sT,
                            void* workspace, size_t workspace_bytes, void* stream) {
    return attn_forward(B, T, H, C, io_dtype, state_dtype, w, q, k, v, a, b, s0, y, scratch, sT, workspace,
                        workspace_bytes, 0, stream);
}

size_t wind_rwkv7_attn_prefill_static_bytes(int B, int T, int H, int C) {
    if (check_shape(B, T, H, C) != WIND_RWKV7_OK) return 0;
    // The query also looks up the current device's copy of the array (once per device), so that a caller who sizes its
    // problem before starting a graph capture has the lookup behind it; without a device it finds nothing and the
    // size is still returned.
    (void)static_scratch();
    return rec_fwd_bytes(B, T, H) + fwd_ws_bytes(B, T, H);
}

int wind_rwkv7_attn_prefill_static(int B, int T, int H, int C, int io_dtype, int state_dtype,
                                   const void* w, const void* q, const void* k, const void* v,
                                   const void* a, const void* b, const void* s0,
                                   void* y, void* sT, void* stream) {
    int rc = check_shape(B, T, H, C);
    if (rc) return rc;
    rc = check_dtypes(io_dtype, state_dtype);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !y || !sT) return WIND_RWKV7_ERR_NULL_POINTER;
    if (wind_rwkv7_attn_prefill_static_bytes(B, T, H, C) > (size_t)WIND_RWKV7_STATIC_SCRATCH_BYTES)
        return WIND_RWKV7_ERR_STATIC_LIMIT;
    char* base = static_cast<char*>(static_scratch());
    if (!base) return WIND_RWKV7_ERR_LAUNCH;
    // the records first (every byte the kernels read of them is written by this call's prepare kernel first), the
    // segment workspace behind them; nothing has to start at zero
    const size_t rec = rec_fwd_bytes(B, T, H);
    return attn_forward(B, T, H, C, io_dtype, state_dtype, w, q, k, v, a, b, s0, y, base, sT, base + rec,
                        fwd_ws_bytes(B, T, H), 0, stream);
}

int wind_rwkv7_attn_backward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                             const void* w, const void* q, const void* k, const void* v,
                             const void* a, const void* b,
                             const void* dy, const void* s, const void* dsT,
                             void* dw, void* dq, void* dk, void* dv, void* da, void* db, void* ds0,
                             void* workspace, size_t workspace_bytes, void* stream_) {
    int rc = check_shape(B, T, H, C, true);
    if (rc) return rc;
    rc = check_dtypes(io_dtype, state_dtype);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !dy || !s) return WIND_RWKV7_ERR_NULL_POINTER;   // (dsT may be null: zero)
    if (!dw || !dq || !dk || !dv || !da || !db) return WIND_RWKV7_ERR_NULL_POINTER;            // (ds0 may be null: not wanted)
    rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, C));
    if (rc) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    Stamp st(1, stream);
    if (C != wkv::HEAD) {
        wkv::wide::launch_backward(B, T, H, C, state_dtype == WIND_RWKV7_F32, w, q, k, v, a, b, dy, s, dsT, ds0, dw, dq, dk,
                                   dv, da, db, workspace,
                                   static_cast<char*>(workspace) + wkv::wide::record_bytes(B, T, H, C, false), stream);
        st.mark("wide::bwd_prepare_kernel + wide::scan_kernel[bwd] + wide::grads_kernel");
        return launch_status();
    }
    wkv::launch_fused_backward_scan(B, T, H, state_dtype == WIND_RWKV7_F32, w, q, a, b, dy, dsT, ds0, workspace,
                                    pair_states(B, T, H), stream, nullptr, nullptr,
                                    static_cast<char*>(workspace) + rec_bwd_bytes(B, T, H));
    st.mark("wkv7_fused_kernel[bwd]");
    wkv::launch_bwd_grads(B, T, H, w, q, k, v, a, b, dy, s, workspace, dw, dq, dk, dv, da, db,
                          pair_states(B, T, H) ? 3 : 1, stream);
    st.mark("bwd_grads_kernel");
    return launch_status();
}

// attn_ln at the head sizes other than 64: the plain operator's kernels for that head size and the epilogue kernels,
// composed here.  The saved tensor is what the plain backward needs followed by the WKV7 output; the backward
// workspace is the plain one, the epilogue's partial records and four sequences (the gradient of the WKV7 output and
// the bonus term's parts of dq, dk, dv, which are added to the plain backward's afterwards).
static size_t wide_seq_bytes(int B, int T, int H, int C) { return (size_t)B * T * H * C * 2; }
// the centres the kept WKV7 output of attn_ln is stored around: one float per token, head and block of 16 channels
static size_t wide_centers_bytes(int B, int T, int H, int C) { return (size_t)B * T * H * (C / 16) * sizeof(float); }
static size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

size_t wind_rwkv7_attn_ln_saved_bytes(int B, int T, int H, int C) {
    if (check_shape(B, T, H, C, true) != WIND_RWKV7_OK) return 0;
    if (C != wkv::HEAD) return wind_rwkv7_attn_saved_bytes(B, T, H, C) + wide_seq_bytes(B, T, H, C) + wide_centers_bytes(B, T, H, C);
    return rec_fwd_bytes(B, T, H) + seq_bytes(B, T, H) + centers_bytes(B, T, H);
}

size_t wind_rwkv7_attn_ln_fwd_workspace_bytes(int B, int T, int H, int C) {
    return wind_rwkv7_attn_fwd_workspace_bytes(B, T, H, C);
}

size_t wind_rwkv7_attn_ln_bwd_workspace_bytes(int B, int T, int H, int C) {
    if (check_shape(B, T, H, C, true) != WIND_RWKV7_OK) return 0;
    if (C != wkv::HEAD)
        return align256(wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, C)) +
               align256(wkv::lnheads::bwd_workspace_bytes((long)B * T, H, C)) + 4 * align256(wide_seq_bytes(B, T, H, C));
    return rec_bwd_bytes(B, T, H, true) + seg_bytes(B, T, H) + seq_bytes(B, T, H) + ddot_bytes(B, T, H) + dpart_bytes(B, T, H);
}

static int attn_ln_forward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                           const void* w, const void* q, const void* k, const void* v,
                           const void* a, const void* b, const void* g, const void* params,
                           const void* s0,
                           void* y, void* s, void* sT,
                           void* workspace, size_t workspace_bytes, int save, void* stream_) {
    int rc = check_shape(B, T, H, C, true);
    if (rc) return rc;
    rc = check_dtypes(io_dtype, state_dtype);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !g || !params || !y || !s || !sT) return WIND_RWKV7_ERR_NULL_POINTER;
    rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_attn_ln_fwd_workspace_bytes(B, T, H, C));
    if (rc) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (C != wkv::HEAD) {
        char* y_wide = static_cast<char*>(s) + wind_rwkv7_attn_saved_bytes(B, T, H, C);
        float* centers = reinterpret_cast<float*>(y_wide + wide_seq_bytes(B, T, H, C));
        rc = attn_forward(B, T, H, C, io_dtype, state_dtype, w, q, k, v, a, b, s0, y_wide, s, sT, workspace, workspace_bytes,
                          save, stream_, centers);
        if (rc) return rc;
        wkv::lnheads::launch_forward((long)B * T, H, C, y_wide, q, k, v, g, params, y, stream, centers);
        return launch_status();
    }
    char* y_wkv = static_cast<char*>(s) + rec_fwd_bytes(B, T, H);
    float* centers = reinterpret_cast<float*>(y_wkv + seq_bytes(B, T, H));
    Stamp st(0, stream);
    // While the plain forward kernel can give every (batch, head) two compute units (two blocks per head, which the
    // epilogue inside the kernel rules out: its statistics span the head, and its three wavefronts take the place of
    // four producers), the plain kernel followed by the epilogue kernel is the faster forward: 55 + 18 us against
    // 86 us at B=8, H=12, T=1024.  With more heads than that the one-kernel form wins (no y_wkv round trip).
    if (2 * B * H <= wkv::compute_units()) {
        wkv::launch_fused_forward(B, T, H, state_dtype == WIND_RWKV7_F32, w, q, k, v, a, b, s0, sT, y_wkv, save ? s : nullptr,
                                  pair_states(B, T, H), stream, nullptr, nullptr, nullptr, centers, workspace);
        st.mark("wkv7_fused_kernel[fwd]");
    } else {
        wkv::launch_fused_forward(B, T, H, state_dtype == WIND_RWKV7_F32, w, q, k, v, a, b, s0, sT, y, save ? s : nullptr,
                                  pair_states(B, T, H), stream,
                                  g, params, y_wkv, centers);
        st.mark("wkv7_fused_kernel[fwd]");
        return launch_status();
    }
    wkv::launch_ln_epilogue(B, T, H, y_wkv, centers, q, k, v, g, params, y, stream);
    st.mark("ln_epilogue_kernel");
    return launch_status();
}

int wind_rwkv7_attn_ln_forward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                               const void* w, const void* q, const void* k, const void* v,
                               const void* a, const void* b, const void* g, const void* params,
                               const void* s0,
                               void* y, void* s, void* sT,
                               void* workspace, size_t workspace_bytes, void* stream) {
    return attn_ln_forward(B, T, H, C, io_dtype, state_dtype, w, q, k, v, a, b, g, params, s0, y, s, sT, workspace,
                           workspace_bytes, 1, stream);
}

int wind_rwkv7_attn_ln_prefill(int B, int T, int H, int C, int io_dtype, int state_dtype,
                               const void* w, const void* q, const void* k, const void* v,
                               const void* a, const void* b, const void* g, const void* params,
                               const void* s0,
                               void* y, void* scratch, void* sT,
                               void* workspace, size_t workspace_bytes, void* stream) {
    return attn_ln_forward(B, T, H, C, io_dtype, state_dtype, w, q, k, v, a, b, g, params, s0, y, scratch, sT, workspace,
                           workspace_bytes, 0, stream);
}

int wind_rwkv7_attn_ln_backward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                                const void* w, const void* q, const void* k, const void* v,
                                const void* a, const void* b, const void* g, const void* params,
                                const void* dy, const void* s, const void* dsT,
                                void* dw, void* dq, void* dk, void* dv, void* da, void* db, void* dg,
                                void* dparams, void* ds0,
                                void* workspace, size_t workspace_bytes, void* stream_) {
    int rc = check_shape(B, T, H, C, true);
    if (rc) return rc;
    rc = check_dtypes(io_dtype, state_dtype);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !g || !params || !dy || !s) return WIND_RWKV7_ERR_NULL_POINTER;
    if (!dw || !dq || !dk || !dv || !da || !db || !dg || !dparams) return WIND_RWKV7_ERR_NULL_POINTER;
    rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_attn_ln_bwd_workspace_bytes(B, T, H, C));
    if (rc) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (C != wkv::HEAD) {
        const char* y_wide = static_cast<const char*>(s) + wind_rwkv7_attn_saved_bytes(B, T, H, C);
        const size_t plain_ws = wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, C);
        const size_t seq = align256(wide_seq_bytes(B, T, H, C));
        char* p = static_cast<char*>(workspace) + align256(plain_ws);
        char* ln_ws = p;
        p += align256(wkv::lnheads::bwd_workspace_bytes((long)B * T, H, C));
        char *dY = p, *dq2 = p + seq, *dk2 = p + 2 * seq, *dv2 = p + 3 * seq;
        wkv::lnheads::launch_backward((long)B * T, H, C, y_wide, q, k, v, g, params, dy, dY, dq2, dk2, dv2, dg, dparams, ln_ws,
                                      stream, reinterpret_cast<const float*>(y_wide + wide_seq_bytes(B, T, H, C)));
        rc = wind_rwkv7_attn_backward(B, T, H, C, io_dtype, state_dtype, w, q, k, v, a, b, dY, s, dsT, dw, dq, dk, dv, da, db,
                                      ds0, workspace, plain_ws, stream_);
        if (rc) return rc;
        void* const dst[3] = {dq, dk, dv};
        const void* const src[3] = {dq2, dk2, dv2};
        wkv::lnheads::launch_accumulate((long)B * T * H * C, dst, src, stream);
        return launch_status();
    }
    const char* y_wkv = static_cast<const char*>(s) + rec_fwd_bytes(B, T, H);
    char* rec = static_cast<char*>(workspace);
    char* seg_ws = rec + rec_bwd_bytes(B, T, H, true);
    char* dY = seg_ws + seg_bytes(B, T, H);
    float* ddot = reinterpret_cast<float*>(dY + seq_bytes(B, T, H));
    float* dpart = reinterpret_cast<float*>(reinterpret_cast<char*>(ddot) + ddot_bytes(B, T, H));
    const float* centers = reinterpret_cast<const float*>(y_wkv + seq_bytes(B, T, H));
    const wkv::LnBackwardBuffers ln{k, v, g, y_wkv, params, centers, dg, dY, dv, ddot, dpart};
    Stamp st(1, stream);
    wkv::launch_ln_epilogue_bwd(B, T, H, q, dy, ln, stream);
    st.mark("ln_epilogue_bwd_kernel");
    // the parameter-gradient partials are complete after the epilogue's backward: where the reverse scan leaves compute
    // units idle its launch reduces them too, else a launch of its own does at the end
    const bool reduce_in_scan = wkv::fused_backward_scan_takes_dparams(B, T, H);
    {
        wkv::launch_fused_backward_scan(B, T, H, state_dtype == WIND_RWKV7_F32, w, q, a, b, dY, dsT, ds0, rec,
                                        pair_states(B, T, H), stream, reduce_in_scan ? dpart : nullptr,
                                        reduce_in_scan ? static_cast<float*>(dparams) : nullptr, seg_ws);
        st.mark("wkv7_fused_kernel[bwd]");
    }
    wkv::launch_bwd_grads(B, T, H, w, q, k, v, a, b, dY, s, rec, dw, dq, dk, dv, da, db,
                          pair_states(B, T, H) ? 3 : 1, stream,
                          static_cast<const float*>(params), ddot);
    st.mark("bwd_grads_kernel");
    if (!reduce_in_scan) {
        wkv::launch_dparams_reduce(B, T, H, dpart, static_cast<float*>(dparams), stream);
        st.mark("dparams_reduce_kernel");
    }
    return launch_status();
}

static int check_decode(int B, int H, int C, int io_dtype, int state_dtype) {
    if (B <= 0 || H <= 0 || C <= 0 || (long long)B * H > (1LL << 30)) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (!wind_rwkv7_attn_head_size_supported(C)) return WIND_RWKV7_ERR_HEAD_SIZE;   // (the single-token kernels cover them all)
    return check_dtypes(io_dtype, state_dtype);
}

int wind_rwkv7_attn_decode(int B, int H, int C, int io_dtype, int state_dtype,
                           const void* w, const void* q, const void* k, const void* v,
                           const void* a, const void* b, void* state, void* y, void* stream_) {
    const int rc = check_decode(B, H, C, io_dtype, state_dtype);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !state || !y) return WIND_RWKV7_ERR_NULL_POINTER;
    if (C != wkv::HEAD)
        wkv::wide::launch_decode(B, H, C, state_dtype == WIND_RWKV7_F32, w, q, k, v, a, b, state, y, static_cast<hipStream_t>(stream_));
    else
        wkv::launch_decode(B, H, state_dtype == WIND_RWKV7_F32, w, q, k, v, a, b, state, y, static_cast<hipStream_t>(stream_));
    return launch_status();
}

int wind_rwkv7_attn_ln_decode(int B, int H, int C, int io_dtype, int state_dtype,
                              const void* w, const void* q, const void* k, const void* v,
                              const void* a, const void* b, const void* g, const void* params,
                              void* state, void* y, void* stream_) {
    const int rc = check_decode(B, H, C, io_dtype, state_dtype);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !g || !params || !state || !y) return WIND_RWKV7_ERR_NULL_POINTER;
    if (C != wkv::HEAD)
        wkv::wide::launch_decode(B, H, C, state_dtype == WIND_RWKV7_F32, w, q, k, v, a, b, state, y,
                                 static_cast<hipStream_t>(stream_), g, params);
    else
        wkv::launch_decode(B, H, state_dtype == WIND_RWKV7_F32, w, q, k, v, a, b, state, y, static_cast<hipStream_t>(stream_), g,
                           params);
    return launch_status();
}

static int check_mixer_decode(int B, int C, int H) {
    if (B <= 0 || C <= 0 || H <= 0 || (long long)B * C > (1LL << 30)) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (C != 64 * H) return WIND_RWKV7_ERR_HEAD_SIZE;
    return WIND_RWKV7_OK;
}

size_t wind_rwkv7_mixer_decode_workspace_bytes(int B, int C) {
    if (B <= 0 || C <= 0 || C % 64 != 0) return 0;
    return wkv::mixer_decode_workspace_bytes(B, C);
}

int wind_rwkv7_mixer_decode(int B, int C, int H, int state_dtype, const wind_rwkv7_mixer_weights* weights,
                            const void* x, const void* x_prev, void* state, void* y, void* x_carry,
                            void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_mixer_decode(B, C, H);
    if (rc) return rc;
    rc = check_dtypes(WIND_RWKV7_BF16, state_dtype);
    if (rc) return rc;
    if (!weights || !x || !x_prev || !state || !y) return WIND_RWKV7_ERR_NULL_POINTER;
    if (x_carry && x_carry == x_prev) return WIND_RWKV7_ERR_BAD_SHAPE;   // (every wavefront reads x_prev after others have stored)
    const void* const* wp = reinterpret_cast<const void* const*>(weights);
    for (size_t i = 0; i < sizeof(*weights) / sizeof(void*); i++)
        if (!wp[i]) return WIND_RWKV7_ERR_NULL_POINTER;
    rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_mixer_decode_workspace_bytes(B, C));
    if (rc) return rc;
    static_assert(sizeof(wkv::MixerWeights) == sizeof(wind_rwkv7_mixer_weights), "the two declarations list the same pointers");
    wkv::MixerWeights mw;
    memcpy(&mw, weights, sizeof(mw));
    wkv::launch_mixer_decode(B, C, H, state_dtype == WIND_RWKV7_F32, mw, x, x_prev, state, y, x_carry, workspace,
                             static_cast<hipStream_t>(stream));
    return launch_status();
}

static int check_ddlerp(int B, int T, int C, int D) {
    if (B <= 0 || T <= 0 || C <= 0 || D <= 0) return WIND_RWKV7_ERR_BAD_SHAPE;
    if ((long long)B * T * C > (1LL << 40)) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (T % 16 != 0) return WIND_RWKV7_ERR_SEQ_MULTIPLE;
    if (C % 64 != 0) return WIND_RWKV7_ERR_CHANNELS;
    if (!wkv::ddlerp_rank_supported(D)) return WIND_RWKV7_ERR_RANK;
    return WIND_RWKV7_OK;
}

int wind_rwkv7_ddlerp_rank_supported(int D) { return wkv::ddlerp_rank_supported(D) ? 1 : 0; }

size_t wind_rwkv7_ddlerp_bwd_workspace_bytes(int B, int T, int C, int D) {
    if (check_ddlerp(B, T, C, D) != WIND_RWKV7_OK) return 0;
    return wkv::ddlerp_bwd_workspace_bytes((long)B * T, C, D);
}

int wind_rwkv7_ddlerp_forward(int B, int T, int C, int D,
                              const void* x, const void* alpha, const void* L, const void* R, const void* beta,
                              void* bmid, void* bder, void* y, void* stream) {
    const int rc = check_ddlerp(B, T, C, D);
    if (rc) return rc;
    if (!x || !alpha || !L || !R || !beta || !bmid || !bder || !y) return WIND_RWKV7_ERR_NULL_POINTER;
    wkv::launch_ddlerp_forward((long)B * T, T, C, D, x, alpha, L, R, beta, bmid, bder, y,
                               static_cast<hipStream_t>(stream));
    return launch_status();
}

int wind_rwkv7_ddlerp_backward(int B, int T, int C, int D,
                               const void* x, const void* alpha, const void* L, const void* R, const void* beta,
                               const void* bmid, const void* bder,
                               const void* dy0, const void* dy1, const void* dy2, const void* dy3,
                               void* dx, void* dalpha, void* dL, void* dR, void* dbeta,
                               void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_ddlerp(B, T, C, D);
    if (rc) return rc;
    if (!x || !alpha || !L || !R || !beta || !bmid || !bder || !dy0 || !dy1 || !dy2 || !dy3) return WIND_RWKV7_ERR_NULL_POINTER;
    if (!dx || !dalpha || !dL || !dR || !dbeta) return WIND_RWKV7_ERR_NULL_POINTER;
    rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_ddlerp_bwd_workspace_bytes(B, T, C, D));
    if (rc) return rc;
    const void* const dy4[4] = {dy0, dy1, dy2, dy3};
    wkv::launch_ddlerp_backward((long)B * T, T, C, D, x, alpha, L, R, beta, bmid, bder, dy4, dx, dalpha, dL, dR, dbeta,
                                workspace, static_cast<hipStream_t>(stream));
    return launch_status();
}

static int check_loras(int B, int T, int C, int D, int head_size) {
    if (B <= 0 || T <= 0 || C <= 0 || D <= 0) return WIND_RWKV7_ERR_BAD_SHAPE;
    if ((long long)B * T * C > (1LL << 40)) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (head_size < 16 || head_size % 16 != 0) return WIND_RWKV7_ERR_HEAD_SIZE;
    if (T % 16 != 0) return WIND_RWKV7_ERR_SEQ_MULTIPLE;
    // the kernels work on blocks of 64 channels whatever the head size
    if (C % wkv::HEAD != 0 || !wkv::expand_loras_head_size_supported(C, head_size)) return WIND_RWKV7_ERR_CHANNELS;
    if (!wkv::expand_loras_rank_supported(D)) return WIND_RWKV7_ERR_RANK;
    return WIND_RWKV7_OK;
}

int wind_rwkv7_expand_loras_rank_supported(int D) { return wkv::expand_loras_rank_supported(D) ? 1 : 0; }

size_t wind_rwkv7_expand_loras_bwd_workspace_bytes(int B, int T, int C, int D) {
    if (check_loras(B, T, C, D, wkv::HEAD) != WIND_RWKV7_OK) return 0;
    return wkv::expand_loras_bwd_workspace_bytes((long)B * T, C, D);
}

int wind_rwkv7_expand_loras_forward(int B, int T, int C, int D, int head_size,
                                    const void* w_in, const void* k_in,
                                    const void* z_in, const void* a_in, const void* ma_in, const void* mk_in,
                                    const void* Wz, const void* Wa, const void* Wma, const void* Wmk,
                                    const void* w_bias, const void* a_bias, const void* ma_bias, const void* mk_bias,
                                    void* w_out, void* k_out, void* kk_out, void* b_out, void* stream) {
    const int rc = check_loras(B, T, C, D, head_size);
    if (rc) return rc;
    const void* const acts[4] = {z_in, a_in, ma_in, mk_in};
    const void* const Ws[4] = {Wz, Wa, Wma, Wmk};
    const void* const biases[4] = {w_bias, a_bias, ma_bias, mk_bias};
    void* const outs[4] = {w_out, k_out, kk_out, b_out};
    if (!w_in || !k_in) return WIND_RWKV7_ERR_NULL_POINTER;
    for (int i = 0; i < 4; i++)
        if (!acts[i] || !Ws[i] || !biases[i] || !outs[i]) return WIND_RWKV7_ERR_NULL_POINTER;
    wkv::launch_expand_loras_forward((long)B * T, C, D, head_size, w_in, k_in, acts, Ws, biases, outs, static_cast<hipStream_t>(stream));
    return launch_status();
}

int wind_rwkv7_expand_loras_backward(int B, int T, int C, int D, int head_size,
                                     const void* w_in, const void* k_in,
                                     const void* z_in, const void* a_in, const void* ma_in, const void* mk_in,
                                     const void* Wz, const void* Wa, const void* Wma, const void* Wmk,
                                     const void* w_bias, const void* a_bias, const void* ma_bias, const void* mk_bias,
                                     const void* dw_out, const void* dk_out, const void* dkk_out, const void* db_out,
                                     void* dw_in, void* dk_in,
                                     void* dz_in, void* da_in, void* dma_in, void* dmk_in,
                                     void* dWz, void* dWa, void* dWma, void* dWmk,
                                     void* dw_bias, void* da_bias, void* dma_bias, void* dmk_bias,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_loras(B, T, C, D, head_size);
    if (rc) return rc;
    const void* const acts[4] = {z_in, a_in, ma_in, mk_in};
    const void* const Ws[4] = {Wz, Wa, Wma, Wmk};
    const void* const biases[4] = {w_bias, a_bias, ma_bias, mk_bias};
    const void* const dys[4] = {dw_out, dk_out, dkk_out, db_out};
    void* const dacts[4] = {dz_in, da_in, dma_in, dmk_in};
    void* const dWs[4] = {dWz, dWa, dWma, dWmk};
    void* const dbiases[4] = {dw_bias, da_bias, dma_bias, dmk_bias};
    if (!w_in || !k_in || !dw_in || !dk_in) return WIND_RWKV7_ERR_NULL_POINTER;
    for (int i = 0; i < 4; i++)
        if (!acts[i] || !Ws[i] || !biases[i] || !dys[i] || !dacts[i] || !dWs[i] || !dbiases[i])
            return WIND_RWKV7_ERR_NULL_POINTER;
    rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_expand_loras_bwd_workspace_bytes(B, T, C, D));
    if (rc) return rc;
    wkv::launch_expand_loras_backward((long)B * T, C, D, head_size, w_in, k_in, acts, Ws, biases, dys, dw_in, dk_in, dacts, dWs,
                                      dbiases, workspace, static_cast<hipStream_t>(stream));
    return launch_status();
}

static int check_epilogue(int B, int T, int H, int C) {
    if (B <= 0 || T <= 0 || H <= 0 || C <= 0) return WIND_RWKV7_ERR_BAD_SHAPE;
    if ((long long)B * T * H * C > (1LL << 40)) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (!wkv::lnheads::head_size_supported(C)) return WIND_RWKV7_ERR_HEAD_SIZE;
    if (T % 16 != 0) return WIND_RWKV7_ERR_SEQ_MULTIPLE;
    return WIND_RWKV7_OK;
}

size_t wind_rwkv7_ln_epilogue_bwd_workspace_bytes(int B, int T, int H, int C) {
    if (check_epilogue(B, T, H, C) != WIND_RWKV7_OK) return 0;
    return wkv::lnheads::bwd_workspace_bytes((long)B * T, H, C);
}

int wind_rwkv7_ln_epilogue_forward(int B, int T, int H, int C, const void* y_wkv, const void* q, const void* k,
                                   const void* v, const void* g, const void* params, void* out, void* stream) {
    const int rc = check_epilogue(B, T, H, C);
    if (rc) return rc;
    if (!y_wkv || !q || !k || !v || !g || !params || !out) return WIND_RWKV7_ERR_NULL_POINTER;
    wkv::lnheads::launch_forward((long)B * T, H, C, y_wkv, q, k, v, g, params, out, static_cast<hipStream_t>(stream));
    return launch_status();
}

int wind_rwkv7_ln_epilogue_backward(int B, int T, int H, int C, const void* y_wkv, const void* q, const void* k,
                                    const void* v, const void* g, const void* params, const void* dout, void* dy_wkv,
                                    void* dq, void* dk, void* dv, void* dg, void* dparams, void* workspace,
                                    size_t workspace_bytes, void* stream) {
    int rc = check_epilogue(B, T, H, C);
    if (rc) return rc;
    if (!y_wkv || !q || !k || !v || !g || !params || !dout || !dy_wkv || !dq || !dk || !dv || !dg || !dparams)
        return WIND_RWKV7_ERR_NULL_POINTER;
    rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_ln_epilogue_bwd_workspace_bytes(B, T, H, C));
    if (rc) return rc;
    wkv::lnheads::launch_backward((long)B * T, H, C, y_wkv, q, k, v, g, params, dout, dy_wkv, dq, dk, dv, dg, dparams,
                                  workspace, static_cast<hipStream_t>(stream));
    return launch_status();
}

int wind_rwkv7_f32_head_size_supported(int C) { return C >= 16 && C <= wkv::WKV7_F32_MAX_HEAD && C % 16 == 0; }

static int check_shape_f32(int B, int T, int H, int C) {
    if (B <= 0 || T <= 0 || H <= 0 || C <= 0) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (!wind_rwkv7_f32_head_size_supported(C)) return WIND_RWKV7_ERR_HEAD_SIZE;
    if (T % wkv::CHUNK != 0) return WIND_RWKV7_ERR_SEQ_MULTIPLE;
    if ((long long)B * T * H * C > (1LL << 40)) return WIND_RWKV7_ERR_BAD_SHAPE;
    return WIND_RWKV7_OK;
}

size_t wind_rwkv7_attn_f32_saved_bytes(int B, int T, int H, int C) {
    if (check_shape_f32(B, T, H, C)) return 0;
    return wkv::wkv7_f32_saved_bytes(B, T, H, C);
}

int wind_rwkv7_attn_f32_forward(int B, int T, int H, int C,
                                const void* w, const void* q, const void* k, const void* v, const void* a, const void* b,
                                const void* s0, void* y, void* s, void* sT, void* stream) {
    const int rc = check_shape_f32(B, T, H, C);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !s0 || !y || !s || !sT) return WIND_RWKV7_ERR_NULL_POINTER;
    auto f = [](const void* p) { return static_cast<const float*>(p); };
    wkv::launch_wkv7_f32_forward(B, T, H, C, f(w), f(q), f(k), f(v), f(a), f(b), f(s0), static_cast<float*>(y),
                                 static_cast<float*>(s), static_cast<float*>(sT), static_cast<hipStream_t>(stream));
    return launch_status();
}

int wind_rwkv7_attn_f32_prefill(int B, int T, int H, int C,
                                const void* w, const void* q, const void* k, const void* v, const void* a, const void* b,
                                const void* s0, void* y, void* sT, void* stream) {
    const int rc = check_shape_f32(B, T, H, C);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !s0 || !y || !sT) return WIND_RWKV7_ERR_NULL_POINTER;
    auto f = [](const void* p) { return static_cast<const float*>(p); };
    wkv::launch_wkv7_f32_forward(B, T, H, C, f(w), f(q), f(k), f(v), f(a), f(b), f(s0), static_cast<float*>(y), nullptr,
                                 static_cast<float*>(sT), static_cast<hipStream_t>(stream));
    return launch_status();
}

int wind_rwkv7_attn_f32_backward(int B, int T, int H, int C,
                                 const void* w, const void* q, const void* k, const void* v, const void* a, const void* b,
                                 const void* dy, const void* s, const void* dsT,
                                 void* dw, void* dq, void* dk, void* dv, void* da, void* db, void* ds0, void* stream) {
    const int rc = check_shape_f32(B, T, H, C);
    if (rc) return rc;
    if (!w || !q || !k || !v || !a || !b || !dy || !s || !dsT || !dw || !dq || !dk || !dv || !da || !db || !ds0)
        return WIND_RWKV7_ERR_NULL_POINTER;
    auto f = [](const void* p) { return static_cast<const float*>(p); };
    auto g = [](void* p) { return static_cast<float*>(p); };
    wkv::launch_wkv7_f32_backward(B, T, H, C, f(w), f(q), f(k), f(v), f(a), f(b), f(dy), f(s), f(dsT), g(dw), g(dq),
                                  g(dk), g(dv), g(da), g(db), g(ds0), static_cast<hipStream_t>(stream));
    return launch_status();
}

static int check_linear(long long tokens, int O, int I) {
    if (tokens <= 0 || O <= 0 || I <= 0 || tokens > (1LL << 40)) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (O % 16 != 0 || I % 16 != 0) return WIND_RWKV7_ERR_CHANNELS;
    return WIND_RWKV7_OK;
}

size_t wind_rwkv7_linear_wgrad_workspace_bytes(long long tokens, int O, int I) {
    if (check_linear(tokens, O, I)) return 0;
    return align_up(wkv::linear_wgrad_plan((long)tokens, O, I).partial_bytes);
}

int wind_rwkv7_linear_wgrad(long long tokens, int O, int I, const void* dy, long long ld_dy, const void* x, long long ld_x,
                            void* dW, int out_dtype, void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_linear(tokens, O, I);
    if (rc) return rc;
    if (!dy || !x || !dW) return WIND_RWKV7_ERR_NULL_POINTER;
    if (out_dtype != WIND_RWKV7_BF16 && out_dtype != WIND_RWKV7_F32) return WIND_RWKV7_ERR_DTYPE;
    // rows are read in 16-byte pieces
    if (ld_dy < O || ld_x < I || ld_dy % 8 != 0 || ld_x % 8 != 0) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(dy) % 16 != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0)
        return WIND_RWKV7_ERR_BAD_SHAPE;
    rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_linear_wgrad_workspace_bytes(tokens, O, I));
    if (rc) return rc;
    wkv::launch_linear_wgrad((long)tokens, O, I, dy, (long)ld_dy, x, (long)ld_x, dW, out_dtype == WIND_RWKV7_F32, workspace,
                             static_cast<hipStream_t>(stream));
    return launch_status();
}

size_t wind_rwkv7_linear_wgrad_group_workspace_bytes(int n, long long tokens, const int* O, const int* I) {
    if (n < 1 || n > WIND_RWKV7_WGRAD_GROUP_MAX || !O || !I) return 0;
    for (int j = 0; j < n; j++)
        if (check_linear(tokens, O[j], I[j])) return 0;
    return align_up(wkv::linear_wgrad_group_workspace_bytes(n, (long)tokens, O, I));
}

int wind_rwkv7_linear_wgrad_group(int n, long long tokens, const int* O, const int* I, const void* const* dy,
                                  const long long* ld_dy, const void* const* x, const long long* ld_x, void* const* dW,
                                  int out_dtype, void* workspace, size_t workspace_bytes, void* stream) {
    if (n < 1 || n > WIND_RWKV7_WGRAD_GROUP_MAX) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (!O || !I || !dy || !ld_dy || !x || !ld_x || !dW) return WIND_RWKV7_ERR_NULL_POINTER;
    if (out_dtype != WIND_RWKV7_BF16 && out_dtype != WIND_RWKV7_F32) return WIND_RWKV7_ERR_DTYPE;
    long ldy[WIND_RWKV7_WGRAD_GROUP_MAX], ldx[WIND_RWKV7_WGRAD_GROUP_MAX];
    for (int j = 0; j < n; j++) {
        const int rc = check_linear(tokens, O[j], I[j]);
        if (rc) return rc;
        if (!dy[j] || !x[j] || !dW[j]) return WIND_RWKV7_ERR_NULL_POINTER;
        if (ld_dy[j] < O[j] || ld_x[j] < I[j] || ld_dy[j] % 8 != 0 || ld_x[j] % 8 != 0) return WIND_RWKV7_ERR_BAD_SHAPE;
        if (reinterpret_cast<uintptr_t>(dy[j]) % 16 != 0 || reinterpret_cast<uintptr_t>(x[j]) % 16 != 0)
            return WIND_RWKV7_ERR_BAD_SHAPE;
        ldy[j] = (long)ld_dy[j];
        ldx[j] = (long)ld_x[j];
    }
    const int rc = check_workspace(workspace, workspace_bytes, wind_rwkv7_linear_wgrad_group_workspace_bytes(n, tokens, O, I));
    if (rc) return rc;
    if (!wkv::launch_linear_wgrad_group(n, (long)tokens, O, I, dy, ldy, x, ldx, dW, out_dtype == WIND_RWKV7_F32, workspace,
                                        static_cast<hipStream_t>(stream)))
        return WIND_RWKV7_ERR_CHANNELS;
    return launch_status();
}

int wind_rwkv7_copy_columns(long long M, int n, const void* const* src, const long long* src_ld, const int* src_col0,
                            void* const* dst, const long long* dst_ld, const int* dst_col0, const int* width,
                            const int* op, const void* const* aux, void* stream) {
    if (M < 0 || M > (1LL << 36) || n < 0 || n > 256) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (n == 0 || M == 0) return WIND_RWKV7_OK;
    if (!src || !src_ld || !src_col0 || !dst || !dst_ld || !dst_col0 || !width || !op) return WIND_RWKV7_ERR_NULL_POINTER;
    wkv::ColumnPiece pieces[256];
    for (int t = 0; t < n; t++) {
        if (width[t] <= 0 || width[t] % 8 != 0) return WIND_RWKV7_ERR_CHANNELS;
        if (op[t] != wkv::COLS_COPY && op[t] != wkv::COLS_TANH && op[t] != wkv::COLS_TANH_GRAD) return WIND_RWKV7_ERR_BAD_SHAPE;
        if (!dst[t]) return WIND_RWKV7_ERR_NULL_POINTER;
        if (op[t] == wkv::COLS_TANH_GRAD && (!aux || !aux[t])) return WIND_RWKV7_ERR_NULL_POINTER;
        // 16-byte accesses on both sides
        if (dst_col0[t] < 0 || dst_col0[t] % 8 != 0 || dst_ld[t] < dst_col0[t] + width[t] || dst_ld[t] % 8 != 0 ||
            reinterpret_cast<uintptr_t>(dst[t]) % 16 != 0)
            return WIND_RWKV7_ERR_BAD_SHAPE;
        if (src[t] && (src_col0[t] < 0 || src_col0[t] % 8 != 0 || src_ld[t] < src_col0[t] + width[t] || src_ld[t] % 8 != 0 ||
                       reinterpret_cast<uintptr_t>(src[t]) % 16 != 0))
            return WIND_RWKV7_ERR_BAD_SHAPE;
        if (op[t] == wkv::COLS_TANH_GRAD && reinterpret_cast<uintptr_t>(aux[t]) % 16 != 0) return WIND_RWKV7_ERR_BAD_SHAPE;
        pieces[t] = wkv::ColumnPiece{src[t], aux ? aux[t] : nullptr, dst[t], src_ld[t], dst_ld[t],
                                     src_col0[t], dst_col0[t], width[t], op[t]};
    }
    wkv::launch_copy_columns(M, n, pieces, static_cast<hipStream_t>(stream));
    return launch_status();
}

int wind_rwkv7_cast_to_bf16(int n, const void* const* src, const int* src_dtype, const long long* numel,
                            const long long* dst_offset, void* dst, void* stream) {
    if (n < 0 || n > 4096) return WIND_RWKV7_ERR_BAD_SHAPE;
    if (n == 0) return WIND_RWKV7_OK;
    if (!src || !src_dtype || !numel || !dst) return WIND_RWKV7_ERR_NULL_POINTER;
    int f32[4096];
    long long total = 0;
    for (int t = 0; t < n; t++) {
        if (numel[t] < 0 || numel[t] > (1LL << 40)) return WIND_RWKV7_ERR_BAD_SHAPE;
        if (dst_offset && (dst_offset[t] < 0 || dst_offset[t] > (1LL << 40))) return WIND_RWKV7_ERR_BAD_SHAPE;
        if (numel[t] > 0 && !src[t]) return WIND_RWKV7_ERR_NULL_POINTER;
        if (src_dtype[t] != WIND_RWKV7_BF16 && src_dtype[t] != WIND_RWKV7_F32) return WIND_RWKV7_ERR_DTYPE;
        f32[t] = src_dtype[t] == WIND_RWKV7_F32;
        total += numel[t];
    }
    if (total / 2048 + n > 0x7fffffffLL) return WIND_RWKV7_ERR_BAD_SHAPE;   // one block per 2048 elements
    wkv::launch_cast_to_bf16(n, src, f32, numel, dst_offset, dst, static_cast<hipStream_t>(stream));
    return launch_status();
}

int wind_rwkv7_profile_enable(int on) {
    if (on && !g_prof.on) {
        for (int d = 0; d < 2; d++)
            for (int i = 0; i <= WIND_RWKV7_PROFILE_SLOTS; i++)
                if (hipEventCreate(&g_prof.ev[d][i]) != hipSuccess) return WIND_RWKV7_ERR_LAUNCH;
        g_prof.count[0] = g_prof.count[1] = 0;
        g_prof.on = true;
    } else if (!on && g_prof.on) {
        g_prof.on = false;
        for (int d = 0; d < 2; d++)
            for (int i = 0; i <= WIND_RWKV7_PROFILE_SLOTS; i++) (void)hipEventDestroy(g_prof.ev[d][i]);
    }
    return WIND_RWKV7_OK;
}

int wind_rwkv7_profile_read(int direction, float* ms, int n) {
    if (!ms) return -WIND_RWKV7_ERR_NULL_POINTER;
    if (direction < 0 || direction > 1 || !g_prof.on) return -WIND_RWKV7_ERR_BAD_SHAPE;
    const int have = g_prof.count[direction];
    if (have <= 0) return 0;
    if (hipEventSynchronize(g_prof.ev[direction][have]) != hipSuccess) return -WIND_RWKV7_ERR_LAUNCH;
    int written = 0;
    for (int i = 0; i < have && i < n; i++) {
        if (hipEventElapsedTime(&ms[i], g_prof.ev[direction][i], g_prof.ev[direction][i + 1]) != hipSuccess)
            return -WIND_RWKV7_ERR_LAUNCH;
        written++;
    }
    return written;
}

const char* wind_rwkv7_profile_kernel_name(int direction, int i) {
    if (direction < 0 || direction > 1 || i < 0 || i >= WIND_RWKV7_PROFILE_SLOTS) return nullptr;
    return g_prof.name[direction][i];
}

}  // extern "C"
