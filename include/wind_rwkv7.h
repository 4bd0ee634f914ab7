/* wind_rwkv7.h - C ABI of the MI355X (gfx950) RWKV-7 time-mixer kernels.
 *
 * This is the drop-in boundary: plain pointers and sizes, no torch types.  Every entry point
 * replaces one launcher / operator of johanwind/wind-rwkv7 (cited per function below as file:line
 * in that repository).
 *
 * Conventions
 *   - All data pointers are DEVICE pointers.  The library never allocates, frees or synchronises;
 *     outputs and workspaces are allocated by the caller (as in the reference, where Python
 *     allocates every output: rwkv7_attn.py:5-16).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Work is only enqueued.
 *   - Tensors are contiguous, row-major: sequences [B,T,H,C] (token stride H*C, as attn.cu:25,29),
 *     states [B,H,C,C] indexed [value row i][key column j] (attn.cu:42).
 *     Every tensor starts on a 16-byte boundary (the kernels use 16-byte accesses; any allocator's memory does).
 *   - `io_dtype` is the element type of sequences; `state_dtype` that of s0/sT/dsT/ds0
 *     (WIND_RWKV7_BF16 or WIND_RWKV7_F32).  The reference fixes both to bf16 (rwkv7_attn.py:24).
 *   - Every function returns 0 on success or a WIND_RWKV7_ERR_* code; arguments are validated on
 *     the host before anything is enqueued, so a failing call has no effect.
 */
#ifndef WIND_RWKV7_H
#define WIND_RWKV7_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WIND_RWKV7_ABI_VERSION 1

enum {
    WIND_RWKV7_OK = 0,
    WIND_RWKV7_ERR_NULL_POINTER = 1,   /* a required pointer is NULL */
    WIND_RWKV7_ERR_BAD_SHAPE = 2,      /* B, T, H or C not positive, or sizes overflow: more than 2^30 chunks of 16
                                        * tokens x heads, or at head size 64 a batch element's rows of one tensor
                                        * (T*H*64 bf16) of 2 GiB or more */
    WIND_RWKV7_ERR_HEAD_SIZE = 3,      /* C is not a head size these kernels were built for */
    WIND_RWKV7_ERR_SEQ_MULTIPLE = 4,   /* T is not a multiple of the chunk length (16; rwkv7_attn.py:22) */
    WIND_RWKV7_ERR_DTYPE = 5,          /* unsupported io_dtype / state_dtype */
    WIND_RWKV7_ERR_WORKSPACE = 6,      /* workspace missing, too small or misaligned (256 bytes) */
    WIND_RWKV7_ERR_LAUNCH = 7,         /* the HIP runtime refused a launch */
    WIND_RWKV7_ERR_RANK = 8,           /* unsupported LoRA rank D */
    WIND_RWKV7_ERR_CHANNELS = 9,       /* channel count is not a multiple of 64 (or of the head size) */
    WIND_RWKV7_ERR_STATIC_LIMIT = 10   /* wind_rwkv7_attn_prefill_static: problem larger than the built-in scratch */
};

enum { WIND_RWKV7_BF16 = 0, WIND_RWKV7_F32 = 1 };

/* ABI version of the loaded library (== WIND_RWKV7_ABI_VERSION of the header it was built from). */
int wind_rwkv7_abi_version(void);

/* Static description of an error code. */
const char* wind_rwkv7_strerror(int code);

/* 1 if head size C is supported, else 0.  Replaces the compile-time -D_C_ of the reference's JIT build
 * (rwkv7_attn.py:46-51, attn.cu:8): head size is a runtime argument here. */
int wind_rwkv7_head_size_supported(int C);

/* The same for the plain WKV7 entry points, wind_rwkv7_attn_{forward,prefill,backward} and their size queries, and for
 * the single-token entry points wind_rwkv7_attn_decode / wind_rwkv7_attn_ln_decode, which
 * also have kernels for the other head sizes: multiples of 16 up to 128.  The reference serves those by
 * recompiling attn.cu per head size (rwkv7_attn.py:46-51) and, for large heads, with the Triton kernels of
 * rwkv7_attn_triton_bighead.py:31-322. */
int wind_rwkv7_attn_head_size_supported(int C);

/* Tokens per chunk (16): the unit of the dense products on the matrix cores.  T must be a multiple of it.  The
 * reference's kernels are written for this length (attn.cu:48, rwkv7_attn_triton.py:162). */
int wind_rwkv7_chunk_len(void);

/* Tokens between the states that the training forward keeps for the backward pass (and the backward scan for the
 * gradient kernel): 32 (default) or 16.  At 32 the chunks work in pairs - two-level chunking: 16-token products, a
 * 64x64 checkpoint only every second chunk, and the gradient kernel carries the state across the pair itself, which
 * moves 512 bytes less per token and head in each direction.  At 16 there is a checkpoint per chunk, as in the
 * reference (attn.cu:92-94).  32 applies to sequences with an even number of chunks (long sequences on few heads,
 * which run as segments of at least 32 chunks, always have one); an odd number keeps a state per chunk whatever the setting.  It
 * concerns head size 64; the kernels of the other head sizes keep a state per chunk.  The setting is process-wide and is read by the size queries, the
 * forward and the backward entry points alike: a forward call, the queries that size its buffers and its backward call
 * must all run under the same value.  Results agree within the rounding of a bf16 state (both are held to the same
 * tolerance against the fp64 recurrence).  The reference has no such switch.
 * set: 0, or WIND_RWKV7_ERR_BAD_SHAPE for a value other than 16 and 32. */
int wind_rwkv7_checkpoint_interval(void);
int wind_rwkv7_set_checkpoint_interval(int tokens);

/* ---- WKV7 ("attn") ------------------------------------------------------------------------------ */

/* Bytes of the tensor saved by forward for backward: the reference's `s`, rwkv7_attn.py:9
 * ([B,H,T/16,C,C] bf16 there).  Its layout is private to the library. */
size_t wind_rwkv7_attn_saved_bytes(int B, int T, int H, int C);

/* Bytes of scratch the forward / backward call needs (contents undefined afterwards). */
size_t wind_rwkv7_attn_fwd_workspace_bytes(int B, int T, int H, int C);
size_t wind_rwkv7_attn_bwd_workspace_bytes(int B, int T, int H, int C);

/* y, sT = WKV7(w, q, k, v, a, b, s0), and `s` for backward.
 * Replaces cuda_forward (attn.cu:108-128) / the operator wind::forward (attn.cpp:10-13,25).
 *   S_t = S_{t-1} diag(exp(-exp(w_t))) + (S_{t-1} a_t) b_t^T + v_t k_t^T ;  y_t = S_t q_t
 * w,q,k,v,a,b,y: [B,T,H,C] io_dtype;  s0,sT: [B,H,C,C] state_dtype;  s: wind_rwkv7_attn_saved_bytes.
 * s0 may be NULL: the sequence starts from a zero state (no tensor of zeros has to be made for it); this holds for
 * every bf16-sequence entry point that takes an s0. */
int wind_rwkv7_attn_forward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                            const void* w, const void* q, const void* k, const void* v,
                            const void* a, const void* b, const void* s0,
                            void* y, void* s, void* sT,
                            void* workspace, size_t workspace_bytes, void* stream);

/* The same y and sT for a caller that will not differentiate (prompt processing, evaluation): what only the
 * backward pass would read (10 KiB per chunk of 16 tokens) is not stored, a fifth of the call's memory traffic.  The
 * reference has one forward for both uses (attn.cu:108-128 always fills s and sa).  `scratch` has the size and
 * alignment of `s` above, and its contents are undefined afterwards: it must not be handed to
 * wind_rwkv7_attn_backward, and may be one buffer reused by every call on the stream. */
int wind_rwkv7_attn_prefill(int B, int T, int H, int C, int io_dtype, int state_dtype,
                            const void* w, const void* q, const void* k, const void* v,
                            const void* a, const void* b, const void* s0,
                            void* y, void* scratch, void* sT,
                            void* workspace, size_t workspace_bytes, void* stream);

/* wind_rwkv7_attn_prefill for callers that cannot allocate or pass device scratch: code under HIP-graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The scratch and
 * workspace of wind_rwkv7_attn_prefill live in a device array that is part of the library's code object
 * (WIND_RWKV7_STATIC_SCRATCH_BYTES per GPU, held from the library's load on that GPU until the process ends), so the
 * call allocates nothing and takes inputs and outputs only.  y and sT are bit-identical to wind_rwkv7_attn_prefill.
 * Limit: wind_rwkv7_attn_prefill_static_bytes(B,T,H,C) <= WIND_RWKV7_STATIC_SCRATCH_BYTES (about 3200 chunks of
 * 16 tokens x heads, e.g. B*H*T <= 52 000 at C = 64), else WIND_RWKV7_ERR_STATIC_LIMIT and nothing is enqueued.
 * All calls on one GPU share that GPU's array: two calls whose kernels may overlap in time (different streams, or
 * threads, without ordering between them) race; calls on one stream are ordered and safe.
 * The array's device address is looked up once per GPU, by the first wind_rwkv7_attn_prefill_static_bytes or
 * wind_rwkv7_attn_prefill_static call with that GPU current: make that first call outside a graph capture. */
#define WIND_RWKV7_STATIC_SCRATCH_BYTES (32u << 20)
size_t wind_rwkv7_attn_prefill_static_bytes(int B, int T, int H, int C);
int wind_rwkv7_attn_prefill_static(int B, int T, int H, int C, int io_dtype, int state_dtype,
                                   const void* w, const void* q, const void* k, const void* v,
                                   const void* a, const void* b, const void* s0,
                                   void* y, void* sT, void* stream);

/* Gradients of wind_rwkv7_attn_forward.  Replaces cuda_backward (attn.cu:328-348) / wind::backward (attn.cpp:17-22,26).
 * dy: [B,T,H,C]; dsT: [B,H,C,C]; outputs dw,dq,dk,dv,da,db: [B,T,H,C]; ds0: [B,H,C,C].
 * dsT may be NULL (the final state has no gradient: zero) and ds0 may be NULL (not wanted, not written); the same
 * holds for wind_rwkv7_attn_ln_backward. */
int wind_rwkv7_attn_backward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                             const void* w, const void* q, const void* k, const void* v,
                             const void* a, const void* b,
                             const void* dy, const void* s, const void* dsT,
                             void* dw, void* dq, void* dk, void* dv, void* da, void* db, void* ds0,
                             void* workspace, size_t workspace_bytes, void* stream);

/* ---- WKV7 + per-head GroupNorm + bonus + gate ("attn_ln") -------------------------------------------- */

/* Same as the attn functions with the fused epilogue of the reference's attn_ln:
 *   out = (group_norm(y; eps = 64e-5) * ln_w + ln_b + (sum_c q_c k_c bonus_c) * v) * g
 * g: [B,T,H,C] io_dtype;  params: [3, H*C] FLOAT32 = stack(ln_w, ln_b, bonus) (rwkv7_attn_ln.py:26,29).
 * forward replaces cuda_forward of attn_ln.cu:214-234 (operator schema attn_ln.cpp:25), backward replaces
 * cuda_backward of attn_ln.cu:466-486 (attn_ln.cpp:26).  dparams [3, H*C] float32 is OVERWRITTEN with a
 * sum taken in a fixed order (the reference accumulates into a pre-zeroed tensor with atomicAdd,
 * attn_ln.cu:450-463, rwkv7_attn_ln.py:15); it need not be zeroed.
 * Head sizes: those of wind_rwkv7_attn_head_size_supported.  At 64 (wind_rwkv7_head_size_supported) the epilogue
 * runs inside the WKV7 kernels or right behind them; at the others these functions run the plain entry points and
 * wind_rwkv7_ln_epilogue_* below, with the WKV7 output kept behind the plain saved tensor.
 * At every head size the WKV7 output is kept (for the epilogue when it runs as a kernel of its own, and for the backward
 * pass) as bf16 values CENTRED per token and block of 16 channels, with the fp32 centres beside them: GroupNorm then
 * sees it as accurately as the reference's epilogue sees its fp32 accumulators (attn_ln.cu:11-22, :192) at bf16
 * traffic, also when a head's mean is many times its spread. */
size_t wind_rwkv7_attn_ln_saved_bytes(int B, int T, int H, int C);
size_t wind_rwkv7_attn_ln_fwd_workspace_bytes(int B, int T, int H, int C);
size_t wind_rwkv7_attn_ln_bwd_workspace_bytes(int B, int T, int H, int C);

int wind_rwkv7_attn_ln_forward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                               const void* w, const void* q, const void* k, const void* v,
                               const void* a, const void* b, const void* g, const void* params,
                               const void* s0,
                               void* y, void* s, void* sT,
                               void* workspace, size_t workspace_bytes, void* stream);

/* Forward for a caller that will not differentiate: see wind_rwkv7_attn_prefill (the reference's forward,
 * attn_ln.cu:214-234, always stores s and sa).  `scratch`: wind_rwkv7_attn_ln_saved_bytes, contents undefined
 * afterwards. */
int wind_rwkv7_attn_ln_prefill(int B, int T, int H, int C, int io_dtype, int state_dtype,
                               const void* w, const void* q, const void* k, const void* v,
                               const void* a, const void* b, const void* g, const void* params,
                               const void* s0,
                               void* y, void* scratch, void* sT,
                               void* workspace, size_t workspace_bytes, void* stream);

int wind_rwkv7_attn_ln_backward(int B, int T, int H, int C, int io_dtype, int state_dtype,
                                const void* w, const void* q, const void* k, const void* v,
                                const void* a, const void* b, const void* g, const void* params,
                                const void* dy, const void* s, const void* dsT,
                                void* dw, void* dq, void* dk, void* dv, void* da, void* db, void* dg,
                                void* dparams, void* ds0,
                                void* workspace, size_t workspace_bytes, void* stream);

/* ---- single-token step (autoregressive decoding) ------------------------------------------------------ */

/* One token of WKV7 per sequence on a state that stays in device memory between calls:
 *   y = WKV7 step(w, q, k, v, a, b; state), state updated IN PLACE.
 * w,q,k,v,a,b,y: [B,H,C] io_dtype (one token);  state: [B,H,C,C] state_dtype, value row x key column, the same
 * tensor as s0 / sT of the sequence entry points - a prompt is run with wind_rwkv7_attn_forward (any multiple
 * of the chunk length) and its sT handed to this function.  The reference has no single-token kernel; this
 * replaces the per-token loop of its PyTorch path (ref_attn, time_mixer.py:6-16).  No workspace. */
int wind_rwkv7_attn_decode(int B, int H, int C, int io_dtype, int state_dtype,
                           const void* w, const void* q, const void* k, const void* v,
                           const void* a, const void* b, void* state, void* y, void* stream);

/* The same with the attn_ln epilogue (GroupNorm + bonus + gate); g: [B,H,C] io_dtype, params: [3, H*C] float32. */
int wind_rwkv7_attn_ln_decode(int B, int H, int C, int io_dtype, int state_dtype,
                              const void* w, const void* q, const void* k, const void* v,
                              const void* a, const void* b, const void* g, const void* params,
                              void* state, void* y, void* stream);

/* ---- the attn_ln epilogue on its own ------------------------------------------------------------------- */

/* GroupNorm over each head + bonus + gate, as the reference's fw_post_process / bw_post_process compute them
 * inside its attn_ln kernels (attn_ln.cu:11-37, :40-104; spec tests/test_attn_ln.py:18-21), for head sizes C that
 * are multiples of 16 up to 128.  At head size 64 wind_rwkv7_attn_ln_* have the epilogue inside; for the other head
 * sizes, which the reference serves by recompiling attn_ln.cu (rwkv7_attn_ln.py:11-17), attn_ln is
 * wind_rwkv7_attn_forward followed by this forward, and this backward followed by wind_rwkv7_attn_backward
 * (wind_rwkv7_attn_ln_* do exactly that; these are for callers that hold the WKV7 output themselves).
 *   forward:  y_wkv, q, k, v, g [B,T,H,C] bf16, params [3,H*C] float32 (ln weight, ln bias, bonus) -> out bf16
 *   backward: + dout -> dy_wkv (gradient of the WKV7 output), dq, dk, dv (the bonus term's contributions, to be
 *             added to those of the WKV7 backward), dg, all [B,T,H,C] bf16, and FLOAT32 dparams [3,H*C],
 *             overwritten, summed in a fixed order.
 * Requires T % 16 == 0. */
size_t wind_rwkv7_ln_epilogue_bwd_workspace_bytes(int B, int T, int H, int C);
int wind_rwkv7_ln_epilogue_forward(int B, int T, int H, int C,
                                   const void* y_wkv, const void* q, const void* k, const void* v, const void* g,
                                   const void* params, void* out, void* stream);
int wind_rwkv7_ln_epilogue_backward(int B, int T, int H, int C,
                                    const void* y_wkv, const void* q, const void* k, const void* v, const void* g,
                                    const void* params, const void* dout,
                                    void* dy_wkv, void* dq, void* dk, void* dv, void* dg, void* dparams,
                                    void* workspace, size_t workspace_bytes, void* stream);

/* One token per sequence through the WHOLE time mixer (TimeMixer of time_mixer.py:18-167 taken at T = 1): token
 * shift, projections, LoRAs, the WKV7 step with GroupNorm / bonus / gate, output projection - five kernel launches.
 * The reference's block has no single-token form; its forward (time_mixer.py:96-167) is the specification, with the
 * previous token x_prev and the WKV7 state carried by the caller.  Head size 64, C = 64 H, the block's LoRA ranks
 * (mix 32, decay 64, gate 128, the others 16).  Every parameter is a bf16 device array laid out as the module's
 * parameter of that name, except ln_params. */
typedef struct wind_rwkv7_mixer_weights {
    const void *time_maa_x, *time_maa, *time_maa_w1, *time_maa_w2;                     /* [C] [4,C] [128,C] [4,C,32] */
    const void *Wr, *Wk, *Wv, *Wo;                                                     /* [C,C] */
    const void *gate_w1, *time_decay_w1, *time_kkk_w1, *mk_w1, *time_aaa_w1, *ma_w1;   /* [rank,C] */
    const void *gate_w2, *time_decay_w2, *time_kkk_w2, *mk_w2, *time_aaa_w2, *ma_w2;   /* [C,rank] */
    const void *time_decay, *time_aaaaa, *time_misc_a, *time_misc_k;                   /* [C] */
    const void* ln_params;   /* [3,C] float32: ln_x.weight, ln_x.bias, time_faaaa */
} wind_rwkv7_mixer_weights;

size_t wind_rwkv7_mixer_decode_workspace_bytes(int B, int C);

/* x, x_prev: [B,C] bf16 (the token and the one before it); state: [B,H,64,64] state_dtype, updated IN PLACE;
 * y: [B,C] bf16; x_carry: NULL or [B,C] bf16 that receives a copy of x, to be the next call's x_prev (another
 * buffer than x_prev).  workspace: wind_rwkv7_mixer_decode_workspace_bytes(B, C) bytes, 256-byte aligned. */
int wind_rwkv7_mixer_decode(int B, int C, int H, int state_dtype, const wind_rwkv7_mixer_weights* weights,
                            const void* x, const void* x_prev, void* state, void* y, void* x_carry,
                            void* workspace, size_t workspace_bytes, void* stream);

/* ---- ddlerp: data-dependent token-shift interpolation ------------------------------------------------ */

/* Replaces the Triton kernels behind DDLerp (rwkv7_ddlerp.py:306-336; launches :43-48, :76-83, :132-138,
 * :159-166, :251-264, :296-302).  Spec tests/test_ddlerp.py:5-13.
 *   x [B,T,C] bf16;  alpha [C], L [4D,C], R [4,C,D], beta [4,C]: bf16 (the reference casts its fp32
 *   parameters to bf16 before its kernels, rwkv7_ddlerp.py:309).
 *   forward: bmid = tanh(.) and bder = 1 - tanh(.)^2, both [B,T,4D] bf16, saved for backward (the reference
 *   saves only bmid, :321, and recomputes the derivative from the rounded value); y [4,B,T,C] bf16.
 *   backward: dy0..dy3 [B,T,C] bf16 -> dx [B,T,C] bf16 and FLOAT32 dalpha [C], dL [4D,C], dR [4,C,D],
 *   dbeta [4,C], all overwritten, summed in a fixed order (the reference uses atomics, :237-246, :289-291).
 * Requires C % 64 == 0, T % 16 == 0 and a supported rank D (32 or 64).  A smaller rank runs at the next of the two
 * with zero rows appended to each of L's four blocks and zero columns to R (tanh(0) = 0 against a zero weight: the same
 * result); the caller drops the padding's gradients (the Python operator does this, rwkv7/token_shift.py). */
int wind_rwkv7_ddlerp_rank_supported(int D);
size_t wind_rwkv7_ddlerp_bwd_workspace_bytes(int B, int T, int C, int D);
int wind_rwkv7_ddlerp_forward(int B, int T, int C, int D,
                              const void* x, const void* alpha, const void* L, const void* R, const void* beta,
                              void* bmid, void* bder, void* y, void* stream);
int wind_rwkv7_ddlerp_backward(int B, int T, int C, int D,
                               const void* x, const void* alpha, const void* L, const void* R, const void* beta,
                               const void* bmid, const void* bder,
                               const void* dy0, const void* dy1, const void* dy2, const void* dy3,
                               void* dx, void* dalpha, void* dL, void* dR, void* dbeta,
                               void* workspace, size_t workspace_bytes, void* stream);

/* ---- expand_loras: second halves of four rank-D LoRAs + the elementwise tail --------------------------- */

/* Replaces the Triton kernels behind ExpandLoras (rwkv7_expand_loras.py:214-241; launches :72-79, :192-211).
 * Spec tests/test_expand_loras.py:6-19.  All tensors bf16 unless noted:
 *   w_in, k_in [B,T,C];  z_in, a_in, ma_in, mk_in [B,T,D];  Wz, Wa, Wma, Wmk [C,D];
 *   w_bias, a_bias, ma_bias, mk_bias [C];  outputs w_out, k_out, kk_out, b_out [B,T,C].
 * backward: dw_out, dk_out, dkk_out, db_out [B,T,C] -> dw_in, dk_in [B,T,C], dz_in, da_in, dma_in, dmk_in
 * [B,T,D] (bf16) and FLOAT32 dWz, dWa, dWma, dWmk [C,D], dw_bias, da_bias, dma_bias, dmk_bias [C], all
 * overwritten and summed in a fixed order (the reference uses atomics, :181-189, and sums the per-head
 * partials of the rank-space gradients on the host, :207-210).
 * Requires head_size a multiple of 16 that divides C (the reference passes it on, :72-79), C % 64 == 0,
 * T % 16 == 0, D in {16, 32, 64}.  The backward workspace size does not depend on the head size. */
int wind_rwkv7_expand_loras_rank_supported(int D);
size_t wind_rwkv7_expand_loras_bwd_workspace_bytes(int B, int T, int C, int D);
int wind_rwkv7_expand_loras_forward(int B, int T, int C, int D, int head_size,
                                    const void* w_in, const void* k_in,
                                    const void* z_in, const void* a_in, const void* ma_in, const void* mk_in,
                                    const void* Wz, const void* Wa, const void* Wma, const void* Wmk,
                                    const void* w_bias, const void* a_bias, const void* ma_bias, const void* mk_bias,
                                    void* w_out, void* k_out, void* kk_out, void* b_out, void* stream);
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
                                     void* workspace, size_t workspace_bytes, void* stream);

/* ---- WKV7 in fp32 (accuracy mode, and head sizes other than 64) ------------------------------------- */

/* The same operator with fp32 sequences, fp32 state and fp32 arithmetic throughout (no matrix cores): results
 * within 1e-4 of the fp64 recurrence, where the bf16 entry points above are within 1e-2.  Replaces the
 * reference's Triton kernels run with dot_prec='fp32' (fw_attn_triton / bw_attn_triton,
 * rwkv7_attn_triton.py:27-156, precision switch :182-190; fp32 checkpoints :67,167) and, for head sizes other
 * than 64, its large-head variant (rwkv7_attn_triton_bighead.py:31-322; `assert C%16 == 0`, :335).
 * All tensors are float32: w,q,k,v,a,b,y,dy and the six gradients [B,T,H,C]; s0,sT,dsT,ds0 [B,H,C,C];
 * s = wind_rwkv7_attn_f32_saved_bytes bytes (the state every 16 tokens and a [B,T,H,C] tensor of row sums).
 * No workspace.  The backward zeroes dq, dk, da, db, dw itself and adds two parts per element onto them (atomics; the result does not depend on their order).  C a multiple of 16 from 16 to 128 (wind_rwkv7_f32_head_size_supported), T % 16 == 0. */
int wind_rwkv7_f32_head_size_supported(int C);
size_t wind_rwkv7_attn_f32_saved_bytes(int B, int T, int H, int C);
int wind_rwkv7_attn_f32_forward(int B, int T, int H, int C,
                                const void* w, const void* q, const void* k, const void* v,
                                const void* a, const void* b, const void* s0,
                                void* y, void* s, void* sT, void* stream);
/* Forward for a caller that will not differentiate: the same y and sT, no saved states (the reference's Triton
 * forward always stores them, rwkv7_attn_triton.py:67). */
int wind_rwkv7_attn_f32_prefill(int B, int T, int H, int C,
                                const void* w, const void* q, const void* k, const void* v,
                                const void* a, const void* b, const void* s0,
                                void* y, void* sT, void* stream);
int wind_rwkv7_attn_f32_backward(int B, int T, int H, int C,
                                 const void* w, const void* q, const void* k, const void* v,
                                 const void* a, const void* b,
                                 const void* dy, const void* s, const void* dsT,
                                 void* dw, void* dq, void* dk, void* dv, void* da, void* db, void* ds0,
                                 void* stream);

/* ---- projection weight gradient ------------------------------------------------------------------ */

/* dW[o][i] = sum_t dy[t][o] * x[t][i]: the weight gradient of a bias-free projection y = x W^T.
 * Replaces the BLAS call torch autograd issues for the weights of the r/k/v/gate/output projections and the
 * LoRA first halves of TimeMixer.forward (time_mixer.py:120-131, :167); the reference has no kernel of its own
 * for it.  Both operands are token-major, so the contraction runs over the slow index of both.
 *   dy [tokens, O] bf16, row stride ld_dy elements;  x [tokens, I] bf16, row stride ld_x elements;
 *   dW [O, I] contiguous, out_dtype (WIND_RWKV7_F32 or WIND_RWKV7_BF16), overwritten; fp32 accumulation,
 *   token ranges summed in a fixed order.
 * Requires O % 16 == 0, I % 16 == 0, strides multiples of 8 elements, dy and x 16-byte aligned. */
size_t wind_rwkv7_linear_wgrad_workspace_bytes(long long tokens, int O, int I);
int wind_rwkv7_linear_wgrad(long long tokens, int O, int I,
                            const void* dy, long long ld_dy, const void* x, long long ld_x,
                            void* dW, int out_dtype,
                            void* workspace, size_t workspace_bytes, void* stream);

/* n <= WIND_RWKV7_WGRAD_GROUP_MAX such weight gradients in one launch (and one launch for the sums of the partial
 * tiles), for products whose upstream gradients are available together - in the time mixer the projections of the four
 * shifted streams (r and the gate's first factor, k and two LoRA factors, v, the decay/a/ma factors), and the second
 * factors of gate and decay.  Same operands and requirements per problem as wind_rwkv7_linear_wgrad, all with the same
 * token count and out_dtype; each problem gets the tile shape that suits it.  With all tiles in one grid a block
 * covers a longer token range, so fewer fp32 partial tiles are written and summed, and problems too small to fill the
 * machine on their own share one launch.  The reference has no counterpart (its weight gradients are autograd's BLAS
 * calls, time_mixer.py:120-131). */
#define WIND_RWKV7_WGRAD_GROUP_MAX 8
size_t wind_rwkv7_linear_wgrad_group_workspace_bytes(int n, long long tokens, const int* O, const int* I);
int wind_rwkv7_linear_wgrad_group(int n, long long tokens, const int* O, const int* I,
                                  const void* const* dy, const long long* ld_dy,
                                  const void* const* x, const long long* ld_x,
                                  void* const* dW, int out_dtype,
                                  void* workspace, size_t workspace_bytes, void* stream);

/* Column blocks of token-major bf16 matrices, moved in one launch: piece t is width[t] columns of M rows, read at
 * src[t] (row stride src_ld[t] elements, first column src_col0[t]; a null src reads as zeros) and written at
 * dst[t] (dst_ld[t], dst_col0[t]), with op[t] = 0 copy, 1 tanh, 2 multiplication by 1 - aux^2 (aux[t]: the
 * contiguous [M, width] tanh output; the derivative).  Replaces the `.split(...)` of the concatenated LoRA first
 * halves, the tanh between the halves and their autograd counterparts in TimeMixer.forward
 * (time_mixer.py:124-131).  Widths, offsets and strides are multiples of 8 elements, bases 16-byte aligned;
 * all arrays are HOST arrays of n entries (aux may be NULL when no piece has op 2); n <= 256. */
int wind_rwkv7_copy_columns(long long M, int n,
                            const void* const* src, const long long* src_ld, const int* src_col0,
                            void* const* dst, const long long* dst_ld, const int* dst_col0,
                            const int* width, const int* op, const void* const* aux, void* stream);

/* bf16 working copies of n parameter tensors in one launch: tensor t (src[t], contiguous, numel[t] elements of
 * src_dtype[t] = WIND_RWKV7_F32 or WIND_RWKV7_BF16) is written, rounded to nearest even, to element offset
 * dst_offset[t] of dst; with dst_offset NULL, right after tensor t-1, so that weights one product uses
 * together come out as one contiguous matrix.  Replaces the per-operand `.to(th.bfloat16)` casts of
 * TimeMixer.forward (time_mixer.py:120-131, :167), DDLerp.forward (rwkv7_ddlerp.py:309) and
 * ExpandLoras.forward (rwkv7_expand_loras.py:218).  src, src_dtype, numel and dst_offset are HOST arrays (read
 * before the call returns); the tensors and dst are device memory; the destination ranges must not overlap.
 * n <= 4096. */
int wind_rwkv7_cast_to_bf16(int n, const void* const* src, const int* src_dtype, const long long* numel,
                            const long long* dst_offset, void* dst, void* stream);

/* ---- measurement aid ----------------------------------------------------------------------------- */

/* Per-kernel timing with HIP events recorded on the caller's stream, for benchmarks.  No counterpart in
 * the reference (its scripts time whole calls with cuda.synchronize(), tests/utils.py:86-93).
 * enable(1) creates the events, enable(0) destroys them; while enabled, every attn forward/backward
 * call brackets each of its kernels with events.  read() waits for the last recorded call of the given
 * direction (0 = forward, 1 = backward) and writes the duration in milliseconds of its kernels, in launch
 * order, to ms[0..n) (n <= WIND_RWKV7_PROFILE_SLOTS); returns the number written, or a negative error code.
 * Process-global and not thread-safe: use from one thread, for measurement only. */
#define WIND_RWKV7_PROFILE_SLOTS 6
int wind_rwkv7_profile_enable(int on);
int wind_rwkv7_profile_read(int direction, float* ms, int n);
/* Name of the kernel timed in slot `i` of `direction`, or NULL. */
const char* wind_rwkv7_profile_kernel_name(int direction, int i);

#ifdef __cplusplus
}
#endif
#endif /* WIND_RWKV7_H */
