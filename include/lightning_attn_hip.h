/*
 * C ABI of liblightning_attn_hip.so -- hand-written HIP kernels for gfx950 (MI355X).
 *
 * The reference (OpenNLPLab/lightning-attention) has no native ABI: its device
 * code is Triton-JIT launched from torch.autograd.Function bodies.  Each entry
 * point below replaces one of those launch sites; the citation names the
 * reference lines whose work it does.  The Python package binds these symbols
 * with ctypes (lightning_attn/ops/hip/_lib.py).
 *
 * Conventions
 *   - all pointers are device pointers owned by the caller (row-major,
 *     contiguous unless a stride argument says otherwise);
 *   - every call only enqueues work on `stream` (a hipStream_t passed as
 *     void*; NULL = the default stream): no allocation, no host sync;
 *   - the return value is 0 on success, a negative LA_E_* code for argument
 *     errors detected on the host before anything is launched, or a positive
 *     hipError_t reported by the launch.  la_error_string() names either;
 *   - dtype: LA_BF16 = 0, LA_FP16 = 1, LA_FP32 = 2 (element type of q,k,v,o and
 *     of the gradients; x,y,dy,dx for the norm).  Slopes, rstd and every
 *     accumulator are float32;
 *   - nothing is read from the process environment: how a call is mapped onto launches depends on
 *     its arguments (la_launch_opts below, where a caller wants to override the library's choices)
 *     and on the compute-unit count of the current device;
 *   - calls are thread-safe and may overlap on different streams, with one exception: la_fwd_static,
 *     whose calls share one scratch array per GPU (one call in flight per GPU, see there);
 *   - what the library remembers, per device and until the process ends: the device's compute-unit
 *     count (asked once; launch plans and workspace sizes depend on it), one flag per kernel
 *     instantiation saying that its dynamic-LDS limit has been raised (hipFuncSetAttribute, made before
 *     that kernel's first launch) and the address of la_fwd_static's array.  The first use of a kernel on a
 *     device therefore does more than enqueue work, which stream capture does not allow: call la_init()
 *     on the device beforehand, or make the first call of each shape outside the capture.
 */
#ifndef LIGHTNING_ATTN_HIP_H
#define LIGHTNING_ATTN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { LA_BF16 = 0, LA_FP16 = 1, LA_FP32 = 2 };

enum {
    LA_OK = 0,
    LA_E_NULLPTR = -1,     /* a required pointer is NULL                      */
    LA_E_SHAPE = -2,       /* a dimension is <= 0 or exceeds the index range  */
    LA_E_UNSUPPORTED = -3, /* head dims / dtype outside la_supported()        */
    LA_E_WORKSPACE = -4,   /* workspace too small for the requested plan       */
    LA_E_ALIGN = -5        /* a pointer or stride is not 16-byte aligned      */
};

/*
 * One-time work for the current device, done up front instead of at first use: the compute-unit count,
 * the dynamic-LDS limit of every kernel instantiation and the address of la_fwd_static's array.  After it
 * every other entry point only enqueues kernels on that device, so first calls may sit inside a stream
 * capture.  Optional otherwise; idempotent; returns 0 or the hipError_t of the failing runtime call.
 * No counterpart in the reference (Triton compiles and configures its kernels at their first launch,
 * lightning_attn/ops/triton/lightning_attn2.py:416).
 */
int la_init(void);

/* Host-only helpers (usable without a GPU). */
const char *la_version(void);
const char *la_error_string(int code);
/* 1 when the attention kernels accept head dims (d, e) at this dtype:
 * d and e multiples of 8, 8 <= d,e <= 256 (<= 128 for float32).  Replaces the dimension gate
 * lightning_attn/ops/lightning_attn_interface.py:8-9,26 (is_support). */
int la_supported(int64_t d, int64_t e, int dtype);
/* Bytes of device scratch la_fwd (which=0) / la_bwd (which=1) can use for these shapes: 0 unless
 * there are so few (batch, head) sequences that the walk over a long sequence is cut into chunks
 * (the job of the reference's variant="parallel", lightning_attn/ops/triton/lightning_attn2_parallel.py:835-1072).
 * The scratch then holds one d x e float state per chunk.  It is optional: with workspace == NULL,
 * or fewer bytes than this, the chunks rebuild their incoming state by walking the blocks before
 * them instead, which gives bit-identical results to the single walk and is several times slower
 * for long sequences.  16-byte aligned; contents need not survive the call, and calls that follow
 * each other on one stream may share it.  0 for shapes la_fwd / la_bwd reject. */
size_t la_workspace_bytes(int which, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype);

/*
 * How a call is mapped onto kernel launches.  A zero-filled struct (or a NULL pointer where one is
 * taken) leaves every choice to the library, which is what production callers want; the fields
 * exist for measurements and for tests that compare the launch forms with each other.  Results
 * are bit-identical across all settings except `scan` / `chunks` with a workspace (chunk states
 * summed in another order: equal to rounding).
 */
enum { LA_OPT_AUTO = 0, LA_OPT_OFF = 1, LA_OPT_ON = 2, LA_OPT_ALL = 3 };
typedef struct la_launch_opts {
    int32_t chunks; /* sequence chunks per (batch, head, column slice): 0 = library's choice, > 0 forced
                       (at most 64 from scanned states, 8 with warm-up blocks, never more than blocks) */
    int32_t scan;   /* start chunks from scanned states in the workspace: LA_OPT_AUTO (where estimated
                       faster and the workspace suffices) / LA_OPT_OFF (warm-up blocks only)            */
    int32_t wide;   /* output columns per workgroup: AUTO / OFF (64) / ON (128, or two equal slices) /
                       LA_OPT_ALL (d and e in 129..192: all columns of a sequence in one workgroup;
                       as AUTO elsewhere)                                                               */
    int32_t paired; /* backward, d == e: dK and dV in one launch: AUTO (yes) / OFF (one after the other) */
    int32_t once;   /* backward, few sequences: every sweep in one launch: AUTO / OFF / ON               */
} la_launch_opts;

/*
 * Forward of decayed causal linear attention, O = (Q K^T * M_h) V with
 * M_h[i][j] = exp(-s[h] (i-j)) for i >= j, else 0.   s == NULL means no decay
 * (M = tril(1)).  q,k: (b,h,n,d); v,o: (b,h,n,e); s: h floats.
 * Replaces LightningAttention2.forward + _fwd_kernel
 * (lightning_attn/ops/triton/lightning_attn2.py:8-85, 400-434) and the no-decay
 * twin (lightning_attn/ops/triton/lightning_attn2_no_decay.py:8-77, 369-401).
 */
int la_fwd(const void *q, const void *k, const void *v, const float *s, void *o,
           int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
           void *workspace, size_t ws_bytes, void *stream);

/*
 * Backward of the same operator: given dO (b,h,n,e) writes dq,dk (b,h,n,d) and
 * dv (b,h,n,e), each exactly once (no read-modify-write of the gradients).
 * Replaces LightningAttention2.backward + _bwd_intra_kernel + _bwd_inter_kernel
 * (lightning_attn/ops/triton/lightning_attn2.py:88-395, 437-504) and the
 * no-decay twin (lightning_attn2_no_decay.py:80-364, 404-468).
 */
int la_bwd(const void *q, const void *k, const void *v, const float *s, const void *dout,
           void *dq, void *dk, void *dv,
           int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
           void *workspace, size_t ws_bytes, void *stream);

/*
 * la_fwd / la_bwd on tensors that are not plain (b,h,n,d) arrays: every tensor argument gets
 * three strides in ELEMENTS (batch, head, token), in the order of the pointer arguments
 * (la_fwd_strided: q,k,v,o = 12 values; la_bwd_strided: q,k,v,dout,dq,dk,dv = 21 values); the
 * feature dim stays contiguous.  A projection output (b,n,h*d) is then used in place with
 * strides {n*h*d, d, h*d}, and o / dq / dk / dv can be written in that layout too.  This removes
 * the copies the reference makes around the operator: `.contiguous()` on q,k,v,do
 * (lightning_attn/ops/triton/lightning_attn2.py:402-405, 439-442) after the caller's
 * `rearrange(x, "b n (h d) -> b h n d")` and the copy behind `rearrange(o, "b h n d -> b n (h d)")`
 * (examples/module/tnl_attn.py:56-64).  Strides must be multiples of 16 bytes, token stride >=
 * the feature dim, one (batch, head) sequence below 2 GiB; bf16 / fp16 only (float32 tensors must
 * be plain: LA_E_UNSUPPORTED otherwise).
 */
int la_fwd_strided(const void *q, const void *k, const void *v, const float *s, void *o,
                   const int64_t *strides,
                   int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                   void *workspace, size_t ws_bytes, void *stream);
int la_bwd_strided(const void *q, const void *k, const void *v, const float *s, const void *dout,
                   void *dq, void *dk, void *dv, const int64_t *strides,
                   int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                   void *workspace, size_t ws_bytes, void *stream);

/*
 * The same entry points with explicit launch options: `strides` as in la_fwd_strided /
 * la_bwd_strided or NULL for plain (b,h,n,d) tensors; `opts` NULL for the library's own choices
 * (then they are exactly la_fwd / la_bwd / la_fwd_strided / la_bwd_strided / la_workspace_bytes).
 * A workspace sized by la_workspace_bytes_opts with the same opts is always large enough.
 * No counterpart in the reference, whose launch shapes are constants
 * (lightning_attn/ops/triton/lightning_attn2.py:410-414, 454-458).
 */
size_t la_workspace_bytes_opts(int which, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                               const la_launch_opts *opts);
int la_fwd_opts(const void *q, const void *k, const void *v, const float *s, void *o,
                const int64_t *strides,
                int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                void *workspace, size_t ws_bytes, const la_launch_opts *opts, void *stream);
int la_bwd_opts(const void *q, const void *k, const void *v, const float *s, const void *dout,
                void *dq, void *dk, void *dv, const int64_t *strides,
                int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                void *workspace, size_t ws_bytes, const la_launch_opts *opts, void *stream);

/*
 * la_fwd_opts on pre-activations: O = attention(silu(q), silu(k), silu(v)), silu(t) = t / (1 + exp(-t))
 * evaluated in float32 and rounded to the tensors' type where the tiles are loaded, so that the activated
 * tensors never exist in memory.  This is the forward pass of the reference's attention block without its
 * three activation passes (`F.silu(self.q_proj(x))` ..., examples/module/tnl_attn.py:51-54) for callers that
 * need no backward pass (inference): 0.36 against 0.56 ms at b4 h32 n8192 d=e=128.  bf16 / fp16 with
 * d, e <= 128 (la_fwd_silu_supported; LA_E_UNSUPPORTED otherwise: apply the activation first and call la_fwd).
 * Workspace as for la_fwd.
 */
int la_fwd_silu_supported(int64_t d, int64_t e, int dtype);
int la_fwd_silu(const void *q, const void *k, const void *v, const float *s, void *o,
                const int64_t *strides,
                int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                void *workspace, size_t ws_bytes, const la_launch_opts *opts, void *stream);

/*
 * Forward and backward pass as a pair: the forward pass leaves its d x e float state K^T V at a few
 * token boundaries, and the dQ sweep of the backward pass - whose state V^T K is the transpose - starts
 * one chunk of each sequence at each of them.  It then needs neither warm-up blocks nor collect and scan
 * launches to run as several workgroups per sequence, which is what lets it use 128-column workgroups
 * when b*h alone gives the chip one or two workgroups per compute unit (b*h of 65 .. 128 on 256 CUs,
 * 64 < d <= 128, e <= 128, bf16 / fp16) - or, with d and e both in 129 .. 192, workgroups that take all
 * columns of a sequence.  The reference recomputes that state in its backward pass
 * (lightning_attn/ops/triton/lightning_attn2.py:240-280) and saves the inputs only (:432); keeping a few
 * states as well is a deviation made for speed.  Gradients agree with la_bwd's to rounding (the state is
 * summed in the same order but its operands are rounded to the tensors' dtype in the other role).
 *
 * la_saved_state_bytes: bytes the pair uses for these shapes and options, 0 where it would not help (then
 * la_fwd_save is la_fwd_opts and la_bwd_saved is la_bwd_opts).  Layout: for each of the b*h sequences
 * m = bytes / (b*h*d*e*4) row-major d x e float matrices, matrix j being
 *     sum over tokens t < T of exp(-s[h] (T - t)) k_t^T v_t,   T = (j + 1) * la_saved_state_interval(...).
 * la_fwd_save: la_fwd_opts that also fills `saved` (16-byte aligned, saved_bytes >= la_saved_state_bytes;
 * otherwise, and with saved == NULL, nothing is saved).  la_bwd_saved: la_bwd_opts that uses `saved` as left
 * by la_fwd_save for the same tensors, shapes and options (same conditions; otherwise exactly la_bwd_opts).
 */
size_t la_saved_state_bytes(int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                            const la_launch_opts *opts);
int64_t la_saved_state_interval(int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                                const la_launch_opts *opts);
int la_fwd_save(const void *q, const void *k, const void *v, const float *s, void *o,
                const int64_t *strides,
                int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                void *workspace, size_t ws_bytes, const la_launch_opts *opts,
                float *saved, size_t saved_bytes, void *stream);
int la_bwd_saved(const void *q, const void *k, const void *v, const float *s, const void *dout,
                 void *dq, void *dk, void *dv, const int64_t *strides,
                 int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                 void *workspace, size_t ws_bytes, const la_launch_opts *opts,
                 const float *saved, size_t saved_bytes, void *stream);

/*
 * la_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc) and so cannot supply the workspace that makes few
 * long sequences fast: same arguments without the workspace pair, same results bit for bit as la_fwd
 * given la_workspace_bytes(0, ...) bytes.  The chunk states go into a static device array of
 * LA_STATIC_SCRATCH_BYTES inside the library, which every GPU the library runs on holds until the
 * process ends.  The call allocates and frees nothing.  Shapes whose plan needs more than the array
 * holds are rejected with LA_E_WORKSPACE before anything is launched (the plans the library makes for
 * a chip of up to 256 compute units always fit).  All calls on one GPU share the array: calls that
 * follow each other on one stream are safe, calls that overlap on one GPU (different streams or
 * threads) race on it.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress); make it outside graph capture.
 * No counterpart in the reference (its operators allocate through torch,
 * lightning_attn/ops/triton/lightning_attn2.py:408).
 */
#define LA_STATIC_SCRATCH_BYTES (48u << 20)
int la_fwd_static(const void *q, const void *k, const void *v, const float *s, void *o,
                  int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype, void *stream);

/*
 * SimpleRMSNorm forward: rstd[r] = 1/sqrt(mean(x[r,:]^2) + eps), y = x * rstd.
 * x,y: rows x cols with `row_stride` elements between rows; rstd: rows floats.
 * Replaces _SrmsNorm.forward + srms_norm_fw
 * (lightning_attn/ops/triton/srmsnorm.py:12-33, 78-122).
 */
int srmsnorm_fwd(const void *x, void *y, float *rstd, int64_t rows, int64_t cols, int64_t row_stride,
                 float eps, int dtype, void *stream);

/*
 * SimpleRMSNorm backward: xhat = x*rstd; dx = (dy - xhat*mean(xhat*dy)) * rstd.
 * Only x has `row_stride`; dy and dx are dense rows x cols arrays (the reference makes dy
 * contiguous and allocates dx like it, srmsnorm.py:149-151).
 * Replaces _SrmsNorm.backward + srms_norm_bwd_dx_fused
 * (lightning_attn/ops/triton/srmsnorm.py:38-74, 125-175).
 */
int srmsnorm_bwd(const void *x, const void *dy, const float *rstd, void *dx,
                 int64_t rows, int64_t cols, int64_t row_stride, int dtype, void *stream);

/*
 * Gated output norm of the TNL attention block, the caller of the attention operator:
 *     y = LayerNorm(o; weight, bias, eps) * sigmoid(g)        o, g, y: rows x cols, dense
 * with weight, bias of cols elements in the tensors' dtype and mean, rstd (rows floats) kept for the
 * backward pass.  One pass over o and g instead of the three PyTorch operators of
 * examples/module/tnl_attn.py:66-69 (`self.norm(output)`, `F.sigmoid(...)`, `output * output_gate`).
 * cols must be a multiple of 8 (4 for float32) and at most 8192 (4096): norm_gate_supported().
 */
int norm_gate_supported(int64_t cols, int dtype);
int norm_gate_fwd(const void *o, const void *g, const void *weight, const void *bias, void *y,
                  float *mean, float *rstd, int64_t rows, int64_t cols, float eps, int dtype, void *stream);
/*
 * Its backward pass: given dy writes d_o and d_g (rows x cols) and the column sums dweight, dbias
 * (cols elements, tensor dtype; accumulated in float32 in a fixed order, so results are
 * deterministic).  The partial column sums pass through `workspace`, which must hold
 * norm_gate_workspace_bytes(rows, cols, dtype) bytes (LA_E_WORKSPACE otherwise); its contents need
 * not survive the call.  Replaces the autograd chain of the same three operators.
 */
size_t norm_gate_workspace_bytes(int64_t rows, int64_t cols, int dtype);
int norm_gate_bwd(const void *o, const void *g, const void *weight, const void *bias,
                  const float *mean, const float *rstd, const void *dy,
                  void *d_o, void *d_g, void *dweight, void *dbias,
                  void *workspace, size_t ws_bytes, int64_t rows, int64_t cols, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LIGHTNING_ATTN_HIP_H */
