// extern "C" entry points of the attention path (see include/lightning_attn_hip.h).
#include <algorithm>

#include "la_sweep_common.h"
#include "lightning_attn_hip.h"

namespace la {
int sweep(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
          bool reverse, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st);
int sweep_silu(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
               void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st);
int sweep_bwd_once(const SweepIO& dq, const SweepIO& dk, const SweepIO& dv, const float* s, int64_t bh, int64_t h, int64_t n,
                   int64_t d, int dtype, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st);
int sweep_fwd_rev_once(const SweepIO& fwd, const SweepIO& rev, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk,
                       int64_t dv, int dtype, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st);
int sweep2(const SweepIO& io0, const SweepIO& io1, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv,
           int dtype, bool reverse, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st);
size_t sweep_workspace_bytes(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, int dtype, const Opts& opts);
SavedPlan plan_saved(int64_t bh, int64_t n, int64_t d, int64_t e, int dtype, const Opts& opts);
int sweep_saving(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
                 float* save, int save_len, int width, hipStream_t st);
int sweep_resumed(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
                  const float* saved, int nchunk, int chunk_len, int width, hipStream_t st);
int prepare_srmsnorm();   // srmsnorm.hip
int prepare_norm_gate();  // norm_gate.hip
int sweep_f32(const void* x, const void* y, const void* z, void* out, const float* s, int64_t bh, int64_t h,
              int64_t n, int64_t dk, int64_t dv, bool reverse, int chunks, hipStream_t st);
int sweep_f32_bwd_once(const void* q, const void* k, const void* v, const void* dout, void* dq, void* dk, void* dv,
                       const float* s, int64_t bh, int64_t h, int64_t n, int64_t d, int chunks, hipStream_t st);

// A tensor argument: device pointer + where its (batch, head, token) rows start.
struct Tensor {
    const void* p;
    Layout l;
};
static Tensor dense(const void* p, int64_t h, int64_t n, int64_t cols) { return Tensor{p, Layout{h * n * cols, n * cols, cols}}; }
static Tensor strided(const void* p, const int64_t* st) { return Tensor{p, Layout{st[0], st[1], st[2]}}; }
static bool is_dense(const Tensor& t, int64_t h, int64_t n, int64_t cols) {
    return t.l.ts == cols && t.l.hs == n * cols && t.l.bs == h * n * cols;
}

static SweepIO io(const Tensor& x, const Tensor& y, const Tensor& z, const Tensor& out) {
    return SweepIO{x.p, y.p, z.p, const_cast<void*>(out.p), x.l, y.l, z.l, out.l};
}

// caller's scratch memory (may be absent)
struct Scratch {
    void* p;
    size_t bytes;
};

// one directional sweep at the element type named by dtype
static int run(const Tensor& x, const Tensor& y, const Tensor& z, const Tensor& out, const float* s, int64_t bh, int64_t h,
               int64_t n, int64_t dk, int64_t dv, int dtype, bool reverse, const Scratch& ws, const Opts& opts, hipStream_t st) {
    if (dtype == LA_FP32) {
        // the float32 accuracy kernel takes plain (b, h, n, d) tensors only
        if (!is_dense(x, h, n, dk) || !is_dense(y, h, n, dk) || !is_dense(z, h, n, dv) || !is_dense(out, h, n, dv))
            return LA_E_UNSUPPORTED;
        return sweep_f32(x.p, y.p, z.p, const_cast<void*>(out.p), s, bh, h, n, dk, dv, reverse, opts.chunks, st);
    }
    return sweep(io(x, y, z, out), s, bh, h, n, dk, dv, dtype, reverse, ws.p, ws.bytes, opts, st);
}

static inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static int check_dims(int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype) {
    if (b < 0 || h <= 0 || n < 0 || d <= 0 || e <= 0) return LA_E_SHAPE;
    if (b * h > 0x7fffffffLL / 64) return LA_E_SHAPE;
    // the kernels address one (batch, head) slice with 32-bit byte offsets below 2 GiB
    if (n * (d > e ? d : e) * 4 >= (1LL << 31)) return LA_E_SHAPE;
    if (!la_supported(d, e, dtype)) return LA_E_UNSUPPORTED;
    return LA_OK;
}

static int check_opts(const Opts& o) {
    if (o.chunks < 0) return LA_E_SHAPE;
    for (int v : {o.scan, o.paired, o.once})
        if (v != LA_OPT_AUTO && v != LA_OPT_OFF && v != LA_OPT_ON) return LA_E_SHAPE;
    if (o.wide != LA_OPT_AUTO && o.wide != LA_OPT_OFF && o.wide != LA_OPT_ON && o.wide != LA_OPT_ALL) return LA_E_SHAPE;
    return LA_OK;
}
static const Opts kAuto = {0, LA_OPT_AUTO, LA_OPT_AUTO, LA_OPT_AUTO, LA_OPT_AUTO};

// pointer and strides of one tensor with `cols` features per row
static int check_tensor(const Tensor& t, int64_t b, int64_t h, int64_t n, int64_t cols, int dtype) {
    if (!t.p) return LA_E_NULLPTR;
    const int64_t elt = dtype == LA_FP32 ? 4 : 2;
    if (!al16(t.p) || (t.l.bs * elt) % 16 || (t.l.hs * elt) % 16 || (t.l.ts * elt) % 16) return LA_E_ALIGN;
    if (t.l.ts < cols || t.l.hs < 0 || t.l.bs < 0) return LA_E_SHAPE;
    if (b > 1 && t.l.bs == 0) return LA_E_SHAPE;
    if (h > 1 && t.l.hs == 0) return LA_E_SHAPE;
    // one (batch, head) sequence is addressed with 32-bit byte offsets below 2 GiB
    if (((n - 1) * t.l.ts + cols) * elt >= (1LL << 31)) return LA_E_SHAPE;
    return LA_OK;
}

// States for the backward pass (may be absent): memory the forward pass writes / the backward pass reads.
struct Saved {
    float* p;
    size_t bytes;
};
static bool saved_usable(const Saved& sv, const SavedPlan& pl) {
    return pl.nchunk > 1 && sv.p && sv.bytes >= pl.bytes && al16(sv.p);
}

static int fwd(const Tensor& q, const Tensor& k, const Tensor& v, const float* s, const Tensor& o, int64_t b, int64_t h,
               int64_t n, int64_t d, int64_t e, int dtype, const Scratch& ws, const Opts& opts, const Saved& sv, hipStream_t st,
               bool silu = false) {
    int rc = check_dims(b, h, n, d, e, dtype);
    if (rc != LA_OK) return rc;
    if ((rc = check_opts(opts)) != LA_OK) return rc;
    if (b == 0 || n == 0) return LA_OK;  // nothing to do; empty tensors may carry null pointers
    const Tensor* ts[4] = {&q, &k, &v, &o};
    const int64_t cols[4] = {d, d, e, e};
    for (int i = 0; i < 4; ++i)
        if (!ts[i]->p) return LA_E_NULLPTR;
    for (int i = 0; i < 4; ++i)
        if ((rc = check_tensor(*ts[i], b, h, n, cols[i], dtype)) != LA_OK) return rc;
    if (silu) return sweep_silu(io(q, k, v, o), s, b * h, h, n, d, e, dtype, ws.p, ws.bytes, opts, st);
    if (sv.p) {
        const SavedPlan pl = plan_saved(b * h, n, d, e, dtype, opts);
        if (saved_usable(sv, pl)) return sweep_saving(io(q, k, v, o), s, b * h, h, n, d, e, dtype, sv.p, pl.chunk_len, pl.fwd_width, st);
    }
    return run(q, k, v, o, s, b * h, h, n, d, e, dtype, false, ws, opts, st);
}

static int bwd(const Tensor& q, const Tensor& k, const Tensor& v, const float* s, const Tensor& dout, const Tensor& dq,
               const Tensor& dk, const Tensor& dv, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
               const Scratch& ws, const Opts& opts, const Saved& sv, hipStream_t st) {
    int rc = check_dims(b, h, n, d, e, dtype);
    if (rc != LA_OK) return rc;
    if ((rc = check_opts(opts)) != LA_OK) return rc;
    if (b == 0 || n == 0) return LA_OK;
    const Tensor* ts[7] = {&q, &k, &v, &dout, &dq, &dk, &dv};
    const int64_t cols[7] = {d, d, e, e, d, d, e};
    for (int i = 0; i < 7; ++i)
        if (!ts[i]->p) return LA_E_NULLPTR;
    for (int i = 0; i < 7; ++i)
        if ((rc = check_tensor(*ts[i], b, h, n, cols[i], dtype)) != LA_OK) return rc;
    // dQ_i = sum_{j<=i} lam^(i-j) (dO_i . v_j) k_j
    // (the launches follow each other on one stream, so they can all use the same scratch memory)
    if (d == e && dtype == LA_FP32 && opts.paired != LA_OPT_OFF) {
        // float32: the three sweeps always share a launch (plain tensors only, as in run())
        for (int i = 0; i < 7; ++i)
            if (!is_dense(*ts[i], h, n, d)) return LA_E_UNSUPPORTED;
        return sweep_f32_bwd_once(q.p, k.p, v.p, dout.p, const_cast<void*>(dq.p), const_cast<void*>(dk.p),
                                  const_cast<void*>(dv.p), s, b * h, h, n, d, opts.chunks, st);
    }
    if (d == e && dtype != LA_FP32) {
        // few sequences: all three gradients in one launch, side by side (LA_E_UNSUPPORTED: not this time)
        rc = sweep_bwd_once(io(dout, v, k, dq), io(v, dout, q, dk), io(k, q, dout, dv), s, b * h, h, n, d, dtype, ws.p,
                            ws.bytes, opts, st);
        if (rc != LA_E_UNSUPPORTED) return rc;
    }
    if (d != e && dtype != LA_FP32) {
        // dQ and dK have one shape and opposite directions: with few sequences, one launch for the two
        rc = sweep_fwd_rev_once(io(dout, v, k, dq), io(v, dout, q, dk), s, b * h, h, n, e, d, dtype, ws.p, ws.bytes, opts, st);
        if (rc == LA_OK) return run(k, q, dout, dv, s, b * h, h, n, d, e, dtype, true, ws, opts, st);
        if (rc != LA_E_UNSUPPORTED) return rc;
    }
    const SavedPlan pl = sv.p ? plan_saved(b * h, n, d, e, dtype, opts) : SavedPlan{1, 0, 0, 0, 0};
    if (saved_usable(sv, pl) && d == e) {
        // dK + dV first: their reverse walk starts at the end of the sequences, where the forward pass has just
        // been (what the last-level cache still holds of k, v, q is read there: -0.8 % per step at b4 h32 n8192
        // d128), and ends at their start, where the first dQ chunk begins
        rc = sweep2(io(v, dout, q, dk), io(k, q, dout, dv), s, b * h, h, n, d, e, dtype, true, ws.p, ws.bytes, opts, st);
        if (rc != LA_OK) return rc;
        return sweep_resumed(io(dout, v, k, dq), s, b * h, h, n, e, d, dtype, sv.p, pl.nchunk, pl.chunk_len, pl.dq_width, st);
    }
    if (saved_usable(sv, pl))  // the chunks of dQ start from the states the forward pass left
        rc = sweep_resumed(io(dout, v, k, dq), s, b * h, h, n, e, d, dtype, sv.p, pl.nchunk, pl.chunk_len, pl.dq_width, st);
    else
        rc = run(dout, v, k, dq, s, b * h, h, n, e, d, dtype, false, ws, opts, st);
    if (rc != LA_OK) return rc;
    // dK_j = sum_{i>=j} lam^(i-j) (v_j . dO_i) q_i   and   dV_j = sum_{i>=j} lam^(i-j) (k_j . q_i) dO_i
    // have the same shape when d == e: one launch, in which they share the reads of dO and q
    if (d == e && dtype != LA_FP32)
        return sweep2(io(v, dout, q, dk), io(k, q, dout, dv), s, b * h, h, n, d, e, dtype, true, ws.p, ws.bytes, opts, st);
    rc = run(v, dout, q, dk, s, b * h, h, n, e, d, dtype, true, ws, opts, st);
    if (rc != LA_OK) return rc;
    return run(k, q, dout, dv, s, b * h, h, n, d, e, dtype, true, ws, opts, st);
}
}  // namespace la

extern "C" const char* la_version(void) { return "lightning_attn_hip 0.1.0 (gfx950)"; }

extern "C" const char* la_error_string(int code) {
    switch (code) {
        case LA_OK: return "success";
        case LA_E_NULLPTR: return "a required pointer is NULL";
        case LA_E_SHAPE: return "a dimension is out of range";
        case LA_E_UNSUPPORTED: return "head dims / dtype not supported (need d,e multiples of 8 in [8,256]; [8,128] for float32)";
        case LA_E_WORKSPACE: return "workspace too small for the requested plan";
        case LA_E_ALIGN: return "pointer not 16-byte aligned";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown error";
}

extern "C" int la_supported(int64_t d, int64_t e, int dtype) {
    if (dtype != LA_BF16 && dtype != LA_FP16 && dtype != LA_FP32) return 0;
    const int64_t hi = dtype == LA_FP32 ? 128 : 256;
    if (d < 8 || e < 8 || d > hi || e > hi) return 0;
    if ((d % 8) || (e % 8)) return 0;
    return 1;
}

extern "C" size_t la_workspace_bytes_opts(int which, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                                          const la_launch_opts* opts) {
    const la::Opts& o = opts ? *opts : la::kAuto;
    // nothing for empty tensors and for shapes the entry points reject
    if (b <= 0 || n <= 0 || la::check_dims(b, h, n, d, e, dtype) != LA_OK || la::check_opts(o) != LA_OK) return 0;
    using la::sweep_workspace_bytes;
    const int64_t bh = b * h;
    if (which == 0) return sweep_workspace_bytes(bh, n, d, e, 1, dtype, o);  // O = sweep(q, k, v)
    // dQ = sweep(dO, v, k); then dK and dV, together when d == e
    size_t need = sweep_workspace_bytes(bh, n, e, d, 1, dtype, o);
    const size_t rest = d == e && o.paired != LA_OPT_OFF
                            ? sweep_workspace_bytes(bh, n, d, e, 2, dtype, o)
                            : std::max(sweep_workspace_bytes(bh, n, e, d, 1, dtype, o), sweep_workspace_bytes(bh, n, d, e, 1, dtype, o));
    return std::max(need, rest);
}

extern "C" size_t la_workspace_bytes(int which, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype) {
    return la_workspace_bytes_opts(which, b, h, n, d, e, dtype, nullptr);
}

extern "C" int la_fwd_save(const void* q, const void* k, const void* v, const float* s, void* o, const int64_t* strides,
                           int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype, void* workspace,
                           size_t ws_bytes, const la_launch_opts* opts, float* saved, size_t saved_bytes, void* stream) {
    const la::Scratch ws = {workspace, workspace ? ws_bytes : 0};
    const la::Saved sv = {saved, saved ? saved_bytes : 0};
    const la::Opts& op = opts ? *opts : la::kAuto;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    using la::dense;
    using la::strided;
    if (!strides)
        return la::fwd(dense(q, h, n, d), dense(k, h, n, d), dense(v, h, n, e), s, dense(o, h, n, e), b, h, n, d, e, dtype, ws, op, sv, st);
    return la::fwd(strided(q, strides), strided(k, strides + 3), strided(v, strides + 6), s, strided(o, strides + 9), b, h, n,
                   d, e, dtype, ws, op, sv, st);
}

extern "C" int la_fwd_silu_supported(int64_t d, int64_t e, int dtype) {
    return (dtype == LA_BF16 || dtype == LA_FP16) && d <= 128 && e <= 128 && la_supported(d, e, dtype);
}

extern "C" int la_fwd_silu(const void* q, const void* k, const void* v, const float* s, void* o, const int64_t* strides,
                           int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype, void* workspace,
                           size_t ws_bytes, const la_launch_opts* opts, void* stream) {
    if (la_supported(d, e, dtype) && !la_fwd_silu_supported(d, e, dtype)) return LA_E_UNSUPPORTED;
    const la::Scratch ws = {workspace, workspace ? ws_bytes : 0};
    const la::Saved none = {nullptr, 0};
    const la::Opts& op = opts ? *opts : la::kAuto;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    using la::dense;
    using la::strided;
    if (!strides)
        return la::fwd(dense(q, h, n, d), dense(k, h, n, d), dense(v, h, n, e), s, dense(o, h, n, e), b, h, n, d, e, dtype, ws, op, none, st, true);
    return la::fwd(strided(q, strides), strided(k, strides + 3), strided(v, strides + 6), s, strided(o, strides + 9), b, h, n,
                   d, e, dtype, ws, op, none, st, true);
}

extern "C" int la_fwd_opts(const void* q, const void* k, const void* v, const float* s, void* o, const int64_t* strides,
                           int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype, void* workspace,
                           size_t ws_bytes, const la_launch_opts* opts, void* stream) {
    return la_fwd_save(q, k, v, s, o, strides, b, h, n, d, e, dtype, workspace, ws_bytes, opts, nullptr, 0, stream);
}

extern "C" size_t la_saved_state_bytes(int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                                       const la_launch_opts* opts) {
    const la::Opts& o = opts ? *opts : la::kAuto;
    if (b <= 0 || n <= 0 || la::check_dims(b, h, n, d, e, dtype) != LA_OK || la::check_opts(o) != LA_OK) return 0;
    return la::plan_saved(b * h, n, d, e, dtype, o).bytes;
}

extern "C" int64_t la_saved_state_interval(int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                                           const la_launch_opts* opts) {
    const la::Opts& o = opts ? *opts : la::kAuto;
    if (b <= 0 || n <= 0 || la::check_dims(b, h, n, d, e, dtype) != LA_OK || la::check_opts(o) != LA_OK) return 0;
    const la::SavedPlan pl = la::plan_saved(b * h, n, d, e, dtype, o);
    return pl.nchunk > 1 ? (int64_t)pl.chunk_len * 64 : 0;
}

extern "C" int la_bwd_saved(const void* q, const void* k, const void* v, const float* s, const void* dout, void* dq,
                            void* dk, void* dv, const int64_t* strides, int64_t b, int64_t h, int64_t n, int64_t d,
                            int64_t e, int dtype, void* workspace, size_t ws_bytes, const la_launch_opts* opts,
                            const float* saved, size_t saved_bytes, void* stream) {
    const la::Scratch ws = {workspace, workspace ? ws_bytes : 0};
    const la::Saved sv = {const_cast<float*>(saved), saved ? saved_bytes : 0};
    const la::Opts& op = opts ? *opts : la::kAuto;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    using la::dense;
    using la::strided;
    if (!strides)
        return la::bwd(dense(q, h, n, d), dense(k, h, n, d), dense(v, h, n, e), s, dense(dout, h, n, e), dense(dq, h, n, d),
                       dense(dk, h, n, d), dense(dv, h, n, e), b, h, n, d, e, dtype, ws, op, sv, st);
    return la::bwd(strided(q, strides), strided(k, strides + 3), strided(v, strides + 6), s, strided(dout, strides + 9),
                   strided(dq, strides + 12), strided(dk, strides + 15), strided(dv, strides + 18), b, h, n, d, e, dtype, ws,
                   op, sv, st);
}

extern "C" int la_bwd_opts(const void* q, const void* k, const void* v, const float* s, const void* dout, void* dq,
                           void* dk, void* dv, const int64_t* strides, int64_t b, int64_t h, int64_t n, int64_t d,
                           int64_t e, int dtype, void* workspace, size_t ws_bytes, const la_launch_opts* opts, void* stream) {
    return la_bwd_saved(q, k, v, s, dout, dq, dk, dv, strides, b, h, n, d, e, dtype, workspace, ws_bytes, opts, nullptr, 0, stream);
}

extern "C" int la_fwd(const void* q, const void* k, const void* v, const float* s, void* o, int64_t b, int64_t h,
                      int64_t n, int64_t d, int64_t e, int dtype, void* workspace, size_t ws_bytes, void* stream) {
    return la_fwd_opts(q, k, v, s, o, nullptr, b, h, n, d, e, dtype, workspace, ws_bytes, nullptr, stream);
}

extern "C" int la_bwd(const void* q, const void* k, const void* v, const float* s, const void* dout, void* dq,
                      void* dk, void* dv, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                      void* workspace, size_t ws_bytes, void* stream) {
    return la_bwd_opts(q, k, v, s, dout, dq, dk, dv, nullptr, b, h, n, d, e, dtype, workspace, ws_bytes, nullptr, stream);
}

// ---- forward without any allocation: the chunk states live in a static device array ----------------
// Each GPU the library runs on holds its own copy of the array, at its own address, until the process
// ends.  In host code the array's name is only a handle: the address kernels can use comes from
// hipGetSymbolAddress, asked once per device with that device current, and is kept per device.
namespace la {
static __device__ __align__(256) unsigned char scratch[LA_STATIC_SCRATCH_BYTES];
static void* scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device.
static int static_scratch(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return LA_E_UNSUPPORTED;
    void* p = __atomic_load_n(&scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        // (two threads arriving together both ask and both get the same answer)
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return (int)hipErrorInvalidSymbol;
        __atomic_store_n(&scratch_ptr[dev], p, __ATOMIC_RELEASE);
    }
    *out = p;
    return LA_OK;
}
}  // namespace la

extern "C" int la_init(void) {
    int rc = la::prepare_plans();
    if (rc == LA_OK) rc = la::prepare_pipe();
    if (rc == LA_OK) rc = la::prepare_f32();
    if (rc == LA_OK) rc = la::prepare_srmsnorm();
    if (rc == LA_OK) rc = la::prepare_norm_gate();
    void* p = nullptr;
    if (rc == LA_OK) rc = la::static_scratch(&p);
    return rc;
}

extern "C" int la_fwd_static(const void* q, const void* k, const void* v, const float* s, void* o, int64_t b, int64_t h,
                             int64_t n, int64_t d, int64_t e, int dtype, void* stream) {
    // what la_fwd would use of a caller's workspace for this shape; host arithmetic only
    const size_t need = la_workspace_bytes(0, b, h, n, d, e, dtype);
    if (need > (size_t)LA_STATIC_SCRATCH_BYTES) return LA_E_WORKSPACE;
    void* ws = nullptr;
    if (need > 0) {
        const int rc = la::static_scratch(&ws);
        if (rc != LA_OK) return rc;
    }
    // Every state slot the scan reads is written by the collect launch before it (state waves without
    // live columns write zeros), so nothing in the array has to start at zero and what an earlier call
    // left there does not matter.
    return la_fwd(q, k, v, s, o, b, h, n, d, e, dtype, ws, need, stream);
}

extern "C" int la_fwd_strided(const void* q, const void* k, const void* v, const float* s, void* o,
                              const int64_t* strides, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                              void* workspace, size_t ws_bytes, void* stream) {
    if (!strides) return LA_E_NULLPTR;
    return la_fwd_opts(q, k, v, s, o, strides, b, h, n, d, e, dtype, workspace, ws_bytes, nullptr, stream);
}

extern "C" int la_bwd_strided(const void* q, const void* k, const void* v, const float* s, const void* dout, void* dq,
                              void* dk, void* dv, const int64_t* strides, int64_t b, int64_t h, int64_t n, int64_t d,
                              int64_t e, int dtype, void* workspace, size_t ws_bytes, void* stream) {
    if (!strides) return LA_E_NULLPTR;
    return la_bwd_opts(q, k, v, s, dout, dq, dk, dv, strides, b, h, n, d, e, dtype, workspace, ws_bytes, nullptr, stream);
}
