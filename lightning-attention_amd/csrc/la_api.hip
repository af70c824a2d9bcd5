// extern "C" entry points of the attention path (see include/lightning_attn_hip.h).
#include "la_common.h"
#include "lightning_attn_hip.h"

namespace la {
int sweep(const void* x, const void* y, const void* z, void* out, const float* s, int64_t bh, int64_t h, int64_t n,
          int64_t dk, int64_t dv, int dtype, bool reverse, hipStream_t st);
int sweep_f32(const void* x, const void* y, const void* z, void* out, const float* s, int64_t bh, int64_t h,
              int64_t n, int64_t dk, int64_t dv, bool reverse, hipStream_t st);

// one directional sweep at the element type named by dtype
static int run(const void* x, const void* y, const void* z, void* out, const float* s, int64_t bh, int64_t h,
               int64_t n, int64_t dk, int64_t dv, int dtype, bool reverse, hipStream_t st) {
    if (dtype == LA_FP32) return sweep_f32(x, y, z, out, s, bh, h, n, dk, dv, reverse, st);
    return sweep(x, y, z, out, s, bh, h, n, dk, dv, dtype, reverse, st);
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
}  // namespace la

extern "C" const char* la_version(void) { return "lightning_attn_hip 0.1.0 (gfx950)"; }

extern "C" const char* la_error_string(int code) {
    switch (code) {
        case LA_OK: return "success";
        case LA_E_NULLPTR: return "a required pointer is NULL";
        case LA_E_SHAPE: return "a dimension is out of range";
        case LA_E_UNSUPPORTED: return "head dims / dtype not supported (need d,e multiples of 8 in [8,256]; [8,128] for float32)";
        case LA_E_WORKSPACE: return "workspace too small";
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

extern "C" size_t la_workspace_bytes(int which, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype) {
    (void)which; (void)b; (void)h; (void)n; (void)d; (void)e; (void)dtype;
    return 0;
}

extern "C" int la_fwd(const void* q, const void* k, const void* v, const float* s, void* o, int64_t b, int64_t h,
                      int64_t n, int64_t d, int64_t e, int dtype, void* workspace, size_t ws_bytes, void* stream) {
    (void)workspace; (void)ws_bytes;
    int rc = la::check_dims(b, h, n, d, e, dtype);
    if (rc != LA_OK) return rc;
    if (b == 0 || n == 0) return LA_OK;  // nothing to do; empty tensors may carry null pointers
    if (!q || !k || !v || !o) return LA_E_NULLPTR;
    if (!la::al16(q) || !la::al16(k) || !la::al16(v) || !la::al16(o)) return LA_E_ALIGN;
    return la::run(q, k, v, o, s, b * h, h, n, d, e, dtype, false, static_cast<hipStream_t>(stream));
}

extern "C" int la_bwd(const void* q, const void* k, const void* v, const float* s, const void* dout, void* dq,
                      void* dk, void* dv, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e, int dtype,
                      void* workspace, size_t ws_bytes, void* stream) {
    (void)workspace; (void)ws_bytes;
    int rc = la::check_dims(b, h, n, d, e, dtype);
    if (rc != LA_OK) return rc;
    if (b == 0 || n == 0) return LA_OK;
    if (!q || !k || !v || !dout || !dq || !dk || !dv) return LA_E_NULLPTR;
    if (!la::al16(q) || !la::al16(k) || !la::al16(v) || !la::al16(dout) || !la::al16(dq) || !la::al16(dk) ||
        !la::al16(dv))
        return LA_E_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // dQ_i = sum_{j<=i} lam^(i-j) (dO_i . v_j) k_j
    rc = la::run(dout, v, k, dq, s, b * h, h, n, e, d, dtype, false, st);
    if (rc != LA_OK) return rc;
    // dK_j = sum_{i>=j} lam^(i-j) (v_j . dO_i) q_i
    rc = la::run(v, dout, q, dk, s, b * h, h, n, e, d, dtype, true, st);
    if (rc != LA_OK) return rc;
    // dV_j = sum_{i>=j} lam^(i-j) (k_j . q_i) dO_i
    return la::run(k, q, dout, dv, s, b * h, h, n, d, e, dtype, true, st);
}
