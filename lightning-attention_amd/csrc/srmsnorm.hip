// SimpleRMSNorm forward / backward row kernels for gfx950.
//
// A row is read once with 16-byte loads straight into registers, reduced, and
// written once.  Up to 1024 chunks of 16 bytes: one 64-lane wavefront per row and
// workgroup, cross-lane shuffles, no LDS, no barrier (one row per workgroup measured
// against 2, 4 and 8 at 1024 to 4096 columns: never slower); short rows share a
// wavefront (4 .. 32 lanes each); rows up to 64 KB take a four-wavefront workgroup.
// Only the packed inputs are kept across the reduction (the second pass converts them
// again): carrying the converted floats cost the backward kernel 168 registers and
// half of its waves in flight (5.7 -> 6.2 TB/s with 79 registers).
// Replaces srms_norm_fw / srms_norm_bwd_dx_fused
// (lightning_attn/ops/triton/srmsnorm.py:12-33, 38-74).
#include "la_rows.h"
#include "lightning_attn_hip.h"

namespace la {

template <typename T, int NV, int TPR>
__global__ __launch_bounds__(TPR == 256 ? 256 : 64) void srms_fwd_vec(const T* __restrict__ x, T* __restrict__ y,
                                                                     float* __restrict__ rstd, int64_t rows, int cols,
                                                                     int64_t stride, float eps) {
    constexpr int E = Pack16<T>::N;
    constexpr int RPG = TPR == 256 ? 1 : 64 / TPR;  // rows per workgroup
    __shared__ float red[4];
    const int l = threadIdx.x % TPR;
    const int64_t row = (int64_t)blockIdx.x * RPG + threadIdx.x / TPR;
    const bool row_ok = row < rows;
    const T* xr = x + row * stride;
    T* yr = y + row * stride;
    Pack16<T> buf[NV];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int c = (u * TPR + l) * E;
        if (row_ok && c < cols) buf[u] = load16(xr + c);
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int c = (u * TPR + l) * E;
        if (row_ok && c < cols) {
#pragma unroll
            for (int t = 0; t < E; ++t) {
                const float f = (float)buf[u].v[t];
                ss += f * f;
            }
        }
    }
    ss = row_sum<TPR>(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)cols + eps);
    if (l == 0 && row_ok) rstd[row] = rs;
#pragma unroll
    for (int u = 0; u < NV; ++u) forget(buf[u]);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int c = (u * TPR + l) * E;
        if (row_ok && c < cols) {
            Pack16<T> o;
#pragma unroll
            for (int t = 0; t < E; ++t) o.v[t] = (T)((float)buf[u].v[t] * rs);
            store16(yr + c, o);
        }
    }
}

template <typename T, int NV, int TPR>
__global__ __launch_bounds__(TPR == 256 ? 256 : 64) void srms_bwd_vec(const T* __restrict__ x, const T* __restrict__ dy,
                                                                     const float* __restrict__ rstd, T* __restrict__ dx,
                                                                     int64_t rows, int cols, int64_t stride) {
    constexpr int E = Pack16<T>::N;
    constexpr int RPG = TPR == 256 ? 1 : 64 / TPR;
    __shared__ float red[4];
    const int l = threadIdx.x % TPR;
    const int64_t row = (int64_t)blockIdx.x * RPG + threadIdx.x / TPR;
    const bool row_ok = row < rows;
    const T* xr = x + row * stride;
    const T* gr = dy + row * (int64_t)cols;  // dy and dx are dense (rows, cols)
    T* dr = dx + row * (int64_t)cols;
    Pack16<T> bx[NV], bg[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int c = (u * TPR + l) * E;
        if (row_ok && c < cols) {
            bx[u] = load16(xr + c);
            bg[u] = load16(gr + c);
        }
    }
    const float rs = row_ok ? rstd[row] : 0.f;
    float acc = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int c = (u * TPR + l) * E;
        if (row_ok && c < cols) {
#pragma unroll
            for (int t = 0; t < E; ++t) acc += ((float)bx[u].v[t] * rs) * (float)bg[u].v[t];
        }
    }
    acc = row_sum<TPR>(acc, red);
    const float m = acc / (float)cols;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        forget(bx[u]);
        forget(bg[u]);
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int c = (u * TPR + l) * E;
        if (row_ok && c < cols) {
            Pack16<T> o;
#pragma unroll
            for (int t = 0; t < E; ++t) {
                const float xh = (float)bx[u].v[t] * rs;
                o.v[t] = (T)(((float)bg[u].v[t] - xh * m) * rs);
            }
            store16(dr + c, o);
        }
    }
}

// ---- any cols / any alignment: one workgroup per row, scalar accesses ------
template <typename T>
__global__ __launch_bounds__(256) void srms_fwd_any(const T* __restrict__ x, T* __restrict__ y,
                                                    float* __restrict__ rstd, int64_t rows, int64_t cols,
                                                    int64_t stride, float eps) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const T* xr = x + row * stride;
    T* yr = y + row * stride;
    float ss = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += 256) {
        const float f = (float)xr[c];
        ss += f * f;
    }
    ss = block_sum_256(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)cols + eps);
    if (threadIdx.x == 0) rstd[row] = rs;
    for (int64_t c = threadIdx.x; c < cols; c += 256) yr[c] = (T)((float)xr[c] * rs);
}

template <typename T>
__global__ __launch_bounds__(256) void srms_bwd_any(const T* __restrict__ x, const T* __restrict__ dy,
                                                    const float* __restrict__ rstd, T* __restrict__ dx,
                                                    int64_t rows, int64_t cols, int64_t stride) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const T* xr = x + row * stride;
    const T* gr = dy + row * cols;
    T* dr = dx + row * cols;
    const float rs = rstd[row];
    float acc = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += 256) acc += ((float)xr[c] * rs) * (float)gr[c];
    acc = block_sum_256(acc, red);
    const float m = acc / (float)cols;
    for (int64_t c = threadIdx.x; c < cols; c += 256) {
        const float xh = (float)xr[c] * rs;
        dr[c] = (T)(((float)gr[c] - xh * m) * rs);
    }
}

// Shape of the register-resident kernels for a row of `chunks` 16-byte chunks: threads per row and
// chunks per thread (0 = too wide).
static void vec_shape(int64_t chunks, int* tpr, int* nv) {
    *nv = 0;
    if (chunks <= 32) {
        *tpr = 4;
        while (*tpr < chunks) *tpr *= 2;
        *nv = 1;
    } else if (chunks <= 64 * 16) {
        *tpr = 64;
        *nv = 1;
        while (64 * *nv < chunks) *nv *= 2;
    } else if (chunks <= 256 * 16) {
        *tpr = 256;
        *nv = 8;
        while (256 * *nv < chunks) *nv *= 2;
    }
}

#define LA_SRMS_DISPATCH(KERNEL, ...)                                                                      \
    do {                                                                                                   \
        const unsigned rpg = tpr == 256 ? 1u : 64u / (unsigned)tpr;                                        \
        const dim3 grid((unsigned)((rows + rpg - 1) / rpg)), block(tpr == 256 ? 256 : 64);                 \
        if (tpr == 4) hipLaunchKernelGGL((KERNEL<T, 1, 4>), grid, block, 0, st, __VA_ARGS__);              \
        else if (tpr == 8) hipLaunchKernelGGL((KERNEL<T, 1, 8>), grid, block, 0, st, __VA_ARGS__);         \
        else if (tpr == 16) hipLaunchKernelGGL((KERNEL<T, 1, 16>), grid, block, 0, st, __VA_ARGS__);       \
        else if (tpr == 32) hipLaunchKernelGGL((KERNEL<T, 1, 32>), grid, block, 0, st, __VA_ARGS__);       \
        else if (tpr == 64 && nv == 1) hipLaunchKernelGGL((KERNEL<T, 1, 64>), grid, block, 0, st, __VA_ARGS__);   \
        else if (tpr == 64 && nv == 2) hipLaunchKernelGGL((KERNEL<T, 2, 64>), grid, block, 0, st, __VA_ARGS__);   \
        else if (tpr == 64 && nv == 4) hipLaunchKernelGGL((KERNEL<T, 4, 64>), grid, block, 0, st, __VA_ARGS__);   \
        else if (tpr == 64 && nv == 8) hipLaunchKernelGGL((KERNEL<T, 8, 64>), grid, block, 0, st, __VA_ARGS__);   \
        else if (tpr == 64) hipLaunchKernelGGL((KERNEL<T, 16, 64>), grid, block, 0, st, __VA_ARGS__);      \
        else if (nv == 8) hipLaunchKernelGGL((KERNEL<T, 8, 256>), grid, block, 0, st, __VA_ARGS__);        \
        else hipLaunchKernelGGL((KERNEL<T, 16, 256>), grid, block, 0, st, __VA_ARGS__);                    \
    } while (0)

template <typename T>
static int launch_fwd(const void* x, void* y, float* rstd, int64_t rows, int64_t cols, int64_t stride,
                      float eps, hipStream_t st) {
    constexpr int E = 16 / sizeof(T);
    const T* xp = static_cast<const T*>(x);
    T* yp = static_cast<T*>(y);
    int tpr = 0, nv = 0;
    if ((cols % E == 0) && (stride % E == 0) && aligned16(x) && aligned16(y)) vec_shape(cols / E, &tpr, &nv);
    if (nv) {
        LA_SRMS_DISPATCH(srms_fwd_vec, xp, yp, rstd, rows, (int)cols, stride, eps);
    } else {
        hipLaunchKernelGGL((srms_fwd_any<T>), dim3((unsigned)rows), dim3(256), 0, st, xp, yp, rstd, rows, cols, stride, eps);
    }
    return (int)hipGetLastError();
}

template <typename T>
static int launch_bwd(const void* x, const void* dy, const float* rstd, void* dx, int64_t rows, int64_t cols,
                      int64_t stride, hipStream_t st) {
    constexpr int E = 16 / sizeof(T);
    const T* xp = static_cast<const T*>(x);
    const T* gp = static_cast<const T*>(dy);
    T* dp = static_cast<T*>(dx);
    int tpr = 0, nv = 0;
    if ((cols % E == 0) && (stride % E == 0) && aligned16(x) && aligned16(dy) && aligned16(dx)) vec_shape(cols / E, &tpr, &nv);
    if (nv) {
        LA_SRMS_DISPATCH(srms_bwd_vec, xp, gp, rstd, dp, rows, (int)cols, stride);
    } else {
        hipLaunchKernelGGL((srms_bwd_any<T>), dim3((unsigned)rows), dim3(256), 0, st, xp, gp, rstd, dp, rows, cols, stride);
    }
    return (int)hipGetLastError();
}
#undef LA_SRMS_DISPATCH

}  // namespace la

// Makes the runtime load this file's code object now (it otherwise does at the first launch from it).
namespace la {
int prepare_srmsnorm() {
    hipFuncAttributes attr;
    return (int)hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(&srms_fwd_any<float>));
}
}  // namespace la

extern "C" int srmsnorm_fwd(const void* x, void* y, float* rstd, int64_t rows, int64_t cols, int64_t row_stride,
                            float eps, int dtype, void* stream) {
    if (rows < 0 || cols <= 0 || row_stride < cols || rows > 0x7fffffffLL) return LA_E_SHAPE;
    if (dtype != LA_BF16 && dtype != LA_FP16 && dtype != LA_FP32) return LA_E_UNSUPPORTED;
    if (rows == 0) return LA_OK;  // empty tensors may carry null pointers
    if (!x || !y || !rstd) return LA_E_NULLPTR;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case LA_BF16: return la::launch_fwd<__bf16>(x, y, rstd, rows, cols, row_stride, eps, st);
        case LA_FP16: return la::launch_fwd<_Float16>(x, y, rstd, rows, cols, row_stride, eps, st);
        case LA_FP32: return la::launch_fwd<float>(x, y, rstd, rows, cols, row_stride, eps, st);
        default: return LA_E_UNSUPPORTED;
    }
}

extern "C" int srmsnorm_bwd(const void* x, const void* dy, const float* rstd, void* dx, int64_t rows, int64_t cols,
                            int64_t row_stride, int dtype, void* stream) {
    if (rows < 0 || cols <= 0 || row_stride < cols || rows > 0x7fffffffLL) return LA_E_SHAPE;
    if (dtype != LA_BF16 && dtype != LA_FP16 && dtype != LA_FP32) return LA_E_UNSUPPORTED;
    if (rows == 0) return LA_OK;
    if (!x || !dy || !rstd || !dx) return LA_E_NULLPTR;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case LA_BF16: return la::launch_bwd<__bf16>(x, dy, rstd, dx, rows, cols, row_stride, st);
        case LA_FP16: return la::launch_bwd<_Float16>(x, dy, rstd, dx, rows, cols, row_stride, st);
        case LA_FP32: return la::launch_bwd<float>(x, dy, rstd, dx, rows, cols, row_stride, st);
        default: return LA_E_UNSUPPORTED;
    }
}
