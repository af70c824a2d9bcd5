// Gated output norm of the TNL attention block for gfx950:
//     y = LayerNorm(o; weight, bias, eps) * sigmoid(g)
// forward and backward as row kernels (examples/module/tnl_attn.py:66-69 of the reference, where it
// is three separate PyTorch operators: LayerNorm, sigmoid and a product - seven passes over
// (tokens, embed_dim) tensors forward and eleven backward; here three and five).
//
// Same data movement as the SimpleRMSNorm kernels: a row of o, g (and dy) is read once with 16-byte
// non-temporal loads into registers, reduced, and the results written once.  TPR threads share a row:
// one or two wavefronts (four or two rows to a workgroup of 256 threads) or a whole workgroup of 256,
// 512 or 1024 threads.  The forward kernel takes one group of rows per workgroup and fetches weight and
// bias from the caches.  The backward kernel walks the rows with a grid stride and gives every thread one
// 16-byte chunk of the row: a thread always holds the same columns, so weight and bias stay in registers
// as floats and the column sums (d weight, d bias) are accumulated in registers over all rows a thread
// sees (118 registers: four waves per SIMD; with more chunks per thread it ran at two).  Those partial
// sums go to a scratch buffer, one row per workgroup, and a second small kernel adds them up in a fixed
// order: deterministic, no atomics.
//
// Per element, float32 throughout:
//   forward   xh = (o - mean) rstd ; ln = xh w + b ; sg = 1 / (1 + exp(-g)) ; y = ln sg
//   backward  dln = dy sg ; dg = dy ln sg (1 - sg) ; dxh = dln w ;
//             do = rstd (dxh - mean_c(dxh) - xh mean_c(dxh xh)) ; dw += dln xh ; db += dln
#include "la_rows.h"
#include "lightning_attn_hip.h"

namespace la {

// Threads of a workgroup: TPR threads share a row; rows of one or two wavefronts travel four or two to a
// workgroup of 256, wider rows take a workgroup of 256, 512 or 1024 threads to themselves.
constexpr int ng_threads(int tpr) { return tpr >= 256 ? tpr : 256; }

// both sums over the TPR threads of a row at once (every thread of the workgroup takes part)
template <int TPR>
__device__ __forceinline__ void row_sum2(float& a, float& b, float* red) {
    if (TPR >= 128) {
        constexpr int NWV = TPR / 64;  // wavefronts per row
        a = wave_sum(a);
        b = wave_sum(b);
        const int w = threadIdx.x >> 6, w0 = w / NWV * NWV;
        if ((threadIdx.x & 63) == 0) {
            red[w] = a;
            red[16 + w] = b;
        }
        __syncthreads();
        a = b = 0.f;
#pragma unroll
        for (int i = 0; i < NWV; ++i) {
            a += red[w0 + i];
            b += red[16 + w0 + i];
        }
        __syncthreads();
        return;
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        a += __shfl_xor(a, m, 64);
        b += __shfl_xor(b, m, 64);
    }
}

// 1 / (1 + exp(-x)) with the hardware's exp2 and reciprocal (about 1 ulp each); an IEEE division
// would cost more instructions than the rest of the element's arithmetic
__device__ __forceinline__ float sigmoidf(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896340736f));
}

template <typename T, int NV, int TPR>
__global__ __launch_bounds__(ng_threads(TPR)) void norm_gate_fwd_kernel(const T* __restrict__ o, const T* __restrict__ g,
                                                                  const T* __restrict__ w, const T* __restrict__ b,
                                                                  T* __restrict__ y, float* __restrict__ mean,
                                                                  float* __restrict__ rstd, int64_t rows, int cols, float eps) {
    constexpr int E = Pack16<T>::N;
    constexpr int RPG = ng_threads(TPR) / TPR;  // rows a workgroup holds at a time
    __shared__ float red[32];
    const int l = threadIdx.x % TPR;
    const float inv = 1.0f / (float)cols;
    for (int64_t row0 = (int64_t)blockIdx.x * RPG; row0 < rows; row0 += (int64_t)gridDim.x * RPG) {
        const int64_t row = row0 + threadIdx.x / TPR;
        const bool row_ok = row < rows;
        const T* orow = o + row * (int64_t)cols;
        const T* grow = g + row * (int64_t)cols;
        T* yrow = y + row * (int64_t)cols;
        Pack16<T> po[NV], pg[NV];
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int c = (u * TPR + l) * E;
            if (row_ok && c < cols) {
                po[u] = load16(orow + c);
                pg[u] = load16(grow + c);
            }
        }
        float s = 0.f, dummy = 0.f;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int c = (u * TPR + l) * E;
            if (row_ok && c < cols) {
#pragma unroll
                for (int t = 0; t < E; ++t) s += (float)po[u].v[t];
            }
        }
        row_sum2<TPR>(s, dummy, red);
        const float mu = s * inv;
        // only the packed inputs live across the reductions: the passes convert them again
#pragma unroll
        for (int u = 0; u < NV; ++u) forget(po[u]);
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int c = (u * TPR + l) * E;
            if (row_ok && c < cols) {
#pragma unroll
                for (int t = 0; t < E; ++t) {
                    const float dlt = (float)po[u].v[t] - mu;
                    ss += dlt * dlt;
                }
            }
        }
        row_sum2<TPR>(ss, dummy, red);
        const float rs = 1.0f / sqrtf(ss * inv + eps);
#pragma unroll
        for (int u = 0; u < NV; ++u) forget(po[u]);
        if (l == 0 && row_ok) {
            mean[row] = mu;
            rstd[row] = rs;
        }
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int c = (u * TPR + l) * E;
            if (row_ok && c < cols) {
                // weight and bias come from the caches (every row reads the same cols elements)
                const Pack16<T> pw = *reinterpret_cast<const Pack16<T>*>(w + c);
                const Pack16<T> pb = *reinterpret_cast<const Pack16<T>*>(b + c);
                Pack16<T> out;
#pragma unroll
                for (int t = 0; t < E; ++t) {
                    const float ln = ((float)po[u].v[t] - mu) * rs * (float)pw.v[t] + (float)pb.v[t];
                    out.v[t] = (T)(ln * sigmoidf((float)pg[u].v[t]));
                }
                store16(yrow + c, out);
            }
        }
    }
}

// `part`: gridDim.x rows of [d weight | d bias] partial column sums, 2 * cols floats each.
template <typename T, int NV, int TPR>
__global__ __launch_bounds__(ng_threads(TPR)) void norm_gate_bwd_kernel(const T* __restrict__ o, const T* __restrict__ g,
                                                                  const T* __restrict__ w, const T* __restrict__ b,
                                                                  const float* __restrict__ mean, const float* __restrict__ rstd,
                                                                  const T* __restrict__ dy, T* __restrict__ d_o,
                                                                  T* __restrict__ d_g, float* __restrict__ part,
                                                                  int64_t rows, int cols) {
    constexpr int E = Pack16<T>::N;
    constexpr int RPG = ng_threads(TPR) / TPR;
    __shared__ float red[32];
    __shared__ float comb[RPG > 1 ? (RPG - 1) * TPR * NV * E * 2 : 1];  // column sums of the rows beside the first
    const int l = threadIdx.x % TPR;
    float wf[NV][E], bf[NV][E];  // this thread's columns of weight and bias
    float aw[NV][E], ab[NV][E];  // ... and of the column sums
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int c = (u * TPR + l) * E;
#pragma unroll
        for (int t = 0; t < E; ++t) {
            wf[u][t] = c < cols ? (float)w[c + t] : 0.f;
            bf[u][t] = c < cols ? (float)b[c + t] : 0.f;
            aw[u][t] = ab[u][t] = 0.f;
        }
    }
    const float inv = 1.0f / (float)cols;
    for (int64_t row0 = (int64_t)blockIdx.x * RPG; row0 < rows; row0 += (int64_t)gridDim.x * RPG) {
        const int64_t row = row0 + threadIdx.x / TPR;
        const bool row_ok = row < rows;
        const T* orow = o + row * (int64_t)cols;
        const T* grow = g + row * (int64_t)cols;
        const T* yrow = dy + row * (int64_t)cols;
        Pack16<T> po[NV], pg[NV], py[NV];
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int c = (u * TPR + l) * E;
            if (row_ok && c < cols) {
                po[u] = load16(orow + c);
                pg[u] = load16(grow + c);
                py[u] = load16(yrow + c);
            }
        }
        const float mu = row_ok ? mean[row] : 0.f, rs = row_ok ? rstd[row] : 0.f;
        // Kept from the first pass for the second: xh, dln and 1 - sigmoid(g) (one exp and one
        // reciprocal per element in all; the kernel is close to its VALU budget, not only to HBM's).
        float xh[NV][E], dln[NV][E], cs[NV][E];
        float s1 = 0.f, s2 = 0.f;
        const float shift = -mu * rs;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int c = (u * TPR + l) * E;
            if (row_ok && c < cols) {
#pragma unroll
                for (int t = 0; t < E; ++t) {
                    xh[u][t] = (float)po[u].v[t] * rs + shift;
                    const float sv = sigmoidf((float)pg[u].v[t]);
                    cs[u][t] = 1.0f - sv;
                    dln[u][t] = (float)py[u].v[t] * sv;
                    const float dxh = dln[u][t] * wf[u][t];
                    s1 += dxh;
                    s2 += dxh * xh[u][t];
                    aw[u][t] += dln[u][t] * xh[u][t];
                    ab[u][t] += dln[u][t];
                }
            }
        }
        row_sum2<TPR>(s1, s2, red);
        const float k1 = s1 * inv * rs, k2 = s2 * inv * rs;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int c = (u * TPR + l) * E;
            if (row_ok && c < cols) {
                Pack16<T> out_o, out_g;
#pragma unroll
                for (int t = 0; t < E; ++t) {
                    // do = rstd (dxh - mean(dxh) - xh mean(dxh xh)) ; dg = dy ln sg (1 - sg) = dln ln (1 - sg)
                    out_o.v[t] = (T)(dln[u][t] * wf[u][t] * rs - k1 - xh[u][t] * k2);
                    const float ln = xh[u][t] * wf[u][t] + bf[u][t];
                    out_g.v[t] = (T)(dln[u][t] * ln * cs[u][t]);
                }
                store16(d_o + row * (int64_t)cols + c, out_o);
                store16(d_g + row * (int64_t)cols + c, out_g);
            }
        }
    }
    // column sums of this workgroup: the thread groups of its rows hold the same columns and are
    // added up in row order first
    if (RPG > 1) {
        const int grp = threadIdx.x / TPR;
        if (grp > 0) {
#pragma unroll
            for (int u = 0; u < NV; ++u)
#pragma unroll
                for (int t = 0; t < E; ++t) {
                    comb[((((grp - 1) * NV + u) * E + t) * 2 + 0) * TPR + l] = aw[u][t];
                    comb[((((grp - 1) * NV + u) * E + t) * 2 + 1) * TPR + l] = ab[u][t];
                }
        }
        __syncthreads();
        if (grp > 0) return;
#pragma unroll
        for (int k = 0; k < RPG - 1; ++k)
#pragma unroll
            for (int u = 0; u < NV; ++u)
#pragma unroll
                for (int t = 0; t < E; ++t) {
                    aw[u][t] += comb[(((k * NV + u) * E + t) * 2 + 0) * TPR + l];
                    ab[u][t] += comb[(((k * NV + u) * E + t) * 2 + 1) * TPR + l];
                }
    }
    float* prow = part + (size_t)blockIdx.x * 2 * cols;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int c = (u * TPR + l) * E;
        if (c < cols) {
#pragma unroll
            for (int t = 0; t < E; ++t) {
                prow[c + t] = aw[u][t];
                prow[cols + c + t] = ab[u][t];
            }
        }
    }
}

// d weight[c] = sum over the partial rows, in a fixed order: 32 columns per workgroup, 32 interleaved
// partial sums per column (eight independent loads in flight each) combined through LDS.
constexpr int kRedCols = 32, kRedGroups = 32;
template <typename T>
__global__ __launch_bounds__(kRedCols * kRedGroups) void norm_gate_reduce_kernel(const float* __restrict__ part, int nparts,
                                                                                 int cols, T* __restrict__ dweight,
                                                                                 T* __restrict__ dbias) {
    __shared__ float acc[kRedGroups][2 * kRedCols];
    const int lane = threadIdx.x % kRedCols, grp = threadIdx.x / kRedCols;
    const int c = blockIdx.x * kRedCols + lane;
    float sw = 0.f, sb = 0.f;
    if (c < cols) {
        constexpr int U = 8;
        for (int p0 = grp; p0 < nparts; p0 += kRedGroups * U) {
            float vw[U], vb[U];
#pragma unroll
            for (int i = 0; i < U; ++i) {
                const int p = p0 + i * kRedGroups;
                vw[i] = p < nparts ? part[(size_t)p * 2 * cols + c] : 0.f;
                vb[i] = p < nparts ? part[(size_t)p * 2 * cols + cols + c] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < U; ++i) {
                sw += vw[i];
                sb += vb[i];
            }
        }
    }
    acc[grp][lane] = sw;
    acc[grp][kRedCols + lane] = sb;
    __syncthreads();
    if (grp == 0 && c < cols) {
        float tw = 0.f, tb = 0.f;
#pragma unroll
        for (int k = 0; k < kRedGroups; ++k) {
            tw += acc[k][lane];
            tb += acc[k][kRedCols + lane];
        }
        dweight[c] = (T)tw;
        dbias[c] = (T)tb;
    }
}

// Threads per row and 16-byte chunks per thread for rows of `chunks` chunks (nv = 0: too wide).  The
// forward kernel holds little per column and gives a wavefront rows of up to 512 chunks; the backward
// kernel carries weight, bias and two column sums per column and spreads rows over the workgroup earlier.
static void ng_shape(int64_t chunks, bool backward, int* tpr, int* nv) {
    *nv = 0;
    if (backward) {
        // one chunk per thread: the kernel keeps ~7 floats per element of a thread's columns
        if (chunks > 1024) return;
        *nv = 1;
        *tpr = chunks <= 64 ? 64 : chunks <= 128 ? 128 : chunks <= 256 ? 256 : chunks <= 512 ? 512 : 1024;
        return;
    }
    if (chunks <= 64 * 4) {
        *tpr = 64;
        *nv = 1;
        while (64 * *nv < chunks) *nv *= 2;
    } else if (chunks <= 256 * 4) {
        *tpr = 256;
        *nv = chunks <= 256 ? 1 : chunks <= 512 ? 2 : 4;
    }
}

// workgroups of a launch: enough to keep every CU's memory pipeline full, never more than row groups
static int64_t ng_grid(int64_t rows, int tpr, bool backward) {
    const int64_t threads = ng_threads(tpr), rpg = threads / tpr, groups = (rows + rpg - 1) / rpg;
    if (!backward) return groups;  // nothing is carried from row to row: one group of rows per workgroup
    const int64_t cap = 4 * (int64_t)num_cus() * 256 / threads;  // ~16 wavefronts per CU
    return groups < cap ? groups : cap;
}

#define LA_NG_GO(KERNEL, NV, TPR, ...) hipLaunchKernelGGL((KERNEL<T, NV, TPR>), grid, dim3(ng_threads(TPR)), 0, st, __VA_ARGS__)
#define LA_NG_DISPATCH_FWD(KERNEL, ...)                               \
    do {                                                              \
        if (tpr == 64 && nv == 1) LA_NG_GO(KERNEL, 1, 64, __VA_ARGS__);       \
        else if (tpr == 64 && nv == 2) LA_NG_GO(KERNEL, 2, 64, __VA_ARGS__);  \
        else if (tpr == 64) LA_NG_GO(KERNEL, 4, 64, __VA_ARGS__);             \
        else if (nv == 1) LA_NG_GO(KERNEL, 1, 256, __VA_ARGS__);              \
        else if (nv == 2) LA_NG_GO(KERNEL, 2, 256, __VA_ARGS__);              \
        else LA_NG_GO(KERNEL, 4, 256, __VA_ARGS__);                           \
    } while (0)
#define LA_NG_DISPATCH_BWD(KERNEL, ...)                               \
    do {                                                              \
        if (tpr == 64) LA_NG_GO(KERNEL, 1, 64, __VA_ARGS__);          \
        else if (tpr == 128) LA_NG_GO(KERNEL, 1, 128, __VA_ARGS__);   \
        else if (tpr == 256) LA_NG_GO(KERNEL, 1, 256, __VA_ARGS__);   \
        else if (tpr == 512) LA_NG_GO(KERNEL, 1, 512, __VA_ARGS__);   \
        else LA_NG_GO(KERNEL, 1, 1024, __VA_ARGS__);                  \
    } while (0)

template <typename T>
static int ng_fwd(const void* o, const void* g, const void* w, const void* b, void* y, float* mean, float* rstd, int64_t rows,
                  int64_t cols, float eps, hipStream_t st) {
    int tpr = 0, nv = 0;
    ng_shape(cols / (16 / (int64_t)sizeof(T)), false, &tpr, &nv);
    if (!nv) return LA_E_UNSUPPORTED;
    const dim3 grid((unsigned)ng_grid(rows, tpr, false));
    LA_NG_DISPATCH_FWD(norm_gate_fwd_kernel, static_cast<const T*>(o), static_cast<const T*>(g), static_cast<const T*>(w),
                   static_cast<const T*>(b), static_cast<T*>(y), mean, rstd, rows, (int)cols, eps);
    return (int)hipGetLastError();
}

template <typename T>
static int ng_bwd(const void* o, const void* g, const void* w, const void* b, const float* mean, const float* rstd,
                  const void* dy, void* d_o, void* d_g, void* dweight, void* dbias, float* part, int64_t rows, int64_t cols,
                  hipStream_t st) {
    int tpr = 0, nv = 0;
    ng_shape(cols / (16 / (int64_t)sizeof(T)), true, &tpr, &nv);
    if (!nv) return LA_E_UNSUPPORTED;
    const dim3 grid((unsigned)ng_grid(rows, tpr, true));
    LA_NG_DISPATCH_BWD(norm_gate_bwd_kernel, static_cast<const T*>(o), static_cast<const T*>(g), static_cast<const T*>(w),
                   static_cast<const T*>(b), mean, rstd, static_cast<const T*>(dy), static_cast<T*>(d_o), static_cast<T*>(d_g),
                   part, rows, (int)cols);
    int rc = (int)hipGetLastError();
    if (rc != 0) return rc;
    hipLaunchKernelGGL((norm_gate_reduce_kernel<T>), dim3((unsigned)((cols + kRedCols - 1) / kRedCols)),
                       dim3(kRedCols * kRedGroups), 0, st, part, (int)grid.x, (int)cols, static_cast<T*>(dweight),
                       static_cast<T*>(dbias));
    return (int)hipGetLastError();
}
#undef LA_NG_DISPATCH_FWD
#undef LA_NG_DISPATCH_BWD
#undef LA_NG_GO

static int ng_check(int64_t rows, int64_t cols, int dtype) {
    if (rows < 0 || cols <= 0 || rows > 0x7fffffffLL) return LA_E_SHAPE;
    if (dtype != LA_BF16 && dtype != LA_FP16 && dtype != LA_FP32) return LA_E_UNSUPPORTED;
    return norm_gate_supported(cols, dtype) ? LA_OK : LA_E_UNSUPPORTED;
}

}  // namespace la

// Makes the runtime load this file's code object now (it otherwise does at the first launch from it).
namespace la {
int prepare_norm_gate() {
    hipFuncAttributes attr;
    return (int)hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(&norm_gate_reduce_kernel<float>));
}
}  // namespace la

extern "C" int norm_gate_supported(int64_t cols, int dtype) {
    if (dtype != LA_BF16 && dtype != LA_FP16 && dtype != LA_FP32) return 0;
    const int64_t e = dtype == LA_FP32 ? 4 : 8;
    return cols > 0 && cols % e == 0 && cols / e <= 1024;
}

extern "C" size_t norm_gate_workspace_bytes(int64_t rows, int64_t cols, int dtype) {
    if (rows <= 0 || !norm_gate_supported(cols, dtype)) return 0;
    int tpr = 0, nv = 0;
    la::ng_shape(cols / (dtype == LA_FP32 ? 4 : 8), true, &tpr, &nv);
    return (size_t)la::ng_grid(rows, tpr, true) * 2 * (size_t)cols * sizeof(float);
}

extern "C" int norm_gate_fwd(const void* o, const void* g, const void* weight, const void* bias, void* y, float* mean,
                             float* rstd, int64_t rows, int64_t cols, float eps, int dtype, void* stream) {
    int rc = la::ng_check(rows, cols, dtype);
    if (rc != LA_OK) return rc;
    if (rows == 0) return LA_OK;
    if (!o || !g || !weight || !bias || !y || !mean || !rstd) return LA_E_NULLPTR;
    for (const void* p : {o, g, weight, bias, (const void*)y})
        if (!la::aligned16(p)) return LA_E_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case LA_BF16: return la::ng_fwd<__bf16>(o, g, weight, bias, y, mean, rstd, rows, cols, eps, st);
        case LA_FP16: return la::ng_fwd<_Float16>(o, g, weight, bias, y, mean, rstd, rows, cols, eps, st);
        default: return la::ng_fwd<float>(o, g, weight, bias, y, mean, rstd, rows, cols, eps, st);
    }
}

extern "C" int norm_gate_bwd(const void* o, const void* g, const void* weight, const void* bias, const float* mean,
                             const float* rstd, const void* dy, void* d_o, void* d_g, void* dweight, void* dbias,
                             void* workspace, size_t ws_bytes, int64_t rows, int64_t cols, int dtype, void* stream) {
    int rc = la::ng_check(rows, cols, dtype);
    if (rc != LA_OK) return rc;
    if (!dweight || !dbias) return LA_E_NULLPTR;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (rows == 0) {
        // no rows: the column sums are zero (the reduction over zero partial rows writes them)
        const dim3 grid((unsigned)((cols + la::kRedCols - 1) / la::kRedCols)), block(la::kRedCols * la::kRedGroups);
        if (dtype == LA_BF16) hipLaunchKernelGGL((la::norm_gate_reduce_kernel<__bf16>), grid, block, 0, st, nullptr, 0, (int)cols, static_cast<__bf16*>(dweight), static_cast<__bf16*>(dbias));
        else if (dtype == LA_FP16) hipLaunchKernelGGL((la::norm_gate_reduce_kernel<_Float16>), grid, block, 0, st, nullptr, 0, (int)cols, static_cast<_Float16*>(dweight), static_cast<_Float16*>(dbias));
        else hipLaunchKernelGGL((la::norm_gate_reduce_kernel<float>), grid, block, 0, st, nullptr, 0, (int)cols, static_cast<float*>(dweight), static_cast<float*>(dbias));
        return (int)hipGetLastError();
    }
    if (!o || !g || !weight || !bias || !mean || !rstd || !dy || !d_o || !d_g) return LA_E_NULLPTR;
    for (const void* p : {o, g, weight, bias, dy, (const void*)d_o, (const void*)d_g})
        if (!la::aligned16(p)) return LA_E_ALIGN;
    if (!workspace || ws_bytes < norm_gate_workspace_bytes(rows, cols, dtype) || (reinterpret_cast<uintptr_t>(workspace) & 3u))
        return LA_E_WORKSPACE;
    float* part = static_cast<float*>(workspace);
    switch (dtype) {
        case LA_BF16: return la::ng_bwd<__bf16>(o, g, weight, bias, mean, rstd, dy, d_o, d_g, dweight, dbias, part, rows, cols, st);
        case LA_FP16: return la::ng_bwd<_Float16>(o, g, weight, bias, mean, rstd, dy, d_o, d_g, dweight, dbias, part, rows, cols, st);
        default: return la::ng_bwd<float>(o, g, weight, bias, mean, rstd, dy, d_o, d_g, dweight, dbias, part, rows, cols, st);
    }
}
