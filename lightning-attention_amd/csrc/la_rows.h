// Helpers shared by the row kernels (SimpleRMSNorm, the gated LayerNorm): 16-byte packed accesses and
// sums over the threads that share a row.
#pragma once
#include "la_common.h"

namespace la {

template <typename T>
struct alignas(16) Pack16 {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
};

template <typename T>
__device__ __forceinline__ Pack16<T> load16(const T* p) {
    Pack16<T> r;
    *reinterpret_cast<u32x4*>(&r) = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return r;
}
template <typename T>
__device__ __forceinline__ void store16(T* p, const Pack16<T>& r) {
    __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(&r), reinterpret_cast<u32x4*>(p));
}

// ---- register-resident rows -------------------------------------------------
// TPR threads share a row (4 .. 64: 64 / TPR rows per single-wavefront workgroup, cross-lane
// reduction; 256: one four-wavefront workgroup per row, reduction through LDS), each holding NV
// 16-byte chunks of it: cols <= TPR * NV * (16 / sizeof T).

// Makes the optimiser forget what it knows about a packed register quartet, so that values derived
// from it before this point (float conversions) are not kept alive for later use.
template <typename T>
__device__ __forceinline__ void forget(Pack16<T>& p) {
    asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&p)));
}

__device__ __forceinline__ float block_sum_256(float v, float* red) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    const float t = red[0] + red[1] + red[2] + red[3];
    __syncthreads();
    return t;
}

// sum over the TPR threads of a row (every thread of the workgroup takes part)
template <int TPR>
__device__ __forceinline__ float row_sum(float v, float* red) {
    if (TPR == 256) return block_sum_256(v, red);
#pragma unroll
    for (int m = TPR / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace la
