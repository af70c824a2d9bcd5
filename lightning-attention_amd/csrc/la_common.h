// Shared device/host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace la {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 f16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;

typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2;

constexpr int kWave = 64;

// Raw buffer access with hardware bounds checking: a load whose byte offset lies at
// or beyond `bytes` returns zeros and such a store is dropped, so ragged tails need
// no branches.  kOob is an offset that is out of range for every buffer used here
// (all are smaller than 2 GiB).
constexpr unsigned kOob = 0x80000000u;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
// Cache policy of a buffer access (the instruction's auxiliary bits on gfx950): kCached = default; kStream = the nt
// bit, for data that is touched once - it then does not displace what other accesses of the launch will come back to.
constexpr int kCached = 0, kStream = 2;
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, unsigned off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
}
template <int POLICY>
__device__ __forceinline__ u32x4 buf_load16p(__amdgpu_buffer_rsrc_t r, unsigned off, unsigned soff = 0u) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, off, soff, POLICY);
}
template <int POLICY>
__device__ __forceinline__ void buf_store16p(__amdgpu_buffer_rsrc_t r, unsigned off, unsigned soff, u32x4 v) {
    __builtin_amdgcn_raw_buffer_store_b128(v, r, off, soff, POLICY);
}
__device__ __forceinline__ void buf_store8(__amdgpu_buffer_rsrc_t r, unsigned off, u32x2 v) {
    __builtin_amdgcn_raw_buffer_store_b64(v, r, off, 0, 0);
}
__device__ __forceinline__ void buf_store16(__amdgpu_buffer_rsrc_t r, unsigned off, unsigned soff, u32x4 v) {
    __builtin_amdgcn_raw_buffer_store_b128(v, r, off, soff, 0);
}
// The same with a wave-uniform byte offset `soff` added to the per-lane one.  `soff` must lie
// inside the buffer (the hardware compares the per-lane offset with the range left after it).
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, unsigned off, unsigned soff) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, off, soff, 0);
}
__device__ __forceinline__ void buf_store8(__amdgpu_buffer_rsrc_t r, unsigned off, unsigned soff, u32x2 v) {
    __builtin_amdgcn_raw_buffer_store_b64(v, r, off, soff, 0);
}

template <typename T>
struct ElemTraits;
template <>
struct ElemTraits<__bf16> {
    static constexpr int kDtype = 0;
};
template <>
struct ElemTraits<_Float16> {
    static constexpr int kDtype = 1;
};
template <>
struct ElemTraits<float> {
    static constexpr int kDtype = 2;
};

// Compute units of the current device (256 if it cannot be asked), asked once per device: launch plans and
// workspace sizes depend on it.
constexpr int kMaxDevices = 64;
inline int num_cus() {
    static int cache[kMaxDevices];  // 0: not asked yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    const bool cached = dev >= 0 && dev < kMaxDevices;
    if (cached) {
        const int c = __atomic_load_n(&cache[dev], __ATOMIC_RELAXED);
        if (c > 0) return c;
    }
    int n = 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    if (cached) __atomic_store_n(&cache[dev], n, __ATOMIC_RELAXED);
    return n;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

}  // namespace la
