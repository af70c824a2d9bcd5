// Single-sweep decayed linear attention for gfx950 (bf16 / fp16 MFMA, fp32 state).
//
// One generic "sweep" computes, per (batch, head),
//     forward  direction:  out_i = sum_{j<=i} lam^(i-j) (x_i . y_j) z_j
//     reverse  direction:  out_i = sum_{j>=i} lam^(j-i) (x_i . y_j) z_j
// with lam = exp(-s_h).  The four products of the operator are instances of it:
//     O  = sweep_fwd(Q , K , V )      dQ = sweep_fwd(dO, V , K )
//     dK = sweep_rev(V , dO, Q )      dV = sweep_rev(K , Q , dO)
// (lightning_attn/ops/triton/lightning_attn2.py:8-85 forward, :88-395 backward.)
//
// The sequence is cut into blocks of 64 tokens.  A workgroup (4 wavefronts)
// owns one (batch, head, 64-column slice of z/out) and walks the blocks in
// order, carrying the dk x 64 slice of the state  S = sum lam^.. y_j^T z_j  in
// fp32 MFMA accumulators.  Wavefront w owns 16 of the 64 columns:
//     1. S^T tile  (y x^T) for its 16 tokens i        -> decay/mask -> P in LDS
//     2. out^T[c,i] = Lout[i] * (state^T x^T) + z^T P^T    (two MFMA chains)
//     3. state     = lam^64 * state + y^T (z * Lupd)
// State and z^T fragments never leave registers: the accumulator layout of one
// MFMA is reused as the A operand of the next with a matching permutation of
// the contraction index on the B side.  Transposed operands (y^T, z^T) are
// fetched with the LDS transpose read ds_read_b64_tr_b16.
#include "la_common.h"
#include "lightning_attn_hip.h"

namespace la {

struct SweepArgs {
    const void* x;  // (bh, n, dk)
    const void* y;  // (bh, n, dk)
    const void* z;  // (bh, n, dv)
    void* out;      // (bh, n, dv)
    const float* s; // h decay rates or nullptr
    int64_t n;
    int dk, dv, h, bh, nslice;
};

template <typename T>
struct Mma;
template <>
struct Mma<__bf16> {
    typedef bf16x8 V8;
    typedef bf16x4 V4;
    static __device__ __forceinline__ f32x4 mma(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ __bf16 cvt(float f) { return (__bf16)f; }
};
template <>
struct Mma<_Float16> {
    typedef f16x8 V8;
    typedef f16x4 V4;
    static __device__ __forceinline__ f32x4 mma(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    // fp16 saturates instead of overflowing to inf when a state entry is large
    static __device__ __forceinline__ _Float16 cvt(float f) {
        return (_Float16)__builtin_fminf(__builtin_fmaxf(f, -65504.f), 65504.f);
    }
};

// LDS transpose read: the 16 lanes of a group each point at 4 consecutive
// 16-bit elements; lane i of the group receives element (i % 4) of the lanes
// 4e + i/4, e = 0..3.  With lane L pointing at row L/4, columns 4(L%4).. of a
// row-major tile, lane i ends up with column i of rows 0..3.
template <typename V4>
__device__ __forceinline__ V4 lds_tr4(const void* p) {
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
    return __builtin_bit_cast(V4, v);
}
template <typename V8, typename V4>
__device__ __forceinline__ V8 cat(V4 a, V4 b) {
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

template <typename T, int DKP, bool REVERSE, bool DECAY>
__global__ __launch_bounds__(256, 1) void la_sweep_kernel(SweepArgs a) {
    typedef Mma<T> M;
    typedef typename M::V8 V8;
    typedef typename M::V4 V4;
    constexpr int XS = DKP + 8;   // row stride (elements) of the x / y tiles
    constexpr int ZS = 64 + 8;    // row stride of the z slice and the P tile
    constexpr int KS = DKP / 32;  // 32-wide contraction steps over the feature dim
    constexpr int KT = DKP / 16;  // 16-row state tiles
    constexpr int XC = DKP / 32;  // 16-byte chunks per thread for an x / y tile
    extern __shared__ __align__(16) unsigned char smem[];
    T* Xs = reinterpret_cast<T*>(smem);
    T* Ys = Xs + 64 * XS;
    T* Zs = Ys + 64 * XS;
    T* Ps = Zs + 64 * ZS;

    // Workgroups are dealt round-robin to the 8 XCDs by linear id; keep the
    // column slices of one head on one XCD so their x / y re-reads share an L2.
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int unit = xcd + 8 * (local / a.nslice);
    const int slice = local % a.nslice;
    if (unit >= a.bh) return;

    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int64_t n = a.n;
    const int dk = a.dk, dv = a.dv;
    const T* xg = static_cast<const T*>(a.x) + (int64_t)unit * n * dk;
    const T* yg = static_cast<const T*>(a.y) + (int64_t)unit * n * dk;
    const T* zg = static_cast<const T*>(a.z) + (int64_t)unit * n * dv;
    T* og = static_cast<T*>(a.out) + (int64_t)unit * n * dv;
    const int col0 = slice * 64;
    const bool wave_active = (col0 + 16 * w) < dv;

    float rate = 0.f;
    if (DECAY) rate = a.s[unit % a.h];

    // ---- per-lane decay tables (every factor <= 1) --------------------------
    float dfac[4][4];  // mask * decay of the S^T tile: token i = 16w + r, j = 16jt + 4g + v
    float ofac[4];     // scale of the inter-block term for token i = 16it + r
    float zfac[2][8];  // scale of token j = 32ks + 8g + u in the state update
    float lamB = 1.f;
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int i = 16 * w + r, j = 16 * jt + 4 * g + v;
            const int diff = REVERSE ? (j - i) : (i - j);
            dfac[jt][v] = diff >= 0 ? (DECAY ? expf(-rate * (float)diff) : 1.f) : 0.f;
        }
    if (DECAY) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int i = 16 * it + r;
            ofac[it] = expf(-rate * (float)(REVERSE ? 64 - i : i));
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = 32 * ks + 8 * g + u;
                zfac[ks][u] = expf(-rate * (float)(REVERSE ? j : 64 - j));
            }
        lamB = expf(-rate * 64.f);
    }

    f32x4 st[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) st[kt] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int64_t nblk = (n + 63) / 64;
    uint4 xr[XC], yr[XC], zr[2];

    auto load_block = [&](int64_t t) {
        const int64_t tok0 = t * 64;
#pragma unroll
        for (int u = 0; u < XC; ++u) {
            const int c = tid + 256 * u;
            const int row = c / (DKP / 8), col = (c % (DKP / 8)) * 8;
            const bool ok = (tok0 + row < n) && (col < dk);
            xr[u] = ok ? *reinterpret_cast<const uint4*>(xg + (tok0 + row) * dk + col) : make_uint4(0, 0, 0, 0);
            yr[u] = ok ? *reinterpret_cast<const uint4*>(yg + (tok0 + row) * dk + col) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int c = tid + 256 * u;
            const int row = c / 8, col = (c % 8) * 8;
            const bool ok = (tok0 + row < n) && (col0 + col < dv);
            zr[u] = ok ? *reinterpret_cast<const uint4*>(zg + (tok0 + row) * dv + col0 + col) : make_uint4(0, 0, 0, 0);
        }
    };
    auto stage_block = [&]() {
#pragma unroll
        for (int u = 0; u < XC; ++u) {
            const int c = tid + 256 * u;
            const int row = c / (DKP / 8), col = (c % (DKP / 8)) * 8;
            *reinterpret_cast<uint4*>(Xs + row * XS + col) = xr[u];
            *reinterpret_cast<uint4*>(Ys + row * XS + col) = yr[u];
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int c = tid + 256 * u;
            const int row = c / 8, col = (c % 8) * 8;
            *reinterpret_cast<uint4*>(Zs + row * ZS + col) = zr[u];
        }
    };

    // zero P once: tiles on the masked side of the diagonal are never written
    for (int c = tid; c < 64 * ZS / 8; c += 256) reinterpret_cast<uint4*>(Ps)[c] = make_uint4(0, 0, 0, 0);
    load_block(REVERSE ? nblk - 1 : 0);
    stage_block();
    __syncthreads();

    const int jlo = REVERSE ? w : 0, jhi = REVERSE ? 3 : w;

    for (int64_t it = 0; it < nblk; ++it) {
        const int64_t t = REVERSE ? nblk - 1 - it : it;
        const bool have_next = it + 1 < nblk;
        if (have_next) load_block(REVERSE ? t - 1 : t + 1);

        // ---- 1. S^T tiles for tokens i in [16w, 16w+16) ----------------------
        {
            f32x4 sacc[4];
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) sacc[jt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const V8 bx = *reinterpret_cast<const V8*>(Xs + (16 * w + r) * XS + 32 * ks + 8 * g);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
                    if (jt >= jlo && jt <= jhi) {
                        const V8 ay = *reinterpret_cast<const V8*>(Ys + (16 * jt + r) * XS + 32 * ks + 8 * g);
                        sacc[jt] = M::mma(ay, bx, sacc[jt]);
                    }
                }
            }
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                if (jt >= jlo && jt <= jhi) {
                    V4 p;
#pragma unroll
                    for (int v = 0; v < 4; ++v) p[v] = M::cvt(sacc[jt][v] * dfac[jt][v]);
                    *reinterpret_cast<V4*>(Ps + (16 * w + r) * ZS + 16 * jt + 4 * g) = p;
                }
            }
        }
        __syncthreads();

        if (wave_active) {
            // z^T fragments: rows (tokens) 32ks + 8g + u, column 16w + r
            V8 zf[2];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const T* pz = Zs + (32 * ks + 8 * g + (r >> 2)) * ZS + 16 * w + 4 * (r & 3);
                zf[ks] = cat<V8, V4>(lds_tr4<V4>(pz), lds_tr4<V4>(pz + 4 * ZS));
            }
            // ---- 2a. inter-block term: out^T = state^T x^T -------------------
            V8 sb[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    sb[ks][v] = M::cvt(st[2 * ks][v]);
                    sb[ks][4 + v] = M::cvt(st[2 * ks + 1][v]);
                }
            }
            f32x4 oacc[4];
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                oacc[i4] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const T* px = Xs + (16 * i4 + r) * XS + 32 * ks + 4 * g;
                    const V8 bx = cat<V8, V4>(*reinterpret_cast<const V4*>(px), *reinterpret_cast<const V4*>(px + 16));
                    oacc[i4] = M::mma(sb[ks], bx, oacc[i4]);
                }
                if (DECAY) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) oacc[i4][v] *= ofac[i4];
                }
            }
            // ---- 2b. intra-block term: out^T += z^T P^T ----------------------
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const bool need = REVERSE ? (ks >= i4 / 2) : (ks <= i4 / 2);
                    if (need) {
                        const V8 bp = *reinterpret_cast<const V8*>(Ps + (16 * i4 + r) * ZS + 32 * ks + 8 * g);
                        oacc[i4] = M::mma(zf[ks], bp, oacc[i4]);
                    }
                }
            }
            // ---- store out[token][16w + 4g .. +3] ----------------------------
            const int col = col0 + 16 * w + 4 * g;
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int64_t tok = t * 64 + 16 * i4 + r;
                if (tok < n && col < dv) {
                    V4 o;
#pragma unroll
                    for (int v = 0; v < 4; ++v) o[v] = (T)oacc[i4][v];
                    *reinterpret_cast<V4*>(og + tok * dv + col) = o;
                }
            }
            // ---- 3. state = lam^64 state + y^T (z * Lupd) ---------------------
            if (have_next) {
                if (DECAY) {
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                        for (int u = 0; u < 8; ++u) zf[ks][u] = (T)((float)zf[ks][u] * zfac[ks][u]);
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                        for (int v = 0; v < 4; ++v) st[kt][v] *= lamB;
                }
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const T* py = Ys + (32 * ks + 8 * g + (r >> 2)) * XS + 16 * kt + 4 * (r & 3);
                        const V8 ay = cat<V8, V4>(lds_tr4<V4>(py), lds_tr4<V4>(py + 4 * XS));
                        st[kt] = M::mma(ay, zf[ks], st[kt]);
                    }
                }
            }
        }
        __syncthreads();
        if (have_next) {
            stage_block();
            __syncthreads();
        }
    }
}

template <typename T, int DKP, bool REVERSE, bool DECAY>
static int launch_one(const SweepArgs& a, hipStream_t st) {
    constexpr size_t lds = (size_t)(2 * 64 * (DKP + 8) + 2 * 64 * 72) * sizeof(T);
    auto kern = la_sweep_kernel<T, DKP, REVERSE, DECAY>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    const int units8 = (a.bh + 7) / 8 * 8;
    const unsigned grid = (unsigned)(units8 * a.nslice);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, st, a);
    return (int)hipGetLastError();
}

template <typename T, bool REVERSE>
static int launch_dir(const SweepArgs& a, hipStream_t st) {
    const bool decay = a.s != nullptr;
#define LA_GO(DKP) (decay ? launch_one<T, DKP, REVERSE, true>(a, st) : launch_one<T, DKP, REVERSE, false>(a, st))
    if (a.dk <= 32) return LA_GO(32);
    if (a.dk <= 64) return LA_GO(64);
    if (a.dk <= 128) return LA_GO(128);
    if (a.dk <= 192) return LA_GO(192);
    return LA_GO(256);
#undef LA_GO
}

// x,y: (bh,n,dk)  z,out: (bh,n,dv)
int sweep(const void* x, const void* y, const void* z, void* out, const float* s, int64_t bh, int64_t h, int64_t n,
          int64_t dk, int64_t dv, int dtype, bool reverse, hipStream_t st) {
    SweepArgs a;
    a.x = x; a.y = y; a.z = z; a.out = out; a.s = s;
    a.n = n; a.dk = (int)dk; a.dv = (int)dv; a.h = (int)h; a.bh = (int)bh;
    a.nslice = (int)((dv + 63) / 64);
    if (dtype == LA_BF16) return reverse ? launch_dir<__bf16, true>(a, st) : launch_dir<__bf16, false>(a, st);
    if (dtype == LA_FP16) return reverse ? launch_dir<_Float16, true>(a, st) : launch_dir<_Float16, false>(a, st);
    return LA_E_UNSUPPORTED;
}

}  // namespace la
