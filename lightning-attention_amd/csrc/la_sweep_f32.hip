// float32 variant of the sweep (see la_sweep.hip for the algorithm): the same
// block recurrence and work split, with every product on the fp32 matrix
// instruction v_mfma_f32_16x16x4_f32 (one A and one B element per lane:
// row/column = lane % 16, contraction slot = lane / 16).  Nothing is rounded
// below float32, so the result is within float32 accumulation error of the
// exact value.  This is the accuracy path, not the throughput path.
//
// Every operand but z comes out of LDS in 16-byte reads.  A contraction may visit its index in any
// order as long as both operands agree, and the rows of a state tile may stand for any 16 features
// as long as the products that write and read the state agree:
//   scores        step (kt, v) of slot g contracts feature 16kt + 4g + v: x and y rows read 4 floats at a time;
//   state tiles   come in groups of four (kt = 4K + q); row rho of tile kt is feature
//                 64K + 4 pi(rho) + q with pi(rho) = 4 (rho % 4) + rho / 4, so that one 16-byte read of a
//                 y row (state update) or an x row (inter-block term) feeds the four tiles of a group.
#include "la_sweep_common.h"
#include "lightning_attn_hip.h"

namespace la {

#ifndef LA_F32_XPAD
#define LA_F32_XPAD 8  // floats of padding per x / y row
#endif

struct SweepArgsF32 {
    const float* x;
    const float* y;
    const float* z;
    float* out;
    const float* s;
    int64_t n;
    int dk, dv, h, bh, nslice;
    // sequence chunks (few sequences): the workgroup of chunk c produces the blocks chunk_start[c] ..
    // chunk_start[c + 1] - 1 of the walk, after running over the blocks before them with the state
    // update alone (no workspace, same results bit for bit)
    int nchunk;
    int chunk_start[9];
};


__device__ __forceinline__ f32x4 mma4(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// `bid`: number of the workgroup within its part of the launch.
template <int DKP, bool REVERSE, bool DECAY>
__device__ __forceinline__ void sweep_f32_body(const SweepArgsF32& a, const unsigned bid) {
    constexpr int XS = DKP + LA_F32_XPAD;  // row stride (floats) of the x / y tiles
    constexpr int ZS = 64 + 4;    // row stride of the z slice and the P tile
    constexpr int KT = DKP / 16;  // 16-row state tiles
    constexpr int KG = DKP / 64;  // groups of four state tiles
    constexpr int XC = DKP / 16;  // 16-byte chunks per thread for an x / y tile
    extern __shared__ __align__(16) unsigned char smem[];
    float* Xs = reinterpret_cast<float*>(smem);
    float* Ys = Xs + 64 * XS;
    float* Zs = Ys + 64 * XS;
    float* Ps = Zs + 64 * ZS;

    const int xcd = bid & 7, local = bid >> 3;
    const int per_unit = a.nslice * a.nchunk;
    const int unit = xcd + 8 * (local / per_unit);
    const int slice = (local % per_unit) % a.nslice;
    const int chunk = (local % per_unit) / a.nslice;
    if (unit >= a.bh) return;

    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int64_t n = a.n;
    const int dk = a.dk, dv = a.dv;
    const float* xg = a.x + (int64_t)unit * n * dk;
    const float* yg = a.y + (int64_t)unit * n * dk;
    const float* zg = a.z + (int64_t)unit * n * dv;
    float* og = a.out + (int64_t)unit * n * dv;
    const int col0 = slice * 64;
    const bool wave_active = (col0 + 16 * w) < dv;

    float rate = 0.f;
    if (DECAY) rate = a.s[unit % a.h];

    float dfac[4][4], ofac[4], zfac[4][4], lamB = 1.f;
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int i = 16 * w + r, j = 16 * jt + 4 * g + v;
            const int diff = REVERSE ? (j - i) : (i - j);
            dfac[jt][v] = diff >= 0 ? (DECAY ? expf(-rate * (float)diff) : 1.f) : 0.f;
            zfac[jt][v] = DECAY ? expf(-rate * (float)(REVERSE ? j : 64 - j)) : 1.f;
        }
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int i = 16 * it + r;
        ofac[it] = DECAY ? expf(-rate * (float)(REVERSE ? 64 - i : i)) : 1.f;
    }
    if (DECAY) lamB = expf(-rate * 64.f);

    f32x4 st[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) st[kt] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int64_t nblk = (n + 63) / 64;
    const int64_t it_first = a.chunk_start[chunk], it_end = a.chunk_start[chunk + 1];
    uint4 xr[XC], yr[XC], zr[4];

    // block number `it` of the walk; x is not needed for a warm-up block
    auto load_block = [&](int64_t it) {
        const int64_t tok0 = (REVERSE ? nblk - 1 - it : it) * 64;
        const bool need_x = it >= it_first;
#pragma unroll
        for (int u = 0; u < XC; ++u) {
            const int c = tid + 256 * u;
            const int row = c / (DKP / 4), col = (c % (DKP / 4)) * 4;
            const bool ok = (tok0 + row < n) && (col < dk);
            xr[u] = ok && need_x ? *reinterpret_cast<const uint4*>(xg + (tok0 + row) * dk + col) : make_uint4(0, 0, 0, 0);
            yr[u] = ok ? *reinterpret_cast<const uint4*>(yg + (tok0 + row) * dk + col) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = tid + 256 * u;
            const int row = c / 16, col = (c % 16) * 4;
            const bool ok = (tok0 + row < n) && (col0 + col < dv);
            zr[u] = ok ? *reinterpret_cast<const uint4*>(zg + (tok0 + row) * dv + col0 + col) : make_uint4(0, 0, 0, 0);
        }
    };
    auto stage_block = [&]() {
#pragma unroll
        for (int u = 0; u < XC; ++u) {
            const int c = tid + 256 * u;
            const int row = c / (DKP / 4), col = (c % (DKP / 4)) * 4;
            *reinterpret_cast<uint4*>(Xs + row * XS + col) = xr[u];
            *reinterpret_cast<uint4*>(Ys + row * XS + col) = yr[u];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = tid + 256 * u;
            const int row = c / 16, col = (c % 16) * 4;
            *reinterpret_cast<uint4*>(Zs + row * ZS + col) = zr[u];
        }
    };

    for (int c = tid; c < 64 * ZS / 4; c += 256) reinterpret_cast<uint4*>(Ps)[c] = make_uint4(0, 0, 0, 0);
    load_block(0);
    stage_block();
    __syncthreads();

    const int jlo = REVERSE ? w : 0, jhi = REVERSE ? 3 : w;

    for (int64_t it = 0; it < it_end; ++it) {
        const int64_t t = REVERSE ? nblk - 1 - it : it;
        const bool have_next = it + 1 < it_end;
        const bool warm = it < it_first;  // warm-up block: state update only
        if (have_next) load_block(it + 1);

        // 1. S^T tiles (rows j, columns i in [16w, 16w+16)) -> masked, decayed P[i][j]
        if (!warm) {
            f32x4 sacc[4];
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) sacc[jt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const f32x4 bx = *reinterpret_cast<const f32x4*>(Xs + (16 * w + r) * XS + 16 * kt + 4 * g);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
                    if (jt >= jlo && jt <= jhi) {
                        const f32x4 ay = *reinterpret_cast<const f32x4*>(Ys + (16 * jt + r) * XS + 16 * kt + 4 * g);
#pragma unroll
                        for (int v = 0; v < 4; ++v) sacc[jt] = mma4(ay[v], bx[v], sacc[jt]);
                    }
                }
            }
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                if (jt >= jlo && jt <= jhi) {
                    f32x4 p;
#pragma unroll
                    for (int v = 0; v < 4; ++v) p[v] = sacc[jt][v] * dfac[jt][v];
                    *reinterpret_cast<f32x4*>(Ps + (16 * w + r) * ZS + 16 * jt + 4 * g) = p;
                }
            }
        }
        __syncthreads();

        if (wave_active) {
            // z[j][16w + r] for the 16 tokens j = 16jt + 4g + v this lane contracts over
            float zf[4][4];
#pragma unroll
            for (int jt = 0; jt < 4; ++jt)
#pragma unroll
                for (int v = 0; v < 4; ++v) zf[jt][v] = Zs[(16 * jt + 4 * g + v) * ZS + 16 * w + r];

            f32x4 oacc[4];
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                if (warm) continue;  // (block-uniform) no output from a warm-up block
                oacc[i4] = (f32x4){0.f, 0.f, 0.f, 0.f};
                // 2a. inter-block: st[4K + q][v] holds row 4g + v of its tile, feature 64K + 16v + 4g + q
#pragma unroll
                for (int K = 0; K < KG; ++K) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const f32x4 bx = *reinterpret_cast<const f32x4*>(Xs + (16 * i4 + r) * XS + 64 * K + 16 * v + 4 * g);
#pragma unroll
                        for (int q = 0; q < 4; ++q) oacc[i4] = mma4(st[4 * K + q][v], bx[q], oacc[i4]);
                    }
                }
                if (DECAY) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) oacc[i4][v] *= ofac[i4];
                }
                // 2b. intra-block: slot g of step (jt, v) is token 16jt + 4g + v
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
                    const bool need = REVERSE ? (jt >= i4) : (jt <= i4);
                    if (need) {
                        const f32x4 bp = *reinterpret_cast<const f32x4*>(Ps + (16 * i4 + r) * ZS + 16 * jt + 4 * g);
#pragma unroll
                        for (int v = 0; v < 4; ++v) oacc[i4] = mma4(zf[jt][v], bp[v], oacc[i4]);
                    }
                }
            }
            const int col = col0 + 16 * w + 4 * g;
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int64_t tok = t * 64 + 16 * i4 + r;
                if (!warm && tok < n && col < dv) *reinterpret_cast<f32x4*>(og + tok * dv + col) = oacc[i4];
            }
            // 3. state = lam^64 state + y^T (z * Lupd)
            if (have_next) {
                if (DECAY) {
#pragma unroll
                    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
                        for (int v = 0; v < 4; ++v) zf[jt][v] *= zfac[jt][v];
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                        for (int v = 0; v < 4; ++v) st[kt][v] *= lamB;
                }
                // row r of tile 4K + q is feature 64K + 16 (r % 4) + 4 (r / 4) + q
#pragma unroll
                for (int K = 0; K < KG; ++K) {
#pragma unroll
                    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            const f32x4 ay = *reinterpret_cast<const f32x4*>(Ys + (16 * jt + 4 * g + v) * XS + 64 * K +
                                                                             16 * (r & 3) + 4 * (r >> 2));
#pragma unroll
                            for (int q = 0; q < 4; ++q) st[4 * K + q] = mma4(ay[q], zf[jt][v], st[4 * K + q]);
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

// (70 KB of LDS at DKP = 64: two workgroups fit a CU when the registers do, which the second bound asks for)
template <int DKP, bool REVERSE, bool DECAY>
__global__ __launch_bounds__(256, DKP <= 64 ? 2 : 1) void la_sweep_f32_kernel(SweepArgsF32 a) {
    sweep_f32_body<DKP, REVERSE, DECAY>(a, blockIdx.x);
}

// The three sweeps of a backward pass with d == e in one launch: part 0 walks forward (dQ), parts 1 and 2
// backward (dK, dV); the parts have the same number of workgroups (a multiple of 8).
struct SweepTrioF32 {
    SweepArgsF32 a[3];
    unsigned per_part;
};
template <int DKP, bool DECAY>
__global__ __launch_bounds__(256, DKP <= 64 ? 2 : 1) void la_sweep_f32_trio_kernel(SweepTrioF32 t) {
    const unsigned part = blockIdx.x / t.per_part, bid = blockIdx.x % t.per_part;
    if (part == 0) sweep_f32_body<DKP, false, DECAY>(t.a[0], bid);
    else sweep_f32_body<DKP, true, DECAY>(t.a[part == 1 ? 1 : 2], bid);
}

template <int DKP, bool DECAY>
static int prep_trio_f32() {
    constexpr size_t lds = (size_t)(2 * 64 * (DKP + LA_F32_XPAD) + 2 * 64 * 68) * sizeof(float);
    static unsigned char lds_allowed[kMaxDevices];
    return allow_lds(la_sweep_f32_trio_kernel<DKP, DECAY>, lds, lds_allowed);
}
template <int DKP, bool REVERSE, bool DECAY>
static int prep_one_f32() {
    constexpr size_t lds = (size_t)(2 * 64 * (DKP + LA_F32_XPAD) + 2 * 64 * 68) * sizeof(float);
    static unsigned char lds_allowed[kMaxDevices];
    return allow_lds(la_sweep_f32_kernel<DKP, REVERSE, DECAY>, lds, lds_allowed);
}
// Every instantiation of this file made ready for its first launch on the current device.
int prepare_f32() {
    int e = 0;
#define LA_P(DKP, D) \
    if (!e) e = prep_trio_f32<DKP, D>(); \
    if (!e) e = prep_one_f32<DKP, false, D>(); \
    if (!e) e = prep_one_f32<DKP, true, D>();
    LA_P(64, false) LA_P(64, true) LA_P(128, false) LA_P(128, true)
#undef LA_P
    return e;
}

template <int DKP, bool DECAY>
static int launch_trio_f32(const SweepTrioF32& t, hipStream_t st) {
    constexpr size_t lds = (size_t)(2 * 64 * (DKP + LA_F32_XPAD) + 2 * 64 * 68) * sizeof(float);
    auto kern = la_sweep_f32_trio_kernel<DKP, DECAY>;
    if (const int e = prep_trio_f32<DKP, DECAY>()) return e;
    hipLaunchKernelGGL(kern, dim3(3 * t.per_part), dim3(256), lds, st, t);
    return (int)hipGetLastError();
}

template <int DKP, bool REVERSE, bool DECAY>
static int launch_one_f32(const SweepArgsF32& a, hipStream_t st) {
    constexpr size_t lds = (size_t)(2 * 64 * (DKP + LA_F32_XPAD) + 2 * 64 * 68) * sizeof(float);
    auto kern = la_sweep_f32_kernel<DKP, REVERSE, DECAY>;
    if (const int e = prep_one_f32<DKP, REVERSE, DECAY>()) return e;
    const int units8 = (a.bh + 7) / 8 * 8;
    hipLaunchKernelGGL(kern, dim3((unsigned)(units8 * a.nslice * a.nchunk)), dim3(256), lds, st, a);
    return (int)hipGetLastError();
}

template <bool REVERSE>
static int launch_dir_f32(const SweepArgsF32& a, hipStream_t st) {
    const bool decay = a.s != nullptr;
#define LA_GO(DKP) (decay ? launch_one_f32<DKP, REVERSE, true>(a, st) : launch_one_f32<DKP, REVERSE, false>(a, st))
    if (a.dk <= 64) return LA_GO(64);
    return LA_GO(128);
#undef LA_GO
}

static SweepArgsF32 make_args_f32(const void* x, const void* y, const void* z, void* out, const float* s, int64_t bh, int64_t h,
                                  int64_t n, int64_t dk, int64_t dv) {
    SweepArgsF32 a;
    a.x = static_cast<const float*>(x); a.y = static_cast<const float*>(y); a.z = static_cast<const float*>(z);
    a.out = static_cast<float*>(out); a.s = s;
    a.n = n; a.dk = (int)dk; a.dv = (int)dv; a.h = (int)h; a.bh = (int)bh;
    a.nslice = (int)((dv + 63) / 64);
    a.nchunk = 1;
    for (int i = 0; i < 9; ++i) a.chunk_start[i] = i == 0 ? 0 : (int)((n + 63) / 64);
    return a;
}

int sweep_f32(const void* x, const void* y, const void* z, void* out, const float* s, int64_t bh, int64_t h,
              int64_t n, int64_t dk, int64_t dv, bool reverse, int chunks, hipStream_t st) {
    if (dk > 128) return LA_E_UNSUPPORTED;
    SweepArgsF32 a = make_args_f32(x, y, z, out, s, bh, h, n, dk, dv);
    plan_warm_up_chunks((bh + 7) / 8 * 8 * a.nslice, (n + 63) / 64, chunks, &a.nchunk, a.chunk_start);
    return reverse ? launch_dir_f32<true>(a, st) : launch_dir_f32<false>(a, st);
}

// float32 backward pass with d == e: dQ = fwd(dO, v, k), dK = rev(v, dO, q), dV = rev(k, q, dO) in one
// launch (the sweeps are independent; with few sequences they run side by side).
int sweep_f32_bwd_once(const void* q, const void* k, const void* v, const void* dout, void* dq, void* dk, void* dv,
                       const float* s, int64_t bh, int64_t h, int64_t n, int64_t d, int chunks, hipStream_t st) {
    if (d > 128) return LA_E_UNSUPPORTED;
    SweepTrioF32 t;
    t.a[0] = make_args_f32(dout, v, k, dq, s, bh, h, n, d, d);
    t.a[1] = make_args_f32(v, dout, q, dk, s, bh, h, n, d, d);
    t.a[2] = make_args_f32(k, q, dout, dv, s, bh, h, n, d, d);
    plan_warm_up_chunks((bh + 7) / 8 * 8 * t.a[0].nslice * 3, (n + 63) / 64, chunks, &t.a[0].nchunk, t.a[0].chunk_start);
    for (int i = 1; i < 3; ++i) {
        t.a[i].nchunk = t.a[0].nchunk;
        for (int j = 0; j < 9; ++j) t.a[i].chunk_start[j] = t.a[0].chunk_start[j];
    }
    t.per_part = (unsigned)((bh + 7) / 8 * 8 * t.a[0].nslice * t.a[0].nchunk);
    const bool decay = s != nullptr;
    if (d <= 64) return decay ? launch_trio_f32<64, true>(t, st) : launch_trio_f32<64, false>(t, st);
    return decay ? launch_trio_f32<128, true>(t, st) : launch_trio_f32<128, false>(t, st);
}

}  // namespace la
