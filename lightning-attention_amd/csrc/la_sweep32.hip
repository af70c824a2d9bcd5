// Decayed linear attention sweep for gfx950, feature dim dk <= 128
// (bf16 / fp16 MFMA 32x32x16, fp32 state).  See la_sweep.hip for the
// definition of a sweep and how the four products of the operator map onto it.
//
// A workgroup of 4 wavefronts owns one (batch, head, 64-column slice of z/out)
// and walks the 64-token blocks in order, one barrier per block:
//
//   waves 0,1  "state" waves.  Wave s owns columns [32s, 32s+32) of the slice and
//              the dk x 32 slab of the state S = sum lam^.. y_j^T z_j in fp32 MFMA
//              accumulators.  Per block:  out^T = Lout * (S^T x^T) + z^T P^T
//              (stored straight from the accumulators), then
//              S = lam^64 S + y^T (z * Lupd).  The accumulator layout of one MFMA
//              is reused as the A operand of the next (state -> bf16 fragments)
//              with the matching permutation of the contraction index on the x
//              side; y^T and z^T fragments come from the LDS transpose read.
//   waves 2,3  "score" waves, one block ahead of the state waves.  Each loads a
//              32-row band of x and of y straight from global memory in MFMA
//              fragment layout (16 B per lane), computes the non-masked 32x32
//              quadrants of S^T = y x^T (wave 2: the first diagonal and the
//              off-diagonal one, wave 3: the second diagonal one), applies mask
//              and decay, writes P to LDS, and forwards its x / y fragments
//              (wave 3 also z and z * Lupd) to the LDS tiles the state waves
//              read.  Loads run two blocks ahead.
//
// x/y/z tiles and P are double-buffered in LDS; nothing else is shared.
#include "la_common.h"
#include "lightning_attn_hip.h"

namespace la {

struct Sweep32Args {
    const void* x;  // (bh, n, dk)
    const void* y;  // (bh, n, dk)
    const void* z;  // (bh, n, dv)
    void* out;      // (bh, n, dv)
    const float* s; // h decay rates or nullptr
    int64_t n;
    int dk, dv, h, bh, nslice;
#ifdef LA_SWEEP32_TIMING
    long long* dbg;  // [wave][block][8] cycle stamps of workgroup 0
#endif
};

#ifdef LA_SWEEP32_TIMING
#define LA_STAMP(slot) do { if (blockIdx.x == 0 && lane == 0 && it < 64) a.dbg[(wave * 64 + it) * 8 + (slot)] = clock64(); } while (0)
#else
#define LA_STAMP(slot) do { } while (0)
#endif

template <typename T>
struct Mma32;
template <>
struct Mma32<__bf16> {
    typedef bf16x8 V8;
    typedef bf16x4 V4;
    static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ __bf16 cvt(float f) { return (__bf16)f; }
};
template <>
struct Mma32<_Float16> {
    typedef f16x8 V8;
    typedef f16x4 V4;
    static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    // fp16 saturates instead of overflowing to inf when a state entry is large
    static __device__ __forceinline__ _Float16 cvt(float f) {
        return (_Float16)__builtin_fminf(__builtin_fmaxf(f, -65504.f), 65504.f);
    }
};

// LDS transpose read (ds_read_b64_tr_b16): within a group of 16 lanes, lane i
// receives element (i % 4) of the 8-byte words addressed by lanes 4e + i/4,
// e = 0..3.  With lane L addressing row L/4, columns 4(L%4).. of a row-major
// tile, lane i ends up with column i of rows 0..3.
template <typename V4>
__device__ __forceinline__ V4 lds_tr4_32(const void* p) {
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
    return __builtin_bit_cast(V4, v);
}
template <typename V8, typename V4>
__device__ __forceinline__ V8 cat32(V4 a, V4 b) {
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

template <int DKP>
struct Sweep32Lds {
    static constexpr int XS = DKP + 8;  // row stride (elements) of the x / y tiles
    static constexpr int ZS = 64 + 8;   // row stride of the z slice and the P tile
    static constexpr int XY = 2 * 64 * XS;  // elements of one x + y buffer (ring of 3)
    static constexpr int ZZ = 2 * 64 * ZS;  // elements of one z + (z * Lupd) buffer (ring of 2)
    static constexpr int PT = 64 * ZS;      // elements of one P buffer (ring of 2)
    static constexpr size_t bytes(size_t elt) { return (size_t)(3 * XY + 2 * ZZ + 2 * PT) * elt; }
};

template <typename T, int DKP, bool REVERSE, bool DECAY>
__global__ __launch_bounds__(256, 1) void la_sweep32_kernel(Sweep32Args a) {
    typedef Mma32<T> M;
    typedef typename M::V8 V8;
    typedef typename M::V4 V4;
    typedef Sweep32Lds<DKP> L;
    constexpr int XS = L::XS, ZS = L::ZS;
    constexpr int KS = DKP / 16;  // 16-wide contraction steps over the feature dim
    constexpr int KT = DKP / 32;  // 32-row state tiles
    extern __shared__ __align__(16) unsigned char smem[];
    T* XYbuf = reinterpret_cast<T*>(smem);
    T* Zbuf = XYbuf + 3 * L::XY;
    T* Pbuf = Zbuf + 2 * L::ZZ;

    // Workgroups are dealt round-robin to the 8 XCDs by linear id; keep the
    // column slices of one head on one XCD so their x / y reads share an L2.
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int unit = xcd + 8 * (local / a.nslice);
    const int slice = local % a.nslice;
    if (unit >= a.bh) return;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int r32 = lane & 31, G = lane >> 5;  // 32x32x16 operand row / contraction half
    const int q = lane >> 4, L16 = lane & 15;  // 16-lane group of the transpose read
    const int64_t n = a.n;
    const int dk = a.dk, dv = a.dv;
    // one bounds-checked buffer per (batch, head) slice: rows >= n read as zero / are not written
    const __amdgpu_buffer_rsrc_t xb = make_rsrc(static_cast<const T*>(a.x) + (int64_t)unit * n * dk, (unsigned)(n * dk * sizeof(T)));
    const __amdgpu_buffer_rsrc_t yb = make_rsrc(static_cast<const T*>(a.y) + (int64_t)unit * n * dk, (unsigned)(n * dk * sizeof(T)));
    const __amdgpu_buffer_rsrc_t zb = make_rsrc(static_cast<const T*>(a.z) + (int64_t)unit * n * dv, (unsigned)(n * dv * sizeof(T)));
    const __amdgpu_buffer_rsrc_t ob = make_rsrc(static_cast<T*>(a.out) + (int64_t)unit * n * dv, (unsigned)(n * dv * sizeof(T)));
    const int col0 = slice * 64;
    const int64_t nblk = (n + 63) / 64;
    float rate = 0.f;
    if (DECAY) rate = a.s[unit % a.h];

    if (wave >= 2) {
        // ===================== score waves ====================================
        // Wave A (band 0) stages rows 0-31 of the x, y and z tiles, wave B (band 1) rows
        // 32-63: coalesced 16-byte loads (16 lanes per 256-byte row) into registers, two
        // blocks ahead, then into LDS.  From the LDS tiles of block it+1 wave A computes
        // the quadrants (0,0) and the off-diagonal one ((1,0) forward, (0,1) reverse) of
        // S^T = y x^T, wave B the quadrant (1,1); (ib, jb) = band of token i, of token j.
        const int band = wave - 2;
        const bool isA = band == 0;
        f32x16 dfacD, dfacO;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int i = r32, j = 8 * (v / 4) + 4 * G + (v % 4);
            const int diff = REVERSE ? (j - i) : (i - j);
            dfacD[v] = diff >= 0 ? (DECAY ? expf(-rate * (float)diff) : 1.f) : 0.f;
            dfacO[v] = DECAY ? expf(-rate * (float)(32 + diff)) : 1.f;  // 32 + diff >= 1
        }
        constexpr int CPR = DKP / 8;      // 16-byte chunks per x / y row
        constexpr int NXY = CPR / 2;      // x (or y) chunks per lane for a 32-row band
        // z rows staged by this lane: 32*band + (lane + 64u)/8, u = 0..3; Lupd of those rows
        float zrow[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int j = 32 * band + ((lane + 64 * u) >> 3);
            zrow[u] = DECAY ? expf(-rate * (float)(REVERSE ? j : 64 - j)) : 1.f;
        }
        u32x4 fx0[NXY], fy0[NXY], fx1[NXY], fy1[NXY], fz0[4], fz1[4];

        // Blocks past the end (b >= nblk) read as zeros.
        auto load_xy = [&](int64_t b, u32x4 (&fx)[NXY], u32x4 (&fy)[NXY]) {
            const int64_t t = REVERSE ? nblk - 1 - b : b;
            const bool blk_ok = b < nblk;
            const unsigned tok0 = (unsigned)(t * 64) + 32 * band;
#pragma unroll
            for (int u = 0; u < NXY; ++u) {
                const int c = lane + 64 * u;
                const int row = c / CPR, col = (c % CPR) * 8;
                const bool ok = blk_ok && col < dk;  // columns dk..DKP-1 are zero padding
                const unsigned off = ((tok0 + row) * (unsigned)dk + col) * (unsigned)sizeof(T);
                fx[u] = buf_load16(xb, ok ? off : kOob);
                fy[u] = buf_load16(yb, ok ? off : kOob);
            }
        };
        auto load_z = [&](int64_t b, u32x4 (&fz)[4]) {
            const int64_t t = REVERSE ? nblk - 1 - b : b;
            const bool blk_ok = b < nblk;
            const unsigned tok0 = (unsigned)(t * 64) + 32 * band;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = lane + 64 * u;
                const int row = c >> 3, col = (c & 7) * 8;
                const bool ok = blk_ok && (col0 + col < dv);
                fz[u] = buf_load16(zb, ok ? ((tok0 + row) * (unsigned)dv + col0 + col) * (unsigned)sizeof(T) : kOob);
            }
        };
        auto stage_xy = [&](int64_t b, const u32x4 (&fx)[NXY], const u32x4 (&fy)[NXY]) {
            T* Xd = XYbuf + (int)(b % 3) * L::XY + 32 * band * XS;
            T* Yd = Xd + 64 * XS;
#pragma unroll
            for (int u = 0; u < NXY; ++u) {
                const int c = lane + 64 * u;
                const int row = c / CPR, col = (c % CPR) * 8;
                *reinterpret_cast<u32x4*>(Xd + row * XS + col) = fx[u];
                *reinterpret_cast<u32x4*>(Yd + row * XS + col) = fy[u];
            }
        };
        auto stage_z = [&](int64_t b, const u32x4 (&fz)[4]) {
            T* Zd = Zbuf + (int)(b & 1) * L::ZZ + 32 * band * ZS;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = lane + 64 * u;
                const int row = c >> 3, col = (c & 7) * 8;
                *reinterpret_cast<u32x4*>(Zd + row * ZS + col) = fz[u];
                if (DECAY) {
                    V8 zv = __builtin_bit_cast(V8, fz[u]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) zv[e] = (T)((float)zv[e] * zrow[u]);
                    *reinterpret_cast<V8*>(Zd + 64 * ZS + row * ZS + col) = zv;
                }
            }
        };
        auto write_p = [&](T* Pd, const f32x16 sacc, const f32x16 df, const int ib, const int jb) {
            // S^T[j][i]: lane holds column i = r32, rows j = 8m + 4G + (0..3), m = 0..3
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                V4 p;
#pragma unroll
                for (int e = 0; e < 4; ++e) p[e] = M::cvt(sacc[4 * m + e] * df[4 * m + e]);
                *reinterpret_cast<V4*>(Pd + (32 * ib + r32) * ZS + 32 * jb + 8 * m + 4 * G) = p;
            }
        };
        auto scores = [&](int64_t b) {
            const T* Xs = XYbuf + (int)(b % 3) * L::XY;
            const T* Ys = Xs + 64 * XS;
            T* Pd = Pbuf + (int)(b & 1) * L::PT;
            const T* xd = Xs + (32 * band + r32) * XS + 8 * G;  // own band
            const T* yd = Ys + (32 * band + r32) * XS + 8 * G;
            f32x16 sacc, sacc2;
#pragma unroll
            for (int v = 0; v < 16; ++v) sacc[v] = sacc2[v] = 0.f;
            if (isA) {
                // off-diagonal: forward y band 0 against x band 1; reverse y band 1 against x band 0
                const T* xo = REVERSE ? xd : xd + 32 * XS;
                const T* yo = REVERSE ? yd + 32 * XS : yd;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    sacc = M::mma(*reinterpret_cast<const V8*>(yd + 16 * ks), *reinterpret_cast<const V8*>(xd + 16 * ks), sacc);
                    sacc2 = M::mma(*reinterpret_cast<const V8*>(yo + 16 * ks), *reinterpret_cast<const V8*>(xo + 16 * ks), sacc2);
                }
                write_p(Pd, sacc, dfacD, 0, 0);
                write_p(Pd, sacc2, dfacO, REVERSE ? 0 : 1, REVERSE ? 1 : 0);
            } else {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    sacc = M::mma(*reinterpret_cast<const V8*>(yd + 16 * ks), *reinterpret_cast<const V8*>(xd + 16 * ks), sacc);
                write_p(Pd, sacc, dfacD, 1, 1);
            }
        };

        // prologue: x/y of blocks 0,1 and z, P of block 0 in LDS; sets 0/1 hold blocks 2/3 (x,y), 1/2 (z)
        load_xy(0, fx0, fy0);
        load_xy(1, fx1, fy1);
        load_z(0, fz0);
        load_z(1, fz1);
        stage_xy(0, fx0, fy0);
        stage_z(0, fz0);
        load_xy(2, fx0, fy0);
        load_z(2, fz0);
        __syncthreads();
        scores(0);
        stage_xy(1, fx1, fy1);
        load_xy(3, fx1, fy1);
        __syncthreads();
        for (int64_t it = 0; it < nblk; it += 2) {
            // state waves work on block it: publish x/y of block it+2, z and P of block it+1
            LA_STAMP(0);
            stage_xy(it + 2, fx0, fy0);
            stage_z(it + 1, fz1);
            LA_STAMP(1);
            load_xy(it + 4, fx0, fy0);
            load_z(it + 3, fz1);
            LA_STAMP(2);
            if (it + 1 < nblk) scores(it + 1);
            LA_STAMP(3);
            __syncthreads();
            LA_STAMP(4);
            if (it + 1 < nblk) {
                stage_xy(it + 3, fx1, fy1);
                stage_z(it + 2, fz0);
                load_xy(it + 5, fx1, fy1);
                load_z(it + 4, fz0);
                if (it + 2 < nblk) scores(it + 2);
                __syncthreads();
            }
        }
    } else {
        // ===================== state waves ====================================
        const int cs = 32 * wave;  // first column of this wave's slab inside the slice
        const bool cols_active = (col0 + cs) < dv;
        float ofac[2];      // scale of the inter-block term for token i = 32*itile + r32
        float lamB = 1.f;
        if (DECAY) {
#pragma unroll
            for (int itile = 0; itile < 2; ++itile) {
                const int i = 32 * itile + r32;
                ofac[itile] = expf(-rate * (float)(REVERSE ? 64 - i : i));
            }
            lamB = expf(-rate * 64.f);
        }
        f32x16 st[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int v = 0; v < 16; ++v) st[kt][v] = 0.f;

        __syncthreads();
        __syncthreads();
        for (int64_t it = 0; it < nblk; ++it) {
            const int64_t t = REVERSE ? nblk - 1 - it : it;
            const int buf = (int)(it & 1);
            const T* Xs = XYbuf + (int)(it % 3) * L::XY;
            const T* Ys = Xs + 64 * XS;
            const T* Zs = Zbuf + buf * L::ZZ;
            const T* Z2 = Zs + 64 * ZS;
            const T* Ps = Pbuf + buf * L::PT;
            LA_STAMP(0);
            if (cols_active) {
                // One software-pipelined chain of MFMA steps: inter (2 KS) -> update (4 KT)
                // -> intra (6).  The LDS operands of step s+PRE are requested before step s
                // issues, so that no more than about a dozen LDS reads are in flight (the
                // hardware counter that orders them saturates at 15) and their latency hides
                // behind the matrix pipe; the elementwise work sits in the MFMA shadow.
                constexpr int NI = 2 * KS, NU = 4 * KT, PRE = 4;
                const bool upd = it + 1 < nblk;
                V8 bx[NI], ay[NU], zs[4], zf[4], bp[2][4];
                auto load_bx = [&](int s_) {  // inter step s_: ks = s_/2, itile = s_%2
                    // state tile kt, accumulator v  <->  k = 32kt + 8(v/4) + 4G + v%4: x is read
                    // with the same permutation of the contraction index
                    const T* px = Xs + (32 * (s_ % 2) + r32) * XS + 16 * (s_ / 2) + 4 * G;
                    bx[s_] = cat32<V8, V4>(*reinterpret_cast<const V4*>(px), *reinterpret_cast<const V4*>(px + 8));
                };
                auto load_z = [&](const T* Zt, int ks) {  // z^T fragment: column cs + r32, tokens 16ks + 8G + u
                    const int zo = (16 * ks + 8 * G + (L16 >> 2)) * ZS + cs + 16 * (q & 1) + 4 * (L16 & 3);
                    return cat32<V8, V4>(lds_tr4_32<V4>(Zt + zo), lds_tr4_32<V4>(Zt + zo + 4 * ZS));
                };
                auto load_upd = [&](int u_) {  // update step u_: ks = u_/KT, kt = u_%KT
                    const int ks = u_ / KT, kt = u_ % KT;
                    if (kt == 0) zs[ks] = load_z(DECAY ? Z2 : Zs, ks);
                    const T* py = Ys + (16 * ks + 8 * G + (L16 >> 2)) * XS + 32 * kt + 16 * (q & 1) + 4 * (L16 & 3);
                    ay[u_] = cat32<V8, V4>(lds_tr4_32<V4>(py), lds_tr4_32<V4>(py + 4 * XS));
                };
                // intra steps in ks-major order; a step exists only on the unmasked side
                auto intra_needed = [&](int ks, int itile) { return REVERSE ? (ks / 2 >= itile) : (ks / 2 <= itile); };
                auto load_intra = [&](int ks) {
                    zf[ks] = (DECAY || !upd) ? load_z(Zs, ks) : zs[ks];
#pragma unroll
                    for (int itile = 0; itile < 2; ++itile)
                        if (intra_needed(ks, itile))
                            bp[itile][ks] = *reinterpret_cast<const V8*>(Ps + (32 * itile + r32) * ZS + 16 * ks + 8 * G);
                };

#pragma unroll
                for (int s_ = 0; s_ < PRE; ++s_) load_bx(s_);
                V8 sb[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int u = 0; u < 8; ++u) sb[ks][u] = M::cvt(st[ks / 2][8 * (ks % 2) + u]);
                f32x16 oacc[2];
#pragma unroll
                for (int itile = 0; itile < 2; ++itile)
#pragma unroll
                    for (int v = 0; v < 16; ++v) oacc[itile][v] = 0.f;
                // ---- inter-block term: out^T[c][i] = sum_k S[k][c] x[i][k] ------------------
#pragma unroll
                for (int s_ = 0; s_ < NI; ++s_) {
                    if (s_ + PRE < NI) load_bx(s_ + PRE);
                    else if (upd) load_upd(s_ + PRE - NI);
                    oacc[s_ % 2] = M::mma(sb[s_ / 2], bx[s_], oacc[s_ % 2]);
                    if (DECAY && upd) {  // lam^64 on the state, 64/NI registers per step
#pragma unroll
                        for (int e = 0; e < 64 / NI * KT / 4; ++e) {
                            const int idx = s_ * (64 / NI * KT / 4) + e;
                            st[idx / 16][idx % 16] *= lamB;
                        }
                    }
                }
                LA_STAMP(1);
                // ---- state = lam^64 state + y^T (z * Lupd) ----------------------------------
                if (upd) {
#pragma unroll
                    for (int u_ = 0; u_ < NU; ++u_) {
                        if (u_ + PRE < NU) load_upd(u_ + PRE);
                        else load_intra(u_ + PRE - NU);
                        st[u_ % KT] = M::mma(ay[u_], zs[u_ / KT], st[u_ % KT]);
                    }
                } else {
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) load_intra(ks);
                }
                LA_STAMP(2);
                if (DECAY) {
#pragma unroll
                    for (int itile = 0; itile < 2; ++itile)
#pragma unroll
                        for (int v = 0; v < 16; ++v) oacc[itile][v] *= ofac[itile];
                }
                // ---- intra-block term: out^T += z^T P^T -------------------------------------
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                    for (int itile = 0; itile < 2; ++itile)
                        if (intra_needed(ks, itile)) oacc[itile] = M::mma(zf[ks], bp[itile][ks], oacc[itile]);
                LA_STAMP(3);
                // ---- store out[token][cs + 8m + 4G .. +3] -----------------------------------
#pragma unroll
                for (int itile = 0; itile < 2; ++itile) {
                    const unsigned tok = (unsigned)(t * 64) + 32 * itile + r32;
#pragma unroll
                    for (int m = 0; m < 4; ++m) {
                        const int col = col0 + cs + 8 * m + 4 * G;
                        V4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = (T)oacc[itile][4 * m + e];
                        const unsigned off = col < dv ? (tok * (unsigned)dv + col) * (unsigned)sizeof(T) : kOob;
                        buf_store8(ob, off, __builtin_bit_cast(u32x2, o));
                    }
                }
            }
            LA_STAMP(4);
            __syncthreads();
            LA_STAMP(5);
        }
    }
}

template <typename T, int DKP, bool REVERSE, bool DECAY>
static int launch32_one(const Sweep32Args& a, hipStream_t st) {
    constexpr size_t lds = Sweep32Lds<DKP>::bytes(sizeof(T));
    static_assert(lds <= 160 * 1024, "LDS budget");
    auto kern = la_sweep32_kernel<T, DKP, REVERSE, DECAY>;
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
static int launch32_dir(const Sweep32Args& a, hipStream_t st) {
    const bool decay = a.s != nullptr;
#define LA_GO(DKP) (decay ? launch32_one<T, DKP, REVERSE, true>(a, st) : launch32_one<T, DKP, REVERSE, false>(a, st))
    if (a.dk <= 64) return LA_GO(64);
    return LA_GO(128);
#undef LA_GO
}

#ifdef LA_SWEEP32_TIMING
long long* g_sweep32_dbg = nullptr;
extern "C" void la_dbg_set(long long* p) { g_sweep32_dbg = p; }
#endif

// x,y: (bh,n,dk)  z,out: (bh,n,dv); dk <= 128
int sweep32(const void* x, const void* y, const void* z, void* out, const float* s, int64_t bh, int64_t h, int64_t n,
            int64_t dk, int64_t dv, int dtype, bool reverse, hipStream_t st) {
    Sweep32Args a;
    a.x = x; a.y = y; a.z = z; a.out = out; a.s = s;
    a.n = n; a.dk = (int)dk; a.dv = (int)dv; a.h = (int)h; a.bh = (int)bh;
    a.nslice = (int)((dv + 63) / 64);
#ifdef LA_SWEEP32_TIMING
    a.dbg = g_sweep32_dbg;
#endif
    if (dtype == LA_BF16) return reverse ? launch32_dir<__bf16, true>(a, st) : launch32_dir<__bf16, false>(a, st);
    if (dtype == LA_FP16) return reverse ? launch32_dir<_Float16, true>(a, st) : launch32_dir<_Float16, false>(a, st);
    return LA_E_UNSUPPORTED;
}

}  // namespace la
