// Single-sweep decayed linear attention for gfx950, feature dims 129 .. 256, wide workgroups:
// one workgroup covers up to 96 (feature dim <= 192) or 128 (<= 256) columns of z / out instead
// of the 64 of la_sweep.hip, with two 16-column accumulator slabs per state wave.
//
// Why: with many (batch, head) sequences the 64-column form needs three (e = 192) or four (e = 256)
// workgroups per sequence - 384 or 512 workgroups for 128 heads on 256 CUs, i.e. two rounds, the
// second of them half empty at e = 192.  96- / 128-column workgroups make it two per sequence: one
// round, the x / y tiles staged and the score tile computed once per 96 / 128 instead of once per 64
// output columns, and every x and y^T fragment read from LDS feeds two MFMAs.
//
// Same operator, same walk over 64-token blocks, same division of labour as la_sweep.hip (waves 0-3
// "score" waves: masked score tile P, then out^T = inter + z^T P^T and the stores; waves 4-7 "state"
// waves: inter = Lout * (state^T x^T), then state = lam^64 state + y^T (z * Lupd)), two barriers per
// block, and the same arithmetic per output column in the same order: results are bit-identical to
// the 64-column form.  What differs, to make room for a state twice as wide:
//   - the two kinds of waves run separate copies of the loop, and the score waves alone fetch and
//     stage the tiles, so the state waves (96 / 128 accumulator registers of state) hold no
//     prefetch registers;
//   - the z slice has a single LDS buffer: it is only read in the second phase of a block, so the
//     next block's slice is written at the start of that block's first phase;
//   - feature dim <= 192: x / y double-buffered, three state waves in use (96 columns); <= 256: one
//     x / y buffer (a third barrier per block), four state waves (128 columns).
// (lightning_attn/ops/triton/lightning_attn2.py:8-85 forward, :88-395 backward.)
#include <type_traits>

#include "la_sweep_common.h"
#include "lightning_attn_hip.h"

namespace la {

template <int DKP>
struct WideLds {
    static constexpr int XS = DKP + 16;            // row stride (elements) of the x / y tiles
    static constexpr int NW = DKP <= 192 ? 3 : 4;  // state waves in use
    static constexpr int ZW = 32 * NW;             // columns of z / out per workgroup, at most
    static constexpr int ZS = ZW + 8;              // row stride of the z slice
    static constexpr int PS = 64 + 8;              // row stride of the P tile
    static constexpr int NBUF = DKP <= 192 ? 2 : 1;
    static constexpr int XY = 2 * 64 * XS;         // elements of one x + y buffer
    static constexpr int ZT = 64 * ZS;
    static constexpr int PT = 64 * PS;
    static constexpr size_t OB = (size_t)NW * 2 * 4 * 64 * 16;  // bytes of the inter-block tile, float32
    static constexpr size_t bytes(size_t elt) { return (size_t)(NBUF * XY + ZT + PT) * elt + OB; }
};

template <typename T, int DKP, bool REVERSE, bool DECAY>
__device__ __forceinline__ void sweep_wide_body(const SweepPair& pair, const unsigned bid) {
    typedef Mma<T> M;
    typedef typename M::V8 V8;
    typedef typename M::V4 V4;
    typedef WideLds<DKP> L;
    constexpr int XS = L::XS, ZS = L::ZS, PS = L::PS, NBUF = L::NBUF, NW = L::NW;
    constexpr int KS = DKP / 32;  // 32-wide contraction steps over the feature dim
    constexpr int KT = DKP / 16;  // 16-row state tiles
    constexpr int NH = 2;         // 16-column slabs per state wave
    constexpr int NL = 256;       // loader threads: the score waves
    constexpr int CPX = DKP / 8;  // 16-byte chunks per row of an x / y tile
    constexpr int XC = 64 * CPX / NL;
    constexpr int CPZ = L::ZW / 8;  // ... of the z slice
    constexpr int ZC = 64 * CPZ / NL;
    extern __shared__ __align__(16) unsigned char smem[];
    T* const tiles = reinterpret_cast<T*>(smem);
    T* const Zs = tiles + NBUF * L::XY;
    T* const Ps = Zs + L::ZT;
    f32x4* const Ob = reinterpret_cast<f32x4*>(Ps + L::PT);  // [wave][slab][i4][lane]

    // workgroup -> (sequence, sweep of a pair, column slice, sequence chunk), as in la_sweep.hip
    const int xcd = bid & 7, local = bid >> 3;
    const int nslice = pair.a[0].nslice, nprod = pair.nprod;
    const int per_unit = nslice * pair.a[0].nchunk * nprod;
    const int unit = xcd + 8 * (local / per_unit);
    const int sub = local % per_unit;
    const SweepArgs& a = pair.a[sub % nprod];
    const int slice = (sub / nprod) % nslice;
    const int chunk = sub / (nprod * nslice);
    if (unit >= a.bh) return;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool state_role = wave >= 4;
    const int w = wave & 3;
    const int lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int64_t n = a.n;
    const int dk = a.dk, dv = a.dv;
    const __amdgpu_buffer_rsrc_t xb = seq_rsrc<T>(a.x, a.lx, unit, a.h, n, dk);
    const __amdgpu_buffer_rsrc_t yb = seq_rsrc<T>(a.y, a.ly, unit, a.h, n, dk);
    const __amdgpu_buffer_rsrc_t zb = seq_rsrc<T>(a.z, a.lz, unit, a.h, n, dv);
    const __amdgpu_buffer_rsrc_t ob = seq_rsrc<T>(a.out, a.lo, unit, a.h, n, dv);
    const unsigned xts = (unsigned)a.lx.ts, yts = (unsigned)a.ly.ts, zts = (unsigned)a.lz.ts, ots = (unsigned)a.lo.ts;
    const unsigned nrows = (unsigned)n;
    const int col0 = slice * a.zw;
    const int colend = min(dv, col0 + a.zw);  // this workgroup's columns: [col0, colend)
    const int cbase = 32 * w;                 // first of this wave's 32 columns within the slice
    const bool wave_active = w < NW && (col0 + cbase) < colend;

    float rate = 0.f;
    if (DECAY) rate = a.s[unit % a.h];

    const int64_t nblk = (n + 63) / 64;
    const int mode = pair.mode;
    const int nchunk = pair.a[0].nchunk;
    if (mode == kCollect && chunk == nchunk - 1) return;  // nobody needs the state after the last chunk
    const int64_t cbeg = mode == kWarmUp ? (int64_t)a.chunk_start[chunk] : min((int64_t)chunk * pair.chunk_len, nblk);
    const int64_t cend = mode == kWarmUp ? (int64_t)a.chunk_start[chunk + 1] : min((int64_t)(chunk + 1) * pair.chunk_len, nblk);
    const int64_t it0 = mode == kWarmUp ? 0 : cbeg;           // first block this workgroup walks
    const int64_t it_first = mode == kCollect ? cend : cbeg;  // first block whose output it produces
    const int64_t it_end = cend;

    if (!state_role) {
        // =====================================================================================
        // score waves: memory traffic, the score tile, the intra-block product and the stores
        // =====================================================================================
        TileDeal deal = kDeal[w];
        if (REVERSE) {
            deal.itA = 3 - deal.itA; deal.jt0 = 3 - deal.jt0;
            if (deal.itB >= 0) { deal.itB = 3 - deal.itB; deal.jt1 = 3 - deal.jt1; deal.jt2 = 3 - deal.jt2; }
        }
        const int itA = __builtin_amdgcn_readfirstlane(deal.itA), jt0 = __builtin_amdgcn_readfirstlane(deal.jt0);
        const int itB = __builtin_amdgcn_readfirstlane(deal.itB), jt1 = __builtin_amdgcn_readfirstlane(deal.jt1);
        const int jt2 = __builtin_amdgcn_readfirstlane(deal.jt2);
        float dfac[3][4];
        {
            const int its[3] = {itA, itB, itB}, jts[3] = {jt0, jt1, jt2};
#pragma unroll
            for (int sl = 0; sl < 3; ++sl)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int i = 16 * its[sl] + r, j = 16 * jts[sl] + 4 * g + v;
                    const int diff = REVERSE ? (j - i) : (i - j);
                    dfac[sl][v] = diff >= 0 ? (DECAY ? expf(-rate * (float)diff) : 1.f) : 0.f;
                }
        }
        // this thread's chunks of a tile: chunk c = tid + 256 u lies in row c / chunks-per-row
        int xrow[XC], zrow[ZC];
        unsigned lane_x[XC], lane_y[XC], lane_z[ZC], stage_x[XC], stage_z[ZC];
#pragma unroll
        for (int u = 0; u < XC; ++u) {
            const int c = tid + NL * u;
            const int row = c / CPX, col = (c % CPX) * 8;
            xrow[u] = row;
            lane_x[u] = col < dk ? (row * xts + col) * (unsigned)sizeof(T) : kOob;
            lane_y[u] = col < dk ? (row * yts + col) * (unsigned)sizeof(T) : kOob;
            stage_x[u] = (unsigned)(row * XS + col);
        }
#pragma unroll
        for (int u = 0; u < ZC; ++u) {
            const int c = tid + NL * u;
            const int row = c / CPZ, col = col0 + (c % CPZ) * 8;
            zrow[u] = row;
            lane_z[u] = col < colend ? (row * zts + col) * (unsigned)sizeof(T) : kOob;
            stage_z[u] = (unsigned)(row * ZS + (c % CPZ) * 8);
        }
        u32x4 xr[XC], yr[XC], zr[ZC];
        // Blocks at or beyond it_end, and the x tile of warm-up blocks, are fetched at the out-of-range
        // offset: zeros, no memory traffic, the same sequence of loads on every path.
        auto load_xy = [&](int64_t b) {
            const int64_t t = REVERSE ? nblk - 1 - b : b;
            const bool valid = b < it_end, need_x = valid && b >= it_first;
            const unsigned tok0 = valid ? (unsigned)(t * 64) : 0u;
            const int rows = valid ? (int)min(64u, nrows - tok0) : 0, rows_x = need_x ? rows : 0;
#pragma unroll
            for (int u = 0; u < XC; ++u) {
                xr[u] = buf_load16(xb, xrow[u] < rows_x ? lane_x[u] : kOob, tok0 * xts * (unsigned)sizeof(T));
                yr[u] = buf_load16(yb, xrow[u] < rows ? lane_y[u] : kOob, tok0 * yts * (unsigned)sizeof(T));
            }
        };
        auto load_z = [&](int64_t b) {
            const int64_t t = REVERSE ? nblk - 1 - b : b;
            const bool valid = b < it_end;
            const unsigned tok0 = valid ? (unsigned)(t * 64) : 0u;
            const int rows = valid ? (int)min(64u, nrows - tok0) : 0;
#pragma unroll
            for (int u = 0; u < ZC; ++u)
                zr[u] = buf_load16(zb, zrow[u] < rows ? lane_z[u] : kOob, tok0 * zts * (unsigned)sizeof(T));
        };
        auto stage_xy = [&](int buf) {
            T* Xd = tiles + buf * L::XY;
            T* Yd = Xd + 64 * XS;
#pragma unroll
            for (int u = 0; u < XC; ++u) {
                *reinterpret_cast<u32x4*>(Xd + stage_x[u]) = xr[u];
                *reinterpret_cast<u32x4*>(Yd + stage_x[u]) = yr[u];
            }
        };
        auto stage_zs = [&]() {
#pragma unroll
            for (int u = 0; u < ZC; ++u) *reinterpret_cast<u32x4*>(Zs + stage_z[u]) = zr[u];
        };

        // zero P once: tiles on the masked side of the diagonal are never written
        for (int c = tid; c < L::PT / 8; c += NL) reinterpret_cast<uint4*>(Ps)[c] = make_uint4(0, 0, 0, 0);
        load_xy(it0);
        load_z(it0);
        stage_xy(NBUF == 2 ? (int)(it0 & 1) : 0);
        load_xy(it0 + 1);
        __syncthreads();

        for (int64_t it = it0; it < it_end; ++it) {
            const int64_t t = REVERSE ? nblk - 1 - it : it;
            const bool warm = it < it_first;  // warm-up block: state update only
            const int buf = NBUF == 2 ? (int)(it & 1) : 0;
            const T* Xs = tiles + buf * L::XY;
            const T* Ys = Xs + 64 * XS;
            // the z slice of this block (its buffer was last read in the second phase of the block
            // before), and the next one on its way
            stage_zs();
            load_z(it + 1);
            // ---- phase 1: S^T tiles of this wave -> masked, decayed P[i][j] ----
            if (!warm) {
                f32x4 sacc[3];
#pragma unroll
                for (int sl = 0; sl < 3; ++sl) sacc[sl] = (f32x4){0.f, 0.f, 0.f, 0.f};
                const T* xa = Xs + (16 * itA + r) * XS + 8 * g;
                const T* y0 = Ys + (16 * jt0 + r) * XS + 8 * g;
                constexpr int SB = 2;  // contraction steps per batch of fragment reads
                if (itB >= 0) {
                    const T* xb2 = Xs + (16 * itB + r) * XS + 8 * g;
                    const T* y1 = Ys + (16 * jt1 + r) * XS + 8 * g;
                    const T* y2 = Ys + (16 * jt2 + r) * XS + 8 * g;
#pragma unroll
                    for (int k0 = 0; k0 < KS; k0 += SB) {
                        V8 fxa[SB], fxb[SB], fy0[SB], fy1[SB], fy2[SB];
#pragma unroll
                        for (int ks = 0; ks < SB; ++ks) {
                            fxa[ks] = *reinterpret_cast<const V8*>(xa + 32 * (k0 + ks));
                            fy0[ks] = *reinterpret_cast<const V8*>(y0 + 32 * (k0 + ks));
                            fxb[ks] = *reinterpret_cast<const V8*>(xb2 + 32 * (k0 + ks));
                            fy1[ks] = *reinterpret_cast<const V8*>(y1 + 32 * (k0 + ks));
                            fy2[ks] = *reinterpret_cast<const V8*>(y2 + 32 * (k0 + ks));
                        }
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int ks = 0; ks < SB; ++ks) {
                            sacc[0] = M::mma(fy0[ks], fxa[ks], sacc[0]);
                            sacc[1] = M::mma(fy1[ks], fxb[ks], sacc[1]);
                            sacc[2] = M::mma(fy2[ks], fxb[ks], sacc[2]);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
#pragma unroll
                    for (int k0 = 0; k0 < KS; k0 += SB) {
                        V8 fxa[SB], fy0[SB];
#pragma unroll
                        for (int ks = 0; ks < SB; ++ks) {
                            fxa[ks] = *reinterpret_cast<const V8*>(xa + 32 * (k0 + ks));
                            fy0[ks] = *reinterpret_cast<const V8*>(y0 + 32 * (k0 + ks));
                        }
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int ks = 0; ks < SB; ++ks) sacc[0] = M::mma(fy0[ks], fxa[ks], sacc[0]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                {
                    V4 p;
#pragma unroll
                    for (int v = 0; v < 4; ++v) p[v] = M::cvt(sacc[0][v] * dfac[0][v]);
                    *reinterpret_cast<V4*>(Ps + (16 * itA + r) * PS + 16 * jt0 + 4 * g) = p;
                }
                if (itB >= 0) {
                    V4 p;
#pragma unroll
                    for (int v = 0; v < 4; ++v) p[v] = M::cvt(sacc[1][v] * dfac[1][v]);
                    *reinterpret_cast<V4*>(Ps + (16 * itB + r) * PS + 16 * jt1 + 4 * g) = p;
#pragma unroll
                    for (int v = 0; v < 4; ++v) p[v] = M::cvt(sacc[2][v] * dfac[2][v]);
                    *reinterpret_cast<V4*>(Ps + (16 * itB + r) * PS + 16 * jt2 + 4 * g) = p;
                }
            }
            __syncthreads();
            // ---- phase 2: out^T = inter + z^T P^T for this wave's 32 columns, then the stores ----
            if (!warm && wave_active) {
                V8 bp[4][2];
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const bool need = REVERSE ? (ks >= i4 / 2) : (ks <= i4 / 2);
                        if (need) bp[i4][ks] = *reinterpret_cast<const V8*>(Ps + (16 * i4 + r) * PS + 32 * ks + 8 * g);
                    }
                }
                // the inter-block tiles of both slabs first: their place in LDS then takes this wave's output tile
                f32x4 oacc[NH][4];
#pragma unroll
                for (int h = 0; h < NH; ++h)
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) oacc[h][i4] = Ob[((w * NH + h) * 4 + i4) * 64 + lane];
#pragma unroll
                for (int h = 0; h < NH; ++h) {
                    if (col0 + cbase + 16 * h >= colend) continue;
                    V8 zf[2];
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const T* pz = Zs + (32 * ks + 8 * g + (r >> 2)) * ZS + cbase + 16 * h + 4 * (r & 3);
                        zf[ks] = cat<V8, V4>(lds_tr4<V4>(pz), lds_tr4<V4>(pz + 4 * ZS));
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) {
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks) {
                            const bool need = REVERSE ? (ks >= i4 / 2) : (ks <= i4 / 2);
                            if (need) oacc[h][i4] = M::mma(zf[ks], bp[i4][ks], oacc[h][i4]);
                        }
                    }
                }
                // Out of the accumulators a store covers 32 bytes of a row; through LDS (this wave's own
                // part of the inter-block tile buffer, 64 rows x 32 columns with padded rows) it covers 64.
                constexpr int OS = 40;  // row stride of the staged tile, elements
                T* const otile = reinterpret_cast<T*>(Ob + (size_t)w * NH * 4 * 64);
                // (wavefront-scope fences: the compiler must keep the reads of the inter-block tile above, the
                // writes of the staged tile and its reads below in this order; LDS itself serves a wave in order)
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
                for (int h = 0; h < NH; ++h)
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) {
                        V4 o;
#pragma unroll
                        for (int v = 0; v < 4; ++v) o[v] = (T)oacc[h][i4][v];
                        *reinterpret_cast<V4*>(otile + (16 * i4 + r) * OS + 16 * h + 4 * g) = o;
                    }
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                {
                    const int orow = lane >> 2, ocol = col0 + cbase + 8 * (lane & 3);
                    const unsigned tok0 = (unsigned)(t * 64);
#pragma unroll
                    for (int p4 = 0; p4 < 4; ++p4) {
                        const int row = orow + 16 * p4;
                        const u32x4 val = *reinterpret_cast<const u32x4*>(otile + row * OS + 8 * (lane & 3));
                        const unsigned tok = tok0 + 16 * p4;  // wave-uniform first token of these 16 rows
                        const unsigned off = (ocol < colend && tok + orow < nrows) ? (orow * ots + ocol) * (unsigned)sizeof(T) : kOob;
                        buf_store16(ob, off, tok < nrows ? tok * ots * (unsigned)sizeof(T) : 0u, val);
                    }
                }
            }
            if (NBUF == 2) {
                stage_xy((int)((it + 1) & 1));
                load_xy(it + 2);
                __syncthreads();
            } else {
                __syncthreads();
                stage_xy(0);
                load_xy(it + 2);
                __syncthreads();
            }
        }
        return;
    }

    // =========================================================================================
    // state waves: the state, the inter-block term and the state update
    // =========================================================================================
    float ofac[4];     // scale of the inter-block term for token i = 16it + r
    float zfac[2][8];  // scale of token j = 32ks + 8g + u in the state update
    float lamB = 1.f;
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
    // state slots: [unit][sweep][slice][chunk 0 .. nchunk-2][state wave][slab][tile][lane] accumulator quartets
    constexpr size_t SF = (size_t)4 * NH * KT * 64 * 4;
    float* const slot0 = pair.state + ((((size_t)unit * nprod + sub % nprod) * nslice + slice) * (size_t)(nchunk - 1)) * SF;
    const size_t lane_slot = ((size_t)w * NH * KT * 64 + lane) * 4;
    f32x4 st[NH][KT];
    {
        const bool resume = mode == kApply && chunk > 0;
        const float* const src = slot0 + (size_t)(chunk - 1) * SF + lane_slot;
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
                st[h][kt] = resume ? *reinterpret_cast<const f32x4*>(src + (size_t)(h * KT + kt) * 256) : (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    __syncthreads();

    for (int64_t it = it0; it < it_end; ++it) {
        const bool have_next = it + 1 < it_end;
        const bool warm = it < it_first;
        const int buf = NBUF == 2 ? (int)(it & 1) : 0;
        const T* Ys = tiles + buf * L::XY + 64 * XS;
        // ---- phase 1: inter-block term out^T[c][i] = Lout[i] * sum_k state[k][c] x[i][k] -> LDS ----
        if (!warm && wave_active) {
            f32x4 oacc[NH][4];
#pragma unroll
            for (int h = 0; h < NH; ++h)
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) oacc[h][i4] = (f32x4){0.f, 0.f, 0.f, 0.f};
            constexpr int IB = DKP <= 192 ? 2 : 1;  // contraction steps per batch of reads
#pragma unroll
            for (int k0 = 0; k0 < KS; k0 += IB) {
                V8 bx[IB][4];
#pragma unroll
                for (int ks = 0; ks < IB; ++ks) {
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) {
                        // two 8-byte reads from base registers the optimiser cannot relate: fused into one
                        // ds_read2_b64 they would conflict on the LDS banks
                        const unsigned xoff = (unsigned)((buf * L::XY + r * XS + 32 * (k0 + ks) + 4 * g) * sizeof(T));
                        unsigned lo = xoff, hi = xoff + 16 * (unsigned)sizeof(T);
                        asm volatile("" : "+v"(lo));
                        asm volatile("" : "+v"(hi));
                        constexpr unsigned ROW = 16 * XS * (unsigned)sizeof(T);
                        bx[ks][i4] = cat<V8, V4>(*reinterpret_cast<const V4*>(smem + lo + i4 * ROW),
                                                 *reinterpret_cast<const V4*>(smem + hi + i4 * ROW));
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < IB; ++ks) {
                    V8 sb[NH];
#pragma unroll
                    for (int h = 0; h < NH; ++h)
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            sb[h][v] = M::cvt(st[h][2 * (k0 + ks)][v]);
                            sb[h][4 + v] = M::cvt(st[h][2 * (k0 + ks) + 1][v]);
                        }
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4)
#pragma unroll
                        for (int h = 0; h < NH; ++h) oacc[h][i4] = M::mma(sb[h], bx[ks][i4], oacc[h][i4]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int h = 0; h < NH; ++h)
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    if (DECAY) {
#pragma unroll
                        for (int v = 0; v < 4; ++v) oacc[h][i4][v] *= ofac[i4];
                    }
                    Ob[((w * NH + h) * 4 + i4) * 64 + lane] = oacc[h][i4];
                }
        }
        __syncthreads();
        // ---- phase 2: state = lam^64 state + y^T (z * Lupd) ----
        if (wave_active && (have_next || mode == kCollect)) {
            V8 zf[NH][2];
#pragma unroll
            for (int h = 0; h < NH; ++h)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const T* pz = Zs + (32 * ks + 8 * g + (r >> 2)) * ZS + cbase + 16 * h + 4 * (r & 3);
                    zf[h][ks] = cat<V8, V4>(lds_tr4<V4>(pz), lds_tr4<V4>(pz + 4 * ZS));
                }
            constexpr int UB = 4;  // state tiles per batch of transposed reads
#pragma unroll
            for (int t0 = 0; t0 < KT; t0 += UB) {
                V8 ay[UB][2];
#pragma unroll
                for (int kt = 0; kt < UB; ++kt) {
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const T* py = Ys + (32 * ks + 8 * g + (r >> 2)) * XS + 16 * (t0 + kt) + 4 * (r & 3);
                        ay[kt][ks] = cat<V8, V4>(lds_tr4<V4>(py), lds_tr4<V4>(py + 4 * XS));
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (DECAY && t0 == 0) {
#pragma unroll
                    for (int h = 0; h < NH; ++h) {
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                            for (int u = 0; u < 8; ++u) zf[h][ks][u] = (T)((float)zf[h][ks][u] * zfac[ks][u]);
#pragma unroll
                        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                            for (int v = 0; v < 4; ++v) st[h][kt][v] *= lamB;
                    }
                }
#pragma unroll
                for (int kt = 0; kt < UB; ++kt) {
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                        for (int h = 0; h < NH; ++h) st[h][t0 + kt] = M::mma(ay[kt][ks], zf[h][ks], st[h][t0 + kt]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
        if (NBUF == 1) __syncthreads();
    }
    if (mode == kCollect) {
        float* const dst = slot0 + (size_t)chunk * SF + lane_slot;
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<f32x4*>(dst + (size_t)(h * KT + kt) * 256) = st[h][kt];
    }
}

template <typename T, int DKP, bool REVERSE, bool DECAY>
__global__ __launch_bounds__(512, 1) void la_sweep_wide_kernel(SweepPair pair) {
    sweep_wide_body<T, DKP, REVERSE, DECAY>(pair, blockIdx.x);
}

template <typename T, int DKP, bool REVERSE, bool DECAY>
static int launch_wide_one(const SweepPair& pair, hipStream_t st) {
    const SweepArgs& a = pair.a[0];
    if (pair.mode != kWarmUp && pipe_state_floats(a.dk, true) != (size_t)4 * 2 * (DKP / 16) * 64 * 4) return LA_E_WORKSPACE;
    // the slice width the host chose must be one the kernel's LDS slot holds
    if (a.zw <= 0 || a.zw % 32 || a.zw > WideLds<DKP>::ZW) return LA_E_UNSUPPORTED;
    constexpr size_t lds = WideLds<DKP>::bytes(sizeof(T));
    static_assert(lds <= 160 * 1024, "LDS budget");
    auto kern = la_sweep_wide_kernel<T, DKP, REVERSE, DECAY>;
    static unsigned char lds_allowed[kMaxDevices];
    if (const int e = allow_lds(kern, lds, lds_allowed)) return e;
    const int units8 = (a.bh + 7) / 8 * 8;
    const unsigned grid = (unsigned)(units8 * a.nslice * a.nchunk * pair.nprod);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, st, pair);
    return (int)hipGetLastError();
}

template <typename T, bool REVERSE>
static int launch_wide_dir(const SweepPair& pair, hipStream_t st) {
    const SweepArgs& a = pair.a[0];
    const bool decay = a.s != nullptr;
#define LA_GO(DKP) (decay ? launch_wide_one<T, DKP, REVERSE, true>(pair, st) : launch_wide_one<T, DKP, REVERSE, false>(pair, st))
    if (a.dk <= 192) return LA_GO(192);
    return LA_GO(256);
#undef LA_GO
}

static int launch_wide_any(const SweepPair& p, int dtype, bool reverse, hipStream_t st) {
    if (dtype == LA_BF16) return reverse ? launch_wide_dir<__bf16, true>(p, st) : launch_wide_dir<__bf16, false>(p, st);
    if (dtype == LA_FP16) return reverse ? launch_wide_dir<_Float16, true>(p, st) : launch_wide_dir<_Float16, false>(p, st);
    return LA_E_UNSUPPORTED;
}

// The wide two-barrier kernel (feature dims 129 .. 256), in one launch or - chunks from scanned states - three.
int sweep_wide(const SweepPair& p, int dtype, bool reverse, hipStream_t st) {
    const SweepArgs& a = p.a[0];
    if (a.dk <= 128 || a.dk > 256 || p.nprod < 1 || p.nprod > 2) return LA_E_UNSUPPORTED;
    SweepPair q = p;
    if (p.mode == kWarmUp || a.nchunk <= 1) {
        q.mode = kWarmUp;
        return launch_wide_any(q, dtype, reverse, st);
    }
    if (!p.state || p.chunk_len < 1) return LA_E_WORKSPACE;
    q.mode = kCollect;
    int rc = launch_wide_any(q, dtype, reverse, st);
    if (rc != LA_OK) return rc;
    rc = launch_state_scan(p, st);
    if (rc != LA_OK) return rc;
    q.mode = kApply;
    return launch_wide_any(q, dtype, reverse, st);
}

}  // namespace la
