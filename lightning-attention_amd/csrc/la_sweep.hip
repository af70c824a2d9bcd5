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
// The sequence is cut into blocks of 64 tokens.  A workgroup of 8 wavefronts owns
// one (batch, head, 64-column slice of z/out) and walks the blocks in order.  The
// wavefronts are specialised so that every SIMD holds two waves with different
// instruction mixes:
//   waves 0-3 ("score" waves)   S^T = y x^T tiles -> decay/mask -> P (LDS);
//                               out^T = inter + z^T P^T ; store out
//   waves 4-7 ("state" waves)   own the dk x 16 column slab of the state
//                               S = sum lam^.. y_j^T z_j in fp32 accumulators;
//                               inter = Lout * (state^T x^T) -> LDS;
//                               state = lam^64 state + y^T (z * Lupd)
// State and z^T fragments never leave registers: the accumulator layout of one
// MFMA is reused as the A operand of the next with a matching permutation of the
// contraction index on the B side.  Transposed operands (y^T, z^T) come from the
// LDS transpose read ds_read_b64_tr_b16.  x/y/z tiles are double-buffered in LDS
// (global -> registers one block ahead -> LDS), two barriers per block.
#include "la_sweep_common.h"
#include "lightning_attn_hip.h"

namespace la {

template <int DKP>
struct SweepLds {
#ifndef LA_XPAD
#define LA_XPAD 16
#endif
#ifndef LA_ZPAD
#define LA_ZPAD 8
#endif
    static constexpr int XS = DKP + LA_XPAD;  // row stride (elements) of the x / y tiles
    static constexpr int ZS = 64 + LA_ZPAD;   // row stride of the z slice and the P tile
    static constexpr int NBUF = DKP <= 192 ? 2 : 1;
    static constexpr int TILE = 2 * 64 * XS + 64 * ZS;  // elements of one x+y+z buffer
    static constexpr size_t bytes(size_t elt) { return (size_t)(NBUF * TILE + 64 * ZS) * elt + 4 * 4 * 64 * 16; }
};

// `bid`: number of the workgroup within its part of the launch.
template <typename T, int DKP, bool REVERSE, bool DECAY>
__device__ __forceinline__ void sweep_body(const SweepPair& pair, const unsigned bid) {
    typedef Mma<T> M;
    typedef typename M::V8 V8;
    typedef typename M::V4 V4;
    typedef SweepLds<DKP> L;
    constexpr int XS = L::XS, ZS = L::ZS, NBUF = L::NBUF;
    constexpr int KS = DKP / 32;  // 32-wide contraction steps over the feature dim
    constexpr int KT = DKP / 16;  // 16-row state tiles
    constexpr int XC = DKP / 64;  // 16-byte chunks per thread for an x / y tile (512 threads)
    extern __shared__ __align__(16) unsigned char smem[];
    T* tiles = reinterpret_cast<T*>(smem);
    T* Ps = tiles + NBUF * L::TILE;
    f32x4* Ob = reinterpret_cast<f32x4*>(Ps + 64 * ZS);  // [wave][i4][lane]

    // Workgroups are dealt round-robin to the 8 XCDs by linear id; keep the
    // column slices of one head on one XCD so their x / y re-reads share an L2.
    const int xcd = bid & 7, local = bid >> 3;
    const int nslice = pair.a[0].nslice, nprod = pair.nprod;
    const int per_unit = nslice * pair.a[0].nchunk * nprod;
    const int unit = xcd + 8 * (local / per_unit);
    const int sub = local % per_unit;
    // the sweeps of a pair alternate fastest, then the column slices, then the sequence chunks
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
    // one bounds-checked buffer per (batch, head) sequence; rows >= n are masked by offset below
    const __amdgpu_buffer_rsrc_t xb = seq_rsrc<T>(a.x, a.lx, unit, a.h, n, dk);
    const __amdgpu_buffer_rsrc_t yb = seq_rsrc<T>(a.y, a.ly, unit, a.h, n, dk);
    const __amdgpu_buffer_rsrc_t zb = seq_rsrc<T>(a.z, a.lz, unit, a.h, n, dv);
    const __amdgpu_buffer_rsrc_t ob = seq_rsrc<T>(a.out, a.lo, unit, a.h, n, dv);
    const unsigned xts = (unsigned)a.lx.ts, yts = (unsigned)a.ly.ts, zts = (unsigned)a.lz.ts, ots = (unsigned)a.lo.ts;
    const unsigned nrows = (unsigned)n;
    const int col0 = slice * 64;  // (a.zw is 64 for this kernel)
    const bool cols_active = (col0 + 16 * w) < dv;

    float rate = 0.f;
    if (DECAY) rate = a.s[unit % a.h];

    // ---- score-wave constants: its tiles and their mask * decay factors -------
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
    // ---- state-wave constants (every factor <= 1) ----------------------------
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

    f32x4 st[KT];
    const int64_t nblk = (n + 63) / 64;
    // Sequence chunking (chunk-parallel variant): this workgroup produces the blocks
    // [it_first, it_end) of the walk.  Without a workspace (kWarmUp) it first runs over the blocks
    // before it_first with the state update only ("warm-up": y and z are read, nothing is written)
    // to rebuild the state its chunk starts from.  With one, the chunks are equally long and a
    // workgroup walks its own chunk only: first with the state update alone, from zero, to leave the
    // state it ends with (kCollect), then - a scan kernel having combined those into the state at the
    // start of every chunk - for good, from that state (kApply).
    const int mode = pair.mode;
    const int nchunk = pair.a[0].nchunk;
    if (mode == kCollect && chunk == nchunk - 1) return;  // nobody needs the state after the last chunk
    const int64_t cbeg = mode == kWarmUp ? (int64_t)a.chunk_start[chunk] : min((int64_t)chunk * pair.chunk_len, nblk);
    const int64_t cend = mode == kWarmUp ? (int64_t)a.chunk_start[chunk + 1] : min((int64_t)(chunk + 1) * pair.chunk_len, nblk);
    const int64_t it0 = mode == kWarmUp ? 0 : cbeg;           // first block this workgroup walks
    const int64_t it_first = mode == kCollect ? cend : cbeg;  // first block whose output it produces
    const int64_t it_end = cend;
    // state slots: [unit][sweep][slice][chunk 0 .. nchunk-2][state wave][tile][lane] accumulator quartets
    constexpr size_t SF = (size_t)4 * KT * 64 * 4;
    float* const slot0 = pair.state + ((((size_t)unit * nprod + sub % nprod) * nslice + slice) * (size_t)(nchunk - 1)) * SF;
    const size_t lane_slot = ((size_t)w * KT * 64 + lane) * 4;
    {
        const bool resume = mode == kApply && chunk > 0 && state_role;
        const float* const src = slot0 + (size_t)(chunk - 1) * SF + lane_slot;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
            st[kt] = resume ? *reinterpret_cast<const f32x4*>(src + (size_t)kt * 256) : (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    // One register set of prefetched tiles (there are no registers to spare for two at these feature
    // dims): while block `it` is worked on, block it+1 is in flight from memory.
    u32x4 xrA[XC], yrA[XC], zrA;

    // Per-lane byte offsets of this thread's 16-byte chunks inside a 64-token block (out of range
    // where the chunk lies in the zero padding dk..DKP-1 or beyond dv); the block's first token goes
    // into the wave-uniform offset of the load.  When a tile row holds a divisor of 512 chunks, a
    // thread's chunks lie whole rows apart in the same columns and only the first one needs registers.
    constexpr bool SAMECOL = 512 % (DKP / 8) == 0;
    constexpr int NLANE = SAMECOL ? 1 : XC;
    constexpr int CROWS = 512 / (DKP / 8);  // rows between two chunks of a thread (SAMECOL)
    int lane_row[NLANE];
    unsigned lane_x[NLANE], lane_y[NLANE];
#pragma unroll
    for (int u = 0; u < NLANE; ++u) {
        const int c = tid + 512 * u;
        const int row = c / (DKP / 8), col = (c % (DKP / 8)) * 8;
        lane_row[u] = row;
        lane_x[u] = col < dk ? (row * xts + col) * (unsigned)sizeof(T) : kOob;
        lane_y[u] = col < dk ? (row * yts + col) * (unsigned)sizeof(T) : kOob;
    }
    const int lane_zrow = tid / 8;
    const unsigned lane_z = (col0 + (tid % 8) * 8 < dv) ? (lane_zrow * zts + col0 + (tid % 8) * 8) * (unsigned)sizeof(T) : kOob;
    // Fetches block number b of the walk.  Blocks at or beyond it_end, and the x tile of warm-up
    // blocks, are fetched at the out-of-range offset: zeros, no memory traffic, and the sequence of
    // loads is the same on every path.
    auto load_block = [&](int64_t b, u32x4 (&xr)[XC], u32x4 (&yr)[XC], u32x4& zr) {
        const int64_t t = REVERSE ? nblk - 1 - b : b;
        const bool valid = b < it_end, need_x = valid && b >= it_first;
        const unsigned tok0 = valid ? (unsigned)(t * 64) : 0u;
        // rows of this block that exist (0 for a block that is not fetched)
        const int rows = valid ? (int)min(64u, nrows - tok0) : 0, rows_x = need_x ? rows : 0;
#pragma unroll
        for (int u = 0; u < XC; ++u) {
            if (SAMECOL) {
                // a wave-uniform offset must stay inside the buffer: 0 when none of these rows exists
                const unsigned tk = u * CROWS < rows ? tok0 + u * CROWS : 0u;
                xr[u] = buf_load16(xb, lane_row[0] < rows_x - u * CROWS ? lane_x[0] : kOob, tk * xts * (unsigned)sizeof(T));
                yr[u] = buf_load16(yb, lane_row[0] < rows - u * CROWS ? lane_y[0] : kOob, tk * yts * (unsigned)sizeof(T));
            } else {
                const int v = u < NLANE ? u : 0;
                xr[u] = buf_load16(xb, lane_row[v] < rows_x ? lane_x[v] : kOob, tok0 * xts * (unsigned)sizeof(T));
                yr[u] = buf_load16(yb, lane_row[v] < rows ? lane_y[v] : kOob, tok0 * yts * (unsigned)sizeof(T));
            }
        }
        zr = buf_load16(zb, lane_zrow < rows ? lane_z : kOob, tok0 * zts * (unsigned)sizeof(T));
    };
    auto stage_block = [&](int buf, const u32x4 (&xr)[XC], const u32x4 (&yr)[XC], const u32x4& zr) {
        T* Xd = tiles + buf * L::TILE;
        T* Yd = Xd + 64 * XS;
        T* Zd = Yd + 64 * XS;
#pragma unroll
        for (int u = 0; u < XC; ++u) {
            const int c = tid + 512 * u;
            const int row = c / (DKP / 8), col = (c % (DKP / 8)) * 8;
            *reinterpret_cast<u32x4*>(Xd + row * XS + col) = xr[u];
            *reinterpret_cast<u32x4*>(Yd + row * XS + col) = yr[u];
        }
        {
            const int row = tid / 8, col = (tid % 8) * 8;
            *reinterpret_cast<u32x4*>(Zd + row * ZS + col) = zr;
        }
    };

    // zero P once: tiles on the masked side of the diagonal are never written
    for (int c = tid; c < 64 * ZS / 8; c += 512) reinterpret_cast<uint4*>(Ps)[c] = make_uint4(0, 0, 0, 0);
    load_block(it0, xrA, yrA, zrA);
    stage_block(NBUF == 2 ? (int)(it0 & 1) : 0, xrA, yrA, zrA);
    load_block(it0 + 1, xrA, yrA, zrA);
    __syncthreads();

    // One block of the walk.  `xr, yr, zr` hold block it+1 on entry and block it+2 on exit.
    auto block_body = [&](const int64_t it, u32x4 (&xr)[XC], u32x4 (&yr)[XC], u32x4& zr) {
        const int64_t t = REVERSE ? nblk - 1 - it : it;
        const bool have_next = it + 1 < it_end;
        const bool warm = it < it_first;  // warm-up block: state update only
        const int buf = NBUF == 2 ? (int)(it & 1) : 0;
        const T* Xs = tiles + buf * L::TILE;
        const T* Ys = Xs + 64 * XS;
        const T* Zs = Ys + 64 * XS;
        // =================== phase 1 =========================================
        if (warm) {
            // nothing: x is not needed and no output is produced
        } else if (!state_role) {
            // S^T tiles of this wave -> masked, decayed P[i][j]
            f32x4 sacc[3];
#pragma unroll
            for (int sl = 0; sl < 3; ++sl) sacc[sl] = (f32x4){0.f, 0.f, 0.f, 0.f};
            const T* xa = Xs + (16 * itA + r) * XS + 8 * g;
            const T* y0 = Ys + (16 * jt0 + r) * XS + 8 * g;
            // all fragment reads of a batch are issued before its MFMAs (the scheduler otherwise
            // sinks each read next to its use and the wave pays one LDS round trip per MFMA)
            constexpr int SB = KS <= 4 ? KS : 2;  // contraction steps per batch
            if (itB >= 0) {
                const T* xb = Xs + (16 * itB + r) * XS + 8 * g;
                const T* y1 = Ys + (16 * jt1 + r) * XS + 8 * g;
                const T* y2 = Ys + (16 * jt2 + r) * XS + 8 * g;
#pragma unroll
                for (int k0 = 0; k0 < KS; k0 += SB) {
                    V8 fxa[SB], fxb[SB], fy0[SB], fy1[SB], fy2[SB];
#pragma unroll
                    for (int ks = 0; ks < SB; ++ks) {
                        fxa[ks] = *reinterpret_cast<const V8*>(xa + 32 * (k0 + ks));
                        fy0[ks] = *reinterpret_cast<const V8*>(y0 + 32 * (k0 + ks));
                        fxb[ks] = *reinterpret_cast<const V8*>(xb + 32 * (k0 + ks));
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
                *reinterpret_cast<V4*>(Ps + (16 * itA + r) * ZS + 16 * jt0 + 4 * g) = p;
            }
            if (itB >= 0) {
                V4 p;
#pragma unroll
                for (int v = 0; v < 4; ++v) p[v] = M::cvt(sacc[1][v] * dfac[1][v]);
                *reinterpret_cast<V4*>(Ps + (16 * itB + r) * ZS + 16 * jt1 + 4 * g) = p;
#pragma unroll
                for (int v = 0; v < 4; ++v) p[v] = M::cvt(sacc[2][v] * dfac[2][v]);
                *reinterpret_cast<V4*>(Ps + (16 * itB + r) * ZS + 16 * jt2 + 4 * g) = p;
            }
        } else if (cols_active) {
            // inter-block term: out^T[c][i] = Lout[i] * sum_k state[k][c] x[i][k]
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
            for (int i4 = 0; i4 < 4; ++i4) oacc[i4] = (f32x4){0.f, 0.f, 0.f, 0.f};
            constexpr int IB = KS <= 4 ? KS : 2;  // contraction steps per batch of reads
#pragma unroll
            for (int k0 = 0; k0 < KS; k0 += IB) {
                V8 bx[IB][4];
#pragma unroll
                for (int ks = 0; ks < IB; ++ks) {
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) {
                        // two 8-byte reads from base registers the optimiser cannot relate: fused
                        // into one ds_read2_b64 they would conflict on the LDS banks
                        const unsigned xoff = (unsigned)((buf * L::TILE + r * XS + 32 * (k0 + ks) + 4 * g) * sizeof(T));
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
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) oacc[i4] = M::mma(sb[k0 + ks], bx[ks][i4], oacc[i4]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                if (DECAY) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) oacc[i4][v] *= ofac[i4];
                }
                Ob[(w * 4 + i4) * 64 + lane] = oacc[i4];
            }
        }
        if (!warm) __syncthreads();  // warm-up blocks share nothing between the two phases

        // =================== phase 2 =========================================
        if (!state_role) {
            if (cols_active && !warm) {
                // out^T = inter + z^T P^T, then store out[token][16w + 4g .. +3]
                V8 zf[2];
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const T* pz = Zs + (32 * ks + 8 * g + (r >> 2)) * ZS + 16 * w + 4 * (r & 3);
                    zf[ks] = cat<V8, V4>(lds_tr4<V4>(pz), lds_tr4<V4>(pz + 4 * ZS));
                }
                f32x4 oacc[4];
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) oacc[i4] = Ob[(w * 4 + i4) * 64 + lane];
                V8 bp[4][2];
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const bool need = REVERSE ? (ks >= i4 / 2) : (ks <= i4 / 2);
                        if (need) bp[i4][ks] = *reinterpret_cast<const V8*>(Ps + (16 * i4 + r) * ZS + 32 * ks + 8 * g);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const bool need = REVERSE ? (ks >= i4 / 2) : (ks <= i4 / 2);
                        if (need) oacc[i4] = M::mma(zf[ks], bp[i4][ks], oacc[i4]);
                    }
                }
                const int col = col0 + 16 * w + 4 * g;
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    const unsigned tok = (unsigned)(t * 64) + 16 * i4;  // wave-uniform first token of the tile
                    V4 o;
#pragma unroll
                    for (int v = 0; v < 4; ++v) o[v] = (T)oacc[i4][v];
                    const unsigned off = (col < dv && tok + r < nrows) ? (r * ots + col) * (unsigned)sizeof(T) : kOob;
                    buf_store8(ob, off, tok < nrows ? tok * ots * (unsigned)sizeof(T) : 0u, __builtin_bit_cast(u32x2, o));
                }
            }
        } else if (cols_active && (have_next || mode == kCollect)) {
            // state = lam^64 state + y^T (z * Lupd)
            V8 zf[2];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const T* pz = Zs + (32 * ks + 8 * g + (r >> 2)) * ZS + 16 * w + 4 * (r & 3);
                zf[ks] = cat<V8, V4>(lds_tr4<V4>(pz), lds_tr4<V4>(pz + 4 * ZS));
            }
            constexpr int UB = KT <= 8 ? KT : 4;  // state tiles per batch of transposed reads
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
                    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                        for (int u = 0; u < 8; ++u) zf[ks][u] = (T)((float)zf[ks][u] * zfac[ks][u]);
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                        for (int v = 0; v < 4; ++v) st[kt][v] *= lamB;
                }
#pragma unroll
                for (int kt = 0; kt < UB; ++kt) {
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) st[t0 + kt] = M::mma(ay[kt][ks], zf[ks], st[t0 + kt]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (NBUF == 2) {
            stage_block((int)((it + 1) & 1), xr, yr, zr);
            load_block(it + 2, xr, yr, zr);
            __syncthreads();
        } else {
            __syncthreads();
            stage_block(0, xr, yr, zr);
            load_block(it + 2, xr, yr, zr);
            __syncthreads();
        }
    };
    for (int64_t it = it0; it < it_end; ++it) block_body(it, xrA, yrA, zrA);
    if (mode == kCollect && state_role) {
        float* const dst = slot0 + (size_t)chunk * SF + lane_slot;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<f32x4*>(dst + (size_t)kt * 256) = st[kt];
    }
}

template <typename T, int DKP, bool REVERSE, bool DECAY>
__global__ __launch_bounds__(512, 1) void la_sweep_kernel(SweepPair pair) {
    sweep_body<T, DKP, REVERSE, DECAY>(pair, blockIdx.x);
}

// Forward-walking and backward-walking sweeps in one launch (SweepBoth).
template <typename T, int DKP, bool DECAY>
__global__ __launch_bounds__(512, 1) void la_sweep_both_kernel(SweepBoth both) {
    if (blockIdx.x < both.nfwd) sweep_body<T, DKP, false, DECAY>(both.fwd, blockIdx.x);
    else sweep_body<T, DKP, true, DECAY>(both.rev, blockIdx.x - both.nfwd);
}

static unsigned part_grid(const SweepPair& p) {
    return (unsigned)((p.a[0].bh + 7) / 8 * 8 * p.a[0].nslice * p.a[0].nchunk * p.nprod);
}

template <typename T, int DKP, bool DECAY>
static int launch_both_one(const SweepBoth& b, hipStream_t st) {
    constexpr size_t lds = SweepLds<DKP>::bytes(sizeof(T));
    auto kern = la_sweep_both_kernel<T, DKP, DECAY>;
    static unsigned char lds_allowed[kMaxDevices];
    if (const int e = allow_lds(kern, lds, lds_allowed)) return e;
    hipLaunchKernelGGL(kern, dim3(b.nfwd + part_grid(b.rev)), dim3(512), lds, st, b);
    return (int)hipGetLastError();
}

template <typename T>
static int launch_both(const SweepBoth& b, hipStream_t st) {
    const bool decay = b.fwd.a[0].s != nullptr;
#define LA_GO(DKP) (decay ? launch_both_one<T, DKP, true>(b, st) : launch_both_one<T, DKP, false>(b, st))
    if (b.fwd.a[0].dk <= 192) return LA_GO(192);
    return LA_GO(256);
#undef LA_GO
}

template <typename T, int DKP, bool REVERSE, bool DECAY>
static int launch_one(const SweepPair& pair, hipStream_t st) {
    const SweepArgs& a = pair.a[0];
    if (pair.mode != kWarmUp && pipe_state_floats(a.dk, false) != (size_t)4 * (DKP / 16) * 64 * 4) return LA_E_WORKSPACE;
    constexpr size_t lds = SweepLds<DKP>::bytes(sizeof(T));
    static_assert(lds <= 160 * 1024, "LDS budget");
    auto kern = la_sweep_kernel<T, DKP, REVERSE, DECAY>;
    static unsigned char lds_allowed[kMaxDevices];
    if (const int e = allow_lds(kern, lds, lds_allowed)) return e;
    const int units8 = (a.bh + 7) / 8 * 8;
    const unsigned grid = (unsigned)(units8 * a.nslice * a.nchunk * pair.nprod);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, st, pair);
    return (int)hipGetLastError();
}

template <typename T, bool REVERSE>
static int launch_dir(const SweepPair& pair, hipStream_t st) {
    const SweepArgs& a = pair.a[0];
    const bool decay = a.s != nullptr;
#define LA_GO(DKP) (decay ? launch_one<T, DKP, REVERSE, true>(pair, st) : launch_one<T, DKP, REVERSE, false>(pair, st))
    if (a.dk <= 192) return LA_GO(192);
    return LA_GO(256);
#undef LA_GO
}

static int num_cus() {
    static const int cus = [] {
        int dev = 0, n = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        return n > 0 ? n : 256;
    }();
    return cus;
}

// Sequence chunks per (batch, head, slice).  With few sequences a single sweep per sequence
// leaves most of the 256 CUs idle; the walk is then cut into up to 8 chunks whose workgroups
// rebuild their incoming state themselves.  A warm-up block costs about half a full block, so
// chunk lengths shrink geometrically (len_c ~ (1 - rho)^c, rho = 0.5) to make all workgroups
// finish together.  The caller's launch options can override the count.
static int64_t warm_up_chunks(int64_t wgs, int64_t nblk) {
    const int64_t cus = num_cus();
    int64_t c = 1;
    if (wgs * 2 <= cus && nblk >= 8) {
        c = cus / wgs;
        if (c > nblk / 4) c = nblk / 4;
    }
    return c > 8 ? 8 : c < 1 ? 1 : c;
}

void plan_warm_up_chunks(int64_t wgs, int64_t nblk, int forced, int* nchunk, int* chunk_start /* [9] */) {
    int64_t c = forced > 0 ? forced : warm_up_chunks(wgs, nblk);
    if (c > 8) c = 8;
    if (c > nblk) c = nblk;
    if (c < 1) c = 1;
    // geometric lengths, at least one block each, summing to nblk
    const double rho = 0.5;
    double wsum = 0.0, wgt = 1.0;
    for (int i = 0; i < c; ++i) { wsum += wgt; wgt *= 1.0 - rho; }
    int64_t start = 0;
    wgt = 1.0;
    for (int i = 0; i < c; ++i) {
        chunk_start[i] = (int)start;
        int64_t len = (int64_t)((double)nblk * wgt / wsum + 0.5);
        const int64_t left_after = c - 1 - i;
        if (len < 1) len = 1;
        if (start + len > nblk - left_after) len = nblk - left_after - start;
        start += len;
        wgt *= 1.0 - rho;
    }
    *nchunk = (int)c;
    for (int i = (int)c; i < 9; ++i) chunk_start[i] = (int)nblk;
}

static void choose_chunks(SweepArgs& a, int nprod, const Opts& opts) {
    plan_warm_up_chunks((int64_t)((a.bh + 7) / 8 * 8) * a.nslice * nprod, (a.n + 63) / 64, opts.chunks, &a.nchunk, a.chunk_start);
}

static SweepArgs make_args(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv) {
    SweepArgs a;
    a.x = io.x; a.y = io.y; a.z = io.z; a.out = io.out; a.s = s;
    a.lx = io.lx; a.ly = io.ly; a.lz = io.lz; a.lo = io.lo;
    a.n = n; a.dk = (int)dk; a.dv = (int)dv; a.h = (int)h; a.bh = (int)bh;
    a.nslice = (int)((dv + 63) / 64);
    a.zw = 64;
    return a;
}

static int launch_classic_one(const SweepPair& p, int dtype, bool reverse, hipStream_t st) {
    if (dtype == LA_BF16) return reverse ? launch_dir<__bf16, true>(p, st) : launch_dir<__bf16, false>(p, st);
    if (dtype == LA_FP16) return reverse ? launch_dir<_Float16, true>(p, st) : launch_dir<_Float16, false>(p, st);
    return LA_E_UNSUPPORTED;
}

// The two-barrier kernel (feature dims 129..256), in one launch or - chunks with scanned states - three.
static int launch_classic(const SweepPair& p, int dtype, bool reverse, hipStream_t st) {
    SweepPair q = p;
    if (p.mode == kWarmUp || p.a[0].nchunk <= 1) {
        q.mode = kWarmUp;
        return launch_classic_one(q, dtype, reverse, st);
    }
    if (!p.state || p.chunk_len < 1) return LA_E_WORKSPACE;
    q.mode = kCollect;
    int rc = launch_classic_one(q, dtype, reverse, st);
    if (rc != LA_OK) return rc;
    rc = launch_state_scan(p, st);
    if (rc != LA_OK) return rc;
    q.mode = kApply;
    return launch_classic_one(q, dtype, reverse, st);
}

// With a workspace the kernels do not rebuild a chunk's incoming state with warm-up blocks: the states
// the chunks end with are collected and scanned, and every chunk starts from the result (three
// launches; equally long chunks, up to 64 of them).  Number of chunks and bytes of workspace for a
// launch of nprod sweeps, 0 bytes where the warm-up form is used (always, with opts.scan == LA_OPT_OFF).
struct ScanPlan {
    int nchunk, chunk_len;
    size_t bytes;
    double us;  // estimated duration of the launch(es)
};

// Estimates, in microseconds, behind the choices below.  A workgroup takes about block_us per 64-token
// block (measured, by feature dim and columns per workgroup) and half of that for a block it only folds
// into the state.  Warm-up blocks: with the geometric chunk lengths of choose_chunks the longest
// workgroup runs the fraction `frac` of a single walk.  Scanned states: a chunk one and a half times,
// plus two more launches and the scan (16 us measured, and 10 for the host's share).
static double block_us(int64_t dk, bool wide) {
    if (dk <= 64) return 1.0;
    if (dk <= 128) return wide ? 1.75 : 1.4;
    if (dk <= 192) return wide ? 3.0 : 2.1;
    return wide ? 4.1 : 2.9;
}
// Column slices per sequence: 64 columns each, or - wide - 128 (feature dim up to 128), 96 (up to 192), 128 (up to 256).
static int64_t wide_slices(int64_t dk, int64_t dv) {
    const int64_t zw = dk <= 128 ? 128 : wide_zw_max((int)dk);
    return (dv + zw - 1) / zw;
}
static int64_t slices(int64_t dk, int64_t dv, bool wide) { return wide ? wide_slices(dk, dv) : (dv + 63) / 64; }
static double warm_up_frac(int64_t wgs, int64_t nblk) {
    static const double frac[9] = {1.0, 1.0, 0.77, 0.71, 0.68, 0.67, 0.66, 0.66, 0.66};
    return frac[warm_up_chunks(wgs, nblk)];
}
static double warm_up_us(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, bool wide) {
    const int64_t nblk = (n + 63) / 64, wgs = (bh + 7) / 8 * 8 * slices(dk, dv, wide) * nprod;
    return warm_up_frac(wgs, nblk) * (double)nblk * block_us(dk, wide);
}

static ScanPlan plan_scan(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, bool wide, const Opts& opts) {
    const ScanPlan none = {1, 0, 0, warm_up_us(bh, n, dk, dv, nprod, wide)};
    ScanPlan pl = none;
    if (opts.scan == LA_OPT_OFF) return none;
    const int forced = opts.chunks;
    const int64_t nblk = (n + 63) / 64, cus = num_cus();
    const int64_t nslice = slices(dk, dv, wide);
    const int64_t wgs = (bh + 7) / 8 * 8 * nslice * nprod;
    int64_t c = 1;
    if (forced > 0) c = forced;
    else if (wgs * 2 <= cus) {
        c = cus / wgs;
        if (c > nblk / 4) c = nblk / 4;  // at least four blocks per chunk
    }
    if (c > 64) c = 64;
    if (c > nblk) c = nblk;
    if (c < 2) return none;
    pl.chunk_len = (int)((nblk + c - 1) / c);
    pl.us = 1.5 * pl.chunk_len * block_us(dk, wide) + 16.0 + 10.0;
    if (forced <= 0 && pl.us >= none.us) return none;
    pl.nchunk = (int)((nblk + pl.chunk_len - 1) / pl.chunk_len);  // no empty chunk
    if (pl.nchunk < 2 || bh * nprod * nslice > 65535) return none;
    pl.bytes = (size_t)(bh * nprod * nslice) * (size_t)(pl.nchunk - 1) * pipe_state_floats((int)dk, wide) * sizeof(float);
    return pl;
}

// The pipelined kernel can give each workgroup 128 columns of z / out instead of 64: the score tile
// and the x / y tiles are then produced once per 128 output columns, and the power-limited kernel
// turns the saved work into time (dK + dV at the headline shape: 0.31 against 0.415 ms) - as long
// as there are workgroups enough.  A 128-column workgroup takes about 1.25 times as long as a
// 64-column one, and there are half as many: compare the rounds of workgroups the chip has to run.
// `scratch`: bytes of workspace the caller has.  opts.wide overrides the choice.
static bool wide_columns(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, size_t scratch, const Opts& opts) {
    if (dk > 128) {
        // Two-barrier kernels: 96- / 128-column workgroups (la_sweep_wide.hip) where that makes fewer slices.
        // They pay when the 64-column form needs more rounds of workgroups than the chip has CUs for
        // (a wide workgroup takes about 1.4 times as long); with few sequences the 64-column form has
        // more workgroups to spread over the CUs and stays.
        const int64_t ws = wide_slices(dk, dv), ns = (dv + 63) / 64;
        if (ws >= ns) return false;
        if (opts.wide != LA_OPT_AUTO) return opts.wide == LA_OPT_ON;
        const int64_t cus = num_cus(), units = (bh + 7) / 8 * 8 * nprod, wide = units * ws, narrow = units * ns;
        if (narrow <= cus) return false;
        return (wide + cus - 1) / cus * 7 < (narrow + cus - 1) / cus * 5;
    }
    if (dv <= 64 || dv > 128) return false;
    if (opts.wide != LA_OPT_AUTO) return opts.wide == LA_OPT_ON;
    if (dk <= 64) return false;  // the 128-column form pads the feature dim to 128
    const int64_t cus = num_cus(), wide = (bh + 7) / 8 * 8 * nprod, narrow = 2 * wide;
    if (narrow <= cus) {
        // Every 64-column workgroup gets a CU of its own.  With so few of them that a long walk is cut
        // into chunks from scanned states, rather half as many workgroups of 128 columns and twice the chunks
        // (b1 h32 n8192 fwd+bwd 0.28 against 0.34 ms, b1 h4 n65536 0.46 against 0.62).
        if (narrow * 2 > cus) return false;
        const ScanPlan w = plan_scan(bh, n, dk, dv, nprod, true, opts), nw = plan_scan(bh, n, dk, dv, nprod, false, opts);
        return w.nchunk > 1 && w.bytes <= scratch && w.us < (nw.bytes <= scratch ? nw.us : warm_up_us(bh, n, dk, dv, nprod, false));
    }
    return (wide + cus - 1) / cus * 5 < (narrow + cus - 1) / cus * 4;
}

// Workspace the kernels can use for one launch of nprod sweeps (0: none).
size_t sweep_workspace_bytes(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, int dtype, const Opts& opts) {
    if (dtype != LA_BF16 && dtype != LA_FP16) return 0;
    return plan_scan(bh, n, dk, dv, nprod, wide_columns(bh, n, dk, dv, nprod, (size_t)-1, opts), opts).bytes;
}

static int launch_planned(SweepPair& p, int64_t bh, int64_t n, int64_t dk, int64_t dv, int dtype, bool reverse, void* ws,
                          size_t ws_bytes, const Opts& opts, hipStream_t st) {
    const bool ws_ok = ws && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
    p.wide = wide_columns(bh, n, dk, dv, p.nprod, ws_ok ? ws_bytes : 0, opts) ? 1 : 0;
    p.mode = kWarmUp;
    p.chunk_len = 0;
    p.state = nullptr;
    for (int i = 0; i < p.nprod; ++i)
        if (p.wide) {
            const int64_t ws = wide_slices(dk, dv);
            p.a[i].nslice = (int)ws;
            // equal slices, a whole number of 32-column state waves each
            p.a[i].zw = dk <= 128 ? 128 : (int)(((dv + ws - 1) / ws + 31) / 32 * 32);
        }
    const ScanPlan pl = plan_scan(bh, n, dk, dv, p.nprod, p.wide != 0, opts);
    if (pl.nchunk > 1 && ws_ok && ws_bytes >= pl.bytes) {
        p.mode = kCollect;  // sweep_pipe runs the three launches
        p.chunk_len = pl.chunk_len;
        p.state = static_cast<float*>(ws);
        for (int i = 0; i < p.nprod; ++i) {
            p.a[i].nchunk = pl.nchunk;
            for (int j = 0; j < 9; ++j) p.a[i].chunk_start[j] = 0;
        }
    } else {
        choose_chunks(p.a[0], p.nprod, opts);
        for (int i = 1; i < p.nprod; ++i) {
            p.a[i].nchunk = p.a[0].nchunk;
            for (int j = 0; j < 9; ++j) p.a[i].chunk_start[j] = p.a[0].chunk_start[j];
        }
    }
    if (p.nprod == 1) p.a[1] = p.a[0];
    if (dk <= 128) return sweep_pipe(p, dtype, reverse, st);  // pipelined kernel, la_sweep_pipe.hip
    if (p.wide) return sweep_wide(p, dtype, reverse, st);     // 96- / 128-column workgroups, la_sweep_wide.hip
    return launch_classic(p, dtype, reverse, st);
}

// x,y: (b,h,n,dk)  z,out: (b,h,n,dv), each with its own batch / head / token strides
int sweep(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
          bool reverse, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st) {
    SweepPair p;
    p.nprod = 1;
    p.a[0] = make_args(io, s, bh, h, n, dk, dv);
    return launch_planned(p, bh, n, dk, dv, dtype, reverse, ws, ws_bytes, opts, st);
}

// States a forward sweep can leave behind for the sweep that follows it over the same tensors in swapped roles.
// O = sweep(q, k, v) carries the state K^T V (d x e); dQ = sweep(dO, v, k) of the backward pass carries V^T K,
// its transpose.  Where the forward pass walks each sequence in one piece and leaves the state at c - 1
// equally spaced block boundaries, the dQ sweep can run as c chunks per sequence from those states - no
// warm-up blocks, no collect and scan launches - and so in 128-column workgroups where 64-column ones
// would otherwise be needed to give every CU a workgroup (b*h around 128 on a 256-CU chip).
// nchunk == 1: not for this shape.
SavedPlan plan_saved(int64_t bh, int64_t n, int64_t d, int64_t e, int dtype, const Opts& opts) {
    const SavedPlan none = {1, 0, 0};
    if (dtype != LA_BF16 && dtype != LA_FP16) return none;
    if (d <= 64 || d > 128 || e > 128) return none;
    if (opts.chunks != 0 || opts.wide == LA_OPT_ON || opts.scan == LA_OPT_ON) return none;
    const int64_t nblk = (n + 63) / 64, cus = num_cus(), units8 = (bh + 7) / 8 * 8;
    // the forward pass as planned: 64-column workgroups, one walk per sequence
    if (wide_columns(bh, n, d, e, 1, (size_t)-1, opts)) return none;
    if (plan_scan(bh, n, d, e, 1, false, opts).nchunk > 1) return none;
    if (warm_up_chunks(units8 * ((e + 63) / 64), nblk) > 1) return none;
    // dQ: one 128-column workgroup per sequence and chunk
    int64_t c = cus / units8;
    if (c > nblk / 4) c = nblk / 4;
    if (c > 64) c = 64;
    if (c < 2) return none;
    SavedPlan pl;
    pl.chunk_len = (int)((nblk + c - 1) / c);
    pl.nchunk = (int)((nblk + pl.chunk_len - 1) / pl.chunk_len);
    if (pl.nchunk < 2) return none;
    // against what the dQ sweep would take by its own plan
    const bool wide = wide_columns(bh, n, e, d, 1, (size_t)-1, opts);
    const ScanPlan own = plan_scan(bh, n, e, d, 1, wide, opts);
    const double own_us = own.nchunk > 1 ? own.us : warm_up_us(bh, n, e, d, 1, wide);
    if ((double)pl.chunk_len * block_us(e, true) >= own_us) return none;
    pl.bytes = (size_t)bh * (size_t)(pl.nchunk - 1) * (size_t)(d * e) * sizeof(float);
    return pl;
}

// The forward sweep as sweep() plans it where plan_saved applies, leaving its state every save_len blocks in `save`.
int sweep_saving(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
                 float* save, int save_len, hipStream_t st) {
    SweepPair p;
    p.nprod = 1;
    p.a[0] = make_args(io, s, bh, h, n, dk, dv);
    p.a[0].nchunk = 1;
    p.a[0].chunk_start[0] = 0;
    for (int j = 1; j < 9; ++j) p.a[0].chunk_start[j] = (int)((n + 63) / 64);
    p.a[1] = p.a[0];
    p.wide = 0;
    p.mode = kWarmUp;
    p.chunk_len = 0;
    p.state = nullptr;
    p.save = save;
    p.save_len = save_len;
    return sweep_pipe(p, dtype, false, st);
}

// The sweep (x, y, z) -> out in nchunk chunks of chunk_len blocks that start from `saved`: what sweep_saving over
// (., z, y) left behind (per sequence nchunk - 1 row-major dv x dk matrices).  128-column workgroups.
int sweep_resumed(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
                  const float* saved, int nchunk, int chunk_len, hipStream_t st) {
    if (dk > 128 || dv > 128 || nchunk < 2 || chunk_len < 1) return LA_E_UNSUPPORTED;
    SweepPair p;
    p.nprod = 1;
    p.a[0] = make_args(io, s, bh, h, n, dk, dv);
    p.a[0].nslice = 1;
    p.a[0].zw = 128;
    p.a[0].nchunk = nchunk;
    for (int j = 0; j < 9; ++j) p.a[0].chunk_start[j] = 0;
    p.a[1] = p.a[0];
    p.wide = 1;
    p.mode = kResume;
    p.chunk_len = chunk_len;
    p.state = const_cast<float*>(saved);
    return sweep_pipe(p, dtype, false, st);
}

// Two sweeps of the same shape and direction in one launch.
int sweep2(const SweepIO& io0, const SweepIO& io1, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv,
           int dtype, bool reverse, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st) {
    if (opts.paired == LA_OPT_OFF) {  // for measurements: two launches
        const int rc = sweep(io0, s, bh, h, n, dk, dv, dtype, reverse, ws, ws_bytes, opts, st);
        return rc != LA_OK ? rc : sweep(io1, s, bh, h, n, dk, dv, dtype, reverse, ws, ws_bytes, opts, st);
    }
    SweepPair p;
    p.nprod = 2;
    p.a[0] = make_args(io0, s, bh, h, n, dk, dv);
    p.a[1] = make_args(io1, s, bh, h, n, dk, dv);
    return launch_planned(p, bh, n, dk, dv, dtype, reverse, ws, ws_bytes, opts, st);
}

// The three sweeps of a backward pass with d == e (dQ forward; dK, dV reverse, paired) in ONE launch,
// where that is the faster way: they fit on the chip together, so they run side by side, each cut into
// the warm-up chunks the CUs left over allow.  Results are bit-identical to separate launches.
// Returns LA_E_UNSUPPORTED when separate launches are to be used (they are estimated faster - scanned
// chunk states on a long walk -, or the sweeps fill the chip anyway).  opts.once = LA_OPT_OFF / LA_OPT_ON:
// never / whenever possible.
int sweep_bwd_once(const SweepIO& dq, const SweepIO& dk, const SweepIO& dv, const float* s, int64_t bh, int64_t h, int64_t n,
                   int64_t d, int dtype, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st) {
    if (dtype != LA_BF16 && dtype != LA_FP16) return LA_E_UNSUPPORTED;
    const int forced = opts.once == LA_OPT_ON ? 1 : opts.once == LA_OPT_OFF ? -1 : 0;
    if (forced < 0 || opts.paired == LA_OPT_OFF) return LA_E_UNSUPPORTED;
    if (forced == 0 && opts.wide == LA_OPT_ON) return LA_E_UNSUPPORTED;  // 128-column workgroups asked for
    const int64_t cus = num_cus(), nblk = (n + 63) / 64, nslice = (d + 63) / 64;
    const int64_t wgs = (bh + 7) / 8 * 8 * nslice * 3;  // one chunk each
    if (forced == 0) {
        if (wgs > cus) return LA_E_UNSUPPORTED;
        // what the separate launches would take, by the estimates behind their own plans
        const bool ws_ok = ws && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
        double separate = 0.0;
        for (int nprod = 1; nprod <= 2; ++nprod) {
            const bool wide = wide_columns(bh, n, d, d, nprod, ws_ok ? ws_bytes : 0, opts);
            const ScanPlan pl = plan_scan(bh, n, d, d, nprod, wide, opts);
            separate += pl.nchunk > 1 && ws_ok && ws_bytes >= pl.bytes ? pl.us : warm_up_us(bh, n, d, d, nprod, wide);
        }
        // here: the longest workgroup of 3 * wgs/3 * c warm-up chunked ones
        if (warm_up_frac(wgs, nblk) * (double)nblk * block_us(d, false) >= separate) return LA_E_UNSUPPORTED;
    }
    SweepBoth b;
    b.fwd.nprod = 1;
    b.fwd.a[0] = make_args(dq, s, bh, h, n, d, d);
    b.rev.nprod = 2;
    b.rev.a[0] = make_args(dk, s, bh, h, n, d, d);
    b.rev.a[1] = make_args(dv, s, bh, h, n, d, d);
    for (SweepPair* p : {&b.fwd, &b.rev}) {
        p->wide = 0;
        p->mode = kWarmUp;
        p->chunk_len = 0;
        p->state = nullptr;
    }
    // the same chunks for every sweep: what all of them together leave room for
    choose_chunks(b.fwd.a[0], 3, opts);
    b.fwd.a[1] = b.fwd.a[0];
    for (int i = 0; i < 2; ++i) {
        b.rev.a[i].nchunk = b.fwd.a[0].nchunk;
        for (int j = 0; j < 9; ++j) b.rev.a[i].chunk_start[j] = b.fwd.a[0].chunk_start[j];
    }
    b.nfwd = part_grid(b.fwd);
    if (d <= 128) return sweep_pipe_both(b, dtype, st);
    if (dtype == LA_BF16) return launch_both<__bf16>(b, st);
    return launch_both<_Float16>(b, st);
}

// The same for two sweeps of one shape and opposite directions (dQ and dK of a backward pass with
// d != e: both contract over e and produce d columns): one launch where they fit on the chip together
// and separate launches are not estimated faster; LA_E_UNSUPPORTED otherwise.
int sweep_fwd_rev_once(const SweepIO& fwd, const SweepIO& rev, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk,
                       int64_t dv, int dtype, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st) {
    if (dtype != LA_BF16 && dtype != LA_FP16) return LA_E_UNSUPPORTED;
    const int forced = opts.once == LA_OPT_ON ? 1 : opts.once == LA_OPT_OFF ? -1 : 0;
    if (forced < 0 || opts.paired == LA_OPT_OFF) return LA_E_UNSUPPORTED;
    if (forced == 0 && opts.wide == LA_OPT_ON) return LA_E_UNSUPPORTED;
    const int64_t cus = num_cus(), nblk = (n + 63) / 64, nslice = (dv + 63) / 64;
    const int64_t wgs = (bh + 7) / 8 * 8 * nslice * 2;
    if (forced == 0) {
        if (wgs > cus) return LA_E_UNSUPPORTED;
        const bool ws_ok = ws && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
        const bool wide = wide_columns(bh, n, dk, dv, 1, ws_ok ? ws_bytes : 0, opts);
        const ScanPlan pl = plan_scan(bh, n, dk, dv, 1, wide, opts);
        const double separate = 2.0 * (pl.nchunk > 1 && ws_ok && ws_bytes >= pl.bytes ? pl.us : warm_up_us(bh, n, dk, dv, 1, wide));
        if (warm_up_frac(wgs, nblk) * (double)nblk * block_us(dk, false) >= separate) return LA_E_UNSUPPORTED;
    }
    SweepBoth b;
    b.fwd.nprod = b.rev.nprod = 1;
    b.fwd.a[0] = make_args(fwd, s, bh, h, n, dk, dv);
    b.rev.a[0] = make_args(rev, s, bh, h, n, dk, dv);
    choose_chunks(b.fwd.a[0], 2, opts);
    b.rev.a[0].nchunk = b.fwd.a[0].nchunk;
    for (int j = 0; j < 9; ++j) b.rev.a[0].chunk_start[j] = b.fwd.a[0].chunk_start[j];
    for (SweepPair* p : {&b.fwd, &b.rev}) {
        p->a[1] = p->a[0];
        p->wide = 0;
        p->mode = kWarmUp;
        p->chunk_len = 0;
        p->state = nullptr;
    }
    b.nfwd = part_grid(b.fwd);
    if (dk <= 128) return sweep_pipe_both(b, dtype, st);
    if (dtype == LA_BF16) return launch_both<__bf16>(b, st);
    return launch_both<_Float16>(b, st);
}

}  // namespace la
