// Single-sweep decayed linear attention for gfx950: the software-pipelined kernel body, one workgroup
// barrier per step, for feature dims up to 256.  Included by la_sweep_pipe.hip (feature dim <= 128) and
// la_sweep_pipe_split.hip (129 .. 256), which instantiate it.
//
// One workgroup of 8 wavefronts per (batch, head, slice of 64, 128 or up to 192 columns of z/out), 64-token blocks
// walked in order, fp32 state in MFMA accumulators.  The two kinds of wavefronts work on different
// data at the same time:
//   waves 0-3 ("score" waves)  do all the memory traffic (two register sets of prefetch, the tiles
//                              published in LDS two steps ahead, the output tile of the block before
//                              written back) and compute the masked, decayed score tile P one step
//                              ahead of the state waves;
//   waves 4-7 ("state" waves)  own one, two or three dk x 16 column slabs of the state and finish the
//                              block: out^T = Lout * (state^T x^T) + z^T P^T, left in LDS, then
//                              state = lam^64 state + y^T (z * Lupd).
// A step is a block (NF = 1, feature dim <= 128) or one of the NF = 2 halves of the feature dim of a
// block (<= 256): the x / y tiles of three blocks of 192 or 256 features do not fit the 160 KB of LDS,
// tiles of half the features do.  Everything that contracts over the feature dim (the score tile, the
// inter-block term) is accumulated over the halves in registers; the state update of a half needs
// the y tile of that half only.  So per step the inter-block term never leaves registers, the state
// waves' serial chain holds no memory instructions, and a single barrier orders
//   - the x/y tiles: three LDS buffers (step s read by the state waves, step s+1 read by the score
//     waves, step s+2 being written);
//   - the P tiles: two LDS buffers (one read, one written);
//   - the output tile of a block, which the state waves write over the z columns they alone read
//     and which leaves for memory as whole row segments when that z slot is refilled.
// NH = 3 (feature dims and column counts of 129 .. 192): a workgroup covers all (up to 192) columns of a sequence,
// every state wave owning three 16-column slabs = 144 accumulator registers of state.  The x and y tiles are then
// staged and multiplied into a score tile once per sequence and block instead of twice, and read from LDS by four
// state waves instead of six (three in each of two 96-column workgroups).  To fit 256 registers the state waves
// fetch their fragments without look-ahead and keep their decay factors in LDS (LEAN below).
// With few (batch, head) sequences the walk is cut into chunks, one workgroup each.  A chunk's
// incoming state comes either from warm-up blocks (the workgroup first walks everything before its
// chunk with the state update alone) or, given a workspace, from a scan: the same kernel run once in
// "collect" mode (every chunk's own blocks, state update alone, end state written out), a small scan
// kernel, and the kernel again in "apply" mode (state read in, the chunk walked for good).
// The chip runs this kernel at its socket power limit, so what counts is the work per output
// element (LDS traffic above all), not the length of any dependency chain: hence the 128-column
// form wherever the launch still has a workgroup for every CU.
// (lightning_attn/ops/triton/lightning_attn2.py:8-85 forward, :88-395 backward.)
#pragma once
#include <type_traits>

#include "la_sweep_common.h"
#include "lightning_attn_hip.h"

namespace la {

// DKP: feature dim as padded; NF: halves it is processed in; NH: 16-column accumulator slabs per state
// wave (a workgroup covers 64 NH columns of z / out; NH = 3 with DKP = 192 only).
template <int DKP, int NF, int NH>
struct PipeLds {
    static_assert(NF == 1 || NF == 2, "one or two feature chunks");
    static constexpr int DKH = DKP / NF;         // features per chunk
    static constexpr int XS = DKH + 16;          // row stride (elements) of the x / y chunk tiles
    static constexpr int ZS = 64 * NH + 8;       // row stride of the z slice
    // z / out slots: one per tile buffer where a block is a step and the slice is narrow; else two,
    // by the parity of the block
    static constexpr int NZ = (NF == 1 && NH == 1) ? 3 : 2;
    static constexpr int PS = 64 + 8;            // row stride of the P tile
    static constexpr int XY = 2 * 64 * XS;       // elements of one x + y buffer
    static constexpr int ZT = 64 * ZS;           // elements of one z buffer
    static constexpr int PT = 64 * PS;           // elements of one P buffer
    // three slabs per state wave: the state waves' decay factors live in LDS, not in registers (512 bytes)
    static constexpr size_t CF = NH > 2 ? 512 : 0;
    static constexpr size_t bytes(size_t elt) { return (size_t)(3 * XY + NZ * ZT + 2 * PT) * elt + CF; }
};

// DENSE: all four tensors are plain (b, h, n, d) arrays; their rows then take a shorter addressing path
// (see load_step).
// `bid`: number of the workgroup within its part of the launch.
// SILU: x, y and z pass through SiLU on their way from memory into LDS (the attention block's activation on
// q, k, v, examples/module/tnl_attn.py:51-54, fused into the forward pass).
template <typename T, int DKP, int NF, int NH, bool REVERSE, bool DECAY, bool DENSE, bool SILU = false>
__device__ __forceinline__ void sweep_pipe_body(const SweepPair& pair, const unsigned bid) {
    typedef Mma<T> M;
    typedef typename M::V8 V8;
    typedef typename M::V4 V4;
    typedef PipeLds<DKP, NF, NH> L;
    constexpr int XS = L::XS, ZS = L::ZS, PS = L::PS, DKH = L::DKH;
    constexpr int KSH = DKH / 32;  // 32-wide contraction steps over one feature chunk
    constexpr int KTH = DKH / 16;  // 16-row state tiles of one feature chunk
    constexpr int KT = DKP / 16;   // 16-row state tiles
    // Threads that fetch, publish and write back the tiles: the 256 of the score waves, which have
    // slack; the state waves' serial chain then holds no memory instructions at all.
    constexpr int NL = 256;
    constexpr int CPX = DKH / 8;             // 16-byte chunks per row of an x / y chunk tile
    constexpr int XC = 64 * CPX / NL;        // ... per loader thread
    constexpr bool ROWAL = NL % CPX == 0;    // a thread's chunks lie a whole number of rows apart
    constexpr int ZW = 64 * NH;              // columns of z / out per workgroup
    constexpr int CPR = ZW / 8;              // 16-byte chunks per row of the z slice
    constexpr int ZC = 64 * CPR / NL;        // chunks per loader thread for the z slice / the output tile
    constexpr bool ZAL = NL % CPR == 0;      // ... which lie a whole number of rows apart (not so at 192 columns)
    constexpr int ZROWS = NL / CPR;          // rows between two of them
    constexpr int NZ = L::NZ;
    // NF = 1, NH = 2: there is room for two z slots only, so the z slice of a block is published one
    // iteration later than its x / y tiles (it is first needed one iteration later, too) and
    // travels one register set behind them.  NF = 2: the z slice travels with the first feature
    // chunk of its block and is published a block ahead.
    constexpr int ZLAG = (NF == 1 && NH == 2) ? 1 : 0;
    constexpr bool TOGETHER = NF == 2 && NH == 3;  // see the load slot of `iteration`
    // Cache policy of the global accesses.  Every tile is needed once per workgroup, and the only second readers
    // are a sibling workgroup that runs beside this one: the other 64-column slice of the head, which reads the same
    // x and y, and the other sweep of a pair, which reads this sweep's y as its z and the other way round.  So the
    // output and the z slice are streamed (nt), and so is x where no slice shares it (128-column workgroups); y stays
    // cached: it is the first of the two touches of a tensor a pair shares (the z slice of a block is fetched one
    // step after its x / y tiles), so the sibling's streamed z read finds it in L2 - and with all four streamed
    // every launch measured slower than with none.  Measured at b4 h32 n8192 d128, ms: la_fwd (64 columns) 0.2253 all
    // cached, 0.2207 as here, 0.2153 with x streamed as well - at 1.137 instead of 1.077 GB of HBM traffic, the
    // sibling slice's read of x then missing L2 now and then: not taken; dQ in 128-column workgroups 0.2078 -> 0.190;
    // dK + dV 0.315 -> 0.302 at 1.616 instead of 1.63 - 1.75 GB.  (A kernel that only streams this access pattern: 5.3 TB/s
    // with cached, 5.9 TB/s with streamed accesses.)  At feature dims above 128 the launches in 64- and 96- / 128-column
    // workgroups are bound by LDS work and the policy made no difference: left cached.  With all columns in one
    // workgroup (NH = 3) they come near the memory side's limit for tiles fetched in half rows (4.6 - 4.8 TB/s for
    // a kernel that only streams that pattern): there the output is streamed, x and y stay cached (the 128-byte
    // line in the middle of a 384-byte row belongs to both halves; with TOGETHER they are asked for in one load
    // slot, and streamed they still lost: la_bwd_saved 0.881 against 0.872 ms at b4 h32 n8192 d192), and
    // z is streamed only when walking forward - walking backward the launch is a dK + dV pair, whose z reads are
    // the sibling sweep's y reads of the same moment (b4 h32 n8192 d192: 2.42 instead of 2.74 GB per launch).
    constexpr bool STREAMS = NF == 1 || NH == 3;  // the forms that come near the memory system's limit
    constexpr int PX = (NF == 1 && NH == 2) ? kStream : kCached;
    constexpr int PY = kCached;
    constexpr int PZ = (NF == 1 || (NH == 3 && !REVERSE)) ? kStream : kCached;
    constexpr int PO = STREAMS ? kStream : kCached;
    extern __shared__ __align__(16) unsigned char smem[];
    // LDS map in bytes: [3][x 64*XS | y 64*XS] tiles, [NZ][64*ZS] z tiles, [2][64*PS] P tiles.
    // All LDS accesses below are written as (per-step base register) + (compile-time
    // constant), which the DS instructions take as register + immediate offset; the bases are
    // made opaque to the optimiser once per step so that it does not keep one address
    // register per access alive across the loop.
    constexpr unsigned E = (unsigned)sizeof(T);
    constexpr unsigned XYB = L::XY * E, ZTB = L::ZT * E, PTB = L::PT * E, YOFF = 64 * XS * E;
    constexpr unsigned ZBASE = 3 * XYB, PBASE = ZBASE + NZ * ZTB;
    constexpr unsigned CFBASE = PBASE + 2 * PTB;  // (NH = 3) float upd[4][16] by lane group g, float out[16][4] by lane row r
    auto opaque = [](unsigned v) {
        asm volatile("" : "+v"(v));
        return v;
    };
    auto ld8 = [&](unsigned addr) { return *reinterpret_cast<const V8*>(smem + addr); };
    auto ld4 = [&](unsigned addr) { return *reinterpret_cast<const V4*>(smem + addr); };
    auto ldt = [&](unsigned addr) { return lds_tr4<V4>(smem + addr); };

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
    // this workgroup's columns of z / out: [col0, colend); a slice may be narrower than the ZW columns LDS holds
    const int col0 = slice * a.zw;
    const int colend = min(dv, col0 + a.zw);
    const int cbase = 16 * NH * w;  // first of this state wave's 16 NH columns within the slice
    const bool cols_active = (col0 + cbase) < colend;

    float rate = 0.f;
    if (DECAY) rate = a.s[unit % a.h];

    // ---- score waves: the tiles of this wave ------------------------------------
    TileDeal deal = kDeal[w];
    if (REVERSE) {
        deal.itA = 3 - deal.itA; deal.jt0 = 3 - deal.jt0;
        if (deal.itB >= 0) { deal.itB = 3 - deal.itB; deal.jt1 = 3 - deal.jt1; deal.jt2 = 3 - deal.jt2; }
    }
    const int itA = __builtin_amdgcn_readfirstlane(deal.itA), jt0 = __builtin_amdgcn_readfirstlane(deal.jt0);
    const int itB = __builtin_amdgcn_readfirstlane(deal.itB), jt1 = __builtin_amdgcn_readfirstlane(deal.jt1);
    const int jt2 = __builtin_amdgcn_readfirstlane(deal.jt2);
    // Per-lane constant factors (all <= 1); the two kinds of waves keep theirs in the same registers.
    //   score waves: cf[4 sl + v]  mask * decay of element v of score tile slot sl
    //   state waves: cf[it]        scale of the inter-block term for token i = 16 it + r
    //                cf[4 + 8 ks + u]  scale of token j = 32 ks + 8 g + u in the state update
    float cf[20];
#pragma unroll
    for (int i = 0; i < 20; ++i) cf[i] = 1.f;
    float lamB = 1.f;
    if (!state_role) {
        const int its[3] = {itA, itB, itB}, jts[3] = {jt0, jt1, jt2};
#pragma unroll
        for (int sl = 0; sl < 3; ++sl)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int i = 16 * its[sl] + r, j = 16 * jts[sl] + 4 * g + v;
                const int diff = REVERSE ? (j - i) : (i - j);
                cf[4 * sl + v] = diff >= 0 ? (DECAY ? expf(-rate * (float)diff) : 1.f) : 0.f;
            }
    }
    if (state_role && DECAY) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int i = 16 * it + r;
            cf[it] = expf(-rate * (float)(REVERSE ? 64 - i : i));
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = 32 * ks + 8 * g + u;
                cf[4 + 8 * ks + u] = expf(-rate * (float)(REVERSE ? j : 64 - j));
            }
        lamB = expf(-rate * 64.f);
        if constexpr (NH > 2) {
            // the factors go to LDS (the same for every state wave; read back where they are used, after the barriers
            // that precede the walk)
            if (w == 0) {
                float* const t = reinterpret_cast<float*>(smem + CFBASE);
                if (r == 0) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) t[16 * g + i] = cf[4 + i];
                }
                if (g == 0) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) t[64 + 4 * r + i] = cf[i];
                }
            }
        }
    }

    f32x4 st[NH][KT];  // the state; zeroed where the state waves start their walk

    const int64_t nblk = (n + 63) / 64;
    // Sequence chunking: this workgroup produces the blocks [it_first, it_end) of the walk.  It
    // first runs over the blocks before it_first with the state update only ("warm-up": y and z
    // are read, nothing is written) to rebuild the state its chunk starts from.
    // With a workspace (pair.mode != kWarmUp) the chunks are equally long and a workgroup walks its own
    // chunk only: first with the state update alone, from zero, to leave the state it ends with
    // (kCollect), then - a scan kernel having combined those into the state at the start of every
    // chunk - for good, from that state (kApply).
    const int mode = pair.mode;
    const int nchunk = pair.a[0].nchunk;
    if (mode == kCollect && chunk == nchunk - 1) return;  // nobody needs the state after the last chunk
    const int64_t cbeg = mode == kWarmUp ? (int64_t)a.chunk_start[chunk] : min((int64_t)chunk * pair.chunk_len, nblk);
    const int64_t cend = mode == kWarmUp ? (int64_t)a.chunk_start[chunk + 1] : min((int64_t)(chunk + 1) * pair.chunk_len, nblk);
    const int64_t it0 = mode == kWarmUp ? 0 : cbeg;           // first block this workgroup walks
    const int64_t it_first = mode == kCollect ? cend : cbeg;  // first block whose output it produces
    const int64_t it_end = cend;
    // the state slot of this workgroup's chunk: [unit][sweep][slice][chunk 0 .. nchunk-2][state waves' accumulators]
    constexpr size_t SF = (size_t)4 * NH * KT * 64 * 4;
    float* const slot0 = pair.state + ((((size_t)unit * nprod + sub % nprod) * nslice + slice) * (size_t)(nchunk - 1)) * SF;

    u32x4 xrA[XC], yrA[XC], zrA[ZC], xrB[XC], yrB[XC], zrB[ZC];

    // Per-lane byte offsets of this thread's first 16-byte chunk inside a 64-token block (out of
    // range where the chunk lies in the zero padding dk..DKP-1 or beyond dv).  Where a row of a
    // chunk tile holds a power-of-two number of chunks (ROWAL), a thread's further chunks lie a
    // whole number of rows below, so they and the block's first token go into the wave-uniform
    // offset of the load; otherwise (96 features: 12 chunks per row) every chunk has a row and a
    // column of its own.
    constexpr int CROWS = ROWAL ? NL / CPX : 1;  // rows between two chunks of a thread
    const int lane_row = tid / CPX, lane_col = (tid % CPX) * 8;
    const int lane_zrow = tid / CPR, lane_zcol = col0 + (tid % CPR) * 8;
    const unsigned lane_z = lane_zcol < colend ? (lane_zrow * zts + lane_zcol) * (unsigned)sizeof(T) : kOob;
    // chunk u of this thread in the z slice / the output tile: row within the block, first column, element offset in
    // the LDS slot (not ZAL: 24 chunks per row, every chunk with a row and a column of its own)
    auto z_row = [&](int u) { return ZAL ? lane_zrow + ZROWS * u : (tid + NL * u) / CPR; };
    auto z_col = [&](int u) { return ZAL ? lane_zcol : col0 + ((tid + NL * u) % CPR) * 8; };
    auto z_lds = [&](int u) { return (unsigned)(z_row(u) * ZS + (z_col(u) - col0)) * (unsigned)sizeof(T); };
    // Fetches feature chunk HC of block number b of the walk and, with its first chunk, the z slice
    // that travels with it.  Blocks at or beyond it_end, and the x tile of warm-up blocks, are fetched
    // at the out-of-range offset: zeros, no memory traffic, and the loads are issued unconditionally
    // (no branches, no draining `s_waitcnt vmcnt(0)` at joins).
    auto load_step = [&](auto hc, int64_t b, u32x4 (&xr)[XC], u32x4 (&yr)[XC], u32x4 (&zr)[ZC]) __attribute__((always_inline)) {
        constexpr int HC = decltype(hc)::value;
        constexpr int FC0 = HC * DKH;  // first feature of the chunk
        const int64_t t = REVERSE ? nblk - 1 - b : b;
        const bool valid = b < it_end, need_x = valid && b >= it_first;
        // the z slice that travels with this block's x / y tiles
        const int64_t bz = b - ZLAG, tz = REVERSE ? nblk - 1 - bz : bz;
        const bool validz = bz >= it0 && bz < it_end;
        if (DENSE) {
            // Plain tensors: one per-lane offset, rows >= n fall outside the buffer and the hardware
            // range check zeroes them.  Kept as its own code path because it is measurably faster
            // (3 % per launch at b4 h32 n8192 d128) than the general form below, whose explicit row
            // mask changes nothing in the memory traffic.
            const unsigned tok0 = (unsigned)(t * 64);
#pragma unroll
            for (int u = 0; u < XC; ++u) {
                const int c = tid + NL * u;
                const int row = c / CPX, col = FC0 + (c % CPX) * 8;
                const unsigned off = col < dk ? ((tok0 + row) * (unsigned)dk + col) * (unsigned)sizeof(T) : kOob;
                xr[u] = buf_load16p<PX>(xb, need_x ? off : kOob);
                yr[u] = buf_load16p<PY>(yb, valid ? off : kOob);
            }
            if constexpr (HC == 0) {
                const unsigned tokz = (unsigned)(tz * 64);
#pragma unroll
                for (int u = 0; u < ZC; ++u) {
                    const int row = z_row(u), zc = z_col(u);
                    const unsigned off = zc < colend ? ((tokz + row) * (unsigned)dv + zc) * (unsigned)sizeof(T) : kOob;
                    zr[u] = buf_load16p<PZ>(zb, validz ? off : kOob);
                }
            }
            return;
        }
        const unsigned tok0 = valid ? (unsigned)(t * 64) : 0u;
        // rows of this block that exist (0 for a block that is not fetched)
        const int rows = valid ? (int)min(64u, nrows - tok0) : 0, rows_x = need_x ? rows : 0;
        if constexpr (ROWAL) {
            const unsigned lane_x = FC0 + lane_col < dk ? (lane_row * xts + FC0 + lane_col) * (unsigned)sizeof(T) : kOob;
            const unsigned lane_y = FC0 + lane_col < dk ? (lane_row * yts + FC0 + lane_col) * (unsigned)sizeof(T) : kOob;
#pragma unroll
            for (int u = 0; u < XC; ++u) {
                // a wave-uniform offset must stay inside the buffer: 0 when none of these rows exists
                const unsigned tk = u * CROWS < rows ? tok0 + u * CROWS : 0u;
                xr[u] = buf_load16p<PX>(xb, lane_row < rows_x - u * CROWS ? lane_x : kOob, tk * xts * (unsigned)sizeof(T));
                yr[u] = buf_load16p<PY>(yb, lane_row < rows - u * CROWS ? lane_y : kOob, tk * yts * (unsigned)sizeof(T));
            }
        } else {
#pragma unroll
            for (int u = 0; u < XC; ++u) {
                const int c = tid + NL * u;
                const int row = c / CPX, col = FC0 + (c % CPX) * 8;
                const unsigned ox = col < dk ? (row * xts + col) * (unsigned)sizeof(T) : kOob;
                const unsigned oy = col < dk ? (row * yts + col) * (unsigned)sizeof(T) : kOob;
                xr[u] = buf_load16p<PX>(xb, row < rows_x ? ox : kOob, tok0 * xts * (unsigned)sizeof(T));
                yr[u] = buf_load16p<PY>(yb, row < rows ? oy : kOob, tok0 * yts * (unsigned)sizeof(T));
            }
        }
        if constexpr (HC == 0) {
            const unsigned tokz = validz ? (unsigned)(tz * 64) : 0u;
            const int rowsz = validz ? (int)min(64u, nrows - tokz) : 0;
#pragma unroll
            for (int u = 0; u < ZC; ++u) {
                if constexpr (ZAL) {
                    const unsigned tk = u * ZROWS < rowsz ? tokz + u * ZROWS : 0u;
                    zr[u] = buf_load16p<PZ>(zb, lane_zrow < rowsz - u * ZROWS ? lane_z : kOob, tk * zts * (unsigned)sizeof(T));
                } else {
                    const int row = z_row(u), zc = z_col(u);
                    const unsigned oz = zc < colend ? (row * zts + zc) * (unsigned)sizeof(T) : kOob;
                    zr[u] = buf_load16p<PZ>(zb, row < rowsz ? oz : kOob, tokz * zts * (unsigned)sizeof(T));
                }
            }
        }
    };
    const unsigned lane_stage_xy = (lane_row * XS + lane_col) * E;
    const unsigned lane_stage_z = (lane_zrow * ZS + (tid % CPR) * 8) * E;
    // Publishes a fetched step in tile buffer `buf`.  With the first feature chunk of a block goes its
    // z slice, into slot `zslot`.  That slot still holds the output tile of the block that used it
    // last (walk index bout; the state waves leave their columns of `out` there, over the z columns
    // they alone read): every thread first takes the 16 bytes its z chunk is about to replace and,
    // if `flush`, sends them to memory - eight (NH = 2: sixteen) lanes write one whole 128-byte
    // (256-byte) row segment.  (Stored straight from the accumulators, each wave would write 32-byte
    // pieces of every row, which the memory system handles far worse: 0.083 against 0.048 ms for the
    // output traffic alone at b4 h32 n8192 d128.)
    const unsigned lane_o = lane_zcol < colend ? (lane_zrow * ots + lane_zcol) * (unsigned)sizeof(T) : kOob;
    auto store_out = [&](int64_t bout, bool flush, const u32x4 (&o)[ZC]) {
        const int64_t t = REVERSE ? nblk - 1 - bout : bout;
#pragma unroll
        for (int u = 0; u < ZC; ++u) {
            if (DENSE) {
                // rows >= n fall outside the buffer and are dropped by the hardware range check
                const int zc = z_col(u);
                const unsigned off = zc < colend ? (((unsigned)(t * 64) + z_row(u)) * (unsigned)dv + zc) * (unsigned)sizeof(T) : kOob;
                buf_store16p<PO>(ob, flush ? off : kOob, 0u, o[u]);
            } else if constexpr (!ZAL) {
                const unsigned tok0 = flush ? (unsigned)(t * 64) : 0u;
                const int rows = flush ? (int)min(64u, nrows - tok0) : 0;
                const int row = z_row(u), zc = z_col(u);
                const unsigned oo = zc < colend ? (row * ots + zc) * (unsigned)sizeof(T) : kOob;
                buf_store16p<PO>(ob, row < rows ? oo : kOob, tok0 * ots * (unsigned)sizeof(T), o[u]);
            } else {
                const unsigned tok0 = flush ? (unsigned)(t * 64) : 0u;
                const int rows = flush ? (int)min(64u, nrows - tok0) : 0;
                const unsigned tk = u * ZROWS < rows ? tok0 + u * ZROWS : 0u;
                buf_store16p<PO>(ob, lane_zrow < rows - u * ZROWS ? lane_o : kOob, tk * ots * (unsigned)sizeof(T), o[u]);
            }
        }
    };
    auto stage_step = [&](auto hc, int buf, int zslot, const u32x4 (&xr)[XC], const u32x4 (&yr)[XC], const u32x4 (&zr)[ZC], int64_t bout, bool flush) __attribute__((always_inline)) {
        constexpr int HC = decltype(hc)::value;
        // SILU: silu(t) = t / (1 + exp(-t)) in float32, rounded back to the tensors' type; padding stays zero
        auto silu16 = [](u32x4 v) {
            typedef T T8 __attribute__((ext_vector_type(8)));
            T8 t = __builtin_bit_cast(T8, v);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float f = (float)t[i];
                t[i] = (T)(f * __builtin_amdgcn_rcpf(1.f + __expf(-f)));
            }
            return __builtin_bit_cast(u32x4, t);
        };
        const unsigned xd = opaque(buf * XYB + (ROWAL ? lane_stage_xy : 0u));
        const unsigned zd = opaque(ZBASE + zslot * ZTB + (ZAL ? lane_stage_z : 0u));
        auto zoff = [&](int u) { return ZAL ? (unsigned)(u * ZROWS * ZS) * E : z_lds(u); };
        u32x4 o[ZC];
        if constexpr (HC == 0) {
#pragma unroll
            for (int u = 0; u < ZC; ++u) o[u] = *reinterpret_cast<const u32x4*>(smem + zd + zoff(u));
        }
#pragma unroll
        for (int u = 0; u < XC; ++u) {
            if constexpr (ROWAL) {
                // chunk c = tid + NL u lies CROWS rows below chunk tid
                *reinterpret_cast<u32x4*>(smem + xd + u * CROWS * XS * E) = SILU ? silu16(xr[u]) : xr[u];
                *reinterpret_cast<u32x4*>(smem + xd + YOFF + u * CROWS * XS * E) = SILU ? silu16(yr[u]) : yr[u];
            } else {
                const int c = tid + NL * u;
                const unsigned so = xd + ((c / CPX) * XS + (c % CPX) * 8) * E;
                *reinterpret_cast<u32x4*>(smem + so) = SILU ? silu16(xr[u]) : xr[u];
                *reinterpret_cast<u32x4*>(smem + so + YOFF) = SILU ? silu16(yr[u]) : yr[u];
            }
        }
        if constexpr (HC == 0) {
            store_out(bout, flush, o);
#pragma unroll
            for (int u = 0; u < ZC; ++u) *reinterpret_cast<u32x4*>(smem + zd + zoff(u)) = SILU ? silu16(zr[u]) : zr[u];
        }
    };

    // Score waves: the part of this wave's S^T tiles that feature chunk HC contributes, for the block
    // whose chunk lies in tile buffer `buf`; with the last chunk the masked, decayed P[i][j] goes to
    // P buffer `pbuf`.  All fragment reads are issued before the MFMAs (the scheduler otherwise sinks
    // each read next to its use and the wave pays one LDS round trip per MFMA).
    const unsigned lane_frag = (r * XS + 8 * g) * E;   // row r, 16-byte chunk g of an x / y tile
    const unsigned lane_pw = (r * PS + 4 * g) * E;     // P[i = r][j = 4g ..] within a 16 x 16 tile
    f32x4 sacc[3];
    auto score_step = [&](auto hc, int buf, int pbuf) __attribute__((always_inline)) {
        constexpr int HC = decltype(hc)::value;
        const unsigned xbase = buf * XYB + lane_frag, pbase = PBASE + pbuf * PTB + lane_pw;
        if constexpr (HC == 0) {
#pragma unroll
            for (int sl = 0; sl < 3; ++sl) sacc[sl] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
        const unsigned xa = opaque(xbase + 16 * itA * XS * E);
        const unsigned y0 = opaque(xbase + YOFF + 16 * jt0 * XS * E);
        if (itB >= 0) {
            const unsigned xb2 = opaque(xbase + 16 * itB * XS * E);
            const unsigned y1 = opaque(xbase + YOFF + 16 * jt1 * XS * E);
            const unsigned y2 = opaque(xbase + YOFF + 16 * jt2 * XS * E);
            V8 fxa[KSH], fxb[KSH], fy0[KSH], fy1[KSH], fy2[KSH];
#pragma unroll
            for (int ks = 0; ks < KSH; ++ks) {
                fxa[ks] = ld8(xa + 32 * ks * E);
                fy0[ks] = ld8(y0 + 32 * ks * E);
                fxb[ks] = ld8(xb2 + 32 * ks * E);
                fy1[ks] = ld8(y1 + 32 * ks * E);
                fy2[ks] = ld8(y2 + 32 * ks * E);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < KSH; ++ks) {
                sacc[0] = M::mma(fy0[ks], fxa[ks], sacc[0]);
                sacc[1] = M::mma(fy1[ks], fxb[ks], sacc[1]);
                sacc[2] = M::mma(fy2[ks], fxb[ks], sacc[2]);
            }
            __builtin_amdgcn_sched_barrier(0);
        } else {
            V8 fxa[KSH], fy0[KSH];
#pragma unroll
            for (int ks = 0; ks < KSH; ++ks) {
                fxa[ks] = ld8(xa + 32 * ks * E);
                fy0[ks] = ld8(y0 + 32 * ks * E);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < KSH; ++ks) sacc[0] = M::mma(fy0[ks], fxa[ks], sacc[0]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (HC == NF - 1) {
            {
                V4 p;
#pragma unroll
                for (int v = 0; v < 4; ++v) p[v] = M::cvt(sacc[0][v] * cf[v]);
                *reinterpret_cast<V4*>(smem + opaque(pbase + (16 * itA * PS + 16 * jt0) * E)) = p;
            }
            if (itB >= 0) {
                V4 p;
#pragma unroll
                for (int v = 0; v < 4; ++v) p[v] = M::cvt(sacc[1][v] * cf[4 + v]);
                *reinterpret_cast<V4*>(smem + opaque(pbase + (16 * itB * PS + 16 * jt1) * E)) = p;
#pragma unroll
                for (int v = 0; v < 4; ++v) p[v] = M::cvt(sacc[2][v] * cf[8 + v]);
                *reinterpret_cast<V4*>(smem + opaque(pbase + (16 * itB * PS + 16 * jt2) * E)) = p;
            }
        }
    };

    // zero both P buffers once: tiles on the masked side of the diagonal are never written
    for (int c = tid; c < 2 * L::PT / 8; c += 512) reinterpret_cast<uint4*>(smem + PBASE)[c] = make_uint4(0, 0, 0, 0);
    // state-wave lane offsets: x fragment halves (row r, columns 4g..), transposed reads of y and
    // of this wave's 16 z columns (row 8g + r/4, columns 4 (r%4)..), P fragments (row r, chunk g)
    const unsigned lane_xq = (r * XS + 4 * g) * E;
    const unsigned lane_yt = ((8 * g + (r >> 2)) * XS + 4 * (r & 3)) * E;
    const unsigned lane_zt = ((8 * g + (r >> 2)) * ZS + cbase + 4 * (r & 3)) * E;
    const unsigned lane_pr = (r * PS + 8 * g) * E;
    const unsigned lane_ow = (r * ZS + cbase + 4 * g) * E;  // out[i = r][cbase + 4 g ..] within 16 rows

    // Forward walk in one piece with `save`: the state after every save_len blocks but the last goes to memory as
    // a plain dk x dv float matrix (this wave's 16 columns of it; 64-byte runs).  Rare - once per chunk
    // of the pass that will start from it -, so the addresses are made where they are used and nothing of
    // this lives in registers across the loop.
    int64_t next_save = pair.save != nullptr && pair.save_len > 0 && pair.save_len < nblk ? (int64_t)pair.save_len : -1;
    auto save_state = [&](const int64_t it) __attribute__((always_inline)) {
        const int64_t nsave = (nblk - 1) / pair.save_len;  // boundaries per unit
        const int64_t j = (it + 1) / pair.save_len - 1;
        const unsigned lr = opaque((unsigned)r), lg = opaque((unsigned)g);
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            const int c = col0 + cbase + 16 * h + (int)lr;
            float* const dst = pair.save + ((size_t)unit * nsave + j) * ((size_t)dk * dv) + c;
            if (c < colend) {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int k = 16 * kt + 4 * (int)lg + v;
                        if (k < dk) dst[(size_t)k * dv] = st[h][kt][v];
                    }
            }
        }
    };
    // the forms a forward pass that saves runs in, and the forms a pass that resumes runs in
    constexpr bool SAVES = !REVERSE && ((NH == 1 && NF == 1) || (NH == 2 && NF == 2));
    constexpr bool RESUMES = !REVERSE && ((NH == 2 && NF == 1) || (NH == 3 && NF == 2));

    f32x4 oacc[NH][4];  // state waves: the output tile of the block in progress, summed over the feature chunks

    // One step: feature chunk HF of block `it`; step number s = NF it + HF.  `xr, yr, zr` hold step
    // s+2 on entry and step s+4 on exit.
    // `role`: 0 the score waves' part of the step, 1 the state waves'.
    auto iteration = [&](auto role, auto hf, const int64_t it, u32x4 (&xr)[XC], u32x4 (&yr)[XC], u32x4 (&zr)[ZC]) __attribute__((always_inline)) {
        constexpr int ROLE = decltype(role)::value;
        constexpr int HF = decltype(hf)::value;
        const bool have_next = it + 1 < it_end;
        const bool warm = it < it_first;  // warm-up block: state update only
        const int bcur = (int)((unsigned)(it * NF + HF) % 3u);
        const int bnext = bcur == 2 ? 0 : bcur + 1;
        const int bstage = bnext == 2 ? 0 : bnext + 1;
        if constexpr (ROLE == 0) {
            // publish step s+2 (its buffer was last read in step s-1; the z slot that goes with it
            // still holds an output tile) and refill the registers with step s+4
            constexpr int HS = (HF + 2) % NF, HL = (HF + 4) % NF, HC = (HF + 1) % NF;
            const int64_t bs = it + (HF + 2) / NF;  // block of the step being published
            const int zslot = NZ == 3 ? bstage : (int)((bs - ZLAG) & 1);
            stage_step(std::integral_constant<int, HS>{}, bstage, zslot, xr, yr, zr, it - 1, it > it_first);
            if constexpr (TOGETHER) {
                // both halves of a block's rows are asked for in one go, after the second half of the block before has
                // been published: the 128-byte line in the middle of a 384-byte row is then fetched once
                if constexpr (HF == NF - 1) {
                    load_step(std::integral_constant<int, 0>{}, it + 2, xrA, yrA, zrA);
                    load_step(std::integral_constant<int, 1>{}, it + 2, xrB, yrB, zrB);
                }
            } else {
                load_step(std::integral_constant<int, HL>{}, it + (HF + 4) / NF, xr, yr, zr);
            }
            // the score tile runs one step ahead of the state waves
            const int64_t bc = it + (HF + 1) / NF;
            if (bc < it_end && bc >= it_first) score_step(std::integral_constant<int, HC>{}, bnext, (int)(bc & 1));
        }
        if (ROLE == 1 && cols_active) {
            const unsigned xq = opaque(bcur * XYB + lane_xq);
            const unsigned yq = opaque(bcur * XYB + YOFF + lane_yt);
            const int zcur = NZ == 3 ? bcur : (int)(it & 1);  // z / out slot of this block
            const unsigned zq = opaque(ZBASE + zcur * ZTB + lane_zt);
            const unsigned pq = opaque(PBASE + (unsigned)(it & 1) * PTB + lane_pr);
            // z^T fragments of this wave's 16-column slabs: A operand of the intra-block product
            // and, scaled, B operand of the state update
            // (three slabs: the state takes 144 registers; the fragments are fetched where they are first needed, the
            // x and P fragments without look-ahead, the y^T fragments two tiles at a time)
            constexpr bool LEAN = NH > 2;
            V8 zf[NH][2];
            auto read_z = [&]() {
#pragma unroll
                for (int h = 0; h < NH; ++h)
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
                        zf[h][ks] = cat<V8, V4>(ldt(zq + (32 * ks * ZS + 16 * h) * E), ldt(zq + ((32 * ks + 4) * ZS + 16 * h) * E));
            };
            if constexpr (!LEAN) read_z();
            if (!warm) {
                // out^T[c][i] = Lout[i] * sum_k state[k][c] x[i][k]  +  sum_j z[j][c] P[i][j]
                // One slab: all x fragments are requested up front; LDS answers in order, so the
                // MFMAs of contraction step ks start as soon as its own fragments are there while
                // the later ones are still on their way.  Two slabs: every fragment feeds both, and
                // there are registers for one step of look-ahead only.
                // (256 features and two slabs: the state takes 128 registers, no look-ahead)
                constexpr int NBX = NH == 1 ? KSH : ((NF == 2 && KTH > 6) || LEAN) ? 1 : 2;
                constexpr bool XALL = NBX == KSH;
                V8 bx[NBX][4];
                V8 bp[LEAN ? 2 : 4][2];
                auto read_x = [&](int ks) {
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) {
                        // 8-byte reads from unrelated base registers (one per contraction step and
                        // half): fused in pairs into ds_read2_b64 they would conflict on the LDS
                        // banks at this row stride
                        const unsigned lo = opaque(xq + 32 * ks * E), hi = opaque(xq + (32 * ks + 16) * E);
                        bx[ks % NBX][i4] = cat<V8, V4>(ld4(lo + 16 * i4 * XS * E), ld4(hi + 16 * i4 * XS * E));
                    }
                    __builtin_amdgcn_sched_barrier(0);  // (keeps the address registers of one step at a time)
                };
                auto read_p = [&]() {
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) {
#pragma unroll
                        for (int k2 = 0; k2 < 2; ++k2) {
                            const bool need = REVERSE ? (k2 >= i4 / 2) : (k2 <= i4 / 2);
                            if (need) bp[i4][k2] = ld8(pq + (16 * i4 * PS + 32 * k2) * E);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                };
#pragma unroll
                for (int ks = 0; ks < (XALL ? KSH : NBX - 1); ++ks) read_x(ks);
                if constexpr (HF == 0) {
#pragma unroll
                    for (int h = 0; h < NH; ++h)
#pragma unroll
                        for (int i4 = 0; i4 < 4; ++i4) oacc[h][i4] = (f32x4){0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int ks = 0; ks < KSH; ++ks) {
                    if (!XALL && NBX == 2 && ks + 1 < KSH) read_x(ks + 1);
                    if (!XALL && NBX == 1) read_x(ks);
                    constexpr int KG0 = HF * KSH;  // contraction steps of the chunks before this one
                    if constexpr (LEAN) {
                        // slab by slab: one converted state fragment at a time
#pragma unroll
                        for (int h = 0; h < NH; ++h) {
                            V8 sb1;
#pragma unroll
                            for (int v = 0; v < 4; ++v) {
                                sb1[v] = M::cvt(st[h][2 * (KG0 + ks)][v]);
                                sb1[4 + v] = M::cvt(st[h][2 * (KG0 + ks) + 1][v]);
                            }
#pragma unroll
                            for (int i4 = 0; i4 < 4; ++i4) oacc[h][i4] = M::mma(sb1, bx[ks % NBX][i4], oacc[h][i4]);
                        }
                    } else {
                    V8 sb[NH];
#pragma unroll
                    for (int h = 0; h < NH; ++h)
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            sb[h][v] = M::cvt(st[h][2 * (KG0 + ks)][v]);
                            sb[h][4 + v] = M::cvt(st[h][2 * (KG0 + ks) + 1][v]);
                        }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4)
#pragma unroll
                        for (int h = 0; h < NH; ++h) oacc[h][i4] = M::mma(sb[h], bx[ks % NBX][i4], oacc[h][i4]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    // the P fragments follow once half of the x fragments have been used up
                    if (HF == NF - 1 && XALL && ks == (KSH - 1) / 2) read_p();
                }
                if constexpr (HF == NF - 1) {
                    if constexpr (LEAN) read_z();
                    if (!XALL && !LEAN) read_p();
                    if (DECAY) {
                        f32x4 co;
                        if constexpr (LEAN) co = *reinterpret_cast<const f32x4*>(smem + opaque(CFBASE + 256 + 16 * r));
#pragma unroll
                        for (int h = 0; h < NH; ++h)
#pragma unroll
                            for (int i4 = 0; i4 < 4; ++i4)
#pragma unroll
                                for (int v = 0; v < 4; ++v) oacc[h][i4][v] *= LEAN ? co[i4] : cf[i4];
                    }
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) {
                        if constexpr (LEAN) {
                            // the P fragments of two 16-row tiles at a time
                            if (i4 % 2 == 0) {
#pragma unroll
                                for (int j = 0; j < 2; ++j)
#pragma unroll
                                    for (int k2 = 0; k2 < 2; ++k2) {
                                        const bool need = REVERSE ? (k2 >= (i4 + j) / 2) : (k2 <= (i4 + j) / 2);
                                        if (need) bp[j][k2] = ld8(pq + (16 * (i4 + j) * PS + 32 * k2) * E);
                                    }
                                __builtin_amdgcn_sched_barrier(0);
                            }
                        }
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks) {
                            const bool need = REVERSE ? (ks >= i4 / 2) : (ks <= i4 / 2);
#pragma unroll
                            for (int h = 0; h < NH; ++h)
                                if (need) oacc[h][i4] = M::mma(zf[h][ks], bp[LEAN ? i4 % 2 : i4][ks], oacc[h][i4]);
                        }
                        if (LEAN && i4 % 2 == 1) __builtin_amdgcn_sched_barrier(0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    // leave the tile in the z slot of this block, over this wave's own z columns (read
                    // above, and by no other wave); the staging of the block after next sends it to memory
                    const unsigned oq = opaque(ZBASE + zcur * ZTB + lane_ow);
#pragma unroll
                    for (int h = 0; h < NH; ++h)
#pragma unroll
                        for (int i4 = 0; i4 < 4; ++i4) {
                            V4 o;
#pragma unroll
                            for (int v = 0; v < 4; ++v) o[v] = (T)oacc[h][i4][v];
                            *reinterpret_cast<V4*>(smem + oq + (16 * i4 * ZS + 16 * h) * E) = o;
                        }
                }
            }
            if (have_next || mode == kCollect) {
                // state = lam^64 state + y^T (z * Lupd), the rows of this feature chunk
                constexpr int KT0 = HF * KTH;
                // transposed y reads in batches where the state leaves no registers for all of them at once
                constexpr int UB = (NF == 2 && NH == 2 && KTH > 6) ? 4 : LEAN ? 2 : KTH;
                if constexpr (LEAN) {
                    if (HF != NF - 1 || warm) read_z();
                    if (DECAY) {
                        // (scaled before the y^T fragments are fetched: the factors and the fragments never share registers)
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks) {
                            const unsigned ca = opaque(CFBASE + (16 * g + 8 * ks) * 4);
                            const f32x4 c0 = *reinterpret_cast<const f32x4*>(smem + ca), c1 = *reinterpret_cast<const f32x4*>(smem + ca + 16);
#pragma unroll
                            for (int h = 0; h < NH; ++h)
#pragma unroll
                                for (int u = 0; u < 8; ++u) zf[h][ks][u] = (T)((float)zf[h][ks][u] * (u < 4 ? c0[u] : c1[u - 4]));
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
#pragma unroll
                for (int t0 = 0; t0 < KTH; t0 += UB) {
                    V8 ay[UB][2];
#pragma unroll
                    for (int kt = 0; kt < UB; ++kt) {
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks) {
                            const unsigned py = yq + (32 * ks * XS + 16 * (t0 + kt)) * E;
                            ay[kt][ks] = cat<V8, V4>(ldt(py), ldt(py + 4 * XS * E));
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if (DECAY && t0 == 0) {
#pragma unroll
                        for (int h = 0; h < NH; ++h) {
#pragma unroll
                            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                                for (int u = 0; u < 8; ++u)
                                    if (!LEAN) zf[h][ks][u] = (T)((float)zf[h][ks][u] * cf[4 + 8 * ks + u]);
#pragma unroll
                            for (int kt = 0; kt < KTH; ++kt)
#pragma unroll
                                for (int v = 0; v < 4; ++v) st[h][KT0 + kt][v] *= lamB;
                        }
                    }
#pragma unroll
                    for (int kt = 0; kt < UB; ++kt) {
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                            for (int h = 0; h < NH; ++h) st[h][KT0 + t0 + kt] = M::mma(ay[kt][ks], zf[h][ks], st[h][KT0 + t0 + kt]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if constexpr (SAVES && HF == NF - 1) {
                // a boundary the next pass over these tensors may start from: leave the state after block `it`
                if (it + 1 == next_save) {
                    save_state(it);
                    next_save += pair.save_len;
                    if (next_save >= nblk) next_save = -1;  // the end of the sequence is no boundary
                }
            }
        }
        __syncthreads();
    };
    typedef std::integral_constant<int, 0> C0;
    typedef std::integral_constant<int, NF - 1> C1;  // (the second feature chunk where there is one)
    // NF = 1: both halves of the unrolled loop always run, so the two register sets are refilled in
    // the same order on every path and the wait before staging one set leaves the other in flight.
    // NF = 2: one register set per feature chunk.
    // The two kinds of waves run separate copies of the loop (one barrier per step in each),
    // so that neither carries the other's registers.
    auto walk = [&](auto role) __attribute__((always_inline)) {
        int64_t it = it0;
        if constexpr (NF == 1) {
            for (; it + 1 < it_end; it += 2) {
                iteration(role, C0{}, it, xrA, yrA, zrA);
                iteration(role, C0{}, it + 1, xrB, yrB, zrB);
            }
            if (it < it_end) iteration(role, C0{}, it, xrA, yrA, zrA);
        } else {
            for (; it < it_end; ++it) {
                iteration(role, C0{}, it, xrA, yrA, zrA);
                iteration(role, C1{}, it, xrB, yrB, zrB);
            }
        }
    };
    // the last block's output tile is still in its z slot when the walk ends
    auto flush_last = [&]() {
        if (it_end <= it_first) return;
        const unsigned zd = ZBASE + (unsigned)(NZ == 3 ? (it_end - 1) % 3 : (it_end - 1) & 1) * ZTB + (ZAL ? lane_stage_z : 0u);
        u32x4 o[ZC];
#pragma unroll
        for (int u = 0; u < ZC; ++u) o[u] = *reinterpret_cast<const u32x4*>(smem + zd + (ZAL ? (unsigned)(u * ZROWS * ZS) * E : z_lds(u)));
        store_out(it_end - 1, true, o);
    };
    // The two kinds of waves part here for good, prologue included (two barriers in each branch):
    // the compiler lays the branches out one after the other and keeps alive, while the first one
    // runs, whatever the second one needs of the values computed before this point - which must
    // therefore not include the score waves' prefetch registers.
    auto prologue = [&]() __attribute__((always_inline)) {
        const int b0 = (int)((unsigned)(it0 * NF) % 3u), b1 = b0 == 2 ? 0 : b0 + 1;
        if constexpr (NF == 1) {
            load_step(C0{}, it0, xrA, yrA, zrA);
            load_step(C0{}, it0 + 1, xrB, yrB, zrB);
            stage_step(C0{}, b0, NZ == 3 ? b0 : (int)((it0 + 1) & 1), xrA, yrA, zrA, 0, false);
            load_step(C0{}, it0 + 2, xrA, yrA, zrA);
            stage_step(C0{}, b1, NZ == 3 ? b1 : (int)(it0 & 1), xrB, yrB, zrB, 0, false);
            load_step(C0{}, it0 + 3, xrB, yrB, zrB);
        } else {
            load_step(C0{}, it0, xrA, yrA, zrA);
            load_step(C1{}, it0, xrB, yrB, zrB);
            stage_step(C0{}, b0, (int)(it0 & 1), xrA, yrA, zrA, 0, false);
            load_step(C0{}, it0 + 1, xrA, yrA, zrA);
            stage_step(C1{}, b1, 0, xrB, yrB, zrB, 0, false);
            load_step(C1{}, it0 + 1, xrB, yrB, zrB);
        }
        __syncthreads();
        if (it0 >= it_first && it0 < it_end) score_step(C0{}, b0, (int)(it0 & 1));
        __syncthreads();
    };
    // the state a workgroup starts from: zero, or what the scan (kApply) or the pass before (kResume) left
    auto init_state = [&]() __attribute__((always_inline)) {
        // this lane's part of a state slot: [wave][slab][tile][lane] accumulator quartets
        const size_t lane_slot = ((size_t)w * NH * KT * 64 + lane) * 4;
        const bool resume = mode == kApply && chunk > 0;
        const float* const src = slot0 + (size_t)(chunk - 1) * SF + lane_slot;
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
                st[h][kt] = resume ? *reinterpret_cast<const f32x4*>(src + (size_t)(h * KT + kt) * 256) : (f32x4){0.f, 0.f, 0.f, 0.f};
        if constexpr (RESUMES) {
            if (mode == kResume && chunk > 0) {
                // state[k][c] = saved[c][k]: this lane's four k of a tile are neighbours in row c of the saved matrix
                const float* const m = pair.state + ((size_t)unit * (nchunk - 1) + (chunk - 1)) * ((size_t)dk * dv);
#pragma unroll
                for (int h = 0; h < NH; ++h) {
                    const int c = col0 + cbase + 16 * h + r;
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) {
                        const int k = 16 * kt + 4 * g;  // dk is a multiple of 8: a quartet lies inside or outside
                        if (c < colend && k < dk) st[h][kt] = *reinterpret_cast<const f32x4*>(m + (size_t)c * dk + k);
                    }
                }
            }
        }
    };
    auto leave_state = [&]() __attribute__((always_inline)) {
        if (mode == kCollect) {
            const size_t lane_slot = ((size_t)w * NH * KT * 64 + lane) * 4;
            float* const dst = slot0 + (size_t)chunk * SF + lane_slot;
#pragma unroll
            for (int h = 0; h < NH; ++h)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<f32x4*>(dst + (size_t)(h * KT + kt) * 256) = st[h][kt];
        }
    };
    if (!state_role) {
        prologue();
        walk(std::integral_constant<int, 0>{});
        flush_last();
    } else {
        __syncthreads();
        __syncthreads();
        // The state waves are the critical path and every SIMD holds one wave of each kind: when both
        // have an instruction ready (right after the barrier all eight waves go for LDS), theirs goes first.
        __builtin_amdgcn_s_setprio(1);
        init_state();
        walk(std::integral_constant<int, 1>{});
        leave_state();
    }
}

template <typename T, int DKP, int NF, int NH, bool REVERSE, bool DECAY, bool DENSE, bool SILU = false>
__global__ __launch_bounds__(512, 1) void la_sweep_pipe_kernel(SweepPair pair) {
    sweep_pipe_body<T, DKP, NF, NH, REVERSE, DECAY, DENSE, SILU>(pair, blockIdx.x);
}

// Forward-walking and backward-walking sweeps in one launch (SweepBoth).
template <typename T, int DKP, int NF, bool DECAY, bool DENSE>
__global__ __launch_bounds__(512, 1) void la_sweep_pipe_both_kernel(SweepBoth both) {
    if (blockIdx.x < both.nfwd) sweep_pipe_body<T, DKP, NF, 1, false, DECAY, DENSE>(both.fwd, blockIdx.x);
    else sweep_pipe_body<T, DKP, NF, 1, true, DECAY, DENSE>(both.rev, blockIdx.x - both.nfwd);
}

// What a kernel instantiation needs once per device before its first launch (its dynamic LDS limit raised).
template <typename T, int DKP, int NF, int NH, bool REVERSE, bool DECAY, bool DENSE, bool SILU = false>
static int prep_one() {
    constexpr size_t lds = PipeLds<DKP, NF, NH>::bytes(sizeof(T));
    static_assert(lds <= 160 * 1024, "LDS budget");
    static unsigned char lds_allowed[kMaxDevices];
    return allow_lds(la_sweep_pipe_kernel<T, DKP, NF, NH, REVERSE, DECAY, DENSE, SILU>, lds, lds_allowed);
}

template <typename T, int DKP, int NF, int NH, bool REVERSE, bool DECAY, bool DENSE, bool SILU = false>
static int launch_one(const SweepPair& pair, hipStream_t st) {
    const SweepArgs& a = pair.a[0];
    constexpr size_t lds = PipeLds<DKP, NF, NH>::bytes(sizeof(T));
    auto kern = la_sweep_pipe_kernel<T, DKP, NF, NH, REVERSE, DECAY, DENSE, SILU>;
    if (const int e = prep_one<T, DKP, NF, NH, REVERSE, DECAY, DENSE, SILU>()) return e;
    if (SILU != (pair.silu != 0)) return LA_E_UNSUPPORTED;
    const int units8 = (a.bh + 7) / 8 * 8;
    // the slice width the host chose must be one this instantiation's LDS slot and state waves hold
    if (a.zw <= 0 || a.zw > 64 * NH || a.zw % (16 * NH)) return LA_E_UNSUPPORTED;
    // the state slots the host sized must be the ones this instantiation reads and writes
    if ((pair.mode == kCollect || pair.mode == kApply) && pipe_state_floats(a.dk, pair.wide) != (size_t)4 * NH * (DKP / 16) * 64 * 4)
        return LA_E_WORKSPACE;
    if (pair.wide != NH - 1) return LA_E_UNSUPPORTED;
    // the plain-matrix forms of the state exist in two instantiations only
    constexpr bool SAVES = !REVERSE && ((NH == 1 && NF == 1) || (NH == 2 && NF == 2));
    constexpr bool RESUMES = !REVERSE && ((NH == 2 && NF == 1) || (NH == 3 && NF == 2));
    if (pair.mode == kResume && (!RESUMES || pair.nprod != 1)) return LA_E_UNSUPPORTED;
    if (pair.save && (!SAVES || pair.nprod != 1 || pair.mode != kWarmUp || a.nchunk != 1)) return LA_E_UNSUPPORTED;
    const unsigned grid = (unsigned)(units8 * a.nslice * a.nchunk * pair.nprod);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, st, pair);
    return (int)hipGetLastError();
}

static inline bool plain(const Layout& l, int64_t h, int64_t n, int64_t cols) {
    return l.ts == cols && l.hs == n * cols && l.bs == h * n * cols;
}
static inline bool all_plain(const SweepPair& p) {
    bool dense = true;
    for (int i = 0; i < p.nprod; ++i) {
        const SweepArgs& c = p.a[i];
        dense = dense && plain(c.lx, c.h, c.n, c.dk) && plain(c.ly, c.h, c.n, c.dk) && plain(c.lz, c.h, c.n, c.dv) &&
                plain(c.lo, c.h, c.n, c.dv);
    }
    return dense;
}

template <typename T, int DKP, int NF, bool DECAY, bool DENSE>
static int prep_both_one() {
    constexpr size_t lds = PipeLds<DKP, NF, 1>::bytes(sizeof(T));
    static unsigned char lds_allowed[kMaxDevices];
    return allow_lds(la_sweep_pipe_both_kernel<T, DKP, NF, DECAY, DENSE>, lds, lds_allowed);
}

template <typename T, int DKP, int NF, bool DECAY, bool DENSE>
static int launch_both_one(const SweepBoth& b, hipStream_t st) {
    constexpr size_t lds = PipeLds<DKP, NF, 1>::bytes(sizeof(T));
    auto kern = la_sweep_pipe_both_kernel<T, DKP, NF, DECAY, DENSE>;
    if (const int e = prep_both_one<T, DKP, NF, DECAY, DENSE>()) return e;
    hipLaunchKernelGGL(kern, dim3(b.nfwd + part_grid(b.rev)), dim3(512), lds, st, b);
    return (int)hipGetLastError();
}

// prep_one / prep_both_one for every direction, decay and layout form of one (element type, shape) family.
template <typename T, int DKP, int NF, int NH>
static int prep_family() {
    int e = 0;
#define LA_P(R, D, S) if (!e) e = prep_one<T, DKP, NF, NH, R, D, S>();
    LA_P(false, false, false) LA_P(false, false, true) LA_P(false, true, false) LA_P(false, true, true)
    LA_P(true, false, false) LA_P(true, false, true) LA_P(true, true, false) LA_P(true, true, true)
#undef LA_P
    if constexpr (NH == 1) {
#define LA_P(D, S) if (!e) e = prep_both_one<T, DKP, NF, D, S>();
        LA_P(false, false) LA_P(false, true) LA_P(true, false) LA_P(true, true)
#undef LA_P
    }
    return e;
}

// The instantiations for feature dims 129 .. 256 live in a translation unit of their own (la_sweep_pipe_split.hip).
int launch_split(const SweepPair& p, int dtype, bool reverse, hipStream_t st);
int launch_split_both(const SweepBoth& b, int dtype, hipStream_t st);
int prepare_split();

}  // namespace la
