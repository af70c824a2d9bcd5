// Decayed linear attention as directional "sweeps", and how a sweep is mapped onto kernel launches (host side).
//
// One generic sweep computes, per (batch, head),
//     forward  direction:  out_i = sum_{j<=i} lam^(i-j) (x_i . y_j) z_j
//     reverse  direction:  out_i = sum_{j>=i} lam^(j-i) (x_i . y_j) z_j
// with lam = exp(-s_h).  The four products of the operator are instances of it:
//     O  = sweep_fwd(Q , K , V )      dQ = sweep_fwd(dO, V , K )
//     dK = sweep_rev(V , dO, Q )      dV = sweep_rev(K , Q , dO)
// (lightning_attn/ops/triton/lightning_attn2.py:8-85 forward, :88-395 backward.)
//
// The kernel is the pipelined one of la_sweep_pipe_body.h for every feature dim up to 256.  This file
// decides, from the shape and the compute units of the device, how many columns of z / out a workgroup
// takes (64 or 128), whether a long walk over few sequences is cut into chunks (from warm-up blocks, or
// from scanned states in a workspace), and which sweeps of a backward pass share a launch.
#include "la_sweep_common.h"
#include "lightning_attn_hip.h"

namespace la {

int prepare_plans() { return num_cus() > 0 ? 0 : (int)hipErrorInvalidDevice; }

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
// `width` of a workgroup: 0 = 64 columns of z / out, 1 = 128 (96 where there are 192 to share out), 2 = all
// (129 .. 192) columns of a sequence in one workgroup.
static const double kWholeBlockUs = 3.9;
static double block_us(int64_t dk, int width) {
    if (dk <= 64) return 1.0;
    if (dk <= 128) return width ? 1.75 : 1.4;
    if (dk <= 192) return width == 2 ? kWholeBlockUs : width ? 3.0 : 2.1;
    return width ? 4.1 : 2.9;
}
// Column slices per sequence: 64 columns each, or 128, or one slice.
static int64_t wide_slices(int64_t dv) { return (dv + 127) / 128; }
static int64_t slices(int64_t dk, int64_t dv, int width) { return width == 2 ? 1 : width ? wide_slices(dv) : (dv + 63) / 64; }
static double warm_up_frac(int64_t wgs, int64_t nblk) {
    static const double frac[9] = {1.0, 1.0, 0.77, 0.71, 0.68, 0.67, 0.66, 0.66, 0.66};
    return frac[warm_up_chunks(wgs, nblk)];
}
static double warm_up_us(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, int wide) {
    const int64_t nblk = (n + 63) / 64, wgs = (bh + 7) / 8 * 8 * slices(dk, dv, wide) * nprod;
    return warm_up_frac(wgs, nblk) * (double)nblk * block_us(dk, wide);
}

static ScanPlan plan_scan(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, int wide, const Opts& opts) {
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

// Estimated duration (us) of one launch of nprod sweeps in workgroups of width code `width`, by the figures
// above: rounds of workgroups where they fill the chip, else the better of the two chunk plans.
static double width_us(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, int width, size_t scratch, const Opts& opts) {
    const int64_t cus = num_cus(), nblk = (n + 63) / 64, wgs = (bh + 7) / 8 * 8 * slices(dk, dv, width) * nprod;
    if (wgs * 2 > cus) return (double)((wgs + cus - 1) / cus) * (double)nblk * block_us(dk, width);
    const ScanPlan pl = plan_scan(bh, n, dk, dv, nprod, width, opts);
    return pl.nchunk > 1 && pl.bytes <= scratch ? pl.us : warm_up_us(bh, n, dk, dv, nprod, width);
}

// The pipelined kernel can give each workgroup 128 columns of z / out instead of 64: the score tile
// and the x / y tiles are then produced once per 128 output columns, and the power-limited kernel
// turns the saved work into time (dK + dV at the headline shape: 0.31 against 0.415 ms) - as long
// as there are workgroups enough.  A 128-column workgroup takes about 1.25 times as long as a
// 64-column one, and there are half as many: compare the rounds of workgroups the chip has to run.
// `scratch`: bytes of workspace the caller has.  opts.wide overrides the choice.
static bool wide_columns(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, size_t scratch, const Opts& opts_in) {
    Opts opts = opts_in;
    if (opts.wide == LA_OPT_ALL) opts.wide = LA_OPT_AUTO;  // (column_width's business)
    if (dk > 128) {
        // Feature dims 129 .. 256: 128-column workgroups where that makes fewer slices.
        // They pay when the 64-column form needs more rounds of workgroups than the chip has CUs for
        // (a wide workgroup takes about 1.4 times as long), and with few sequences on a long walk, where half as
        // many workgroups mean twice the chunks (d = e = 256 fwd+bwd: b1 h8 n16384 0.42 against 0.58 ms, b2 h12 n16384
        // 1.16 against 1.59, b2 h12 n4096 0.33 against 0.41); in between the 64-column form has more workgroups to
        // spread over the CUs and stays.
        const int64_t ws = wide_slices(dv), ns = (dv + 63) / 64;
        if (ws >= ns) return false;
        if (opts.wide != LA_OPT_AUTO) return opts.wide == LA_OPT_ON;
        const int64_t cus = num_cus(), units = (bh + 7) / 8 * 8 * nprod, wide = units * ws, narrow = units * ns;
        if (narrow <= cus) return width_us(bh, n, dk, dv, nprod, 1, scratch, opts) < 0.9 * width_us(bh, n, dk, dv, nprod, 0, scratch, opts);
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
        // (in between: one 128-column workgroup per sequence only where the second 64-column slice would be half
        // empty - d = e = 96, b*h = 96: la_fwd 0.321 against 0.359 ms at n = 16384, la_bwd 0.78 against 0.82)
        if (narrow * 2 > cus) return dv <= 96;
        const ScanPlan w = plan_scan(bh, n, dk, dv, nprod, true, opts), nw = plan_scan(bh, n, dk, dv, nprod, false, opts);
        return w.nchunk > 1 && w.bytes <= scratch && w.us < (nw.bytes <= scratch ? nw.us : warm_up_us(bh, n, dk, dv, nprod, false));
    }
    return (wide + cus - 1) / cus * 5 < (narrow + cus - 1) / cus * 4;
}

// Feature dims and columns of 129 .. 192: one workgroup can take all columns of a sequence (la_sweep_pipe_body.h,
// NH = 3), at kWholeBlockUs per block against 3.0 us for each of two 96-column workgroups or 2.1 us for each of
// three 64-column ones.  Taken where it is estimated at least 3 % faster than the choice among the narrower forms:
// fewer rounds of workgroups with many sequences (b*h = 160 at n = 4096: la_fwd 0.241 against 0.300 ms, la_bwd 0.703
// against 0.878), shorter chunks with few (b*h = 24 at n = 16384: la_fwd 0.185 against 0.309 ms; b*h = 48 at n = 4096:
// 0.104 / 0.272 against 0.141 / 0.317).
// Returns the width code of the launch: 0 / 1 as wide_columns has it, or 2.  opts.wide overrides the choice.
static int column_width(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, size_t scratch, const Opts& opts) {
    const int wide = wide_columns(bh, n, dk, dv, nprod, scratch, opts) ? 1 : 0;
    if (dk <= 128 || dk > 192 || dv <= 128 || dv > 192) return wide;
    if (opts.wide != LA_OPT_AUTO) return opts.wide == LA_OPT_ALL ? 2 : wide;
    return width_us(bh, n, dk, dv, nprod, 2, scratch, opts) < 0.97 * width_us(bh, n, dk, dv, nprod, wide, scratch, opts) ? 2 : wide;
}

// The column slices of a sweep whose workgroups have width code `width` (make_args leaves 64-column slices).
static void set_width(SweepArgs& a, int width, int64_t dv) {
    if (width == 2) {
        a.nslice = 1;
        a.zw = 192;
    } else if (width) {
        // equal slices, a whole number of 32-column state waves each (192 columns: 96 + 96, not 128 + 64)
        const int64_t ws = wide_slices(dv);
        a.nslice = (int)ws;
        a.zw = (int)(((dv + ws - 1) / ws + 31) / 32 * 32);
    }
}

// Workspace the kernels can use for one launch of nprod sweeps (0: none).
size_t sweep_workspace_bytes(int64_t bh, int64_t n, int64_t dk, int64_t dv, int nprod, int dtype, const Opts& opts) {
    if (dtype != LA_BF16 && dtype != LA_FP16) return 0;
    return plan_scan(bh, n, dk, dv, nprod, column_width(bh, n, dk, dv, nprod, (size_t)-1, opts), opts).bytes;
}

static int launch_planned(SweepPair& p, int64_t bh, int64_t n, int64_t dk, int64_t dv, int dtype, bool reverse, void* ws,
                          size_t ws_bytes, const Opts& opts, hipStream_t st) {
    const bool ws_ok = ws && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
    p.wide = column_width(bh, n, dk, dv, p.nprod, ws_ok ? ws_bytes : 0, opts);
    p.mode = kWarmUp;
    p.chunk_len = 0;
    p.state = nullptr;
    for (int i = 0; i < p.nprod; ++i) set_width(p.a[i], p.wide, dv);
    const ScanPlan pl = plan_scan(bh, n, dk, dv, p.nprod, p.wide, opts);
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
    return sweep_pipe(p, dtype, reverse, st);
}

// x,y: (b,h,n,dk)  z,out: (b,h,n,dv), each with its own batch / head / token strides
int sweep(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
          bool reverse, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st) {
    SweepPair p;
    p.nprod = 1;
    p.a[0] = make_args(io, s, bh, h, n, dk, dv);
    return launch_planned(p, bh, n, dk, dv, dtype, reverse, ws, ws_bytes, opts, st);
}

// The forward sweep over silu(x), silu(y), silu(z): the same plan, the activation applied in the tile load.
int sweep_silu(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
               void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st) {
    if (dk > 128 || dv > 128 || (dtype != LA_BF16 && dtype != LA_FP16)) return LA_E_UNSUPPORTED;
    SweepPair p;
    p.nprod = 1;
    p.silu = 1;
    p.a[0] = make_args(io, s, bh, h, n, dk, dv);
    return launch_planned(p, bh, n, dk, dv, dtype, false, ws, ws_bytes, opts, st);
}

// States a forward sweep can leave behind for the sweep that follows it over the same tensors in swapped roles.
// O = sweep(q, k, v) carries the state K^T V (d x e); dQ = sweep(dO, v, k) of the backward pass carries V^T K,
// its transpose.  Where the forward pass walks each sequence in one piece and leaves the state at c - 1
// equally spaced block boundaries, the dQ sweep can run as c chunks per sequence from those states - no
// warm-up blocks, no collect and scan launches - and so in 128-column workgroups where 64-column ones
// would otherwise be needed to give every CU a workgroup (b*h around 128 on a 256-CU chip).
// nchunk == 1: not for this shape.
SavedPlan plan_saved(int64_t bh, int64_t n, int64_t d, int64_t e, int dtype, const Opts& opts) {
    const SavedPlan none = {1, 0, 0, 0, 0};
    if (dtype != LA_BF16 && dtype != LA_FP16) return none;
    // Feature dims up to 128: the forward pass in 64-column workgroups, dQ in 128-column ones.  d and e both in
    // 129 .. 192: the forward pass in two slices of up to 96 columns, dQ with all its columns in one workgroup.
    // (The kernel forms that can leave and pick up the states, la_sweep_pipe_body.h.)
    const bool big = d > 128 && d <= 192 && e > 128 && e <= 192;
    if (!big && (d <= 64 || d > 128 || e > 128)) return none;
    if (opts.chunks != 0 || opts.wide == LA_OPT_ON || opts.wide == LA_OPT_ALL || opts.scan == LA_OPT_ON) return none;
    const int64_t nblk = (n + 63) / 64, cus = num_cus(), units8 = (bh + 7) / 8 * 8;
    // Short sequences: writing the states and starting from them costs what the wider workgroups save
    // (b4 h32 d128 fwd+bwd, with / without: n = 512 0.060 / 0.056 ms, 1024 0.097 / 0.096, 2048 0.176 / 0.181, 4096
    // 0.341 / 0.357; d = 192: n = 1024 0.160 / 0.158, 2048 0.319 / 0.332).
    if (nblk < 24) return none;
    const int fwd_width = big ? 1 : 0, dq_width = big ? 2 : 1;
    // the forward pass as planned: that width, one walk per sequence
    if (column_width(bh, n, d, e, 1, (size_t)-1, opts) != fwd_width) return none;
    if (plan_scan(bh, n, d, e, 1, fwd_width, opts).nchunk > 1) return none;
    if (warm_up_chunks(units8 * slices(d, e, fwd_width), nblk) > 1) return none;
    // dQ: one workgroup of that width per sequence and chunk
    int64_t c = cus / units8;
    if (c > nblk / 4) c = nblk / 4;
    if (c > 64) c = 64;
    if (c < 2) return none;
    SavedPlan pl;
    pl.chunk_len = (int)((nblk + c - 1) / c);
    pl.nchunk = (int)((nblk + pl.chunk_len - 1) / pl.chunk_len);
    if (pl.nchunk < 2) return none;
    // against what the dQ sweep would take by its own plan
    const int wide = column_width(bh, n, e, d, 1, (size_t)-1, opts);
    const ScanPlan own = plan_scan(bh, n, e, d, 1, wide, opts);
    const int64_t own_wgs = units8 * slices(e, d, wide);
    const double own_us = own.nchunk > 1 ? own.us
                          : own_wgs * 2 <= cus ? warm_up_us(bh, n, e, d, 1, wide)
                                               : (double)((own_wgs + cus - 1) / cus) * (double)nblk * block_us(e, wide);
    if ((double)pl.chunk_len * block_us(e, dq_width) >= own_us) return none;
    pl.bytes = (size_t)bh * (size_t)(pl.nchunk - 1) * (size_t)(d * e) * sizeof(float);
    pl.fwd_width = fwd_width;
    pl.dq_width = dq_width;
    return pl;
}

// The forward sweep as sweep() plans it where plan_saved applies, leaving its state every save_len blocks in `save`.
int sweep_saving(const SweepIO& io, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk, int64_t dv, int dtype,
                 float* save, int save_len, int width, hipStream_t st) {
    SweepPair p;
    p.nprod = 1;
    p.a[0] = make_args(io, s, bh, h, n, dk, dv);
    set_width(p.a[0], width, dv);
    p.a[0].nchunk = 1;
    p.a[0].chunk_start[0] = 0;
    for (int j = 1; j < 9; ++j) p.a[0].chunk_start[j] = (int)((n + 63) / 64);
    p.a[1] = p.a[0];
    p.wide = width;
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
                  const float* saved, int nchunk, int chunk_len, int width, hipStream_t st) {
    if (nchunk < 2 || chunk_len < 1 || slices(dk, dv, width) != 1) return LA_E_UNSUPPORTED;
    SweepPair p;
    p.nprod = 1;
    p.a[0] = make_args(io, s, bh, h, n, dk, dv);
    set_width(p.a[0], width, dv);
    p.a[0].nchunk = nchunk;
    for (int j = 0; j < 9; ++j) p.a[0].chunk_start[j] = 0;
    p.a[1] = p.a[0];
    p.wide = width;
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
    if (forced == 0 && (opts.wide == LA_OPT_ON || opts.wide == LA_OPT_ALL)) return LA_E_UNSUPPORTED;  // wider workgroups asked for
    const int64_t cus = num_cus(), nblk = (n + 63) / 64, nslice = (d + 63) / 64;
    const int64_t wgs = (bh + 7) / 8 * 8 * nslice * 3;  // one chunk each
    if (forced == 0) {
        // (up to two rounds of workgroups: on a short walk one launch of twice as many 64-column workgroups as
        // there are CUs still beats two launches - b1 h48 n2048 d192: la_bwd 0.138 against 0.162 ms)
        if (wgs > 2 * cus) return LA_E_UNSUPPORTED;
        // what the separate launches would take, by the estimates behind their own plans
        const bool ws_ok = ws && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
        double separate = 0.0;
        for (int nprod = 1; nprod <= 2; ++nprod) {
            const size_t scratch = ws_ok ? ws_bytes : 0;
            separate += width_us(bh, n, d, d, nprod, column_width(bh, n, d, d, nprod, scratch, opts), scratch, opts);
        }
        // here: the longest workgroup of 3 * wgs/3 * c warm-up chunked ones, or two rounds of single walks
        const double rounds = wgs > cus ? 2.0 : 1.0;
        if (rounds * warm_up_frac(wgs, nblk) * (double)nblk * block_us(d, false) >= separate) return LA_E_UNSUPPORTED;
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
    return sweep_pipe_both(b, dtype, st);
}

// The same for two sweeps of one shape and opposite directions (dQ and dK of a backward pass with
// d != e: both contract over e and produce d columns): one launch where separate launches are not estimated
// faster (they fit on the chip together, or share rounds of workgroups); LA_E_UNSUPPORTED otherwise.
int sweep_fwd_rev_once(const SweepIO& fwd, const SweepIO& rev, const float* s, int64_t bh, int64_t h, int64_t n, int64_t dk,
                       int64_t dv, int dtype, void* ws, size_t ws_bytes, const Opts& opts, hipStream_t st) {
    if (dtype != LA_BF16 && dtype != LA_FP16) return LA_E_UNSUPPORTED;
    const int forced = opts.once == LA_OPT_ON ? 1 : opts.once == LA_OPT_OFF ? -1 : 0;
    if (forced < 0 || opts.paired == LA_OPT_OFF) return LA_E_UNSUPPORTED;
    if (forced == 0 && (opts.wide == LA_OPT_ON || opts.wide == LA_OPT_ALL)) return LA_E_UNSUPPORTED;
    const int64_t cus = num_cus(), nblk = (n + 63) / 64, nslice = (dv + 63) / 64;
    const int64_t wgs = (bh + 7) / 8 * 8 * nslice * 2;
    if (forced == 0) {
        // (up to three rounds of workgroups: where each sweep alone leaves its last round mostly empty, the two
        // together need fewer rounds - d192 e128 b*h = 96, 288 workgroups a sweep: la_bwd 0.215 against 0.261 ms at
        // n = 2048; d256 e128 b*h = 80: 0.229 against 0.274)
        if (wgs > 3 * cus) return LA_E_UNSUPPORTED;
        const bool ws_ok = ws && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
        const size_t scratch = ws_ok ? ws_bytes : 0;
        const double separate = 2.0 * width_us(bh, n, dk, dv, 1, column_width(bh, n, dk, dv, 1, scratch, opts), scratch, opts);
        const int64_t rounds = (wgs + cus - 1) / cus;
        const double share = rounds > 1 ? (double)rounds : warm_up_frac(wgs, nblk);
        if (share * (double)nblk * block_us(dk, false) >= separate) return LA_E_UNSUPPORTED;
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
    return sweep_pipe_both(b, dtype, st);
}

}  // namespace la
