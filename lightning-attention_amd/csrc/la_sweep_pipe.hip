// The pipelined sweep kernel (la_sweep_pipe_body.h) for feature dims up to 128, the scan kernel between the
// collect and apply launches of a chunked walk, and the host entry points of the pipelined kernels.
// (lightning_attn/ops/triton/lightning_attn2.py:8-85 forward, :88-395 backward.)
#include "la_sweep_pipe_body.h"

namespace la {

template <typename T, bool REVERSE>
static int launch_dir(const SweepPair& pair, hipStream_t st) {
    const SweepArgs& a = pair.a[0];
    const bool decay = a.s != nullptr;
    const bool dense = all_plain(pair);
#define LA_GO2(DKP, NH, DENSE) (decay ? launch_one<T, DKP, 1, NH, REVERSE, true, DENSE>(pair, st) : launch_one<T, DKP, 1, NH, REVERSE, false, DENSE>(pair, st))
#define LA_GO(DKP, NH) (dense ? LA_GO2(DKP, NH, true) : LA_GO2(DKP, NH, false))
    if (pair.silu) {
        if constexpr (!REVERSE) {
#define LA_GS2(DKP, NH, DENSE) (decay ? launch_one<T, DKP, 1, NH, false, true, DENSE, true>(pair, st) : launch_one<T, DKP, 1, NH, false, false, DENSE, true>(pair, st))
#define LA_GS(DKP, NH) (dense ? LA_GS2(DKP, NH, true) : LA_GS2(DKP, NH, false))
            if (pair.wide) return LA_GS(128, 2);
            if (a.dk <= 64) return LA_GS(64, 1);
            return LA_GS(128, 1);
#undef LA_GS
#undef LA_GS2
        }
        return LA_E_UNSUPPORTED;
    }
    if (pair.wide) return LA_GO(128, 2);  // 128 columns per workgroup (nslice counts those)
    if (a.dk <= 64) return LA_GO(64, 1);
    return LA_GO(128, 1);
#undef LA_GO
#undef LA_GO2
}

template <typename T>
static int launch_both(const SweepBoth& b, hipStream_t st) {
    const SweepArgs& a = b.fwd.a[0];
    const bool decay = a.s != nullptr;
    const bool dense = all_plain(b.fwd) && all_plain(b.rev);
#define LA_GO2(DKP, DENSE) (decay ? launch_both_one<T, DKP, 1, true, DENSE>(b, st) : launch_both_one<T, DKP, 1, false, DENSE>(b, st))
#define LA_GO(DKP) (dense ? LA_GO2(DKP, true) : LA_GO2(DKP, false))
    if (a.dk <= 64) return LA_GO(64);
    return LA_GO(128);
#undef LA_GO
#undef LA_GO2
}

int sweep_pipe_both(const SweepBoth& b, int dtype, hipStream_t st) {
    const SweepArgs &f = b.fwd.a[0], &r = b.rev.a[0];
    if (f.dk > 256 || f.dk != r.dk || f.dv != r.dv || f.n != r.n || f.bh != r.bh || b.fwd.wide || b.rev.wide ||
        b.fwd.mode != kWarmUp || b.rev.mode != kWarmUp || b.nfwd != part_grid(b.fwd))
        return LA_E_UNSUPPORTED;
    if (f.dk > 128) return launch_split_both(b, dtype, st);
    if (dtype == LA_BF16) return launch_both<__bf16>(b, st);
    if (dtype == LA_FP16) return launch_both<_Float16>(b, st);
    return LA_E_UNSUPPORTED;
}

// Between kCollect and kApply: turns the states the chunks end with (each computed from zero) into the
// states they start from.  Slot c holds S_loc[c] on entry and S_in[c + 1] = lam^(64 len_c) S_in[c] + S_loc[c]
// on exit (S_in[0] = 0).  One thread per accumulator quartet, chunks in order; the layout inside a slot
// does not matter.
__global__ __launch_bounds__(256) void la_state_scan_kernel(float* state, const float* s, int h, int sets_per_unit,
                                                           int nchunk, int chunk_len, int quartets) {
    const int q = blockIdx.x * 256 + threadIdx.x;  // quartet within the slot
    const int64_t set = blockIdx.y;                // (unit, sweep, slice)
    if (q >= quartets) return;
    const float rate = s ? s[(set / sets_per_unit) % h] : 0.f;
    f32x4* slot = reinterpret_cast<f32x4*>(state) + set * (int64_t)(nchunk - 1) * quartets + q;
    // every chunk but the last is chunk_len blocks long
    const float f = s ? expf(-rate * 64.f * (float)chunk_len) : 1.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    // the loads of a batch are independent of the running sum: one memory round trip per batch, not per chunk
    constexpr int BATCH = 16;
    for (int c0 = 0; c0 + 1 < nchunk; c0 += BATCH) {
        f32x4 loc[BATCH];
#pragma unroll
        for (int i = 0; i < BATCH; ++i)
            if (c0 + i + 1 < nchunk) loc[i] = slot[(int64_t)(c0 + i) * quartets];
#pragma unroll
        for (int i = 0; i < BATCH; ++i)
            if (c0 + i + 1 < nchunk) {
                acc = acc * f + loc[i];
                slot[(int64_t)(c0 + i) * quartets] = acc;
            }
    }
}

int launch_state_scan(const SweepPair& p, hipStream_t st) {
    const SweepArgs& a = p.a[0];
    const int quartets = (int)(pipe_state_floats(a.dk, p.wide) / 4);
    const int sets_per_unit = p.nprod * a.nslice;
    hipLaunchKernelGGL(la_state_scan_kernel, dim3((unsigned)((quartets + 255) / 256), (unsigned)(a.bh * sets_per_unit)),
                       dim3(256), 0, st, p.state, a.s, a.h, sets_per_unit, a.nchunk, p.chunk_len, quartets);
    return (int)hipGetLastError();
}

static int launch_any(const SweepPair& p, int dtype, bool reverse, hipStream_t st) {
    if (p.silu && (p.a[0].dk > 128 || reverse || p.nprod != 1)) return LA_E_UNSUPPORTED;
    if (p.a[0].dk > 128) return launch_split(p, dtype, reverse, st);
    if (dtype == LA_BF16) return reverse ? launch_dir<__bf16, true>(p, st) : launch_dir<__bf16, false>(p, st);
    if (dtype == LA_FP16) return reverse ? launch_dir<_Float16, true>(p, st) : launch_dir<_Float16, false>(p, st);
    return LA_E_UNSUPPORTED;
}

// Every instantiation of the pipelined kernel made ready for its first launch on the current device.
int prepare_pipe() {
    int e = prep_family<__bf16, 64, 1, 1>();
    if (!e) e = prep_family<__bf16, 128, 1, 1>();
    if (!e) e = prep_family<__bf16, 128, 1, 2>();
    if (!e) e = prep_family<_Float16, 64, 1, 1>();
    if (!e) e = prep_family<_Float16, 128, 1, 1>();
    if (!e) e = prep_family<_Float16, 128, 1, 2>();
#define LA_PS(T, DKP, NH) \
    if (!e) e = prep_one<T, DKP, 1, NH, false, false, false, true>(); \
    if (!e) e = prep_one<T, DKP, 1, NH, false, false, true, true>();  \
    if (!e) e = prep_one<T, DKP, 1, NH, false, true, false, true>();  \
    if (!e) e = prep_one<T, DKP, 1, NH, false, true, true, true>();
    LA_PS(__bf16, 64, 1) LA_PS(__bf16, 128, 1) LA_PS(__bf16, 128, 2)
    LA_PS(_Float16, 64, 1) LA_PS(_Float16, 128, 1) LA_PS(_Float16, 128, 2)
#undef LA_PS
    if (!e) e = prepare_split();
    return e;
}

int sweep_pipe(const SweepPair& p, int dtype, bool reverse, hipStream_t st) {
    const SweepArgs& a = p.a[0];
    if (a.dk > 256 || p.nprod < 1 || p.nprod > 2) return LA_E_UNSUPPORTED;
    if (p.mode == kWarmUp || a.nchunk <= 1) {
        SweepPair q = p;
        q.mode = kWarmUp;
        return launch_any(q, dtype, reverse, st);
    }
    if (!p.state || p.chunk_len < 1) return LA_E_WORKSPACE;
    if (p.mode == kResume) return launch_any(p, dtype, reverse, st);  // the states are there already
    // three launches: local end states, their scan, the walk proper
    SweepPair q = p;
    q.mode = kCollect;
    int rc = launch_any(q, dtype, reverse, st);
    if (rc != LA_OK) return rc;
    rc = launch_state_scan(p, st);
    if (rc != LA_OK) return rc;
    q.mode = kApply;
    return launch_any(q, dtype, reverse, st);
}

}  // namespace la
