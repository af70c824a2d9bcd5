// The pipelined sweep kernel (la_sweep_pipe_body.h) for feature dims 129 .. 256: the feature dim is padded
// to 192 or 256 and processed in two halves per 64-token block, one workgroup barrier per half.
// (lightning_attn/ops/triton/lightning_attn2.py:8-85 forward, :88-395 backward; the reference serves these
// dims by cutting q / k into 64-wide slices and adding the partial outputs,
// lightning_attn/ops/lightning_attn_interface.py:34-55.)
#include "la_sweep_pipe_body.h"

namespace la {

template <typename T, bool REVERSE>
static int launch_split_dir(const SweepPair& pair, hipStream_t st) {
    const SweepArgs& a = pair.a[0];
    const bool decay = a.s != nullptr;
    const bool dense = all_plain(pair);
#define LA_GO2(DKP, NH, DENSE) (decay ? launch_one<T, DKP, 2, NH, REVERSE, true, DENSE>(pair, st) : launch_one<T, DKP, 2, NH, REVERSE, false, DENSE>(pair, st))
#define LA_GO(DKP, NH) (dense ? LA_GO2(DKP, NH, true) : LA_GO2(DKP, NH, false))
    if (pair.wide == 2) return a.dk <= 192 ? LA_GO(192, 3) : LA_E_UNSUPPORTED;
    if (a.dk <= 192) return pair.wide ? LA_GO(192, 2) : LA_GO(192, 1);
    return pair.wide ? LA_GO(256, 2) : LA_GO(256, 1);
#undef LA_GO
#undef LA_GO2
}

int launch_split(const SweepPair& p, int dtype, bool reverse, hipStream_t st) {
    if (p.a[0].dk <= 128 || p.a[0].dk > 256) return LA_E_UNSUPPORTED;
    if (dtype == LA_BF16) return reverse ? launch_split_dir<__bf16, true>(p, st) : launch_split_dir<__bf16, false>(p, st);
    if (dtype == LA_FP16) return reverse ? launch_split_dir<_Float16, true>(p, st) : launch_split_dir<_Float16, false>(p, st);
    return LA_E_UNSUPPORTED;
}

template <typename T>
static int launch_split_both_t(const SweepBoth& b, hipStream_t st) {
    const SweepArgs& a = b.fwd.a[0];
    const bool decay = a.s != nullptr;
    const bool dense = all_plain(b.fwd) && all_plain(b.rev);
#define LA_GO2(DKP, DENSE) (decay ? launch_both_one<T, DKP, 2, true, DENSE>(b, st) : launch_both_one<T, DKP, 2, false, DENSE>(b, st))
#define LA_GO(DKP) (dense ? LA_GO2(DKP, true) : LA_GO2(DKP, false))
    if (a.dk <= 192) return LA_GO(192);
    return LA_GO(256);
#undef LA_GO
#undef LA_GO2
}

int launch_split_both(const SweepBoth& b, int dtype, hipStream_t st) {
    if (b.fwd.a[0].dk <= 128 || b.fwd.a[0].dk > 256) return LA_E_UNSUPPORTED;
    if (dtype == LA_BF16) return launch_split_both_t<__bf16>(b, st);
    if (dtype == LA_FP16) return launch_split_both_t<_Float16>(b, st);
    return LA_E_UNSUPPORTED;
}

// Every instantiation of this file made ready for its first launch on the current device.
int prepare_split() {
    int e = prep_family<__bf16, 192, 2, 1>();
    if (!e) e = prep_family<__bf16, 192, 2, 2>();
    if (!e) e = prep_family<__bf16, 192, 2, 3>();
    if (!e) e = prep_family<__bf16, 256, 2, 1>();
    if (!e) e = prep_family<__bf16, 256, 2, 2>();
    if (!e) e = prep_family<_Float16, 192, 2, 1>();
    if (!e) e = prep_family<_Float16, 192, 2, 2>();
    if (!e) e = prep_family<_Float16, 192, 2, 3>();
    if (!e) e = prep_family<_Float16, 256, 2, 1>();
    if (!e) e = prep_family<_Float16, 256, 2, 2>();
    return e;
}

}  // namespace la
