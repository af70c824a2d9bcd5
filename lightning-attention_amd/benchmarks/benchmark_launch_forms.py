"""How the launch form of the attention entry points affects their time on one shape: the library's own choice
against forced forms (64- / wide-column workgroups, sequence chunks from scanned states or with warm-up blocks,
paired / separate dK + dV launches), through the C ABI with ``la_launch_opts``; and the same launches on operands
that stay resident in the 256 MB last-level cache against operands that cannot (several sets in rotation), which
tells how much of a launch's time is HBM's.

    python lightning-attention_amd/benchmarks/benchmark_launch_forms.py [--shape B,H,N,D] [--cache]

Default shape: b4 h32 n8192 d=e=128 bf16 (the benchmark shape of the operator).
"""
import ctypes
import os
import statistics
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import torch  # noqa: E402

from lightning_attn.ops.hip import _lib  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402

DEV = "cuda"


def event_times(fn, reps, warm):
    for i in range(warm):
        fn(i)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    torch.cuda.synchronize()
    ev[0].record()
    for i in range(reps):
        fn(i)
        ev[i + 1].record()
    torch.cuda.synchronize()
    ts = [ev[i].elapsed_time(ev[i + 1]) for i in range(reps)]
    return statistics.median(ts), min(ts)


class Case:
    def __init__(self, b, h, n, d, nsets=1):
        self.dims = (b, h, n, d)
        self.s = _build_slope_tensor(h).to(DEV).float().contiguous()
        self.sets = [[torch.randn(b, h, n, d, device=DEV).bfloat16() for _ in range(4)]
                     + [torch.empty(b, h, n, d, device=DEV, dtype=torch.bfloat16) for _ in range(3)] for _ in range(nsets)]
        self.L = _lib.lib()
        self.st = torch.cuda.current_stream().cuda_stream

    def run(self, which, opts, reps=40, warm=10):
        b, h, n, d = self.dims
        L, ob = self.L, (ctypes.byref(opts) if opts is not None else None)
        need = L.la_workspace_bytes_opts(0 if which == "fwd" else 1, b, h, n, d, d, 0, ob)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
        wp = ws.data_ptr() if need else None

        def f(i):
            q, k, v, do, o1, o2, o3 = self.sets[i % len(self.sets)]
            if which == "fwd":
                rc = L.la_fwd_opts(q.data_ptr(), k.data_ptr(), v.data_ptr(), self.s.data_ptr(), o1.data_ptr(), None, b, h, n, d, d,
                                   0, wp, need, ob, self.st)
            else:
                rc = L.la_bwd_opts(q.data_ptr(), k.data_ptr(), v.data_ptr(), self.s.data_ptr(), do.data_ptr(), o1.data_ptr(),
                                   o2.data_ptr(), o3.data_ptr(), None, b, h, n, d, d, 0, wp, need, ob, self.st)
            assert rc == 0, L.la_error_string(rc)

        med, mn = event_times(f, reps, warm)
        return med, mn, need


def main():
    shape = (4, 32, 8192, 128)
    if "--shape" in sys.argv:
        shape = tuple(int(t) for t in sys.argv[sys.argv.index("--shape") + 1].split(","))
    O = _lib.LaunchOpts
    A, OFF, ON = _lib.LA_OPT_AUTO, _lib.LA_OPT_OFF, _lib.LA_OPT_ON
    torch.manual_seed(1)
    case = Case(*shape)
    case.run("fwd", None, reps=60, warm=60)  # bring the chip to its steady state first
    print("launch forms at b%d h%d n%d d=e=%d bf16 (median / min ms, workspace bytes)" % shape)
    forms = [("library's choice", None), ("64-column workgroups", O(0, A, OFF, A, A)), ("wide workgroups, one chunk", O(1, A, ON, A, A)),
             ("wide, 2 chunks, scanned states", O(2, A, ON, A, A)), ("wide, 4 chunks, scanned states", O(4, A, ON, A, A)),
             ("wide, 2 chunks, warm-up blocks", O(2, OFF, ON, A, A)), ("64-column, 2 chunks, scanned states", O(2, A, OFF, A, A)),
             ("64-column, 3 chunks, warm-up blocks", O(3, OFF, OFF, A, A)), ("separate dK and dV launches", O(0, A, A, OFF, A)),
             ("library's choice (again)", None)]
    for name, opts in forms:
        f = case.run("fwd", opts)
        b = case.run("bwd", opts)
        print("  %-38s la_fwd %.4f / %.4f  (%9d)   la_bwd %.4f / %.4f  (%9d)" % ((name,) + f + b), flush=True)
    if "--cache" in sys.argv:
        b, h, _, d = shape
        print("operands resident in the last-level cache (1 set) against streamed from HBM (12 sets in rotation), b%d h%d d=e=%d:" % (b, h, d))
        for n in (512, 1024, 2048):
            mib = b * h * n * d * 2 / 2 ** 20
            for nsets in (1, 12):
                c = Case(b, h, n, d, nsets)
                f = c.run("fwd", None, reps=60, warm=30)
                bw = c.run("bwd", None, reps=60, warm=30)
                print("  n=%5d  %2d set(s) of 7 tensors x %3.0f MiB: la_fwd %.1f us (%.2f us per 64-token block)  la_bwd %.1f us (%.2f)"
                      % (n, nsets, mib, f[0] * 1e3, f[0] * 1e3 / (n / 64), bw[0] * 1e3, bw[0] * 1e3 / (n / 64)), flush=True)
                del c


if __name__ == "__main__":
    main()
