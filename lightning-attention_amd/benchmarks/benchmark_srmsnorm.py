"""Speed and peak-memory tables of SimpleRMSNorm, x of shape (12, n, 2048) bf16, n = 2^9 .. 2^15:
the tables of the reference's benchmarks/benchmark_srmsnorm.py:19-140 (columns: the HIP module,
where the reference has its Triton one, and the plain PyTorch module).

    python lightning-attention_amd/benchmarks/benchmark_srmsnorm.py
"""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import torch  # noqa: E402

from _harness import do_bench, peak_memory_mb, print_table  # noqa: E402
from lightning_attn.ops import SimpleRMSNorm, SimpleRMSNormTorch  # noqa: E402

B, D = 12, 2048


def main():
    dev = torch.device("cuda")
    ns = [2 ** i for i in range(9, 16)]
    tables = {(kind, mode): {} for kind in ("speed", "memory") for mode in ("fwd", "bwd")}
    for n in ns:
        torch.manual_seed(2024)
        x = torch.randn(B, n, D, dtype=torch.bfloat16, device=dev).requires_grad_()
        for name, module in (("Hip", SimpleRMSNorm(D)), ("Torch", SimpleRMSNormTorch(D))):
            fn = lambda: module(x)  # noqa: E731
            tables[("memory", "fwd")].setdefault(name, []).append(peak_memory_mb(fn, dev))
            tables[("speed", "fwd")].setdefault(name, []).append(do_bench(fn))
            y = fn()
            dy = torch.randn(B, n, D, dtype=torch.bfloat16, device=dev)
            bwd = lambda: y.backward(dy, retain_graph=True)  # noqa: E731
            tables[("memory", "bwd")].setdefault(name, []).append(peak_memory_mb(bwd, dev))
            tables[("speed", "bwd")].setdefault(name, []).append(do_bench(bwd, grads=(x,)))
            del y, dy
            x.grad = None
    for (kind, mode), cols in tables.items():
        print_table("srms-%s_%s-batch%d-dim%d-dtype_bf16" % (kind, mode, B, D), ns, list(cols.items()))


if __name__ == "__main__":
    main()
