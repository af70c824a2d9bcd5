"""Speed and peak-memory tables of the attention operators, n = 2^9 .. 2^15 at b4 h32 d=e=128 bf16:
the tables of the reference's benchmarks/benchmark_lightning2.py:55-204 (Lightning2 and
Lightning2NoDecay columns; forward alone, backward alone).  PyTorch's fused causal softmax
attention stands in for the Flash2 / Xformers columns when it runs on this device.

    python lightning-attention_amd/benchmarks/benchmark_lightning2.py [--max-n 32768]
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import torch  # noqa: E402
import torch.nn.functional as F  # noqa: E402

from _harness import do_bench, peak_memory_mb, print_table  # noqa: E402
from lightning_attn.ops import lightning_attn2, lightning_attn2_no_decay  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402

B, H, D, E = 4, 32, 128, 128


def providers(q, k, v, s):
    out = {
        "Lightning2": lambda: lightning_attn2(q, k, v, s),
        "Lightning2NoDecay": lambda: lightning_attn2_no_decay(q, k, v),
    }
    try:
        F.scaled_dot_product_attention(q[:, :, :64], k[:, :, :64], v[:, :, :64], is_causal=True)
        out["TorchSDPA"] = lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True)
    except Exception:
        pass
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--max-n", type=int, default=32768)
    ap.add_argument("--sdpa-max-n", type=int, default=8192, help="longest n the softmax column is run at")
    args = ap.parse_args()
    dev = torch.device("cuda")
    ns = [2 ** i for i in range(9, 16) if 2 ** i <= args.max_n]
    tables = {(kind, mode): {} for kind in ("speed", "memory") for mode in ("fwd", "bwd")}
    for n in ns:
        torch.manual_seed(2024)
        q, k, v = (torch.randn(B, H, n, x, dtype=torch.bfloat16, device=dev).requires_grad_() for x in (D, D, E))
        s = _build_slope_tensor(H).to(dev).to(torch.float32)
        for name, fn in providers(q, k, v, s).items():
            if name == "TorchSDPA" and n > args.sdpa_max_n:
                for key in tables:
                    tables[key].setdefault(name, []).append(float("nan"))
                continue
            # as in the reference: the forward figures with q, k, v alone alive, the backward ones
            # with the output, its upstream gradient and the input gradients as well
            tables[("memory", "fwd")].setdefault(name, []).append(peak_memory_mb(fn, dev))
            tables[("speed", "fwd")].setdefault(name, []).append(do_bench(fn))
            o = fn()
            do = torch.randn(B, H, n, E, dtype=torch.bfloat16, device=dev)
            bwd = lambda: o.backward(do, retain_graph=True)  # noqa: E731
            tables[("memory", "bwd")].setdefault(name, []).append(peak_memory_mb(bwd, dev))
            tables[("speed", "bwd")].setdefault(name, []).append(do_bench(bwd, grads=(q, k, v)))
            del o, do
            q.grad = k.grad = v.grad = None
    for (kind, mode), cols in tables.items():
        print_table("lightning2-%s_%s-batch%d-head%d-qk_dim%d-v_dim%d-dtype_bf16" % (kind, mode, B, H, D, E), ns,
                    list(cols.items()))


if __name__ == "__main__":
    main()
