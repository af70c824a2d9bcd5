"""Forward + backward time of the TNL attention block (examples/module/tnl_attn.py) around the operator,
with the output norm, sigmoid gate and product fused into one row kernel (``norm_gate``) and as the three
separate PyTorch operators of the reference's block (tnl_attn.py:66-69), and the time of the fused kernel
against that chain on its own.

    python lightning-attention_amd/benchmarks/benchmark_tnl_block.py [--quick | --large]

Under ``rocprofv3 --kernel-trace --stats`` the same run gives the split of the block by kernel (projection
GEMMs, the three SiLU passes, the attention sweeps, the norm / gate kernels).
"""
import importlib.util
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import torch  # noqa: E402
import torch.nn.functional as F  # noqa: E402

from _harness import do_bench  # noqa: E402
from lightning_attn.ops.hip import norm_gate  # noqa: E402

_spec = importlib.util.spec_from_file_location("tnl_attn_example", os.path.join(os.path.dirname(HERE), "examples", "module", "tnl_attn.py"))
tnl = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(tnl)


def main():
    quick = "--quick" in sys.argv
    dev = torch.device("cuda")
    torch.manual_seed(2024)
    shapes = [(2, 2048, 1024, 8)] if quick else [(2, 2048, 1024, 8), (4, 4096, 2048, 16), (4, 8192, 4096, 32)]
    if "--large" in sys.argv:  # the block around the benchmark shape of the operator only
        shapes = shapes[-1:]
    print("TNL block, bf16: b, n, embed, heads | block fwd+bwd ms, fused norm-gate / separate operators | "
          "norm-gate alone fwd, bwd ms: fused / separate | block forward without gradients, SiLU in the kernel / separate")
    for b, n, embed, heads in shapes:
        block = tnl.TnlAttention(embed, heads).to(dev).bfloat16()
        x = torch.randn(b, n, embed, device=dev, dtype=torch.bfloat16).requires_grad_()
        g = torch.randn(b, n, embed, device=dev, dtype=torch.bfloat16)
        params = [x] + list(block.parameters())

        def step():
            block(x).backward(g)

        times = {}
        for fused in (True, False):
            block.fused_norm_gate = fused
            times[fused] = do_bench(step, grads=params)
        # inference: the forward pass alone without gradients, SiLU inside the forward kernel / as three PyTorch passes
        infer = {}
        block.fused_norm_gate = True
        for fused in (True, False):
            block.fused_silu = fused
            with torch.no_grad():
                infer[fused] = do_bench(lambda: block(x))
        block.fused_silu = True
        # the norm / gate part on its own
        o, gate = (torch.randn(b * n, embed, device=dev, dtype=torch.bfloat16).requires_grad_() for _ in range(2))
        w, bias = block.norm.weight, block.norm.bias
        dy = torch.randn(b * n, embed, device=dev, dtype=torch.bfloat16)
        parts = {}
        for name, fn in (("fused", lambda: norm_gate(o, gate, w, bias, 1e-5)),
                         ("separate", lambda: F.layer_norm(o, (embed,), w, bias, 1e-5) * torch.sigmoid(gate))):
            y = fn()
            parts[name] = (do_bench(fn), do_bench(lambda: y.backward(dy, retain_graph=True), grads=(o, gate, w, bias)))
            del y
        print("%d %5d %5d %3d | %.4f / %.4f | fwd %.4f / %.4f  bwd %.4f / %.4f | inference fwd, SiLU fused / separate %.4f / %.4f"
              % (b, n, embed, heads, times[True], times[False], parts["fused"][0], parts["separate"][0],
                 parts["fused"][1], parts["separate"][1], infer[True], infer[False]), flush=True)
        del block, x, g, o, gate, dy


if __name__ == "__main__":
    main()
