#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-sweep]

A step is one forward+backward of ``lightning_attn_func`` on synthetic N(0,1)
bf16 inputs at b=4, h=32, n=8192, d=e=128 with slopes from
``_build_slope_tensor(32)`` and an N(0,1) upstream gradient; inputs are resident in
HBM before the timed region.  Prints ONE JSON line.  ``value`` is the algorithmic
MFMA rate of the step (flop count of a 64-token block recurrence, 344064 flop per
token and head, divided by the measured time); ``ms_per_step`` is the same
measurement in milliseconds.  The line also carries the live roofline figures of
the dominant kernel, the SRMSNorm bandwidths, the n-sweep and a CPU baseline
(the oracle's naive path on the host cores, bounded sample).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "lightning-attention_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

METRIC = "fwd+bwd ms & MFMA TFLOP/s at b4 h32 n8192 d128 bf16; SRMSNorm HBM GB/s"
B, H, N, D = 4, 32, 8192, 128
BLOCK = 64
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E


def flops_per_token(d, e, which):
    fwd = 2 * BLOCK * (d + e) + 4 * d * e
    bwd = 2 * BLOCK * (3 * d + 2 * e) + 10 * d * e
    return {"fwd": fwd, "bwd": bwd, "both": fwd + bwd}[which]


def bytes_per_token(d, e, which, elt=2):
    fwd = (2 * d + 2 * e) * elt
    bwd = (4 * d + 3 * e) * elt
    return {"fwd": fwd, "bwd": bwd, "both": fwd + bwd}[which]


def _clear(*tensors):
    for t in tensors:
        t.grad = None


def event_ms(fn, reps, warm=3):
    """Average duration of fn() over reps launches, HIP events on the current stream
    (the stream the operators launch on)."""
    import torch

    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps


def cpu_baseline(n_seq=10):
    """Oracle naive path (float32 arithmetic on the bf16-rounded inputs) for n_seq of the
    128 (batch, head) sequences of the workload, one sequence at a time."""
    import torch

    import oracle

    torch.set_num_threads(os.cpu_count() or 1)
    slopes = oracle.build_slope_tensor(H)
    g = torch.Generator().manual_seed(2024)
    total = 0.0
    done = 0
    for i in range(n_seq + 1):  # first pass is the warm-up
        hi = (i * 9) % H
        q, k, v, do = (torch.randn(1, 1, N, D, generator=g).bfloat16().float() for _ in range(4))
        t0 = time.perf_counter()
        oracle.linear_attn_fwd_bwd(q, k, v, slopes[hi:hi + 1], do, torch.float32)
        dt = time.perf_counter() - t0
        if i > 0:
            total += dt
            done += 1
        if total > 30.0:
            break
    tokens = done * N
    return {
        "value": round(flops_per_token(D, D, "both") * tokens / total / 1e12, 5),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "%d of %d (batch, head) sequences at n=%d, d=e=%d, naive O(n^2) oracle in float32 on bf16-rounded "
                  "inputs, fwd+bwd through autograd; %.2f s per sequence => %.0f ms for the whole step"
                  % (done, B * H, N, D, total / done, total / done * B * H * 1e3),
        "ms_per_step_extrapolated": round(total / done * B * H * 1e3, 1),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-sweep", action="store_true", help="skip the fwd/bwd split and the n sweep")
    ap.add_argument("--no-srms", action="store_true", help="skip the SRMSNorm timings")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU part (every (batch, head) sequence is "
                 "independent); run with --gpus 1")

    import torch

    from lightning_attn.ops import SimpleRMSNorm, lightning_attn_func
    from lightning_attn.ops.hip import _lib
    from lightning_attn.utils import _build_slope_tensor

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")
    dev = torch.device("cuda:0")
    L = _lib.lib()  # fails loudly if the HIP library is not built
    torch.manual_seed(2024)

    def inputs(n):
        q, k, v, do = (torch.randn(B, H, n, D, device=dev, dtype=torch.float32).bfloat16() for _ in range(4))
        return q.requires_grad_(), k.requires_grad_(), v.requires_grad_(), do

    s = _build_slope_tensor(H).to(dev).to(torch.float32)
    q, k, v, do = inputs(N)

    def step():
        o = lightning_attn_func(q, k, v, s)
        o.backward(do)
        q.grad = k.grad = v.grad = None

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps

    tokens = B * H * N
    flop_step = flops_per_token(D, D, "both") * tokens
    bytes_step = bytes_per_token(D, D, "both") * tokens
    tflops = flop_step / (ms * 1e-3) / 1e12

    # ---- dominant kernel: the forward-direction sweep, one launch = O = sweep(Q, K, V) ----
    o_buf = torch.empty_like(v)
    st = torch.cuda.current_stream().cuda_stream

    def fwd_launch():
        rc = L.la_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), o_buf.data_ptr(), B, H, N, D, D, 0,
                      None, 0, st)
        assert rc == 0, rc

    k_ms = event_ms(fwd_launch, 30)
    k_bytes = bytes_per_token(D, D, "fwd") * tokens
    k_flop = flops_per_token(D, D, "fwd") * tokens
    roofline = {
        "kernel": "la_sweep_pipe_kernel<bf16, DKP=128, forward, decay> (one launch: O = sweep(Q,K,V); a step is this, the same for dQ, and one double launch for dK + dV)",
        "bound": "hbm",
        "achieved": round(k_bytes / (k_ms * 1e-3) / 1e9, 1),
        "peak": PEAK_HBM_GBS,
        "unit": "GB/s",
        "frac": round(k_bytes / (k_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
        # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE (x2.0) + WRITE_SIZE (x1.0), see
        # profiles/la_sweep_pipe_kernel_b4_h32_n8192_d128_bf16.md; bench.py cannot read counters itself
        "traffic": 1.0741e9,
        "traffic_unit": "bytes/launch (rocprofv3 counters, committed profile)",
        "algorithmic_bytes": k_bytes,
        "launch_ms": round(k_ms, 4),
        "mfma_tflops": round(k_flop / (k_ms * 1e-3) / 1e12, 1),
        "mfma_frac": round(k_flop / (k_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
    }

    out = {
        "metric": METRIC,
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "lightning_attn_func fwd+bwd, b=4 h=32 n=8192 d=e=128 bf16, slopes(32), N(0,1) inputs "
                               "and upstream gradient (the shape the metric is quoted on; configs[1] is the same at n=4096)"},
        "step_mfma_frac": round(tflops / PEAK_BF16_TFLOPS, 4),
        "step_hbm_frac": round(bytes_step / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
        "roofline": roofline,
    }

    if not args.no_sweep:
        # fwd / bwd split at the metric shape (events, reference protocol: bwd = o.backward(do, retain_graph))
        o = lightning_attn_func(q, k, v, s)

        def bwd_only():
            o.backward(do, retain_graph=True)
            q.grad = k.grad = v.grad = None

        out["fwd_ms"] = round(event_ms(lambda: lightning_attn_func(q, k, v, s), 20), 4)
        out["bwd_ms"] = round(event_ms(bwd_only, 20), 4)
        del o
        sweep = {}
        for n in (512, 1024, 2048, 4096, 8192, 16384, 32768):
            q = k = v = do = None
            q, k, v, do = inputs(n)
            sweep[str(n)] = round(event_ms(step, 10 if n >= 16384 else 20), 4)
        out["n_sweep_fwd_bwd_ms"] = sweep
        # the other GPU configurations (parity-test cases; timings for reference only):
        # configs[1] without decay, config 4 = b2 h12 n2048 d=e=192 with and without decay, and config 4's
        # shape fed token-major (a (b, n, h*d) projection output used in place through the strided entry points)
        q = k = v = do = None
        extra = {}
        q, k, v, do = inputs(4096)
        extra["b4_h32_n4096_d128_no_decay_ms"] = round(event_ms(lambda: (lightning_attn_func(q, k, v, None).backward(do), _clear(q, k, v)), 20), 4)
        q = k = v = do = None
        b4, h4, n4, d4 = 2, 12, 2048, 192
        s4 = _build_slope_tensor(h4).to(dev).to(torch.float32)
        q, k, v, do = (torch.randn(b4, h4, n4, d4, device=dev).bfloat16() for _ in range(4))
        q, k, v = q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
        extra["b2_h12_n2048_d192_ms"] = round(event_ms(lambda: (lightning_attn_func(q, k, v, s4).backward(do), _clear(q, k, v)), 30), 4)
        # the same shape with the C entry points called directly: the two launches of a step without
        # torch's autograd engine in between (its hand-over to the backward thread bounds the figure above)
        o4, dq4, dk4, dv4 = (torch.empty_like(q) for _ in range(4))

        def direct4():
            rc = L.la_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s4.data_ptr(), o4.data_ptr(), b4, h4, n4, d4, d4, 0, None, 0, st)
            rc = rc or L.la_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s4.data_ptr(), do.data_ptr(), dq4.data_ptr(),
                                dk4.data_ptr(), dv4.data_ptr(), b4, h4, n4, d4, d4, 0, None, 0, st)
            assert rc == 0, rc

        extra["b2_h12_n2048_d192_la_fwd_la_bwd_ms"] = round(event_ms(direct4, 30), 4)
        o4 = dq4 = dk4 = dv4 = None
        extra["b2_h12_n2048_d192_no_decay_ms"] = round(event_ms(lambda: (lightning_attn_func(q, k, v, None).backward(do), _clear(q, k, v)), 30), 4)
        qt, kt, vt = (torch.randn(b4, n4, h4, d4, device=dev).bfloat16().transpose(1, 2).requires_grad_() for _ in range(3))
        dot = torch.randn(b4, n4, h4, d4, device=dev).bfloat16().transpose(1, 2)
        extra["b2_h12_n2048_d192_token_major_ms"] = round(event_ms(lambda: (lightning_attn_func(qt, kt, vt, s4).backward(dot), _clear(qt, kt, vt)), 30), 4)
        out["other_configs_fwd_bwd"] = extra
        qt = kt = vt = dot = None
    del q, k, v, do
    if not args.no_srms:
        # SRMSNorm, config 5: [32768, 4096] bf16, 1 % outliers x50
        rows, cols = 32768, 4096
        x = torch.randn(rows, cols, device=dev)
        x = torch.where(torch.rand(rows, cols, device=dev) < 0.01, x * 50, x).bfloat16().requires_grad_()
        dy = torch.randn(rows, cols, device=dev).bfloat16()
        norm = SimpleRMSNorm(cols)
        y = norm(x)

        def nbwd():
            y.backward(dy, retain_graph=True)
            x.grad = None

        f_ms = event_ms(lambda: norm(x), 50)
        b_ms = event_ms(nbwd, 50)
        fb, bb = rows * (2 * 2 * cols + 4), rows * (3 * 2 * cols + 4)
        out["srmsnorm"] = {
            "shape": [rows, cols], "fwd_ms": round(f_ms, 4), "bwd_ms": round(b_ms, 4),
            "fwd_GBps": round(fb / (f_ms * 1e-3) / 1e9, 1), "bwd_GBps": round(bb / (b_ms * 1e-3) / 1e9, 1),
            "fwd_hbm_frac": round(fb / (f_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "bwd_hbm_frac": round(bb / (b_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
        }

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
