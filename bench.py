#!/usr/bin/env python3
"""Benchmark of the scan hot path on one MI355X.

A step is one forward + backward pass of selective_scan_fn over one synthetic batch of the
Mamba-1 benchmark configuration (batch 8, d_inner 5120, seqlen 4096, d_state 16, bf16
activations, fp32 A/D/delta_bias/state), inputs resident in HBM.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def make_inputs(batch, dim, seqlen, dstate, dtype, device, seed=0):
    import torch
    g = torch.Generator(device=device).manual_seed(seed)
    rn = lambda *s: torch.randn(*s, device=device, generator=g).to(dtype)
    dt = torch.exp(torch.rand(dim, device=device, generator=g) * (math.log(1e-1) - math.log(1e-3)) + math.log(1e-3))
    return dict(
        u=rn(batch, dim, seqlen), delta=rn(batch, dim, seqlen), z=rn(batch, dim, seqlen),
        B=rn(batch, 1, dstate, seqlen), C=rn(batch, 1, dstate, seqlen), dout=rn(batch, dim, seqlen),
        A=-torch.arange(1, dstate + 1, device=device, dtype=torch.float32).repeat(dim, 1).contiguous(),
        D=torch.ones(dim, device=device), delta_bias=dt + torch.log(-torch.expm1(-dt)))


def cpu_baseline(seqlen, dstate, full_dim):
    """Oracle (a PyTorch restatement of the reference's selective_scan_ref) forward + backward on the
    host cores, on a batch-1 / 64-channel slice of the workload; channels and batch rows are independent
    in the scan, so tokens/s is scaled by (64 / full_dim)."""
    import torch
    from oracle.mamba1 import selective_scan_oracle, scan_inputs
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    dim = 256
    t = scan_inputs(1, dim, seqlen, dstate, 1, torch.bfloat16, seed=0)
    ins = {k: (v.clone().requires_grad_() if (v is not None and k != "dout") else v) for k, v in t.items()}
    t0 = time.perf_counter()
    out = selective_scan_oracle(ins["u"], ins["delta"], ins["A"], ins["B"], ins["C"], ins["D"], ins["z"],
                                ins["delta_bias"], True)
    out.backward(ins["dout"])
    dt = time.perf_counter() - t0
    return {"value": seqlen * (dim / full_dim) / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"oracle fwd+bwd, batch 1 x {dim} of {full_dim} channels x seqlen {seqlen}, "
                      f"{dt:.1f} s, scaled by {dim}/{full_dim}"}


def copy_calibration(dev):
    """Runs mamba_hip_copy (one 16-byte element per thread) over 1 GiB: 1 GiB read + 1 GiB written."""
    import torch
    from mamba_amd import _lib
    nbytes = 1 << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    lib = _lib.load()
    stream = _lib.current_stream(dev)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    for i in range(6):
        if i == 1:
            ev[0].record()
        _lib.check(lib.mamba_hip_copy(dst.data_ptr(), src.data_ptr(), nbytes, stream), "mamba_hip_copy")
    ev[1].record()
    torch.cuda.synchronize()
    ms = ev[0].elapsed_time(ev[1]) / 5
    print(json.dumps({"kernel": "copy_kernel", "bytes_read": nbytes, "bytes_written": nbytes, "ms": ms,
                      "GB/s": 2 * nbytes / ms / 1e6}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run the library's plain copy kernel over 1 GiB (yardstick for HBM counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the scan has no cross-GPU exchange step); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from mamba_amd.ops import selective_scan_interface as ssi
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn, selective_scan_fwd
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.copy_calibration:
        copy_calibration(dev)
        return
    batch, dim, seqlen, dstate = 8, 5120, 4096, 16
    dtype = torch.bfloat16
    t = make_inputs(batch, dim, seqlen, dstate, dtype, dev)
    leaves = {k: t[k].requires_grad_() for k in ("u", "delta", "A", "B", "C", "D", "z", "delta_bias")}

    def step():
        for v in leaves.values():
            v.grad = None
        out = selective_scan_fn(leaves["u"], leaves["delta"], leaves["A"], leaves["B"], leaves["C"], leaves["D"],
                                z=leaves["z"], delta_bias=leaves["delta_bias"], delta_softplus=True)
        out.backward(t["dout"])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    tokens_per_s = batch * seqlen / (elapsed / args.steps)

    # Dominant kernel (the backward scan) alone, HIP events on the launch stream.
    with torch.no_grad():
        d = {k: v.detach() for k, v in leaves.items()}
        _, ckpt = selective_scan_fwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["z"], d["delta_bias"], True)
        dims = (batch, dim, seqlen, dstate, 1)
        bufs = ssi.ScanBwdBuffers(d["u"], d["delta"], d["B"], d["z"], dims)
        bwd_pre = lambda: ssi.scan_bwd_zero(bufs, dev)  # outside the event pair
        bwd = lambda: ssi.scan_bwd_launch(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["z"],
                                          d["delta_bias"], t["dout"], ckpt, True, bufs, dims)
        fwd = lambda: selective_scan_fwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["z"],
                                         d["delta_bias"], True)

        def kernel_ms(fn, n, pre=None):
            # the library launches on torch's current stream, which is where these events are recorded
            if pre:
                pre()
            fn()
            torch.cuda.synchronize()
            ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
            for a, b in ev:
                if pre:
                    pre()
                a.record()
                fn()
                b.record()
            torch.cuda.synchronize()
            return sum(a.elapsed_time(b) for a, b in ev) / n

        n = max(5, min(args.steps, 50))
        bwd_ms = kernel_ms(bwd, n, bwd_pre)
        fwd_ms = kernel_ms(fwd, n)
    es = 2  # bf16
    E = batch * dim * seqlen * es
    BC = batch * dstate * seqlen * es
    bwd_bytes = 7 * E + 4 * BC   # reads u, delta, z, dout, B, C; writes du, ddelta, dz, dB, dC
    fwd_bytes = 4 * E + 2 * BC   # reads u, delta, z, B, C; writes out
    achieved = bwd_bytes / (bwd_ms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": "scan_bwd_kernel", "achieved": achieved, "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                "kernel_ms": bwd_ms, "algorithmic_bytes": bwd_bytes,
                "fwd_kernel_ms": fwd_ms, "fwd_achieved": fwd_bytes / (fwd_ms * 1e-3) / 1e9,
                "fwd_bwd_frac": (fwd_bytes + bwd_bytes) / ((fwd_ms + bwd_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS}

    result = {
        "metric": "scan fwd+bwd tokens/s at 1 GPU; achieved HBM GB/s and % bf16 MFMA peak",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 in/out, fp32 state and accumulation", "data": "synthetic",
        "config": {"workload": "Mamba-1 selective_scan_fn fwd+bwd: batch 8, d_inner 5120, seqlen 4096, d_state 16, "
                               "bf16 u/delta/B/C/z, fp32 A/D/delta_bias (BASELINE configs[1])",
                   "global_batch": batch, "seq_len": seqlen},
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(seqlen, dstate, dim)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
