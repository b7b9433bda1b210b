#!/usr/bin/env python3
"""Benchmark of the scan hot path on one MI355X.

A step is one forward + backward pass of selective_scan_fn over one synthetic batch of the
Mamba-1 benchmark configuration (batch 8, d_inner 5120, seqlen 4096, d_state 16, bf16
activations, fp32 A/D/delta_bias/state), inputs resident in HBM.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extra]

The line also carries, under "extra", the SSD (configuration 2), decode (configuration 3) and packed-SSD
(configuration 4) workloads timed in the same run, and under "cpu_baseline" the oracle on the host cores.

Side workloads (each prints its own JSON line; they are not the headline metric):
  python bench.py --workload ssd      Mamba-2 mamba_chunk_scan_combined fwd+bwd (batch 4, 80 heads x 64,
                                      seqlen 4096, d_state 128, chunk 256, bf16)
  python bench.py --workload decode [--batch B]   selective_state_update, 1000 consecutive steps (batch 256, 80 heads x 64, d_state 128)
  python bench.py --workload varlen   the same operator on one packed row of 16 sequences, 32768 positions,
                                      64 heads, 8 groups, initial and final states (benchmark configuration 4)
  python bench.py --workload inner    mamba_inner_fn fwd+bwd (conv, projections, scan; d_model 2560)
  python bench.py --workload block    mamba_split_conv1d_scan_combined fwd+bwd (conv, SSD scan, gated norm,
                                      out_proj; d_model 2560)
  python bench.py --copy-calibration  the library's plain copy kernel over 1 GiB
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
PROFILES = os.path.join(ROOT, "profiles")


def source_id():
    """First 16 hex digits of the SHA-256 over the library's sources (mamba_amd/csrc/*.hip, *.hpp, *.cpp and
    include/*.h, in name order).  The counter summaries under profiles/ carry the id of the sources they were
    taken with; figures parsed from a summary whose id differs are reported as null."""
    import hashlib
    h = hashlib.sha256()
    files = []
    for d, exts in ((os.path.join(ROOT, "mamba_amd", "csrc"), (".hip", ".hpp", ".cpp")), (os.path.join(ROOT, "include"), (".h",))):
        files += [os.path.join(d, n) for n in os.listdir(d) if n.endswith(exts)]
    for p in sorted(files):
        h.update(os.path.basename(p).encode())
        h.update(open(p, "rb").read())
    return h.hexdigest()[:16]


_FRESH = {}


def profile_fresh(filename):
    """True when profiles/<filename> says it was taken with the sources this tree holds (a line
    `library sources: <id>`)."""
    if filename not in _FRESH:
        ok = False
        try:
            for line in open(os.path.join(PROFILES, filename)):
                if line.startswith("library sources:"):
                    ok = line.split(":", 1)[1].strip() == source_id()
                    break
        except OSError:
            pass
        _FRESH[filename] = ok
    return _FRESH[filename]


def profile_traffic(filename, kernel):
    """HBM bytes per launch of `kernel` as the FETCH_SIZE / WRITE_SIZE counter runs measured them: the row of
    that kernel in profiles/<filename> (columns ... read MB (scaled), written MB (scaled)).  None when the
    summary or the row is missing or the summary was taken with other sources than this tree's."""
    if not profile_fresh(filename):
        return None
    try:
        for line in open(os.path.join(PROFILES, filename)):
            cols = line.split()
            if len(cols) >= 5 and cols[0].startswith(kernel):
                return (float(cols[-2]) + float(cols[-1])) * 1e6
    except (OSError, ValueError):
        pass
    return None


def profile_traffic_sum(filename):
    """Sum of the scaled read + written bytes over every kernel row of an HBM-counter summary (one step)."""
    if not profile_fresh(filename):
        return None
    total, rows = 0.0, 0
    try:
        seen = False
        for line in open(os.path.join(PROFILES, filename)):
            cols = line.split()
            if cols[:1] == ["kernel"]:
                seen = True
                continue
            if cols[:2] == ["rows", "below:"] or cols[:1] == ["sum"]:
                break  # what follows is not part of a default step
            if seen and len(cols) >= 5:
                try:
                    total += (float(cols[-2]) + float(cols[-1])) * 1e6
                    rows += 1
                except ValueError:
                    pass
    except OSError:
        return None
    return total if rows else None


def profile_counter(filename, kernel, counter):
    """Average per-launch value of one hardware counter from profiles/<filename> (lines `kernel counter value`);
    None when missing or stale."""
    if not profile_fresh(filename):
        return None
    try:
        for line in open(os.path.join(PROFILES, filename)):
            cols = line.split()
            if len(cols) == 3 and cols[0].startswith(kernel) and cols[1] == counter:
                return float(cols[2])
    except (OSError, ValueError):
        pass
    return None


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


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(seqlen, dstate, full_dim):
    """Oracle (a PyTorch restatement of the reference's selective_scan_ref) on the host cores: forward alone and
    forward + backward, each the median of 5 runs (~10 s of CPU work in all), on a batch-1 slice of one sixteenth of
    the channels; channels and batch rows are independent in the scan, so tokens/s of the whole workload is the
    slice's rate x slice / whole."""
    import statistics
    import torch
    from oracle.mamba1 import selective_scan_oracle, scan_inputs
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    dim = full_dim // 16
    t = scan_inputs(1, dim, seqlen, dstate, 1, torch.bfloat16, seed=0)
    names = ("u", "delta", "A", "B", "C", "D", "z", "delta_bias")

    def run(backward):
        ins = {k: (t[k].clone().requires_grad_(backward) if t[k] is not None else None) for k in names}
        t0 = time.perf_counter()
        with torch.set_grad_enabled(backward):
            out = selective_scan_oracle(*[ins[k] for k in names], True)
            if backward:
                out.backward(t["dout"])
        return time.perf_counter() - t0

    fwd = statistics.median(run(False) for _ in range(5))
    both = statistics.median(run(True) for _ in range(5))
    scale = dim / full_dim
    return {"value": seqlen * scale / both, "unit": "tokens/s", "cores": cores, "kind": "port",
            "fwd_only_value": seqlen * scale / fwd, "cpu": cpu_model(),
            "slice_seconds": {"forward": fwd, "forward_backward": both},
            "sample": f"oracle.mamba1.selective_scan_oracle, batch 1 x {dim} of {full_dim} channels x seqlen {seqlen} "
                      f"(1/16 of the channels of one of 8 batch rows): forward {fwd:.2f} s, forward + "
                      f"backward {both:.2f} s (medians of 5); tokens/s of the whole workload = {seqlen} x {dim}/{full_dim} / seconds"}


def cpu_baseline_ssd():
    """The chunked SSD oracle (oracle.ssd.ssd_chunked, the four-step form of the reference's ssd_minimal.py) with
    autograd on the host cores, on one batch row and one sixteenth of configuration 2's heads (heads and batch rows
    are independent); forward + backward, median of 2."""
    import statistics
    import torch
    from oracle.ssd import ssd_chunked, ssd_inputs, dt_pipeline
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    L, H, Hs, P, N, Q = 4096, 80, 5, 64, 128, 256
    t = ssd_inputs(1, L, Hs, P, N, 1, torch.bfloat16, 0)

    def run():
        ins = {k: t[k].clone().float().requires_grad_() for k in ("x", "dt", "B", "C", "z")}
        t0 = time.perf_counter()
        dtv = dt_pipeline(ins["dt"], t["dt_bias"], True)
        out = ssd_chunked(ins["x"], dtv, t["A"], ins["B"], ins["C"], Q, D=t["D"], z=ins["z"])
        out.backward(t["dout"].float())
        return time.perf_counter() - t0

    sec = statistics.median(run() for _ in range(2))
    return {"value": L * (Hs / H) / sec, "unit": "tokens/s", "cores": cores, "kind": "port", "slice_seconds": sec,
            "sample": f"oracle.ssd.ssd_chunked forward + backward, batch 1 x {Hs} of {H} heads x seqlen {L}: {sec:.2f} s "
                      f"(median of 2); tokens/s of the whole workload = {L} x {Hs}/{H} / seconds"}


def cpu_baseline_decode():
    """The decode-step oracle on the host cores: 16 of configuration 3's 256 batch rows, 20 consecutive steps."""
    import torch
    from oracle.step import selective_state_update_oracle
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    rows, batch, H, P, N, steps = 16, 256, 80, 64, 128, 20
    g = torch.Generator().manual_seed(0)
    state = 0.1 * torch.randn(rows, H, P, N, generator=g)
    x, z = (torch.randn(rows, H, P, generator=g).bfloat16() for _ in range(2))
    dt = torch.randn(rows, H, generator=g).bfloat16()[:, :, None].expand(rows, H, P)
    B, C = (torch.randn(rows, 1, N, generator=g).bfloat16() for _ in range(2))
    A = (-(1 + 15 * torch.rand(H, generator=g)))[:, None, None].expand(H, P, N)
    D = torch.rand(H, generator=g)[:, None].expand(H, P)
    dtb = (torch.rand(H, generator=g) - 4)[:, None].expand(H, P)
    one = lambda: selective_state_update_oracle(state, x, dt, A, B, C, D=D, z=z, dt_bias=dtb, dt_softplus=True)
    one()
    t0 = time.perf_counter()
    for _ in range(steps):
        one()
    sec = (time.perf_counter() - t0) / steps
    return {"value": rows / sec, "unit": "tokens/s", "cores": cores, "kind": "port", "slice_seconds_per_step": sec,
            "sample": f"oracle.step.selective_state_update_oracle, {rows} of {batch} batch rows, {steps} consecutive "
                      f"steps: {sec * 1e3:.1f} ms per step; batch rows are independent, so tokens/s = rows / seconds"}


def measured_copy(dev):
    """Runs mamba_hip_copy (one 16-byte element per thread) over 1 GiB: 1 GiB read + 1 GiB written.
    Returns (ms per launch, GB/s): the streaming rate this GPU sustains, beside the published peak."""
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
    return ms, 2 * nbytes / ms / 1e6


def measured_row_pass(dev, batch, seqlen, nheads, n_in):
    """Runs mamba_hip_rows_probe: a bare pass over (batch, seqlen, nheads, 64) bf16 tensors in the order the SSD
    kernels visit them (one workgroup per (batch, 256 positions, head); 128-byte rows, nheads * 128 bytes from one
    position to the next), n_in tensors read and two written.  Returns GB/s: what the layout allows a kernel that
    touches every row once, beside the rate of the linear copy."""
    import ctypes
    import torch
    from mamba_amd import _lib
    seqlen = seqlen // 256 * 256
    t = [torch.empty(batch, seqlen, nheads, 64, dtype=torch.bfloat16, device=dev).fill_(1.0) for _ in range(n_in + 2)]
    ins = (ctypes.c_void_p * n_in)(*[x.data_ptr() for x in t[:n_in]])
    outs = (ctypes.c_void_p * 2)(*[x.data_ptr() for x in t[n_in:]])
    lib = _lib.load()
    stream = _lib.current_stream(dev)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    nbytes = 0
    for i in range(11):
        if i == 1:
            ev[0].record()
        nbytes = lib.mamba_hip_rows_probe(ins, n_in, outs, batch, seqlen, nheads, stream)
        if nbytes <= 0:
            _lib.check(int(nbytes), "mamba_hip_rows_probe")
    ev[1].record()
    torch.cuda.synchronize()
    return nbytes / (ev[0].elapsed_time(ev[1]) / 10) / 1e6


def vs_row_pass(roofline, dev, batch, seqlen, nheads, n_in, moved_bytes):
    """Adds the rate of the bare row pass with this problem's layout (n_in row tensors read, two written) and the
    kernel's own rate over the bytes it moves (`moved_bytes` per launch) as a fraction of it."""
    gbs = measured_row_pass(dev, batch, seqlen, nheads, n_in)
    roofline["row_pass"] = {"gbs": gbs, "tensors_read": n_in, "tensors_written": 2,
                            "kernel_moved_bytes": moved_bytes,
                            "kernel_gbs": moved_bytes / roofline["kernel_ms"] / 1e6,
                            "frac_of_row_pass": moved_bytes / roofline["kernel_ms"] / 1e6 / gbs}
    return roofline


def copy_calibration(dev):
    ms, gbs = measured_copy(dev)
    print(json.dumps({"kernel": "copy_kernel", "bytes_read": 1 << 30, "bytes_written": 1 << 30, "ms": ms, "GB/s": gbs}))


def measured_mfma(dev):
    """TFLOP/s of mamba_hip_mfma_probe: independent bf16 MFMA chains on register operands, 8 workgroups per CU."""
    import torch
    from mamba_amd import _lib
    lib = _lib.load()
    stream = _lib.current_stream(dev)
    sink = torch.zeros(1, device=dev)
    blocks = 8 * torch.cuda.get_device_properties(dev).multi_processor_count
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    flops = 0
    for i in range(4):
        if i == 1:
            ev[0].record()
        flops = lib.mamba_hip_mfma_probe(sink.data_ptr(), 512, blocks, stream)
        if flops <= 0:
            _lib.check(int(flops), "mamba_hip_mfma_probe")
    ev[1].record()
    torch.cuda.synchronize()
    return flops / (ev[0].elapsed_time(ev[1]) / 3) / 1e9


def measured_valu(dev):
    """Per-lane v_fma_f32 instructions per second of mamba_hip_valu_probe (16 independent chains per lane,
    8 workgroups of 4 waves per CU), in T/s."""
    import torch
    from mamba_amd import _lib
    lib = _lib.load()
    stream = _lib.current_stream(dev)
    sink = torch.zeros(1, device=dev)
    blocks = 8 * torch.cuda.get_device_properties(dev).multi_processor_count
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    n = 0
    for i in range(4):
        if i == 1:
            ev[0].record()
        n = lib.mamba_hip_valu_probe(sink.data_ptr(), 2048, blocks, stream)
        if n <= 0:
            _lib.check(int(n), "mamba_hip_valu_probe")
    ev[1].record()
    torch.cuda.synchronize()
    return n / (ev[0].elapsed_time(ev[1]) / 3) / 1e9


def vs_measured_copy(roofline, dev):
    """Adds the streaming-copy rate measured in this run and the kernel's fraction of it."""
    _, gbs = measured_copy(dev)
    roofline["measured_copy_gbs"] = gbs
    roofline["frac_of_measured_copy"] = roofline["achieved"] / gbs
    return roofline


KERNEL_ITERS = 100  # launches per event-timed kernel or pass; the median is reported


def event_stats(fn, n=None, pre=None):
    """HIP-event times of n single calls of fn() on torch's current stream (where the library launches), each
    call in its own event pair; pre() runs outside the pairs.  Returns {"median", "min", "max", "n"} in ms."""
    import statistics
    import torch
    n = n or KERNEL_ITERS
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
    ts = [a.elapsed_time(b) for a, b in ev]
    return {"median": statistics.median(ts), "min": min(ts), "max": max(ts), "n": n}


def event_ms(fn, n=None, pre=None):
    """Median HIP-event time of one call of fn(), in ms."""
    return event_stats(fn, n, pre)["median"]


def timed_steps(step, steps, warmup):
    """The contract's timing: `warmup` untimed steps, then exactly `steps` steps between two device
    synchronisations; returns seconds per step.  Then every step of a second pass of max(steps, KERNEL_ITERS)
    steps in its own event pair: {"median", "min", "max", "n"} in ms."""
    import torch
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / steps
    return sec, event_stats(step, max(steps, KERNEL_ITERS))


def bench_ssd(dev, steps, warmup):
    """Mamba-2 SSD: mamba_chunk_scan_combined forward + backward; the roofline entry is the fused
    C B^T + chunk_scan forward kernel, which is HBM-bound (65 flop per byte against 312 at the ridge)."""
    import torch
    from mamba_amd import _lib
    from mamba_amd.ops.triton import ssd_combined as sc
    batch, L, H, P, N, G, Q = 4, 4096, 80, 64, 128, 1, 256
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    x, z = (rn(batch, L, H, P).to(bf).requires_grad_() for _ in range(2))
    B, C = (rn(batch, L, G, N).to(bf).requires_grad_() for _ in range(2))
    dt = rn(batch, L, H).to(bf).requires_grad_()
    A = (-(1 + 15 * torch.rand(H, device=dev, generator=g))).requires_grad_()
    D = torch.rand(H, device=dev, generator=g).requires_grad_()
    dtb = (torch.rand(H, device=dev, generator=g) - 4).requires_grad_()
    dout = rn(batch, L, H, P).to(bf)
    leaves = (x, z, B, C, dt, A, D, dtb)

    def fwd():
        return sc.mamba_chunk_scan_combined(x, dt, A, B, C, Q, D=D, z=z, dt_bias=dtb, dt_softplus=True)

    def step():
        for v in leaves:
            v.grad = None
        fwd().backward(dout)

    sec, step_stats = timed_steps(step, steps, warmup)
    # the same step in the deterministic mode (integer atomics on fixed-point terms in the backward pass)
    from mamba_amd.utils.determinism import set_deterministic_mode
    set_deterministic_mode(True)
    try:
        step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(max(3, steps // 4)):
            step()
        torch.cuda.synchronize()
        det_sec = (time.perf_counter() - t0) / max(3, steps // 4)
    finally:
        set_deterministic_mode(None)
    with torch.no_grad():
        fwd_ms = event_ms(fwd)
        # the fused scan kernel alone, on the buffers of one forward pass
        lib = _lib.load()
        a = sc._prepare(x, dt, A, B, C, Q, D, z, dtb, None, None)
        ws = sc._workspace(a[0], a[3], Q)
        out, out_x = torch.empty_like(a[0]), torch.empty_like(a[0])
        p = _lib.SsdParams()
        sc._fill_fwd(p, a[0], a[1], a[2], a[3], a[4], Q, a[5], a[6], a[7], None, None, True, (0.0, float("inf")), ws)
        p.out, p.out_x = out.data_ptr(), out_x.data_ptr()
        p.out_bs, p.out_ls, p.out_hs = out.stride(0), out.stride(1), out.stride(2)
        stream = _lib.current_stream(dev)
        _lib.check(lib.ssd_combined_fwd(p, stream), "ssd_combined_fwd")   # fills dA_cumsum and the chunk states
        scan = event_stats(lambda: _lib.check(lib.ssd_chunk_scan_fwd_fused(p, stream), "ssd_chunk_scan_fwd_fused"))
        scan_ms = scan["median"]
    nc = L // Q
    mfma_tflops = measured_mfma(dev)
    flops = batch * nc * (H * (Q * Q * P + 2 * Q * N * P) + G * Q * Q * N)   # causal halves counted once
    nbytes = 2 * (4 * batch * L * H * P + 2 * batch * L * G * N) + 2 * batch * nc * H * P * N  # x z out out_x B C, bf16 states
    prof = "ssd_combined_b4_l4096_h80_p64_n128_q256_bf16"
    step_bytes = 2 * (8 * batch * L * H * P + 6 * batch * L * G * N + 3 * batch * L * H)  # fwd+bwd: 8 X + 6 BC + 3 T
    return ({
        "metric": "SSD mamba_chunk_scan_combined fwd+bwd tokens/s at 1 GPU", "value": batch * L / sec,
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": sec * 1e3,
        "step_ms": step_stats, "fwd_ms": fwd_ms, "deterministic_ms_per_step": det_sec * 1e3, "higher_is_better": True,
        "step_roofline": {"bound": "hbm", "algorithmic_bytes": step_bytes, "achieved": step_bytes / sec / 1e9,
                          "frac": step_bytes / sec / 1e9 / HBM_PEAK_GBS, "unit": "GB/s",
                          "traffic": profile_traffic_sum(prof + "_hbm_counters.txt")},
        "dtype": "bf16 in/out, fp32 accumulation", "data": "synthetic",
        "config": {"workload": f"Mamba-2 SSD fwd+bwd: batch {batch}, seqlen {L}, {H} heads x {P}, d_state {N}, "
                               f"{G} group, chunk {Q}, bf16 (benchmark configuration 2)"},
        "roofline": vs_row_pass(vs_measured_copy({"bound": "hbm", "kernel": "chunk_scan_fwd_paired_kernel", "achieved": nbytes / scan_ms / 1e6,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / scan_ms / 1e6 / HBM_PEAK_GBS,
                     "traffic": profile_traffic(prof + "_hbm_counters.txt", "chunk_scan_fwd_paired_kernel"),
                     "kernel_ms": scan_ms, "kernel_ms_min_max_n": [scan["min"], scan["max"], scan["n"]],
                     "algorithmic_bytes": nbytes,
                     "algorithmic_flops": flops, "mfma_tflops": flops / scan_ms / 1e9,
                     "mfma_frac_of_bf16_peak": flops / scan_ms / 1e9 / 2500.0,
                     # the kernel moves `algorithmic_bytes` for `algorithmic_flops`: at the HBM peak that caps it at
                     "flop_per_byte": flops / nbytes, "mfma_cap_from_hbm_tflops": flops / nbytes * HBM_PEAK_GBS / 1e3,
                     "measured_mfma_tflops": mfma_tflops,
                     "mfma_frac_of_measured": flops / scan_ms / 1e9 / mfma_tflops,
                     "mfma_counters": mfma_counters(prof + "_mfma_counters.txt", "chunk_scan_fwd_paired_kernel")}, dev),
                     dev, batch, L, H, 2, nbytes)})


def mfma_counters(filename, kernel):
    """Matrix-core counters of `kernel` from profiles/<filename> (per launch, summed over the chip): bf16 MFMA
    instructions, and the share of the busy cycles of the compute units in which their matrix cores were
    executing (one matrix core per SIMD, four SIMDs per compute unit)."""
    n = profile_counter(filename, kernel, "SQ_INSTS_VALU_MFMA_BF16")
    busy = profile_counter(filename, kernel, "SQ_VALU_MFMA_BUSY_CYCLES")
    cu = profile_counter(filename, kernel, "SQ_BUSY_CU_CYCLES")
    if n is None or busy is None or cu is None:
        return None
    return {"mfma_bf16_instructions": n, "mfma_busy_cycles": busy, "cu_busy_cycles": cu,
            "mfma_busy_frac_of_cu_busy": busy / (4 * cu) if cu else None}


def bench_decode(dev, steps, warmup, batch=256):
    """Decode: `steps` consecutive selective_state_update calls in place on one state (fp32), the inputs of
    step i taken from a ring of 8 pre-generated sets; the state is read and written once per step."""
    import torch
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    H, P, N, G = 80, 64, 128, 1
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    state = 0.1 * rn(batch, H, P, N)
    ring = [dict(x=rn(batch, H, P).to(bf), z=rn(batch, H, P).to(bf),
                 dt=rn(batch, H).to(bf)[:, :, None].expand(batch, H, P),
                 B=rn(batch, G, N).to(bf), C=rn(batch, G, N).to(bf)) for _ in range(8)]
    A = (-(1 + 15 * torch.rand(H, device=dev, generator=g)))[:, None, None].expand(H, P, N)
    D = torch.rand(H, device=dev, generator=g)[:, None].expand(H, P)
    dtb = (torch.rand(H, device=dev, generator=g) - 4)[:, None].expand(H, P)

    def one(i):
        r = ring[i & 7]
        return selective_state_update(state, r["x"], r["dt"], A, r["B"], r["C"], D=D, z=r["z"], dt_bias=dtb,
                                      dt_softplus=True)

    for i in range(warmup):
        one(i)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        one(i)
    ev[1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) / steps * 1e3
    ms = ev[0].elapsed_time(ev[1]) / steps
    x = ring[0]["x"]
    nbytes = 2 * state.numel() * 4 + 2 * (3 * x.numel() + 2 * ring[0]["B"].numel()) + 2 * batch * H
    return ({
        "metric": "decode selective_state_update tokens/s at 1 GPU", "value": batch / wall_ms * 1e3, "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": wall_ms, "event_ms_per_step": ms,
        "higher_is_better": True, "dtype": "fp32 state, bf16 x/z/B/C/dt", "data": "synthetic",
        "state_finite": bool(torch.isfinite(state).all()),
        "config": {"workload": f"selective_state_update: batch {batch}, {H} heads x {P}, d_state {N}, {G} group, "
                               f"tied A/dt/D per head, {steps} consecutive in-place steps (benchmark configuration 3)"},
        "roofline": vs_measured_copy({"bound": "hbm", "kernel": "state_update_kernel", "achieved": nbytes / ms / 1e6,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / ms / 1e6 / HBM_PEAK_GBS,
                     "traffic": profile_traffic("state_update_b256_h80_p64_n128_bf16_hbm_counters.txt", "state_update_kernel") if batch == 256 else None,
                     "kernel_ms": ms, "algorithmic_bytes": nbytes}, dev)})


def bench_decode_step(dev, steps, warmup, batch):
    """One generated token of a Mamba-2 layer's mixer core, as the reference's step() runs it
    (mamba_ssm/modules/mamba2.py:298-336): causal_conv1d_update over the x/B/C channels, then
    selective_state_update.  Reports wall time per token of the two launches eager and replayed from a
    captured HIP graph, and of each kernel alone in a graph: a single fused kernel cannot be faster than
    the state update alone, so `graph_two_launches - graph_state_update_only` bounds what fusing saves,
    and `eager - graph` is the host side's share (argument checks + parameter fill through ctypes)."""
    import torch
    from mamba_amd.ops.causal_conv1d import causal_conv1d_update
    from mamba_amd.ops.triton.selective_state_update import selective_state_update, mamba2_decode_step
    H, P, N, G, W = 80, 64, 128, 1, 4
    dim, conv_dim = H * P, H * P + 2 * G * N
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    ssm_state = 0.1 * rn(batch, H, P, N)
    conv_state = rn(batch, W, conv_dim).to(bf).transpose(1, 2)   # channel-contiguous, as the reference allocates it
    conv_w, conv_b = (0.4 * rn(conv_dim, W)).to(bf), (0.1 * rn(conv_dim)).to(bf)
    xBC, z, dt = rn(batch, conv_dim).to(bf), rn(batch, H, P).to(bf), rn(batch, H).to(bf)
    A = (-(1 + 15 * torch.rand(H, device=dev, generator=g)))[:, None, None].expand(H, P, N)
    D = torch.rand(H, device=dev, generator=g)[:, None].expand(H, P)
    dtb = (torch.rand(H, device=dev, generator=g) - 4)[:, None].expand(H, P)
    xc0 = rn(batch, conv_dim).to(bf)
    Ah, Dh, dtbh = A[:, 0, 0].contiguous(), D[:, 0].contiguous(), dtb[:, 0].contiguous()

    def fused():
        return mamba2_decode_step(ssm_state, conv_state, xBC, dt, Ah, conv_w, conv_b, D=Dh, z=z, dt_bias=dtbh, ngroups=G,
                                  fuse=True)

    def conv():
        return causal_conv1d_update(xBC, conv_state, conv_w, conv_b, "silu")

    def ssm(xc):
        xs, B, C = torch.split(xc, [dim, G * N, G * N], dim=-1)
        return selective_state_update(ssm_state, xs.reshape(batch, H, P), dt[:, :, None].expand(batch, H, P), A,
                                      B.reshape(batch, G, N), C.reshape(batch, G, N), D=D, z=z, dt_bias=dtb,
                                      dt_softplus=True)

    variants = {"two_launches": lambda: ssm(conv()), "fused": fused, "state_update_only": lambda: ssm(xc0),
                "conv_update_only": conv}

    def wall(fn, n):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e6

    out = {}
    with torch.no_grad():
        for name, fn in variants.items():
            for _ in range(warmup):
                fn()
            out["eager_us_" + name] = wall(fn, steps)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                fn()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(10):   # ten tokens per replay, so that the replay's own launch cost is shared
                    fn()
            graph.replay()
            out["graph_us_" + name] = wall(graph.replay, max(steps // 10, 20)) / 10
    out["fusion_bound_us"] = out["graph_us_two_launches"] - out["graph_us_state_update_only"]
    out["fused_gain_us"] = out["graph_us_two_launches"] - out["graph_us_fused"]
    out["host_share_us"] = out["eager_us_two_launches"] - out["graph_us_two_launches"]
    return {"metric": "decode step (conv update + state update) wall time per token", "unit": "us", "batch": batch,
            "value": out["graph_us_two_launches"], "higher_is_better": False, "steps": steps, "n_gpus": 1,
            "config": {"workload": f"causal_conv1d_update ({conv_dim} channels, width {W}) + selective_state_update: "
                                   f"batch {batch}, {H} heads x {P}, d_state {N}, bf16 inputs, fp32 state"},
            **out}


def bench_varlen(dev, steps, warmup):
    """Configuration 4: one packed row of 16 sequences (lengths uniform in [512, 4096], rescaled to sum to
    32768), seq_idx, nonzero initial states, final states returned; forward + backward."""
    import torch
    from mamba_amd.ops.triton import ssd_combined as sc
    batch, L, H, P, N, G, Q, nseq = 1, 32768, 64, 64, 128, 8, 256, 16
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    x, z = (rn(batch, L, H, P).to(bf).requires_grad_() for _ in range(2))
    B, C = (rn(batch, L, G, N).to(bf).requires_grad_() for _ in range(2))
    dt = rn(batch, L, H).to(bf).requires_grad_()
    A = (-(1 + 15 * torch.rand(H, device=dev, generator=g))).requires_grad_()
    D = torch.rand(H, device=dev, generator=g).requires_grad_()
    dtb = (torch.rand(H, device=dev, generator=g) - 4).requires_grad_()
    init = (0.1 * rn(batch, H, P, N)).requires_grad_()
    dout = rn(batch, L, H, P).to(bf)
    lens = torch.randint(512, 4097, (nseq,), generator=torch.Generator().manual_seed(0)).double()
    lens = (lens / lens.sum() * L).long()
    lens[-1] += L - lens.sum()
    seq_idx = torch.cat([torch.full((int(n),), i, dtype=torch.int32) for i, n in enumerate(lens)])[None].to(dev)
    leaves = (x, z, B, C, dt, A, D, dtb, init)

    def fwd():
        return sc.mamba_chunk_scan_combined(x, dt, A, B, C, Q, D=D, z=z, dt_bias=dtb, initial_states=init,
                                            seq_idx=seq_idx, dt_softplus=True, return_final_states=True)

    def step():
        for v in leaves:
            v.grad = None
        fwd()[0].backward(dout)

    sec, step_stats = timed_steps(step, steps, warmup)
    with torch.no_grad():
        fwd_ms = event_ms(fwd)
        # the fused scan kernel alone (the kernel the roofline entry of configuration 2 names), on the buffers of one
        # forward pass of this packed problem
        from mamba_amd import _lib
        lib = _lib.load()
        a = sc._prepare(x, dt, A, B, C, Q, D, z, dtb, init, seq_idx)
        ws = sc._workspace(a[0], a[3], Q)
        out, out_x = torch.empty_like(a[0]), torch.empty_like(a[0])
        p = _lib.SsdParams()
        sc._fill_fwd(p, a[0], a[1], a[2], a[3], a[4], Q, a[5], a[6], a[7], a[8], a[9], True, (0.0, float("inf")), ws)
        p.out, p.out_x = out.data_ptr(), out_x.data_ptr()
        p.out_bs, p.out_ls, p.out_hs = out.stride(0), out.stride(1), out.stride(2)
        stream = _lib.current_stream(dev)
        _lib.check(lib.ssd_combined_fwd(p, stream), "ssd_combined_fwd")
        scan = event_stats(lambda: _lib.check(lib.ssd_chunk_scan_fwd_fused(p, stream), "ssd_chunk_scan_fwd_fused"))
    nc = L // Q
    scan_bytes = 2 * (4 * batch * L * H * P + 2 * batch * L * G * N) + 2 * batch * nc * H * P * N
    flops = batch * nc * (H * (Q * Q * P + 2 * Q * N * P) + G * Q * Q * N)
    # fwd+bwd, bf16: reads x, z (fwd), x, z, dout (bwd), writes out, dx, dz = 8 X; B, C read twice + dB, dC = 6 BC; dt 3 T
    step_bytes = 2 * (8 * batch * L * H * P + 6 * batch * L * G * N + 3 * batch * L * H)
    prof = "ssd_varlen_b1_l32768_h64_p64_n128_g8_q256_bf16"
    scan_ms = scan["median"]
    return ({
        "metric": "SSD mamba_chunk_scan_combined packed varlen fwd+bwd tokens/s at 1 GPU", "value": batch * L / sec,
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": sec * 1e3,
        "step_ms": step_stats, "fwd_ms": fwd_ms, "higher_is_better": True, "dtype": "bf16 in/out, fp32 accumulation",
        "data": "synthetic",
        "config": {"workload": f"Mamba-2 SSD fwd+bwd, packed: 1 row of {nseq} sequences, {L} positions, {H} heads x {P}, "
                               f"d_state {N}, {G} groups, chunk {Q}, initial + final states (benchmark configuration 4)"},
        "step_roofline": {"bound": "hbm", "algorithmic_bytes": step_bytes, "achieved": step_bytes / sec / 1e9,
                          "frac": step_bytes / sec / 1e9 / HBM_PEAK_GBS, "unit": "GB/s",
                          "traffic": profile_traffic_sum(prof + "_hbm_counters.txt")},
        "roofline": vs_row_pass(vs_measured_copy({"bound": "hbm", "kernel": "chunk_scan_fwd_paired_kernel",
                     "achieved": scan_bytes / scan_ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": scan_bytes / scan_ms / 1e6 / HBM_PEAK_GBS,
                     "traffic": profile_traffic(prof + "_hbm_counters.txt", "chunk_scan_fwd_paired_kernel"),
                     "kernel_ms": scan_ms, "kernel_ms_min_max_n": [scan["min"], scan["max"], scan["n"]],
                     "algorithmic_bytes": scan_bytes, "algorithmic_flops": flops,
                     "mfma_tflops": flops / scan_ms / 1e9, "mfma_frac_of_bf16_peak": flops / scan_ms / 1e9 / 2500.0}, dev),
                     dev, batch, L, H, 2, scan_bytes)})


def bench_inner(dev, steps, warmup):
    """mamba_inner_fn forward + backward: conv1d + SiLU, x_proj, dt_proj, selective scan, out_proj."""
    import torch
    from mamba_amd.ops.selective_scan_interface import mamba_inner_fn
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fwd
    batch, L, dm, di, N, W = 8, 4096, 2560, 5120, 16, 4
    R = math.ceil(dm / 16)
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    xz = rn(batch, 2 * di, L).to(bf).requires_grad_()
    conv_w = (0.3 * rn(di, 1, W)).to(bf).requires_grad_()
    conv_b = (0.1 * rn(di)).to(bf).requires_grad_()
    x_proj = (rn(R + 2 * N, di) / math.sqrt(di)).to(bf).requires_grad_()
    dt_proj = (rn(di, R) / math.sqrt(R)).to(bf).requires_grad_()
    out_proj = (rn(dm, di) / math.sqrt(di)).to(bf).requires_grad_()
    A = (-torch.arange(1, N + 1, device=dev, dtype=torch.float32)[None].repeat(di, 1)).requires_grad_()
    D = torch.ones(di, device=dev).requires_grad_()
    dtb = (torch.rand(di, device=dev, generator=g) - 4).requires_grad_()
    dout = rn(batch, L, dm).to(bf)
    leaves = (xz, conv_w, conv_b, x_proj, dt_proj, out_proj, A, D, dtb)

    def fwd():
        return mamba_inner_fn(xz, conv_w, conv_b, x_proj, dt_proj, out_proj, None, A, None, None, D,
                              delta_bias=dtb, delta_softplus=True)

    def step():
        for v in leaves:
            v.grad = None
        fwd().backward(dout)

    sec, step_stats = timed_steps(step, steps, warmup)
    with torch.no_grad():
        fwd_ms = event_ms(fwd)
        xin = xz[:, :di]
        cw = conv_w.squeeze(1)
        conv_ms = event_ms(lambda: causal_conv1d_fwd(xin, cw, conv_b, activation="silu"))
    nbytes = 2 * 2 * batch * di * L   # the convolution reads x and writes its output once
    return ({
        "metric": "mamba_inner_fn fwd+bwd tokens/s at 1 GPU", "value": batch * L / sec, "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": sec * 1e3, "step_ms": step_stats, "fwd_ms": fwd_ms,
        "higher_is_better": True, "dtype": "bf16 in/out, fp32 state and accumulation", "data": "synthetic",
        "config": {"workload": f"mamba_inner_fn fwd+bwd: batch {batch}, seqlen {L}, d_model {dm}, d_inner {di}, "
                               f"d_state {N}, dt_rank {R}, conv width {W}"},
        "roofline": vs_measured_copy({"bound": "hbm", "kernel": "conv_rows_fwd_kernel", "achieved": nbytes / conv_ms / 1e6,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / conv_ms / 1e6 / HBM_PEAK_GBS,
                     "traffic": None, "kernel_ms": conv_ms, "algorithmic_bytes": nbytes}, dev)})


def bench_block(dev, steps, warmup):
    """mamba_split_conv1d_scan_combined forward + backward: the Mamba-2 block body after in_proj."""
    import torch
    from mamba_amd.ops.triton.ssd_combined import mamba_split_conv1d_scan_combined
    from mamba_amd.ops.triton.layernorm_gated import _layer_norm_fwd
    batch, L, H, P, N, G, Q, W = 4, 4096, 80, 64, 128, 1, 256, 4
    dim = H * P
    dm = dim // 2
    width = 2 * dim + 2 * G * N + H
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    zxbcdt = (0.5 * rn(batch, L, width)).to(bf).requires_grad_()
    conv_w = (0.3 * rn(dim + 2 * G * N, W)).requires_grad_()
    conv_b = (0.1 * rn(dim + 2 * G * N)).requires_grad_()
    dtb = (torch.rand(H, device=dev, generator=g) - 4).requires_grad_()
    A = (-(1 + 15 * torch.rand(H, device=dev, generator=g))).requires_grad_()
    D = torch.rand(H, device=dev, generator=g).requires_grad_()
    norm_w = torch.ones(dim, device=dev).requires_grad_()
    out_w = (rn(dm, dim) / math.sqrt(dim)).to(bf).requires_grad_()
    dout = rn(batch, L, dm).to(bf)
    leaves = (zxbcdt, conv_w, conv_b, dtb, A, D, norm_w, out_w)

    def fwd():
        return mamba_split_conv1d_scan_combined(zxbcdt, conv_w, conv_b, dtb, A, D, Q, rmsnorm_weight=norm_w,
                                                outproj_weight=out_w, headdim=P, ngroups=G, norm_before_gate=False)

    def step():
        for v in leaves:
            v.grad = None
        fwd().backward(dout)

    sec, step_stats = timed_steps(step, steps, warmup)
    with torch.no_grad():
        fwd_ms = event_ms(fwd)
        y = rn(batch * L, dim).to(bf)
        zz = rn(batch * L, dim).to(bf)
        norm_ms = event_ms(lambda: _layer_norm_fwd(y, norm_w, None, 1e-6, z=zz, group_size=dim // G,
                                                   norm_before_gate=False, is_rms_norm=True))
    nbytes = 3 * 2 * batch * L * dim   # the gated norm reads y and z and writes its output once
    return ({
        "metric": "mamba_split_conv1d_scan_combined fwd+bwd tokens/s at 1 GPU", "value": batch * L / sec,
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": sec * 1e3, "step_ms": step_stats, "fwd_ms": fwd_ms,
        "higher_is_better": True, "dtype": "bf16 in/out, fp32 accumulation", "data": "synthetic",
        "config": {"workload": f"Mamba-2 block body fwd+bwd: batch {batch}, seqlen {L}, {H} heads x {P}, d_state {N}, "
                               f"{G} group, chunk {Q}, conv width {W}, gated RMSNorm, out_proj to {dm}"},
        "roofline": vs_measured_copy({"bound": "hbm", "kernel": "norm_fwd_wide_kernel", "achieved": nbytes / norm_ms / 1e6,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / norm_ms / 1e6 / HBM_PEAK_GBS,
                     "traffic": None, "kernel_ms": norm_ms, "algorithmic_bytes": nbytes}, dev)})


def bench_mamba1(dev, steps, warmup):
    """The headline workload: selective_scan_fn forward + backward at benchmark configuration 1."""
    import torch
    from mamba_amd.ops import selective_scan_interface as ssi
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn, selective_scan_fwd
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

    sec, step_stats = timed_steps(step, steps, warmup)
    ms_per_step = sec * 1e3
    tokens_per_s = batch * seqlen / sec

    # Dominant kernel (the backward scan, with the two small kernels that add up its dB / dC partials) alone,
    # HIP events on the launch stream.
    with torch.no_grad():
        d = {k: v.detach() for k, v in leaves.items()}
        _, ckpt = selective_scan_fwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["z"], d["delta_bias"], True)
        dims = (batch, dim, seqlen, dstate, 1)
        bwd_args = (d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["z"], d["delta_bias"], t["dout"], ckpt, True, dims)
        bufs = ssi.scan_bwd_launch(*bwd_args)
        bwd = lambda: ssi.scan_bwd_launch(*bwd_args, bufs=bufs)
        fwd = lambda: selective_scan_fwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["z"], d["delta_bias"], True)
        bwd_st, fwd_st = event_stats(bwd), event_stats(fwd)
        bwd_ms, fwd_ms = bwd_st["median"], fwd_st["median"]
    es = 2  # bf16
    E = batch * dim * seqlen * es
    BC = batch * dstate * seqlen * es
    bwd_bytes = 7 * E + 4 * BC   # reads u, delta, z, dout, B, C; writes du, ddelta, dz, dB, dC
    fwd_bytes = 4 * E + 2 * BC   # reads u, delta, z, B, C; writes out
    achieved = bwd_bytes / (bwd_ms * 1e-3) / 1e9
    prof = "mamba1_scan_b8_d5120_l4096_n16_bf16"
    roofline = {"bound": "hbm", "kernel": "scan_bwd_kernel (+ reduce_parts_kernel x 2)", "achieved": achieved,
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                "traffic": profile_traffic(prof + "_hbm_counters.txt", "scan_bwd_kernel"),
                "kernel_ms": bwd_ms, "kernel_ms_min_max_n": [bwd_st["min"], bwd_st["max"], bwd_st["n"]],
                "algorithmic_bytes": bwd_bytes,
                "fwd_kernel_ms": fwd_ms, "fwd_kernel_ms_min_max_n": [fwd_st["min"], fwd_st["max"], fwd_st["n"]], "fwd_achieved": fwd_bytes / (fwd_ms * 1e-3) / 1e9,
                "fwd_traffic": profile_traffic(prof + "_hbm_counters.txt", "scan_fwd_kernel"),
                "fwd_bwd_frac": (fwd_bytes + bwd_bytes) / ((fwd_ms + bwd_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS}
    vs_measured_copy(roofline, dev)
    # The binding resource of both scan kernels is fp32 vector-ALU issue, not HBM.  A SIMD issues one plain
    # wave64 fp32 instruction every 2 cycles when at least two of its waves are ready (one wave alone: every 4),
    # which is the published 157.3 TFLOP/s = 78.6 T lane-FMA/s; a transcendental (v_exp_f32) holds the port four
    # times as long (measured: 19 T/s).  Slots per (position, channel, state) = the VALU instruction count of the
    # committed counter profile with every transcendental counted four times, over the event time of this run,
    # beside the rate a bare v_fma_f32 loop reaches in this run.
    elems = batch * dim * seqlen * dstate
    probe = measured_valu(dev)
    valu = {"unit": "T lane-instruction slots/s", "measured_fma_probe": probe,
            "nominal_peak": 256 * 4 * 32 * 2.4e9 / 1e12, "element_states": elems}
    for name, ms in (("bwd", bwd_ms), ("fwd", fwd_ms)):
        kern = "scan_%s_kernel" % name
        insts = profile_counter(prof + "_valu_counters.txt", kern, "SQ_INSTS_VALU")
        trans = profile_counter(prof + "_valu_counters.txt", kern, "SQ_INSTS_VALU_TRANS_F32")
        if insts is None or trans is None:
            valu[name] = None
            continue
        slots = (insts + 3 * trans) * 64 / elems
        valu[name] = {"valu_instructions_per_element_state": insts * 64 / elems,
                      "transcendentals_per_element_state": trans * 64 / elems,
                      "slots_per_element_state": slots, "achieved": slots * elems / (ms * 1e-3) / 1e12,
                      "frac_of_probe": slots * elems / (ms * 1e-3) / 1e12 / probe}
    roofline["valu"] = valu
    roofline["profile_is_of_these_sources"] = profile_fresh(prof + "_hbm_counters.txt")
    return {
        "metric": "scan fwd+bwd tokens/s at 1 GPU; achieved HBM GB/s and % bf16 MFMA peak",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "step_ms": step_stats, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 in/out, fp32 state and accumulation", "data": "synthetic",
        "config": {"workload": "Mamba-1 selective_scan_fn fwd+bwd: batch 8, d_inner 5120, seqlen 4096, d_state 16, "
                               "bf16 u/delta/B/C/z, fp32 A/D/delta_bias (benchmark configuration 1)",
                   "global_batch": batch, "seq_len": seqlen},
        "roofline": roofline,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true",
                    help="headline workload only: leave out the SSD, decode and packed-SSD lines under `extra`")
    ap.add_argument("--workload", choices=("mamba1", "ssd", "decode", "decode_step", "varlen", "inner", "block"), default="mamba1")
    ap.add_argument("--batch", type=int, default=256, help="batch of --workload decode")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run the library's plain copy kernel over 1 GiB (yardstick for HBM counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the scan has no cross-GPU exchange step); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.copy_calibration:
        copy_calibration(dev)
        return
    if args.workload == "decode":
        print(json.dumps(bench_decode(dev, max(args.steps, 1000), args.warmup, args.batch)))
        return
    if args.workload == "decode_step":
        print(json.dumps(bench_decode_step(dev, max(args.steps, 200), args.warmup, args.batch)))
        return
    if args.workload != "mamba1":
        fn = {"ssd": bench_ssd, "varlen": bench_varlen, "inner": bench_inner, "block": bench_block}[args.workload]
        print(json.dumps(fn(dev, args.steps, args.warmup)))
        return
    result = bench_mamba1(dev, args.steps, args.warmup)
    if not args.no_extra:
        # the other benchmark configurations, timed in the same run (each entry is the line its own
        # --workload prints): configuration 2 (SSD, with the MFMA figures), 3 (decode, 1000 consecutive
        # steps) and 4 (packed SSD)
        keep = ("value", "unit", "ms_per_step", "step_ms", "step_roofline", "fwd_ms", "deterministic_ms_per_step", "event_ms_per_step", "steps",
                "config", "roofline")
        extra = {}
        for name, fn in (("ssd", lambda: bench_ssd(dev, args.steps, args.warmup)),
                         ("decode", lambda: bench_decode(dev, 1000, 10)),
                         ("varlen", lambda: bench_varlen(dev, args.steps, args.warmup))):
            r = fn()
            extra[name] = {k: r[k] for k in keep if k in r}
        result["extra"] = extra
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(4096, 16, 5120)
        if "extra" in result:
            result["extra"]["ssd"]["cpu_baseline"] = cpu_baseline_ssd()
            result["extra"]["decode"]["cpu_baseline"] = cpu_baseline_decode()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
