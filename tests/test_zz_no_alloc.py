"""mamba1_scan_fwd_noalloc (the forward scan with its tile checkpoints in the library's own fixed
buffer) against mamba1_scan_fwd, through the C ABI: bitwise equal outputs and final states on two
calls in a row, the second on a smaller input, so that stale contents of the shared buffer would show."""
import ctypes

import pytest
import torch

from mamba_amd import _lib
from mamba_amd.ops.selective_scan_interface import _fill_common, scan_tile
from oracle.mamba1 import scan_inputs

pytestmark = pytest.mark.gpu

NAMES = ["u", "delta", "A", "B", "C", "D", "z", "delta_bias"]


def _params(t, out, ckpt):
    batch, dim, seqlen = t["u"].shape
    dims = (batch, dim, seqlen, t["A"].shape[1], t["B"].shape[1])
    p = _lib.MambaScanParams()
    _fill_common(p, *[t[k] for k in NAMES], True, ckpt, dims)
    p.out = out.data_ptr()
    p.out_bs, p.out_ds = out.stride(0), out.stride(1)
    return p


def _both(batch, dim, seqlen, dstate, dtype, seed):
    lib = _lib.load()
    t = {k: (v.cuda() if v is not None else None) for k, v in scan_inputs(batch, dim, seqlen, dstate, 1, dtype, seed=seed).items()}
    ntiles = (seqlen + scan_tile() - 1) // scan_tile()
    stream = _lib.current_stream(t["u"].device)
    # existing entry point: caller workspace
    out_a = torch.empty_like(t["u"])
    ckpt = torch.empty(batch, dim, ntiles, dstate, device="cuda", dtype=torch.float32)
    _lib.check(lib.mamba1_scan_fwd(ctypes.byref(_params(t, out_a, ckpt)), stream), "mamba1_scan_fwd")
    # the entry point under test: no workspace; a poisoned dummy stands in for the ignored ckpt pointer
    out_b = torch.empty_like(t["u"])
    last = torch.full((batch, dim, dstate), float("nan"), device="cuda", dtype=torch.float32)
    dummy = torch.full((1,), float("nan"), device="cuda")
    _lib.check(lib.mamba1_scan_fwd_noalloc(ctypes.byref(_params(t, out_b, dummy)), last.data_ptr(), stream),
               "mamba1_scan_fwd_noalloc")
    torch.cuda.synchronize()
    assert torch.isnan(dummy).all()           # p->ckpt is ignored
    assert torch.equal(out_a, out_b)          # same kernels, same arithmetic: bit for bit
    assert torch.equal(ckpt[:, :, -1], last)
    assert torch.isfinite(last).all()


def test_noalloc_forward_matches_twice_second_smaller():
    assert _lib.load().mamba_hip_init() == 0
    _both(2, 96, 2048 + 40, 16, torch.bfloat16, seed=3)   # 5 tiles, ragged tail
    _both(1, 40, 520, 16, torch.float32, seed=4)          # smaller: 2 tiles


def test_noalloc_rejects_requests_beyond_the_buffer():
    lib = _lib.load()
    p = _lib.MambaScanParams()
    p.batch, p.dim, p.seqlen, p.dstate, p.ngroups = 64, 8192, 8192, 16, 1   # 64*8192*16*16*4 B = 512 MiB
    assert lib.mamba1_scan_fwd_noalloc(ctypes.byref(p), None, None) == -2
