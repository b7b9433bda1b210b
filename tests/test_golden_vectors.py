"""Known-answer vectors of tests/golden/vectors.npz (float64 numpy loops written out position by
position, Mamba-1 gradients by central differences; see tests/golden/make_vectors.py).
The CPU tests hold the oracle to them, the GPU tests the HIP kernels through the C ABI."""
import os

import numpy as np
import pytest
import torch

from oracle.mamba1 import selective_scan_oracle
from oracle.ssd import ssd_oracle
from oracle.step import selective_state_update_oracle

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz"))
M1 = ("u", "delta", "A", "B", "C", "D", "z", "delta_bias")


def _t(name, dtype=torch.float64):
    a = torch.from_numpy(V[name])
    return a if a.dtype in (torch.int32, torch.int64) else a.to(dtype)


def _close(name, got, want, rtol, atol):
    got, want = got.detach().double().cpu(), want.double()
    err = (got - want).abs()
    assert bool((err <= atol + rtol * want.abs()).all()), f"{name}: max err {err.max().item():.3e}"


def _mamba1(fn, dtype, device):
    leaves = {k: _t("m1_" + k, dtype).to(device).requires_grad_() for k in M1}
    out, last = fn(*[leaves[k] for k in M1], True, True)
    (out.double() * _t("m1_dout").to(device)).sum().backward()
    return out, last, {k: leaves[k].grad for k in M1}


def test_oracle_mamba1_vectors():
    out, last, grads = _mamba1(lambda *a: selective_scan_oracle(*a, compute_dtype=torch.float64), torch.float64, "cpu")
    _close("out", out, _t("m1_out"), 1e-9, 1e-10)
    _close("last_state", last, _t("m1_last_state"), 1e-9, 1e-10)
    for k in M1:  # central differences with step 1e-6 in float64
        _close("d" + k, grads[k], _t("m1_d" + k), 1e-5, 1e-6)


def _ssd(fn, dtype, device, **kw):
    g = lambda k: _t("ssd_" + k, dtype).to(device)
    return fn(g("x"), g("dt"), g("A"), g("B"), g("C"), D=g("D"), z=g("z"), dt_bias=g("dt_bias"),
              initial_states=g("init"), seq_idx=_t("ssd_seq_idx").to(device), dt_softplus=True,
              return_final_states=True, **kw)


def test_oracle_ssd_vectors():
    out, fin = _ssd(ssd_oracle, torch.float64, "cpu", compute_dtype=torch.float64)
    _close("out", out, _t("ssd_out"), 1e-9, 1e-10)
    _close("final_states", fin, _t("ssd_final_states"), 1e-9, 1e-10)


def _step(fn, dtype, device, **kw):
    g = lambda k: _t("step_" + k, dtype).to(device)
    state = g("state").clone()
    out = fn(state, g("x"), g("dt"), g("A"), g("B"), g("C"), D=g("D"), z=g("z"), dt_bias=g("dt_bias"), dt_softplus=True,
             **kw)
    return state, out


def test_oracle_step_vectors():
    state, out = _step(selective_state_update_oracle, torch.float64, "cpu", compute_dtype=torch.float64)
    _close("state", state, _t("step_new_state"), 1e-9, 1e-10)
    _close("out", out, _t("step_out"), 1e-9, 1e-10)


@pytest.mark.gpu
def test_hip_mamba1_vectors():
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    out, last, grads = _mamba1(selective_scan_fn, torch.float32, "cuda")
    _close("out", out, _t("m1_out"), 6e-4, 2e-3)
    _close("last_state", last, _t("m1_last_state"), 6e-4, 2e-3)
    for k in M1:
        _close("d" + k, grads[k], _t("m1_d" + k), 1e-3, 5e-3)


@pytest.mark.gpu
def test_hip_ssd_vectors():
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    out, fin = _ssd(lambda *a, **k: mamba_chunk_scan_combined(*a[:5], 8, **k), torch.float32, "cuda")
    _close("out", out, _t("ssd_out"), 6e-4, 2e-3)
    _close("final_states", fin, _t("ssd_final_states"), 6e-4, 2e-3)


@pytest.mark.gpu
def test_hip_step_vectors():
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    state, out = _step(selective_state_update, torch.float32, "cuda")
    _close("state", state, _t("step_new_state"), 6e-4, 2e-3)
    _close("out", out, _t("step_out"), 6e-4, 2e-3)
