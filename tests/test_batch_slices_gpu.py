"""Batches beyond what one launch's grid can index are served in slices at the Python level; with the limit
lowered to 2 rows, the sliced call must equal the plain one (outputs, final states and every gradient)."""
import pytest
import torch

from oracle.mamba1 import scan_inputs
from oracle.ssd import ssd_inputs

pytestmark = pytest.mark.gpu


def test_ssd_batch_slices(monkeypatch):
    from mamba_amd.ops.triton import ssd_combined as sc
    batch, L, H, P, N, G, Q = 5, 192, 4, 32, 32, 2, 64
    t = ssd_inputs(batch, L, H, P, N, G, torch.float32, 3, has_init=True)
    names = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states"]

    def run():
        g = {k: t[k].cuda().requires_grad_() for k in names}
        out, fin = sc.mamba_chunk_scan_combined(g["x"], g["dt"], g["A"], g["B"], g["C"], Q, D=g["D"], z=g["z"],
                                                dt_bias=g["dt_bias"], initial_states=g["initial_states"],
                                                dt_softplus=True, return_final_states=True)
        (out * t["dout"].cuda()).sum().add((fin * t["dfinal"].cuda()).sum()).backward()
        return out, fin, g

    out_a, fin_a, ga = run()
    monkeypatch.setattr(sc, "MAX_GRID_ROWS", 2 * H)   # two batch rows per launch
    out_b, fin_b, gb = run()
    assert torch.equal(out_a, out_b) and torch.equal(fin_a, fin_b)
    for k in names:
        assert torch.allclose(ga[k].grad, gb[k].grad, rtol=1e-5, atol=1e-5), k


def test_mamba1_batch_slices(monkeypatch):
    from mamba_amd.ops import selective_scan_interface as ssi
    t = scan_inputs(5, 8, 160, 8, 1, torch.float32, 5)
    names = ["u", "delta", "A", "B", "C", "D", "z", "delta_bias"]

    def run():
        g = {k: t[k].cuda().requires_grad_() for k in names}
        out, last = ssi.selective_scan_fn(*[g[k] for k in names], delta_softplus=True, return_last_state=True)
        out.backward(t["dout"].cuda())
        return out, last, g

    out_a, last_a, ga = run()
    monkeypatch.setattr(ssi, "MAX_GRID_BATCH", 2)
    out_b, last_b, gb = run()
    assert torch.equal(out_a, out_b) and torch.equal(last_a, last_b)
    for k in names:
        assert torch.allclose(ga[k].grad, gb[k].grad, rtol=1e-5, atol=1e-5), k
