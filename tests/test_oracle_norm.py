"""Pins oracle/norm.py (CPU): against the library routines F.layer_norm / F.rms_norm where the
arguments reduce to them, against a per-element Python loop with the gate on either side, and its
autograd gradients by gradcheck in fp64."""
import math

import torch
import torch.nn.functional as F

from oracle.norm import gated_norm_oracle


def _inputs(rows=5, dim=24, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, dim, generator=g, dtype=torch.float64) * 2 + 0.3
    z = torch.randn(rows, dim, generator=g, dtype=torch.float64)
    w = 1 + 0.2 * torch.randn(dim, generator=g, dtype=torch.float64)
    b = torch.randn(dim, generator=g, dtype=torch.float64)
    return x, z, w, b


def test_reduces_to_library_norms():
    x, z, w, b = _inputs()
    assert torch.allclose(gated_norm_oracle(x, w, b, eps=1e-5), F.layer_norm(x, (24,), w, b, 1e-5), atol=1e-12)
    assert torch.allclose(gated_norm_oracle(x, w, None, eps=1e-5, is_rms_norm=True), F.rms_norm(x, (24,), w, 1e-5), atol=1e-12)
    grouped = gated_norm_oracle(x, w, b, eps=1e-5, group_size=8)
    lib = F.layer_norm(x.reshape(5, 3, 8), (8,), None, None, 1e-5).reshape(5, 24) * w + b
    assert torch.allclose(grouped, lib, atol=1e-12)
    after = gated_norm_oracle(x, w, b, z, eps=1e-5, group_size=8, norm_before_gate=True)
    assert torch.allclose(after, lib * F.silu(z), atol=1e-12)
    before = gated_norm_oracle(x, w, None, z, eps=1e-5, group_size=12, norm_before_gate=False, is_rms_norm=True)
    lib = F.rms_norm((x * F.silu(z)).reshape(5, 2, 12), (12,), None, 1e-5).reshape(5, 24) * w
    assert torch.allclose(before, lib, atol=1e-12)


def test_against_python_loops():
    x, z, w, b = _inputs(rows=3, dim=12, seed=1)
    for is_rms in (False, True):
        for nbg in (False, True):
            got = gated_norm_oracle(x, w, b, z, eps=1e-3, group_size=4, norm_before_gate=nbg, is_rms_norm=is_rms)
            for r in range(3):
                for g in range(3):
                    vals = []
                    for c in range(4 * g, 4 * g + 4):
                        v = float(x[r, c])
                        if not nbg:
                            v *= float(z[r, c]) / (1 + math.exp(-float(z[r, c])))
                        vals.append(v)
                    mean = 0.0 if is_rms else sum(vals) / 4
                    var = sum((v - mean) ** 2 for v in vals) / 4
                    for i, c in enumerate(range(4 * g, 4 * g + 4)):
                        y = (vals[i] - mean) / math.sqrt(var + 1e-3) * float(w[c]) + float(b[c])
                        if nbg:
                            y *= float(z[r, c]) / (1 + math.exp(-float(z[r, c])))
                        assert abs(float(got[r, c]) - y) < 1e-12


def test_gradcheck():
    x, z, w, b = _inputs(rows=2, dim=8, seed=2)
    for t in (x, z, w, b):
        t.requires_grad_()
    for is_rms in (False, True):
        for nbg in (False, True):
            fn = lambda x, w, b, z: gated_norm_oracle(x, w, b, z, 1e-5, 4, nbg, is_rms)
            assert torch.autograd.gradcheck(fn, (x, w, b, z), eps=1e-6, atol=1e-6)
