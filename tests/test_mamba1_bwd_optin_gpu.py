"""The opt-in Mamba-1 backward kernels: the one whose dB / dC sums are formed by the matrix cores
(mamba_amd/csrc/mamba1_scan_bwd_mx.hip, MAMBA_AMD_M1_BWD=mx) and the one with 4 items per lane on 64-position tiles
(mamba1_scan_bwd_k4.hip, MAMBA_AMD_M1_BWD=k4, which also makes the forward kernel write a checkpoint every 64
positions): the output, the last state and every gradient against the CPU oracle at the bf16 tolerance, and
bit-for-bit repeatability.  The library reads the switch once per process, so the kernels run in a child process
that writes its results to a file."""
import os
import subprocess
import sys

import pytest
import torch

from oracle.mamba1 import selective_scan_oracle, scan_inputs

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NAMES = ["u", "delta", "A", "B", "C", "D", "z", "delta_bias"]

CHILD = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
from mamba_amd.ops.selective_scan_interface import selective_scan_fn
t = torch.load(sys.argv[2], weights_only=True)
names = ["u", "delta", "A", "B", "C", "D", "z", "delta_bias"]
outs = []
for rep in range(2):
    x = {k: (t[k].cuda().requires_grad_() if t[k] is not None else None) for k in names}
    out, last = selective_scan_fn(*[x[k] for k in names], delta_softplus=True, return_last_state=True)
    out.backward(t["dout"].cuda())
    torch.cuda.synchronize()
    outs.append({"out": out.detach().cpu(), "last": last.detach().cpu(),
                 **{"d" + k: x[k].grad.cpu() for k in names if x[k] is not None}})
for k in outs[0]:
    assert torch.equal(outs[0][k], outs[1][k]), k + " does not repeat bit for bit"
torch.save(outs[0], sys.argv[3])
"""


@pytest.mark.parametrize("mode", ["mx", "k4"])
@pytest.mark.parametrize("batch,dim,seqlen,dstate,groups,has_z", [
    (2, 96, 1024, 16, 1, True),     # three passes of 32 channels, eight tiles
    (1, 64, 200, 16, 2, False),     # ragged last tile (element-wise loads), two groups, no gate
    (2, 40, 384, 24, 1, True),      # states in two blocks of 16, a partial pass
    (3, 416, 832, 16, 1, True),     # k4: long and short workgroups side by side, a short one past the group's end
    (1, 64, 72, 8, 1, True),        # k4: two 64-position tiles, the second with 8 positions; 8 states
])
def test_optin_backward_against_the_oracle(tmp_path, mode, batch, dim, seqlen, dstate, groups, has_z):
    t = scan_inputs(batch, dim, seqlen, dstate, groups, torch.bfloat16, seed=3)
    if not has_z:
        t["z"] = None
    inp, res = str(tmp_path / "in.pt"), str(tmp_path / "out.pt")
    torch.save({k: t[k] for k in NAMES + ["dout"]}, inp)
    env = dict(os.environ, MAMBA_AMD_M1_BWD=mode)
    r = subprocess.run([sys.executable, "-c", CHILD, ROOT, inp, res], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    got = torch.load(res, weights_only=True)

    x = {k: (t[k].clone().requires_grad_() if t[k] is not None else None) for k in NAMES}
    ref, rlast = selective_scan_oracle(*[x[k] for k in NAMES], delta_softplus=True, return_last_state=True)
    ref.backward(t["dout"])
    rtol, atol = 3e-2, 5e-2

    def close(name, a, b, floor=0.0):
        a, b = a.float(), b.detach().float()
        err = (a - b).abs()
        bound = atol + rtol * b.abs() + floor * b.abs().max()
        assert bool((err <= bound).all()), f"{name}: max err {err.max().item():.3e} (ref max {b.abs().max().item():.3e})"

    close("out", got["out"], ref)
    close("last_state", got["last"], rlast)
    for k in NAMES:
        if x[k] is not None:
            # dA, dD and delta_bias sum over every position of a channel: summation-order noise relative to the
            # largest entry, as in tests/test_mamba1_gpu.py
            close("d" + k, got["d" + k], x[k].grad, floor=2e-3 if k in ("A", "D", "delta_bias") else 0.0)
