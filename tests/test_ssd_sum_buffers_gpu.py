"""Which sum buffers of the SSD backward pass need clearing, and whether it needs CB (ssd_bwd_overwrites in
include/mamba_hip.h): the host sides hand the large buffers (dCB, dB32 / dC32) over uncleared where the library reports
that its kernels store them whole, and skip the C B^T stage where the dCB kernel forms its tiles itself.  Here the allocator's free blocks are filled with NaN first, so an entry that a kernel adds into, or never
writes, although it was reported as stored would come back as NaN; the gradients are then held to the oracle."""
import pytest
import torch

from oracle.ssd import ssd_oracle, ssd_inputs

pytestmark = pytest.mark.gpu

NAMES = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias"]


def _poison(nbytes):
    """NaN into blocks the caching allocator will hand out again."""
    blocks = [torch.full((nbytes // 4,), float("nan"), device="cuda") for _ in range(3)]
    blocks += [torch.full((n,), float("nan"), device="cuda") for n in (1 << 12, 1 << 16, 1 << 20, 1 << 22)]
    torch.cuda.synchronize()
    del blocks


# flags: 8 heads per group and enough (batch, chunk) pairs that the state-path stage gives a whole group to one
# workgroup (2; with few pairs it prefers more, shorter head lists), one head list owns each dCB tile (1) and forms
# its tile of C B^T itself, so that CB is not passed at all (4); 16 heads per group = the dCB tiles and CB only; 32 per
# group = none
@pytest.mark.parametrize("host", ["extension", "python"])
@pytest.mark.parametrize("H,G,L,Q,expect", [(16, 2, 4096, 64, 7), (16, 1, 1024, 256, 5), (32, 1, 1024, 256, 0)])
@pytest.mark.parametrize("packed", [False, True])
def test_uncleared_sum_buffers(monkeypatch, H, G, L, Q, expect, packed, host):
    from mamba_amd import _lib
    from mamba_amd.ops.triton import ssd_combined as sc
    lib = _lib.load()
    seen = []
    if host == "python":
        monkeypatch.setattr(_lib, "torch_ext", lambda: None)
        real = lib.ssd_bwd_overwrites
        monkeypatch.setattr(lib, "ssd_bwd_overwrites", lambda p: seen.append(real(p)) or seen[-1])
    batch, P, N = 1, 64, 128
    t = ssd_inputs(batch, L, H, P, N, G, torch.bfloat16, 12, seq_lens=[L // 3 + 7, L - L // 3 - 7] if packed else None)
    g = {k: t[k].cuda().requires_grad_() for k in NAMES}
    r = {k: t[k].clone().requires_grad_() for k in NAMES}
    seq_idx = t["seq_idx"]
    out = sc.mamba_chunk_scan_combined(g["x"], g["dt"], g["A"], g["B"], g["C"], Q, D=g["D"], z=g["z"], dt_bias=g["dt_bias"],
                                       dt_softplus=True, seq_idx=seq_idx.cuda() if seq_idx is not None else None)
    _poison(4 * (batch * (L // Q) * G * Q * Q + 2 * batch * L * G * N + 4 * batch * H * L))
    out.backward(t["dout"].cuda())
    torch.cuda.synchronize()
    if host == "python":
        assert seen == [expect], f"ssd_bwd_overwrites reported {seen}, expected {expect}"
    ref = ssd_oracle(r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"], dt_softplus=True,
                     seq_idx=seq_idx)
    ref.backward(t["dout"])
    for k in NAMES:
        got, want = g[k].grad.float().cpu(), r[k].grad.float()
        assert bool(torch.isfinite(got).all()), f"d{k} holds non-finite entries: an uncleared buffer was added into"
        # the factors of tests/test_ssd_gpu.py and tests/test_full_size_gpu.py for bf16 (ddt: the gate gradient's rounding)
        f = 3.0 if k == "dt" else 1.5 if k in ("x", "B", "C") else 1.0
        floor = 4e-3 * float(want.abs().max()) if k in ("A", "D", "dt_bias") else 0.0
        err = (got - want).abs()
        assert bool((err <= f * (5e-2 + 3e-2 * want.abs()) + floor).all()), f"d{k}: max err {float(err.max()):.3e}"
