"""GPU parity of the wrappers around the SSD scan: mamba_split_conv1d_scan_combined (the fused
Mamba-2 block body, reference ssd_combined.py:983), ssd_selective_scan (:728), mamba_chunk_scan (:651)
and the *_ref compositions, against the CPU oracles."""
import pytest
import torch

from oracle.block import split_conv1d_scan_oracle
from oracle.ssd import ssd_oracle, ssd_inputs

pytestmark = pytest.mark.gpu


def _tol(dtype):
    return (6e-4, 2e-3) if dtype == torch.float32 else (3e-2, 5e-2)


def _close(name, got, ref, rtol, atol):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    err = (got - ref).abs()
    bound = atol * max(1.0, float(ref.abs().max())) + rtol * ref.abs()
    assert bool((err <= bound).all()), f"{name}: max err {err.max().item():.3e}, ref max {ref.abs().max().item():.3e}"


def _block_inputs(batch, L, nheads, headdim, dstate, ngroups, d_nonssm, d_out, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    dim, width = nheads * headdim, 4
    r = lambda *s: torch.randn(*s, generator=g)
    return dict(
        zxbcdt=r(batch, L, 2 * d_nonssm + 2 * dim + 2 * ngroups * dstate + nheads).to(dtype),
        conv1d_weight=(0.5 * r(dim + 2 * ngroups * dstate, width)).to(dtype),
        conv1d_bias=(0.1 * r(dim + 2 * ngroups * dstate)).to(dtype),
        dt_bias=torch.rand(nheads, generator=g) - 4.0, A=-(1.0 + 15.0 * torch.rand(nheads, generator=g)),
        # D away from 0: with a tiny skip term the scan output right after a sequence start is ~0 for a
        # whole norm group, and 1 / rms then multiplies every rounding difference by hundreds
        D=0.5 + torch.rand(nheads, generator=g), rmsnorm_weight=(1.0 + 0.1 * r(dim)).to(dtype),
        outproj_weight=(0.2 * r(d_out, d_nonssm + dim)).to(dtype), outproj_bias=(0.1 * r(d_out)).to(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("norm,nbg,d_nonssm,packed", [(False, True, 0, False), (True, True, 0, False),
                                                      (True, False, 16, False), (True, True, 0, True)])
def test_mamba_split_conv1d_scan_combined(norm, nbg, d_nonssm, packed, dtype):
    from mamba_amd.ops.triton.ssd_combined import mamba_split_conv1d_scan_combined
    batch, L, nheads, headdim, dstate, ngroups, d_out, chunk = (1 if packed else 2), 384, 4, 64, 32, 2, 48, 128
    t = _block_inputs(batch, L, nheads, headdim, dstate, ngroups, d_nonssm, d_out, 11, dtype)
    seq_idx = None
    if packed:
        lens = [100, 28, 129, 127]
        seq_idx = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(lens)])[None]
    rtol, atol = _tol(dtype)
    names = list(t)
    ref_in = {k: t[k].float().clone().requires_grad_() for k in names}
    gpu_in = {k: t[k].cuda().requires_grad_() for k in names}
    kw = dict(headdim=headdim, ngroups=ngroups, norm_before_gate=nbg)
    out_ref, fin_ref = split_conv1d_scan_oracle(
        ref_in["zxbcdt"], ref_in["conv1d_weight"], ref_in["conv1d_bias"], ref_in["dt_bias"], ref_in["A"], ref_in["D"],
        seq_idx=seq_idx, rmsnorm_weight=ref_in["rmsnorm_weight"] if norm else None,
        outproj_weight=ref_in["outproj_weight"], outproj_bias=ref_in["outproj_bias"], **kw)
    out, fin = mamba_split_conv1d_scan_combined(
        gpu_in["zxbcdt"], gpu_in["conv1d_weight"], gpu_in["conv1d_bias"], gpu_in["dt_bias"], gpu_in["A"], gpu_in["D"], chunk,
        seq_idx=seq_idx.cuda() if packed else None, return_final_states=True,
        rmsnorm_weight=gpu_in["rmsnorm_weight"] if norm else None, outproj_weight=gpu_in["outproj_weight"],
        outproj_bias=gpu_in["outproj_bias"], **kw)
    assert out.dtype == dtype and out.shape == out_ref.shape
    _close("out", out, out_ref, rtol, atol)
    _close("final_states", fin, fin_ref, rtol, atol)
    g = torch.Generator().manual_seed(5)
    dout = torch.randn(out_ref.shape, generator=g)
    out_ref.backward(dout)
    out.backward(dout.to(dtype).cuda())
    for k in names:
        if k == "rmsnorm_weight" and not norm:
            continue
        _close("d" + k, gpu_in[k].grad, ref_in[k].grad, 5 * rtol, 5 * atol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("norm", [False, True])
def test_block_without_projection_with_states_and_3d_conv_weight(norm, dtype):
    """No out_proj, initial states, a gradient arriving through the final states, and the convolution weight
    in nn.Conv1d's (channels, 1, width) shape."""
    from mamba_amd.ops.triton.ssd_combined import mamba_split_conv1d_scan_combined
    batch, L, nheads, headdim, dstate, ngroups, chunk = 2, 200, 4, 32, 16, 1, 64
    t = _block_inputs(batch, L, nheads, headdim, dstate, ngroups, 8, 24, 21, dtype)
    t.pop("outproj_weight")
    t.pop("outproj_bias")
    g = torch.Generator().manual_seed(8)
    t["initial_states"] = 0.3 * torch.randn(batch, nheads, headdim, dstate, generator=g)
    rtol, atol = _tol(dtype)
    names = list(t)
    ref_in = {k: t[k].float().clone().requires_grad_() for k in names}
    gpu_in = {k: t[k].cuda().requires_grad_() for k in names}
    w3 = gpu_in["conv1d_weight"].detach().unsqueeze(1).clone().requires_grad_()
    kw = dict(headdim=headdim, ngroups=ngroups, norm_before_gate=False)
    out_ref, fin_ref = split_conv1d_scan_oracle(
        ref_in["zxbcdt"], ref_in["conv1d_weight"], ref_in["conv1d_bias"], ref_in["dt_bias"], ref_in["A"], ref_in["D"],
        initial_states=ref_in["initial_states"], rmsnorm_weight=ref_in["rmsnorm_weight"] if norm else None, **kw)
    out, fin = mamba_split_conv1d_scan_combined(
        gpu_in["zxbcdt"], w3, gpu_in["conv1d_bias"], gpu_in["dt_bias"], gpu_in["A"], gpu_in["D"], chunk,
        initial_states=gpu_in["initial_states"], return_final_states=True,
        rmsnorm_weight=gpu_in["rmsnorm_weight"] if norm else None, **kw)
    _close("out", out, out_ref, rtol, atol)
    _close("final_states", fin, fin_ref, rtol, atol)
    dout = torch.randn(out_ref.shape, generator=g)
    dfin = torch.randn(fin_ref.shape, generator=g)
    ((out_ref * dout).sum() + (fin_ref * dfin).sum()).backward()
    torch.autograd.backward([out, fin], [dout.to(dtype).cuda(), dfin.cuda()])
    assert w3.grad.shape == w3.shape
    _close("dconv1d_weight", w3.grad.squeeze(1), ref_in["conv1d_weight"].grad, 5 * rtol, 5 * atol)
    for k in names:
        if k == "conv1d_weight" or (k == "rmsnorm_weight" and not norm):
            continue
        _close("d" + k, gpu_in[k].grad, ref_in[k].grad, 5 * rtol, 5 * atol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ssd_selective_scan_and_chunk_scan_wrappers(dtype):
    from mamba_amd.ops.triton.ssd_combined import ssd_selective_scan, mamba_chunk_scan, ssd_chunk_scan_combined_ref
    t = ssd_inputs(2, 300, 4, 32, 16, 2, dtype, 13)
    rtol, atol = _tol(dtype)
    ref = ssd_oracle(t["x"], t["dt"], t["A"], t["B"], t["C"], D=t["D"], z=t["z"], dt_bias=t["dt_bias"], dt_softplus=True)
    cu = lambda v: v.cuda()
    args = [cu(t[k]) for k in ("x", "dt", "A", "B", "C")]
    kw = dict(D=cu(t["D"]), z=cu(t["z"]), dt_bias=cu(t["dt_bias"]), dt_softplus=True)
    _close("ssd_selective_scan", ssd_selective_scan(*args, **kw), ref, rtol, atol)
    _close("mamba_chunk_scan", mamba_chunk_scan(*args, 128, **kw), ref, rtol, atol)
    _close("ssd_chunk_scan_combined_ref", ssd_chunk_scan_combined_ref(*args, 128, **kw), ref, rtol, atol)
    lim = (0.01, 0.05)
    ref2 = ssd_oracle(t["x"], t["dt"], t["A"], t["B"], t["C"], D=t["D"], z=t["z"], dt_bias=t["dt_bias"], dt_softplus=True,
                      dt_limit=lim)
    _close("ssd_selective_scan dt_limit", ssd_selective_scan(*args, dt_limit=lim, **kw), ref2, rtol, atol)


def test_split_conv1d_scan_ref_matches_combined():
    from mamba_amd.ops.triton.ssd_combined import mamba_split_conv1d_scan_combined, mamba_split_conv1d_scan_ref
    t = _block_inputs(2, 256, 4, 32, 16, 1, 0, 24, 17, torch.float32)
    g = {k: v.cuda() for k, v in t.items()}
    kw = dict(rmsnorm_weight=g["rmsnorm_weight"], outproj_weight=g["outproj_weight"], outproj_bias=g["outproj_bias"],
              headdim=32, ngroups=1)
    a = mamba_split_conv1d_scan_combined(g["zxbcdt"], g["conv1d_weight"], g["conv1d_bias"], g["dt_bias"], g["A"], g["D"], 64, **kw)
    b = mamba_split_conv1d_scan_ref(g["zxbcdt"], g["conv1d_weight"], g["conv1d_bias"], g["dt_bias"], g["A"], g["D"], 64, **kw)
    _close("ref vs combined", a, b, 6e-4, 2e-3)
