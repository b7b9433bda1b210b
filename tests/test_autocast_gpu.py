"""The two block-level operators under torch.autocast(bfloat16), the way the reference's modules run them in
mixed-precision training (fp32 parameters, bf16 activations coming out of in_proj): outputs and gradients stay
within the bf16 tolerances of the oracle, and parameter gradients come back in the parameters' dtype."""
import pytest
import torch

from oracle.block import split_conv1d_scan_oracle
from oracle.inner import mamba_inner_oracle

pytestmark = pytest.mark.gpu


def _close(name, got, ref, rtol, atol):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    scale = max(1.0, float(ref.abs().max()))
    err = (got - ref).abs()
    assert bool((err <= atol * scale + rtol * ref.abs()).all()), f"{name}: max err {err.max().item():.3e}, ref max {ref.abs().max().item():.3e}"


def test_mamba_inner_fn_under_autocast():
    from mamba_amd.ops.selective_scan_interface import mamba_inner_fn
    g = torch.Generator().manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=g)
    batch, dim, L, dstate, dt_rank, d_model = 2, 256, 300, 8, 16, 192
    p = dict(xz=r(batch, 2 * dim, L).bfloat16().float(), conv1d_weight=r(dim, 1, 4) * 0.5, conv1d_bias=r(dim) * 0.2,
             x_proj_weight=r(dt_rank + 2 * dstate, dim) * 0.1, delta_proj_weight=0.3 * torch.rand(dim, dt_rank, generator=g),
             out_proj_weight=r(d_model, dim) * 0.1, out_proj_bias=r(d_model) * 0.1,
             A=-0.5 * torch.rand(dim, dstate, generator=g), D=r(dim), delta_bias=0.5 * torch.rand(dim, generator=g))
    order = ["xz", "conv1d_weight", "conv1d_bias", "x_proj_weight", "delta_proj_weight", "out_proj_weight", "out_proj_bias", "A"]
    ref_in = {k: v.clone().requires_grad_() for k, v in p.items()}
    gpu_in = {k: v.cuda().requires_grad_() for k, v in p.items()}
    out_ref = mamba_inner_oracle(*[ref_in[k] for k in order], D=ref_in["D"], delta_bias=ref_in["delta_bias"])
    xz16 = gpu_in["xz"].bfloat16()          # what in_proj hands over under autocast
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = mamba_inner_fn(xz16, *[gpu_in[k] for k in order[1:]], None, None, gpu_in["D"],
                             delta_bias=gpu_in["delta_bias"], delta_softplus=True)
    assert out.dtype == torch.bfloat16
    _close("out", out, out_ref, 3e-2, 5e-2)
    dout = torch.randn(out_ref.shape, generator=g)
    out_ref.backward(dout)
    out.backward(dout.cuda().bfloat16())
    for k in p:
        assert gpu_in[k].grad.dtype == torch.float32, k
        _close("d" + k, gpu_in[k].grad, ref_in[k].grad, 6e-2, 6e-2)


@pytest.mark.parametrize("norm", [False, True])
def test_block_under_autocast(norm):
    from mamba_amd.ops.triton.ssd_combined import mamba_split_conv1d_scan_combined
    g = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=g)
    batch, L, nheads, headdim, dstate, ngroups, d_out, chunk = 2, 200, 4, 32, 16, 1, 40, 64
    dim = nheads * headdim
    p = dict(zxbcdt=(0.7 * r(batch, L, 2 * dim + 2 * ngroups * dstate + nheads)).bfloat16().float(),
             conv1d_weight=0.4 * r(dim + 2 * ngroups * dstate, 4), conv1d_bias=0.1 * r(dim + 2 * ngroups * dstate),
             dt_bias=r(nheads) * 0.5, A=-(0.5 + torch.rand(nheads, generator=g)), D=0.5 + torch.rand(nheads, generator=g),
             rmsnorm_weight=1 + 0.1 * r(dim), outproj_weight=0.2 * r(d_out, dim), outproj_bias=0.1 * r(d_out))
    ref_in = {k: v.clone().requires_grad_() for k, v in p.items()}
    gpu_in = {k: v.cuda().requires_grad_() for k, v in p.items()}
    kw = dict(headdim=headdim, ngroups=ngroups, norm_before_gate=False)
    out_ref, _ = split_conv1d_scan_oracle(
        ref_in["zxbcdt"], ref_in["conv1d_weight"], ref_in["conv1d_bias"], ref_in["dt_bias"], ref_in["A"], ref_in["D"],
        rmsnorm_weight=ref_in["rmsnorm_weight"] if norm else None, outproj_weight=ref_in["outproj_weight"],
        outproj_bias=ref_in["outproj_bias"], **kw)
    z16 = gpu_in["zxbcdt"].bfloat16()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = mamba_split_conv1d_scan_combined(
            z16, gpu_in["conv1d_weight"], gpu_in["conv1d_bias"], gpu_in["dt_bias"], gpu_in["A"], gpu_in["D"], chunk,
            rmsnorm_weight=gpu_in["rmsnorm_weight"] if norm else None, outproj_weight=gpu_in["outproj_weight"],
            outproj_bias=gpu_in["outproj_bias"], **kw)
    assert out.dtype == torch.bfloat16
    _close("out", out, out_ref, 3e-2, 5e-2)
    dout = torch.randn(out_ref.shape, generator=g)
    out_ref.backward(dout)
    out.backward(dout.cuda().bfloat16())
    for k in p:
        if k == "rmsnorm_weight" and not norm:
            continue
        assert gpu_in[k].grad.dtype == torch.float32, k
        _close("d" + k, gpu_in[k].grad, ref_in[k].grad, 6e-2, 6e-2)
