"""GPU parity of mamba_inner_fn against the CPU oracle: output (as the reference's
tests/ops/test_selective_scan.py:160-237 checks) and, beyond the reference's test, every gradient."""
import pytest
import torch

from oracle.inner import mamba_inner_oracle

pytestmark = pytest.mark.gpu


def _params(batch, dim, L, dstate, dt_rank, d_model, g, with_bias):
    r = lambda *s: torch.randn(*s, generator=g)
    p = dict(
        xz=r(batch, 2 * dim, L),
        conv1d_weight=r(dim, 1, 3), conv1d_bias=r(dim),
        x_proj_weight=r(dt_rank + 2 * dstate, dim) * 0.3,
        delta_proj_weight=0.5 * torch.rand(dim, dt_rank, generator=g),
        out_proj_weight=r(d_model, dim) * 0.3,
        out_proj_bias=r(d_model) if with_bias else None,
        A=-0.5 * torch.rand(dim, dstate, generator=g),
        D=r(dim), delta_bias=0.5 * torch.rand(dim, generator=g),
        B_proj_bias=r(dstate) if with_bias else None, C_proj_bias=r(dstate) if with_bias else None,
    )
    return p


@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("L", [128, 700])
def test_mamba_inner_fn(L, with_bias):
    from mamba_amd.ops.selective_scan_interface import mamba_inner_fn, mamba_inner_ref
    g = torch.Generator().manual_seed(0)
    batch, dim, dstate, dt_rank, d_model = 2, 768, 8, 48, 768
    p = _params(batch, dim, L, dstate, dt_rank, d_model, g, with_bias)
    ref_in = {k: (v.clone().requires_grad_() if v is not None else None) for k, v in p.items()}
    gpu_in = {k: (v.cuda().requires_grad_() if v is not None else None) for k, v in p.items()}
    order = ["xz", "conv1d_weight", "conv1d_bias", "x_proj_weight", "delta_proj_weight", "out_proj_weight",
             "out_proj_bias", "A"]
    out_ref = mamba_inner_oracle(*[ref_in[k] for k in order], D=ref_in["D"], delta_bias=ref_in["delta_bias"],
                                 B_proj_bias=ref_in["B_proj_bias"], C_proj_bias=ref_in["C_proj_bias"])
    out = mamba_inner_fn(*[gpu_in[k] for k in order], None, None, gpu_in["D"], delta_bias=gpu_in["delta_bias"],
                         B_proj_bias=gpu_in["B_proj_bias"], C_proj_bias=gpu_in["C_proj_bias"], delta_softplus=True)
    scale = float(out_ref.abs().max())
    # tolerances of tests/ops/test_selective_scan.py:162-168 (fp32), relative to the output scale
    assert torch.allclose(out.cpu(), out_ref, rtol=6e-4, atol=2e-3 * max(1.0, scale)), \
        f"max err {(out.cpu() - out_ref).abs().max().item():.3e} (scale {scale:.2e})"
    # the torch-composed reference of this package agrees too
    with torch.no_grad():
        out2 = mamba_inner_ref(*[gpu_in[k].detach() for k in order[:6]],
                               gpu_in["out_proj_bias"].detach() if with_bias else None, gpu_in["A"].detach(),
                               None, None, gpu_in["D"].detach(), delta_bias=gpu_in["delta_bias"].detach(),
                               B_proj_bias=gpu_in["B_proj_bias"].detach() if with_bias else None,
                               C_proj_bias=gpu_in["C_proj_bias"].detach() if with_bias else None)
    assert torch.allclose(out, out2, rtol=6e-4, atol=2e-3 * max(1.0, scale))
    dout = torch.randn(out_ref.shape, generator=g)
    out_ref.backward(dout)
    out.backward(dout.cuda())
    for k, v in ref_in.items():
        if v is None:
            continue
        got, ref = gpu_in[k].grad.cpu(), v.grad
        s = max(1.0, float(ref.abs().max()))
        assert torch.allclose(got, ref, rtol=5e-3, atol=5e-3 * s), \
            f"d{k}: max err {(got - ref).abs().max().item():.3e}, ref max {ref.abs().max().item():.3e}"


@pytest.mark.parametrize("given", ["B", "C", "BC"])
def test_mamba_inner_fn_given_B_C(given):
    """B and / or C passed in as input-independent (dim, dstate) matrices
    (selective_scan_interface.py:386 B=, C=; is_variable_B / is_variable_C false)."""
    from mamba_amd.ops.selective_scan_interface import mamba_inner_fn
    g = torch.Generator().manual_seed(1)
    batch, dim, dstate, dt_rank, d_model, L = 2, 256, 8, 16, 128, 300
    p = _params(batch, dim, L, dstate, dt_rank, d_model, g, False)
    nproj = dt_rank + dstate * (("B" not in given) + ("C" not in given))
    p["x_proj_weight"] = p["x_proj_weight"][:nproj].contiguous()
    p["B"] = torch.randn(dim, dstate, generator=g) if "B" in given else None
    p["C"] = torch.randn(dim, dstate, generator=g) if "C" in given else None
    ref_in = {k: (v.clone().requires_grad_() if v is not None else None) for k, v in p.items()}
    gpu_in = {k: (v.cuda().requires_grad_() if v is not None else None) for k, v in p.items()}
    order = ["xz", "conv1d_weight", "conv1d_bias", "x_proj_weight", "delta_proj_weight", "out_proj_weight",
             "out_proj_bias", "A"]
    out_ref = mamba_inner_oracle(*[ref_in[k] for k in order], D=ref_in["D"], delta_bias=ref_in["delta_bias"],
                                 B=ref_in["B"], C=ref_in["C"])
    out = mamba_inner_fn(*[gpu_in[k] for k in order], gpu_in["B"], gpu_in["C"], gpu_in["D"],
                         delta_bias=gpu_in["delta_bias"], delta_softplus=True)
    scale = float(out_ref.abs().max())
    assert torch.allclose(out.cpu(), out_ref, rtol=6e-4, atol=2e-3 * max(1.0, scale))
    dout = torch.randn(out_ref.shape, generator=g)
    out_ref.backward(dout)
    out.backward(dout.cuda())
    for k, v in ref_in.items():
        if v is None:
            continue
        got, ref = gpu_in[k].grad.cpu(), v.grad
        s = max(1.0, float(ref.abs().max()))
        assert torch.allclose(got, ref, rtol=5e-3, atol=5e-3 * s), \
            f"d{k}: max err {(got - ref).abs().max().item():.3e}, ref max {ref.abs().max().item():.3e}"


def test_mamba_inner_fn_complex_A():
    """Complex A: x_proj emits (re, im) pairs per state for B and C
    (selective_scan_interface.py:207, :255-258, :268-271)."""
    from mamba_amd.ops.selective_scan_interface import mamba_inner_fn, mamba_inner_ref
    g = torch.Generator().manual_seed(2)
    batch, dim, dstate, dt_rank, d_model, L = 2, 128, 4, 8, 64, 200
    p = _params(batch, dim, L, 2 * dstate, dt_rank, d_model, g, True)   # 2 * dstate projected columns each
    p["A"] = torch.complex(-0.5 * torch.rand(dim, dstate, generator=g), torch.randn(dim, dstate, generator=g))
    ref_in = {k: (v.clone().requires_grad_() if v is not None else None) for k, v in p.items()}
    gpu_in = {k: (v.cuda().requires_grad_() if v is not None else None) for k, v in p.items()}
    order = ["xz", "conv1d_weight", "conv1d_bias", "x_proj_weight", "delta_proj_weight", "out_proj_weight",
             "out_proj_bias", "A"]
    out_ref = mamba_inner_oracle(*[ref_in[k] for k in order], D=ref_in["D"], delta_bias=ref_in["delta_bias"],
                                 B_proj_bias=ref_in["B_proj_bias"], C_proj_bias=ref_in["C_proj_bias"])
    out = mamba_inner_fn(*[gpu_in[k] for k in order], None, None, gpu_in["D"], delta_bias=gpu_in["delta_bias"],
                         B_proj_bias=gpu_in["B_proj_bias"], C_proj_bias=gpu_in["C_proj_bias"], delta_softplus=True)
    scale = max(1.0, float(out_ref.detach().abs().max()))
    assert torch.allclose(out.cpu(), out_ref, rtol=6e-4, atol=2e-3 * scale)
    with torch.no_grad():
        out2 = mamba_inner_ref(*[gpu_in[k].detach() for k in order], None, None, gpu_in["D"].detach(),
                               delta_bias=gpu_in["delta_bias"].detach(), B_proj_bias=gpu_in["B_proj_bias"].detach(),
                               C_proj_bias=gpu_in["C_proj_bias"].detach())
    assert torch.allclose(out, out2, rtol=6e-4, atol=2e-3 * scale)
    dout = torch.randn(out_ref.shape, generator=g)
    out_ref.backward(dout)
    out.backward(dout.cuda())
    for k, v in ref_in.items():
        if v is None:
            continue
        got, ref = gpu_in[k].grad.cpu(), v.grad
        if ref.is_complex():
            got, ref = torch.view_as_real(got), torch.view_as_real(ref)
        s = max(1.0, float(ref.abs().max()))
        assert torch.allclose(got, ref, rtol=5e-3, atol=5e-3 * s), \
            f"d{k}: max err {(got - ref).abs().max().item():.3e}, ref max {ref.abs().max().item():.3e}"


def test_install_as_mamba_ssm_ops():
    import importlib
    import mamba_amd
    mamba_amd.install_as_mamba_ssm_ops()
    m = importlib.import_module("mamba_ssm.ops.selective_scan_interface")
    from mamba_ssm.ops.triton.ssd_combined import mamba_chunk_scan_combined  # noqa: F401
    from mamba_ssm.ops.triton.selective_state_update import selective_state_update  # noqa: F401
    assert m.selective_scan_fn.__module__.startswith("mamba_amd")


@pytest.mark.parametrize("which", ["b", "c", "dt", "all"])
def test_mamba_inner_fn_rms_norms(which):
    """b / c / dt_rms_weight (selective_scan_interface.py:263-274): the value of the norms in the forward pass;
    in the backward pass the reference hands gradients straight through them, and so do the oracle and this."""
    from mamba_amd.ops.selective_scan_interface import mamba_inner_fn
    g = torch.Generator().manual_seed(4)
    batch, dim, dstate, dt_rank, d_model, L = 2, 128, 8, 16, 96, 200
    p = _params(batch, dim, L, dstate, dt_rank, d_model, g, False)
    rms = dict(b_rms_weight=1 + 0.2 * torch.randn(dstate, generator=g) if which in ("b", "all") else None,
               c_rms_weight=1 + 0.2 * torch.randn(dstate, generator=g) if which in ("c", "all") else None,
               dt_rms_weight=0.3 + 0.1 * torch.rand(dim, generator=g) if which in ("dt", "all") else None)
    ref_in = {k: (v.clone().requires_grad_() if v is not None else None) for k, v in p.items()}
    gpu_in = {k: (v.cuda().requires_grad_() if v is not None else None) for k, v in p.items()}
    order = ["xz", "conv1d_weight", "conv1d_bias", "x_proj_weight", "delta_proj_weight", "out_proj_weight",
             "out_proj_bias", "A"]
    out_ref = mamba_inner_oracle(*[ref_in[k] for k in order], D=ref_in["D"], delta_bias=ref_in["delta_bias"],
                                 b_c_dt_rms_eps=1e-5, **rms)
    out = mamba_inner_fn(*[gpu_in[k] for k in order], None, None, gpu_in["D"], delta_bias=gpu_in["delta_bias"],
                         delta_softplus=True, b_c_dt_rms_eps=1e-5,
                         **{k: (v.cuda() if v is not None else None) for k, v in rms.items()})
    scale = float(out_ref.abs().max())
    assert torch.allclose(out.cpu(), out_ref, rtol=6e-4, atol=2e-3 * max(1.0, scale)), \
        f"max err {(out.cpu() - out_ref).abs().max().item():.3e} (scale {scale:.2e})"
    dout = torch.randn(out_ref.shape, generator=g)
    out_ref.backward(dout)
    out.backward(dout.cuda())
    for k, v in ref_in.items():
        if v is None:
            continue
        got, ref = gpu_in[k].grad.cpu(), v.grad
        s = max(1.0, float(ref.abs().max()))
        assert torch.allclose(got, ref, rtol=5e-3, atol=5e-3 * s), \
            f"d{k}: max err {(got - ref).abs().max().item():.3e}, ref max {ref.abs().max().item():.3e}"


def test_mamba_inner_fn_checkpoint_levels_agree():
    """checkpoint_lvl 0 keeps the convolution output and delta, 1 (the default) re-computes them in the
    backward pass (selective_scan_interface.py:279-281, :300-310): same output, same gradients."""
    from mamba_amd.ops.selective_scan_interface import mamba_inner_fn
    g = torch.Generator().manual_seed(6)
    batch, dim, dstate, dt_rank, d_model, L = 2, 96, 8, 8, 64, 260
    p = _params(batch, dim, L, dstate, dt_rank, d_model, g, True)
    order = ["xz", "conv1d_weight", "conv1d_bias", "x_proj_weight", "delta_proj_weight", "out_proj_weight",
             "out_proj_bias", "A"]
    dout = torch.randn(batch, L, d_model, generator=g).cuda()
    res = []
    for lvl in (0, 1):
        t = {k: (v.cuda().requires_grad_() if v is not None else None) for k, v in p.items()}
        out = mamba_inner_fn(*[t[k] for k in order], None, None, t["D"], delta_bias=t["delta_bias"],
                             B_proj_bias=t["B_proj_bias"], C_proj_bias=t["C_proj_bias"], delta_softplus=True,
                             checkpoint_lvl=lvl)
        out.backward(dout)
        res.append((out.detach(), {k: v.grad for k, v in t.items() if v is not None}))
    assert torch.equal(res[0][0], res[1][0])
    for k in res[0][1]:
        a, b = res[0][1][k], res[1][1][k]
        # dB / dC reach the projections through float atomics whose order differs from run to run
        assert torch.allclose(a, b, rtol=1e-4, atol=1e-4 * max(1.0, float(b.abs().max()))), k
