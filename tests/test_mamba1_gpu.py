"""GPU parity of the Mamba-1 selective scan against the CPU oracle.

Mirrors the reference's tests/ops/test_selective_scan.py:38-147 (same shapes, value
distributions and per-gradient tolerances), with the oracle in place of selective_scan_ref,
and adds the bf16 / ragged / strided / multi-tile cases of the benchmark configurations.
"""
import pytest
import torch

from oracle.mamba1 import selective_scan_oracle, scan_inputs

pytestmark = pytest.mark.gpu


def _tols(itype):
    # tests/ops/test_selective_scan.py:43-49
    rtol, atol = (6e-4, 2e-3) if itype == torch.float32 else (3e-3, 5e-3)
    if itype == torch.bfloat16:
        rtol, atol = 3e-2, 5e-2
    rtolw, atolw = max(1e-3, rtol), max(1e-3, atol)
    return rtol, atol, rtolw, atolw


def _close(name, got, ref, rtol, atol, floor=0.0):
    """|got - ref| <= atol + rtol |ref| (+ floor * max |ref|: the fp32 summation-order noise of a
    reduction over batch * seqlen terms, for tensors whose entries differ by orders of magnitude)."""
    got, ref = got.detach().cpu(), ref.detach().cpu()
    if ref.is_complex():
        assert got.is_complex()
        got, ref = torch.view_as_real(got), torch.view_as_real(ref)
    got, ref = got.float(), ref.float()
    err = (got - ref).abs()
    bound = atol + rtol * ref.abs() + floor * ref.abs().max()
    assert bool((err <= bound).all()), (
        f"{name}: max err {err.max().item():.3e}, worst excess {(err - bound).max().item():.3e}, "
        f"ref max {ref.abs().max().item():.3e}")


def _run_case(batch, dim, dstate, seqlen, itype, groups, has_z=True, has_D=True, has_bias=True,
              softplus=True, reference_style=True, seed=0, var_B=True, var_C=True, complex_A=False):
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    dev = "cuda"
    rtol, atol, rtolw, atolw = _tols(itype)
    g = torch.Generator().manual_seed(seed)
    if reference_style:  # distributions of tests/ops/test_selective_scan.py:56-90
        A = -0.5 * torch.rand(dim, dstate, generator=g)
        two = 2 if complex_A else 1
        Bshape = (batch, dstate, seqlen * two) if groups == 0 else (batch, groups, dstate, seqlen * two)
        # input-independent B / C are (dim, dstate) matrices of A's dtype (tests/ops/test_selective_scan.py:64-79)
        mat = lambda: (torch.complex(torch.randn(dim, dstate, generator=g), torch.randn(dim, dstate, generator=g))
                       if complex_A else torch.randn(dim, dstate, generator=g))
        if complex_A:  # wtype complex64 (tests/ops/test_selective_scan.py:59: A = -0.5 * rand, complex)
            A = torch.complex(A, 2.0 * torch.randn(dim, dstate, generator=g))
        B = torch.randn(*Bshape, generator=g).to(itype) if var_B else mat()
        C = torch.randn(*Bshape, generator=g).to(itype) if var_C else mat()
        D = torch.randn(dim, generator=g) if has_D else None
        z = torch.randn(batch, dim, seqlen, generator=g).to(itype) if has_z else None
        delta_bias = 0.5 * torch.rand(dim, generator=g) if has_bias else None
        u = torch.randn(batch, dim, seqlen, generator=g).to(itype)
        delta = (0.5 * torch.rand(batch, dim, seqlen, generator=g)).to(itype)
        dout = torch.randn(batch, dim, seqlen, generator=g).to(itype)
    else:
        t = scan_inputs(batch, dim, seqlen, dstate, max(groups, 1), itype, seed, has_z=has_z, has_D=has_D)
        A, B, C, D, z, delta_bias, u, delta, dout = (t[k] for k in
                                                     ("A", "B", "C", "D", "z", "delta_bias", "u", "delta", "dout"))
        if not has_bias:
            delta_bias = None
    names = ["u", "delta", "A", "B", "C", "D", "z", "delta_bias"]
    cpu = dict(u=u, delta=delta, A=A, B=B, C=C, D=D, z=z, delta_bias=delta_bias)
    ref_in = {k: (v.clone().requires_grad_() if v is not None else None) for k, v in cpu.items()}
    gpu_in = {k: (v.to(dev).requires_grad_() if v is not None else None) for k, v in cpu.items()}

    out_ref, state_ref = selective_scan_oracle(*[ref_in[k] for k in names], delta_softplus=softplus,
                                               return_last_state=True)
    out, state = selective_scan_fn(*[gpu_in[k] for k in names], delta_softplus=softplus, return_last_state=True)
    assert out.dtype == itype and out.shape == out_ref.shape
    _close("out", out, out_ref, rtol, atol)
    _close("last_state", state, state_ref, rtol, atol)

    out_ref.backward(dout)
    out.backward(dout.to(dev))
    gr = lambda k: gpu_in[k].grad
    rr = lambda k: ref_in[k].grad
    # per-gradient tolerances of tests/ops/test_selective_scan.py:135-147
    _close("du", gr("u"), rr("u"), rtol * 2, atol * 2)
    _close("ddelta", gr("delta"), rr("delta"), rtol * 5, atol * 10)
    _close("dA", gr("A"), rr("A"), rtolw, atolw * 5, floor=3e-5 if complex_A else 0.0)
    _close("dB", gr("B"), rr("B"), rtol if var_B else rtolw, atol if var_B else atolw)
    _close("dC", gr("C"), rr("C"), rtol if var_C else rtolw, atol if var_C else atolw)
    if has_D:
        _close("dD", gr("D"), rr("D"), rtolw, atolw)
    if has_z:
        _close("dz", gr("z"), rr("z"), rtolw, atolw)
    if has_bias:
        _close("ddelta_bias", gr("delta_bias"), rr("delta_bias"), rtolw, atolw)
    for k in ("u", "delta", "B", "C", "z"):
        if gpu_in[k] is not None:
            assert gr(k).dtype == gpu_in[k].dtype and gr(k).shape == gpu_in[k].shape
    assert gr("A").dtype == (torch.complex64 if complex_A else torch.float32)


@pytest.mark.parametrize("groups", [0, 1, 2])
@pytest.mark.parametrize("seqlen", [128, 256, 512, 1024, 2048, 4096])
def test_selective_scan_reference_grid(seqlen, groups):
    # the enabled grid of tests/ops/test_selective_scan.py:16-37: fp32, batch 2, dim 4, dstate 8
    _run_case(2, 4, 8, seqlen, torch.float32, groups)


@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("seqlen", [8, 17, 372, 1134])
def test_selective_scan_ragged(seqlen, itype):
    # ragged lengths (no 16-byte path) from the reference's commented-out list, all input dtypes
    _run_case(2, 6, 8, seqlen, itype, 2)


@pytest.mark.parametrize("has_z,has_D,has_bias,softplus", [
    (False, True, True, True), (True, False, True, True), (True, True, False, True), (True, True, True, False),
    (False, False, False, False)])
def test_selective_scan_optional_args(has_z, has_D, has_bias, softplus):
    _run_case(2, 4, 8, 640, torch.float32, 1, has_z=has_z, has_D=has_D, has_bias=has_bias, softplus=softplus)


@pytest.mark.parametrize("dstate", [1, 4, 16, 24, 64])
def test_selective_scan_dstate(dstate):
    _run_case(1, 5, dstate, 700, torch.float32, 1)


@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16])
def test_selective_scan_benchmark_distribution(itype):
    # the benchmark's value distributions (A = -(1..16), softplus^-1 bias) on a slice of its shape
    _run_case(2, 96, 16, 2048, itype, 1, reference_style=False)


@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("var_B,var_C", [(False, True), (True, False), (False, False)])
def test_selective_scan_input_independent_B_C(var_B, var_C, itype):
    # is_variable_B / is_variable_C of tests/ops/test_selective_scan.py:30-33: (dim, dstate) fp32 matrices;
    # several tiles, a ragged tail, more channels than one workgroup holds, dstate above one LDS block
    _run_case(2, 4, 8, 1024, itype, 2, var_B=var_B, var_C=var_C)
    _run_case(2, 40, 16, 700, itype, 1, var_B=var_B, var_C=var_C, has_z=False)
    _run_case(1, 6, 24, 300, itype, 1, var_B=var_B, var_C=var_C, has_bias=False)


@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("var_B,var_C", [(True, True), (False, True), (True, False), (False, False)])
def test_selective_scan_complex_A(var_B, var_C, itype):
    # wtype complex64 of tests/ops/test_selective_scan.py:17: complex state, (re, im)-interleaved B / C
    _run_case(2, 4, 8, 1024, itype, 2, var_B=var_B, var_C=var_C, complex_A=True)
    _run_case(1, 6, 5, 300, itype, 1, var_B=var_B, var_C=var_C, complex_A=True, has_z=False, has_bias=False)
