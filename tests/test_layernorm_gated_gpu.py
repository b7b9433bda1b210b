"""GPU parity of the HIP gated LayerNorm / RMSNorm against oracle/norm.py (pinned on the CPU by
tests/test_oracle_norm.py), forward and every gradient.  The grid follows the reference's own test
(tests/ops/triton/test_layernorm_gated.py: gate on / off, gate order, with and without groups of
64, RMS or not, bias or not, d 2048 and 4096 among the sizes) plus ragged group sizes, strided rows and every team size of the kernels."""
import pytest
import torch

from oracle.norm import gated_norm_oracle

pytestmark = pytest.mark.gpu


def _tol(dtype):
    return (6e-4, 2e-3) if dtype == torch.float32 else ((3e-3, 5e-3) if dtype == torch.float16 else (3e-2, 5e-2))


def _close(name, got, ref, rtol, atol):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    err = (got - ref).abs()
    assert bool((err <= atol + rtol * ref.abs()).all()), f"{name}: max err {err.max().item():.3e}, ref max {ref.abs().max().item():.3e}"


def _case(rows, dim, group_size, dtype, has_z=True, norm_before_gate=True, is_rms=True, has_bias=False,
          wtype=torch.float32, lead=None, row_pad=0, seed=0):
    from mamba_amd.ops.triton.layernorm_gated import layernorm_fn
    g = torch.Generator().manual_seed(seed)
    shape = (rows, dim) if lead is None else (*lead, dim)
    x = (torch.randn(*shape, generator=g) * 1.5 + 0.2).to(dtype)
    z = torch.randn(*shape, generator=g).to(dtype) if has_z else None
    w = (1 + 0.2 * torch.randn(dim, generator=g)).to(wtype)
    b = (0.5 * torch.randn(dim, generator=g)).to(wtype) if has_bias else None
    dy = torch.randn(*shape, generator=g).to(dtype)
    rtol, atol = _tol(dtype)
    leaf = lambda t: t.double().clone().requires_grad_() if t is not None else None
    xr, zr, wr, br = leaf(x), leaf(z), leaf(w), leaf(b)
    ref = gated_norm_oracle(xr, wr, br, zr, 1e-5, group_size, norm_before_gate, is_rms)
    (ref * dy.double()).sum().backward()

    def dev(t):
        if t is None:
            return None
        if row_pad:  # rows of a wider buffer: row stride != dim
            buf = torch.zeros(*t.shape[:-1], dim + row_pad, dtype=t.dtype, device="cuda")
            buf[..., :dim] = t.cuda()
            return buf[..., :dim].detach().requires_grad_()
        return t.cuda().requires_grad_()
    xg, zg, wg, bg = dev(x), dev(z), w.cuda().requires_grad_(), (b.cuda().requires_grad_() if has_bias else None)
    out = layernorm_fn(xg, wg, bg, z=zg, eps=1e-5, group_size=group_size, norm_before_gate=norm_before_gate,
                       is_rms_norm=is_rms)
    assert out.shape == x.shape and out.dtype == dtype
    _close("out", out, ref, rtol, atol)
    out.backward(dy.cuda())
    _close("dx", xg.grad, xr.grad, rtol * 2, atol * 2)
    if has_z:
        _close("dz", zg.grad, zr.grad, rtol * 2, atol * 2)
    nrows = x.numel() // dim
    wt = _tol(wtype)
    # sums over the rows: rounding of the per-row terms grows like sqrt(rows)
    _close("dweight", wg.grad, wr.grad, max(rtol, wt[0]) * 2, max(atol, wt[1]) * 2 * max(1.0, nrows ** 0.5 / 4))
    assert wg.grad.dtype == wtype
    if has_bias:
        _close("dbias", bg.grad, br.grad, max(rtol, wt[0]) * 2, max(atol, wt[1]) * 2 * max(1.0, nrows ** 0.5 / 4))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("has_group", [False, True])
@pytest.mark.parametrize("norm_before_gate", [True, False])
@pytest.mark.parametrize("has_z", [False, True])
@pytest.mark.parametrize("dim", [64, 256, 704, 2048])
def test_reference_grid(dim, has_z, norm_before_gate, has_group, is_rms, dtype):
    _case(0, dim, 64 if has_group else None, dtype, has_z, norm_before_gate, is_rms, has_bias=not is_rms,
          lead=(3, 37))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim,group_size", [(2048, None), (4096, None), (5120, None), (8192, None), (10240, None),
                                            (16384 - 8, None), (5120, 640), (4096, 2048), (24, 12), (30, 5), (1000, None),
                                            (4100, None), (7, 7)])
def test_team_sizes_and_ragged_groups(dim, group_size, dtype):
    _case(19, dim, group_size, dtype, has_z=True, norm_before_gate=False, is_rms=True, has_bias=True, seed=1)
    _case(5, dim, group_size, dtype, has_z=True, norm_before_gate=True, is_rms=False, has_bias=True, seed=2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_strided_rows_and_low_precision_weights(dtype):
    _case(33, 512, 128, dtype, row_pad=64, seed=3)
    _case(33, 520, 104, dtype, row_pad=3, is_rms=False, has_bias=True, seed=4)
    _case(65, 384, None, dtype, wtype=dtype, has_bias=True, is_rms=False, seed=5)


@pytest.mark.parametrize("dim", [16384 + 8, 24576, 32768])
def test_widest_groups_bf16(dim):
    _case(7, dim, None, torch.bfloat16, norm_before_gate=False, has_bias=True, seed=8)
    with pytest.raises(RuntimeError, match="64KB"):
        _case(2, dim, None, torch.float32)


def test_many_rows_bf16():
    # more rows than parts: every team walks several rows; the shape of the Mamba-2 block at 1/16 length
    _case(4 * 1024, 5120, None, torch.bfloat16, norm_before_gate=False, seed=6)
    _case(3000, 1024, 128, torch.bfloat16, norm_before_gate=False, seed=7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_wide_groups_walk_rows(dtype):
    """Groups of 1024 < n <= 8192 channels in multiples of 512 take the kernels that keep one 16-byte piece per thread
    and request the next row ahead: several rows per workgroup, waves past the end of the group (5120 channels on
    1024 threads, 3072 on 512) that only join the sums, two groups per row, LayerNorm's two sums, no gate, padded
    rows."""
    _case(1500, 5120, None, dtype, has_z=False, seed=9)
    _case(1300, 4096, 2048, dtype, norm_before_gate=True, is_rms=False, has_bias=True, row_pad=8, seed=10)
    _case(2100, 3072, None, dtype, norm_before_gate=False, seed=11)
    _case(1100, 8192, None, dtype, norm_before_gate=False, is_rms=False, has_bias=True, seed=12)
    _case(3, 1536, None, dtype, seed=13)


def test_module_and_empty():
    from mamba_amd.ops.triton.layernorm_gated import RMSNorm, LayerNorm, rmsnorm_fn, rms_norm_ref
    m = RMSNorm(256, eps=1e-5, group_size=64, norm_before_gate=False, device="cuda", dtype=torch.float32)
    x = torch.randn(2, 9, 256, device="cuda", dtype=torch.bfloat16)
    z = torch.randn(2, 9, 256, device="cuda", dtype=torch.bfloat16)
    ref = rms_norm_ref(x, m.weight, None, z=z, eps=1e-5, group_size=64, norm_before_gate=False)
    _close("module", m(x, z), ref, 3e-2, 5e-2)
    ln = LayerNorm(256, device="cuda")
    _close("layernorm", ln(x.float()), torch.nn.functional.layer_norm(x.float(), (256,), eps=1e-5), 6e-4, 2e-3)
    xe, ze, we = x[:0].clone().requires_grad_(), z[:0].clone().requires_grad_(), m.weight.detach().clone().requires_grad_()
    empty = rmsnorm_fn(xe, we, None, z=ze)
    assert empty.shape == (0, 9, 256)
    empty.sum().backward()
    assert xe.grad.shape == (0, 9, 256) and float(we.grad.abs().max()) == 0.0
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        rmsnorm_fn(x.cpu(), m.weight.cpu(), None)


def test_backward_with_recomputed_output():
    from mamba_amd.ops.triton.layernorm_gated import _layer_norm_bwd, _layer_norm_fwd
    g = torch.Generator().manual_seed(9)
    x, z, dy = (torch.randn(37, 256, generator=g).cuda() for _ in range(3))
    w = (1 + 0.1 * torch.randn(256, generator=g)).cuda()
    y, _, rstd = _layer_norm_fwd(x, w, None, 1e-5, z=z, group_size=64, norm_before_gate=False, is_rms_norm=True)
    plain = _layer_norm_bwd(dy, x, w, None, 1e-5, None, rstd, z, 64, False, True)
    again = _layer_norm_bwd(dy, x, w, None, 1e-5, None, rstd, z, 64, False, True, recompute_output=True)
    assert len(again) == 5 and torch.equal(again[4], y)
    for a, b in zip(plain, again[:4]):
        assert (a is None and b is None) or torch.equal(a, b)
