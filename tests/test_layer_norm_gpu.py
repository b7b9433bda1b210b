"""GPU parity of the HIP residual-add LayerNorm / RMSNorm against oracle/norm.py applied to
x + residual (pinned on the CPU by tests/test_oracle_norm.py), forward, the handed-on sum, and every
gradient.  The options follow the part of the reference's own test (tests/ops/triton/test_layer_norm.py)
that the Mamba blocks use: residual or not, prenorm or not, fp32 residual stream next to low-precision
activations, RMS or not, bias or not.  The operator's other arguments (rowscale, dropout, the second input x1, the
second set of norm parameters weight1 / bias1; mamba_ssm/ops/triton/layer_norm.py:25-75 states their arithmetic)
are checked the way that arithmetic is stated there: the same sum rebuilt in float64 from the dropout masks the
operator hands back, then the oracle norm on it, forward and every gradient."""
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


def _case(shape, dtype, has_residual=True, prenorm=True, residual_in_fp32=False, is_rms=True, has_bias=False,
          res_dtype=None, seed=0):
    from mamba_amd.ops.triton.layer_norm import layer_norm_fn
    g = torch.Generator().manual_seed(seed)
    dim = shape[-1]
    res_dtype = res_dtype or (torch.float32 if residual_in_fp32 else dtype)
    x = (torch.randn(*shape, generator=g) * 1.5 + 0.2).to(dtype)
    res = torch.randn(*shape, generator=g).to(res_dtype) if has_residual else None
    w = 1 + 0.2 * torch.randn(dim, generator=g)
    b = 0.5 * torch.randn(dim, generator=g) if has_bias else None
    dy = torch.randn(*shape, generator=g).to(dtype)
    sum_dtype = res.dtype if has_residual else (torch.float32 if residual_in_fp32 else dtype)
    dres = torch.randn(*shape, generator=g).to(sum_dtype) if prenorm else None
    rtol, atol = _tol(dtype)
    leaf = lambda t: t.double().clone().requires_grad_() if t is not None else None
    xr, rr, wr, br = leaf(x), leaf(res), leaf(w), leaf(b)
    s = xr + rr if has_residual else xr
    ref = gated_norm_oracle(s, wr, br, None, 1e-5, None, True, is_rms)
    loss = (ref * dy.double()).sum()
    if prenorm:
        loss = loss + (s * dres.double()).sum()
    loss.backward()
    dev = lambda t: t.cuda().requires_grad_() if t is not None else None
    xg, rg, wg, bg = dev(x), dev(res), dev(w), dev(b)
    out = layer_norm_fn(xg, wg, bg, residual=rg, eps=1e-5, prenorm=prenorm, residual_in_fp32=residual_in_fp32,
                        is_rms_norm=is_rms)
    if prenorm:
        out, res_out = out
        assert res_out.dtype == sum_dtype and res_out.shape == x.shape
        st = _tol(sum_dtype)
        _close("residual_out", res_out, s, st[0], st[1])
        torch.autograd.backward([out, res_out], [dy.cuda(), dres.cuda()])
    else:
        out.backward(dy.cuda())
    assert out.dtype == dtype and out.shape == x.shape
    _close("out", out, ref, rtol, atol)
    assert xg.grad.dtype == dtype
    _close("dx", xg.grad, xr.grad, rtol * 2, atol * 2)
    if has_residual:
        assert rg.grad.dtype == res.dtype
        rt = _tol(res.dtype)
        _close("dresidual", rg.grad, rr.grad, max(rt[0], 6e-4) * 2, max(rt[1], 2e-3) * 2)
    nrows = x.numel() // dim
    scale = max(1.0, nrows ** 0.5 / 4)
    _close("dweight", wg.grad, wr.grad, rtol * 2, atol * 2 * scale)
    if has_bias:
        _close("dbias", bg.grad, br.grad, rtol * 2, atol * 2 * scale)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("residual_in_fp32", [False, True])
@pytest.mark.parametrize("prenorm", [False, True])
@pytest.mark.parametrize("has_residual", [False, True])
@pytest.mark.parametrize("dim", [192, 2048, 2560])
def test_block_options(dim, has_residual, prenorm, residual_in_fp32, is_rms, dtype):
    # an fp32 residual stream next to low-precision activations when residual_in_fp32 (block.py:60-66)
    res_dtype = torch.float32 if residual_in_fp32 else dtype
    _case((2, 41, dim), dtype, has_residual, prenorm, residual_in_fp32, is_rms, has_bias=not is_rms,
          res_dtype=res_dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim", [8, 30, 1000, 1024, 4096, 5120, 8192, 8200, 12288, 16384])
def test_team_sizes_and_ragged_dims(dim, dtype):
    _case((23, dim), dtype, residual_in_fp32=True, res_dtype=torch.float32, has_bias=True, seed=dim)
    _case((5, dim), dtype, is_rms=False, has_bias=True, seed=dim + 1)


def test_many_rows_and_module():
    from mamba_amd.ops.triton.layer_norm import RMSNorm, layer_norm_linear_fn, rms_norm_ref
    _case((4 * 1024, 2560), torch.bfloat16, residual_in_fp32=True, res_dtype=torch.float32, seed=9)
    m = RMSNorm(512, device="cuda")
    x = torch.randn(3, 7, 512, device="cuda", dtype=torch.bfloat16)
    res = torch.randn(3, 7, 512, device="cuda", dtype=torch.float32)
    y, r = m(x, residual=res, prenorm=True, residual_in_fp32=True)
    yr, rr = rms_norm_ref(x, m.weight, None, residual=res, eps=m.eps, prenorm=True, upcast=True)
    _close("module out", y, yr, 3e-2, 5e-2)
    _close("module residual", r, rr, 6e-4, 2e-3)
    lw = torch.randn(64, 512, device="cuda", dtype=torch.bfloat16) * 0.05
    out = layer_norm_linear_fn(x, m.weight, None, lw, None, residual=res, eps=m.eps, is_rms_norm=True)
    _close("norm + linear", out, torch.nn.functional.linear(yr.float(), lw.float()), 3e-2, 5e-2)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        m.cpu()(x.cpu())


def _extras_case(shape, dtype, is_rms, has_residual, prenorm, dropout_p, has_rowscale, has_x1, has_w1, has_b1, seed=0):
    from mamba_amd.ops.triton.layer_norm import layer_norm_fn
    g = torch.Generator().manual_seed(seed)
    dim = shape[-1]
    x = (torch.randn(*shape, generator=g) * 1.5 + 0.2).to(dtype)
    x1 = torch.randn(*shape, generator=g).to(dtype) if has_x1 else None
    res = torch.randn(*shape, generator=g).to(torch.float32) if has_residual else None
    rowscale = (0.5 + torch.rand(*shape[:-1], generator=g)).to(dtype) if has_rowscale else None
    w = 1 + 0.2 * torch.randn(dim, generator=g)
    b = 0.5 * torch.randn(dim, generator=g) if not is_rms else None
    w1 = 1 + 0.2 * torch.randn(dim, generator=g) if has_w1 else None
    b1 = 0.5 * torch.randn(dim, generator=g) if has_b1 else None
    dy = torch.randn(*shape, generator=g).to(dtype)
    dy1 = torch.randn(*shape, generator=g).to(dtype) if has_w1 else None
    sum_dtype = torch.float32 if has_residual else dtype
    dres = torch.randn(*shape, generator=g).to(sum_dtype) if prenorm else None
    dev = lambda t: t.cuda().requires_grad_() if t is not None else None
    xg, x1g, rg, wg, bg, w1g, b1g = dev(x), dev(x1), dev(res), dev(w), dev(b), dev(w1), dev(b1)
    outs = layer_norm_fn(xg, wg, bg, residual=rg, x1=x1g, weight1=w1g, bias1=b1g, eps=1e-5, dropout_p=dropout_p,
                         rowscale=rowscale.cuda() if has_rowscale else None, prenorm=prenorm, is_rms_norm=is_rms,
                         return_dropout_mask=True)
    outs = list(outs)
    out = outs.pop(0)
    out1 = outs.pop(0) if has_w1 else None
    res_out = outs.pop(0) if prenorm else None
    mask, mask1 = outs
    if dropout_p > 0:
        assert mask.dtype == torch.bool and mask.shape == x.shape
        kept = mask.float().mean().item()
        assert abs(kept - (1 - dropout_p)) < 0.03, f"kept {kept}"
        assert (mask1 is not None) == has_x1
        if has_x1:
            assert abs(mask1.float().mean().item() - (1 - dropout_p)) < 0.03
            assert (mask ^ mask1).float().mean().item() > 0.1, "the two inputs must not share their draws"
        assert (mask[0] ^ mask[-1]).any(), "rows must not share their draws"
    else:
        assert mask is None and mask1 is None
    # the same arithmetic in float64 (layer_norm.py:46-62), with the operator's own draws
    leaf = lambda t: t.double().clone().requires_grad_() if t is not None else None
    xr, x1r, rr, wr, br, w1r, b1r = leaf(x), leaf(x1), leaf(res), leaf(w), leaf(b), leaf(w1), leaf(b1)
    s = xr * rowscale.double()[..., None] if has_rowscale else xr
    if dropout_p > 0:
        s = s.masked_fill(~mask.cpu(), 0.0) / (1 - dropout_p)
    if has_x1:
        t = x1r.masked_fill(~mask1.cpu(), 0.0) / (1 - dropout_p) if dropout_p > 0 else x1r
        s = s + t
    if has_residual:
        s = s + rr
    ref = gated_norm_oracle(s, wr, br, None, 1e-5, None, True, is_rms)
    loss = (ref * dy.double()).sum()
    if has_w1:
        ref1 = gated_norm_oracle(s, w1r, b1r, None, 1e-5, None, True, is_rms)
        loss = loss + (ref1 * dy1.double()).sum()
    if prenorm:
        loss = loss + (s * dres.double()).sum()
    loss.backward()
    rtol, atol = _tol(dtype)
    _close("out", out, ref, rtol, atol)
    heads, grads = [out], [dy.cuda()]
    if has_w1:
        _close("out1", out1, ref1, rtol, atol)
        heads.append(out1)
        grads.append(dy1.cuda())
    if prenorm:
        st = _tol(sum_dtype)
        _close("residual_out", res_out, s, st[0], st[1])
        heads.append(res_out)
        grads.append(dres.cuda())
    torch.autograd.backward(heads, grads)
    _close("dx", xg.grad, xr.grad, rtol * 2, atol * 2)
    if has_x1:
        _close("dx1", x1g.grad, x1r.grad, rtol * 2, atol * 2)
    if has_residual:
        _close("dresidual", rg.grad, rr.grad, 6e-4 * 2, 2e-3 * 2)
    if dropout_p > 0:
        assert bool((xg.grad[~mask] == 0).all()), "no gradient through a dropped element"
    nrows = x.numel() // dim
    scale = max(1.0, nrows ** 0.5 / 4)
    _close("dweight", wg.grad, wr.grad, rtol * 2, atol * 2 * scale)
    if b is not None:
        _close("dbias", bg.grad, br.grad, rtol * 2, atol * 2 * scale)
    if has_w1:
        _close("dweight1", w1g.grad, w1r.grad, rtol * 2, atol * 2 * scale)
    if has_b1:
        _close("dbias1", b1g.grad, b1r.grad, rtol * 2, atol * 2 * scale)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("variant", ["rowscale", "dropout", "rowscale_dropout", "x1", "x1_dropout", "w1", "x1_w1_b1_dropout"])
@pytest.mark.parametrize("prenorm,has_residual", [(False, False), (True, True)])
def test_rowscale_dropout_second_branch(variant, prenorm, has_residual, is_rms, dtype):
    _extras_case((3, 37, 1000 if dtype == torch.float32 else 2048), dtype, is_rms, has_residual, prenorm,
                 dropout_p=0.25 if "dropout" in variant else 0.0, has_rowscale="rowscale" in variant,
                 has_x1="x1" in variant, has_w1="w1" in variant, has_b1="b1" in variant, seed=len(variant))


def test_dropout_module_and_errors():
    from mamba_amd.ops.triton.layer_norm import RMSNorm, layer_norm_fn
    m = RMSNorm(512, dropout_p=0.5, device="cuda")
    x = torch.randn(64, 512, device="cuda", dtype=torch.bfloat16)
    m.eval()
    y_eval = m(x)
    assert torch.equal(y_eval, RMSNorm(512, device="cuda")(x)), "no dropout outside training"
    m.train()
    y1, y2 = m(x), m(x)
    assert not torch.equal(y1, y2), "two calls draw from torch's generator"
    torch.manual_seed(5)
    a = m(x)
    torch.manual_seed(5)
    assert torch.equal(a, m(x)), "the draws follow torch's seed"
    with pytest.raises(AssertionError):
        layer_norm_fn(x, m.weight, None, x1=x, rowscale=torch.ones(64, device="cuda"))
    with pytest.raises(ValueError):
        layer_norm_fn(x, m.weight, None, dropout_p=1.0)
