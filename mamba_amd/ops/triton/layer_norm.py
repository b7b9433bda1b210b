"""LayerNorm / RMSNorm with the residual add fused in, on the HIP kernels: drop-in for
mamba_ssm/ops/triton/layer_norm.py (`layer_norm_fn` :888, `rms_norm_fn` :922, `RMSNorm` :955,
`layer_norm_linear_fn` :1092; call sites mamba_ssm/modules/block.py:57-66,
mamba_ssm/models/mixer_seq_simple.py:195-204).

Served: residual, prenorm, residual_in_fp32, LayerNorm or RMSNorm, bias or not, and the operator's other
arguments: `rowscale` (a factor per row on x), `dropout_p` (on x and on x1, each with its own draws;
`return_dropout_mask` hands the draws back), the second input `x1` (added to x) and the second set of norm
parameters `weight1` / `bias1` (a second output from the same normalised rows).  The draws come from a hash of
(seed, row, channel) inside the kernel, seeded from torch's generator, so they differ from the reference's
Philox stream bit for bit; the reference's own tests compare through the returned masks, as the tests here do.
There is no CPU or PyTorch fallback: CPU tensors raise.  `layer_norm_ref` / `rms_norm_ref` are the plain-torch
statements of the arithmetic that tests import next to the operators; no operator calls them.
"""
import torch
import torch.nn.functional as F

from mamba_amd import _lib


def _ref_sum(x, residual, x1, dropout_p, rowscale, dropout_mask, dropout_mask1):
    """The row the norm sees: drop(x * rowscale) + drop1(x1) + residual (layer_norm.py:46-62)."""
    if x1 is not None:
        assert rowscale is None, "rowscale is not supported with parallel LayerNorm"
    if rowscale is not None:
        x = x * rowscale[..., None]
    if dropout_p > 0.0:
        keep = 1.0 - dropout_p
        x = x.masked_fill(~dropout_mask, 0.0) / keep if dropout_mask is not None else F.dropout(x, p=dropout_p)
        if x1 is not None:
            x1 = (x1.masked_fill(~dropout_mask1, 0.0) / keep if dropout_mask1 is not None
                  else F.dropout(x1, p=dropout_p))
    if x1 is not None:
        x = x + x1
    if residual is not None:
        x = (x + residual).to(x.dtype)
    return x


def _ref(norm, x, weight, bias, residual, x1, weight1, bias1, eps, dropout_p, rowscale, prenorm, dropout_mask,
         dropout_mask1, upcast):
    dtype = x.dtype
    if upcast:
        up = lambda t: t.float() if t is not None else None
        x, weight, bias, residual, x1, weight1, bias1 = map(up, (x, weight, bias, residual, x1, weight1, bias1))
    x = _ref_sum(x, residual, x1, dropout_p, rowscale, dropout_mask, dropout_mask1)
    out = norm(x, weight, bias, eps).to(dtype)
    if weight1 is None:
        return out if not prenorm else (out, x)
    out1 = norm(x, weight1, bias1, eps).to(dtype)
    return (out, out1) if not prenorm else (out, out1, x)


def _ln(x, weight, bias, eps):
    return F.layer_norm(x.to(weight.dtype), x.shape[-1:], weight=weight, bias=bias, eps=eps)


def _rms(x, weight, bias, eps):
    rstd = torch.rsqrt(x.square().mean(dim=-1, keepdim=True) + eps)
    return x * rstd * weight + bias if bias is not None else x * rstd * weight


def layer_norm_ref(x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                   rowscale=None, prenorm=False, dropout_mask=None, dropout_mask1=None, upcast=False):
    return _ref(_ln, x, weight, bias, residual, x1, weight1, bias1, eps, dropout_p, rowscale, prenorm, dropout_mask,
                dropout_mask1, upcast)


def rms_norm_ref(x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                 rowscale=None, prenorm=False, dropout_mask=None, dropout_mask1=None, upcast=False):
    return _ref(_rms, x, weight, bias, residual, x1, weight1, bias1, eps, dropout_p, rowscale, prenorm, dropout_mask,
                dropout_mask1, upcast)


def _rows(t, what):
    if t.dim() != 2 or t.stride(-1) != 1:
        raise RuntimeError(f"layer_norm: {what} must be (rows, dim) with unit channel stride")
    return t


def _layer_norm_fwd(x, weight, bias, eps, residual=None, x1=None, weight1=None, bias1=None, dropout_p=0.0,
                    rowscale=None, residual_dtype=None, is_rms_norm=False, return_dropout_mask=False):
    """x, residual, x1: (rows, dim).  Returns (y, y1, mean, rstd, residual_out, seeds, dropout_mask, dropout_mask1)
    in the reference's order (layer_norm.py:291): residual_out is the summed row the norm saw, in the residual's
    dtype (or residual_dtype), or x itself when no sum has to be written; seeds are the two words the dropout
    draws of x and x1 derive from (None without dropout)."""
    _lib.require_gpu(x, weight, bias, residual, x1, weight1, bias1, rowscale)
    M, N = _rows(x, "x").shape
    if x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError("layer_norm: x must be fp32, fp16 or bf16")
    if residual is not None:
        assert _rows(residual, "residual").shape == (M, N)
        residual_dtype = residual.dtype
    assert weight.shape == (N,)
    if bias is not None:
        assert bias.shape == (N,)
    if x1 is not None:
        assert _rows(x1, "x1").shape == (M, N) and x1.dtype == x.dtype
        assert rowscale is None, "rowscale is not supported with parallel LayerNorm"
    if weight1 is not None:
        assert weight1.shape == (N,)
    if bias1 is not None:
        assert weight1 is not None and bias1.shape == (N,)
    if rowscale is not None:
        assert rowscale.is_contiguous() and rowscale.shape == (M,)
    if not 0.0 <= dropout_p < 1.0:
        raise ValueError(f"layer_norm: dropout_p must be in [0, 1), got {dropout_p}")
    if N > 65536 // x.element_size():
        raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
    res_dtype = residual_dtype if residual_dtype is not None else x.dtype
    if res_dtype not in (x.dtype, torch.float32):
        raise RuntimeError("layer_norm: the residual stream must be in x's dtype or fp32")
    y = torch.empty(M, N, dtype=x.dtype, device=x.device)
    y1 = torch.empty(M, N, dtype=x.dtype, device=x.device) if weight1 is not None else None
    # the sum is written whenever it is not x itself (layer_norm.py:320-330)
    write_sum = (residual is not None or res_dtype != x.dtype or dropout_p > 0.0 or rowscale is not None
                 or x1 is not None)
    residual_out = torch.empty(M, N, dtype=res_dtype, device=x.device) if write_sum else None
    mean = None if is_rms_norm else torch.empty(M, dtype=torch.float32, device=x.device)
    rstd = torch.empty(M, dtype=torch.float32, device=x.device)
    seeds = dropout_mask = dropout_mask1 = None
    if dropout_p > 0.0:
        seeds = torch.randint(2 ** 32, (2,), device=x.device, dtype=torch.int64)  # torch's generator, no host sync
        if return_dropout_mask:
            dropout_mask = torch.empty(M, N, dtype=torch.bool, device=x.device)
            dropout_mask1 = torch.empty(M, N, dtype=torch.bool, device=x.device) if x1 is not None else None
    if M > 0:
        f32 = lambda t: t.float().contiguous() if t is not None else None
        w32, b32, w132, b132, rs32 = f32(weight), f32(bias), f32(weight1), f32(bias1), f32(rowscale)
        p = _lib.NormResidualParams()
        p.rows, p.dim, p.dtype, p.res_dtype = M, N, _lib.DTYPE_CODE[x.dtype], _lib.DTYPE_CODE[res_dtype]
        p.is_rms, p.eps = int(is_rms_norm), eps
        p.x, p.residual, p.weight, p.bias = x.data_ptr(), _lib.ptr(residual), w32.data_ptr(), _lib.ptr(b32)
        p.out, p.residual_out, p.mean, p.rstd = y.data_ptr(), _lib.ptr(residual_out), _lib.ptr(mean), rstd.data_ptr()
        p.x_rs, p.out_rs = x.stride(0), y.stride(0)
        p.residual_rs = residual.stride(0) if residual is not None else 0
        p.residual_out_rs = residual_out.stride(0) if residual_out is not None else 0
        p.x1, p.x1_rs = _lib.ptr(x1), x1.stride(0) if x1 is not None else 0
        p.rowscale, p.seeds, p.dropout_p = _lib.ptr(rs32), _lib.ptr(seeds), dropout_p
        p.mask, p.mask1 = _lib.ptr(dropout_mask), _lib.ptr(dropout_mask1)
        p.weight1, p.bias1, p.out1 = _lib.ptr(w132), _lib.ptr(b132), _lib.ptr(y1)
        p.out1_rs = y1.stride(0) if y1 is not None else 0
        with torch.cuda.device(x.device):
            _lib.check(_lib.load().norm_residual_fwd(p, _lib.current_stream(x.device)), "norm_residual_fwd")
    return y, y1, mean, rstd, residual_out if residual_out is not None else x, seeds, dropout_mask, dropout_mask1


def _layer_norm_bwd(dy, x, weight, bias, eps, mean, rstd, dresidual=None, dy1=None, weight1=None, bias1=None,
                    seeds=None, dropout_p=0.0, rowscale=None, has_residual=False, has_x1=False, is_rms_norm=False,
                    x_dtype=None):
    """x is the summed row the forward call saved.  Returns (dx, dweight, dbias, dresidual_in, dx1, dweight1,
    dbias1) in the reference's order (layer_norm.py:589): dx, dx1 in x_dtype (default x.dtype); dresidual_in, the
    gradient of the sum, is dx itself where the two are the same tensor (no dropout or rowscale, one dtype)."""
    _lib.require_gpu(dy, x, weight, bias, mean, rstd, dresidual, dy1, weight1, bias1, seeds, rowscale)
    M, N = _rows(x, "x").shape
    assert _rows(dy, "dy").shape == (M, N)
    if dresidual is not None:
        assert _rows(dresidual, "dresidual").shape == (M, N) and dresidual.dtype == x.dtype
    if weight1 is not None:
        assert dy1 is not None and _rows(dy1, "dy1").shape == (M, N)
    if dropout_p > 0.0:
        assert seeds is not None
    x_dtype = x.dtype if x_dtype is None else x_dtype
    if dy.dtype != x_dtype:
        dy = dy.to(x_dtype)
    if dy1 is not None and dy1.dtype != x_dtype:
        dy1 = dy1.to(x_dtype)
    dx = torch.empty(M, N, dtype=x_dtype, device=x.device)
    dx1 = torch.empty(M, N, dtype=x_dtype, device=x.device) if has_x1 else None
    # dx is the gradient of the sum only without dropout / rowscale and in the stream's dtype
    own_dres = has_residual and (x_dtype != x.dtype or dropout_p > 0.0 or rowscale is not None)
    dresidual_in = torch.empty(M, N, dtype=x.dtype, device=x.device) if own_dres else None
    if M == 0:
        z = lambda t: torch.zeros_like(t) if t is not None else None
        return (dx, z(weight), z(bias), dresidual_in if dresidual_in is not None else (dx if has_residual else None),
                dx1, z(weight1), z(bias1))
    team = 64 if N <= 1024 else 256 if N <= 4096 else 512 if N <= 8192 else 1024
    nparts = max(1, min(M, 4096 * 64 // team))
    nb = (2 if bias is not None else 1) + (0 if weight1 is None else 2 if bias1 is not None else 1)
    parts = torch.empty(nb, nparts, N, dtype=torch.float32, device=x.device)
    sums = torch.empty(nb, N, dtype=torch.float32, device=x.device)
    f32 = lambda t: t.float().contiguous() if t is not None else None
    w32, b32, w132, b132, rs32 = f32(weight), f32(bias), f32(weight1), f32(bias1), f32(rowscale)
    p = _lib.NormResidualParams()
    p.rows, p.dim, p.dtype, p.res_dtype = M, N, _lib.DTYPE_CODE[x_dtype], _lib.DTYPE_CODE[x.dtype]
    p.is_rms, p.eps, p.nparts = int(is_rms_norm), eps, nparts
    p.x, p.weight, p.bias, p.mean, p.rstd = x.data_ptr(), w32.data_ptr(), _lib.ptr(b32), _lib.ptr(mean), rstd.data_ptr()
    p.x_rs = x.stride(0)
    p.dy, p.dy_rs, p.dx, p.dx_rs = dy.data_ptr(), dy.stride(0), dx.data_ptr(), dx.stride(0)
    p.dresidual, p.dresidual_rs = _lib.ptr(dresidual), dresidual.stride(0) if dresidual is not None else 0
    p.dresidual_in = _lib.ptr(dresidual_in)
    p.dresidual_in_rs = dresidual_in.stride(0) if dresidual_in is not None else 0
    slot = 0
    p.dweight, p.dw_part = sums[slot].data_ptr(), parts[slot].data_ptr()
    slot += 1
    if bias is not None:
        p.dbias, p.db_part = sums[slot].data_ptr(), parts[slot].data_ptr()
        ib, slot = slot, slot + 1
    p.rowscale, p.seeds, p.dropout_p = _lib.ptr(rs32), _lib.ptr(seeds), dropout_p
    if has_x1:
        p.x1, p.x1_rs = x.data_ptr(), x.stride(0)  # only says that there was a second input: it is not read
        p.dx1, p.dx1_rs = dx1.data_ptr(), dx1.stride(0)
    if weight1 is not None:
        p.weight1, p.bias1 = w132.data_ptr(), _lib.ptr(b132)
        p.dy1, p.dy1_rs = dy1.data_ptr(), dy1.stride(0)
        p.dweight1, p.dw1_part = sums[slot].data_ptr(), parts[slot].data_ptr()
        iw1, slot = slot, slot + 1
        if bias1 is not None:
            p.dbias1, p.db1_part = sums[slot].data_ptr(), parts[slot].data_ptr()
            ib1 = slot
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().norm_residual_bwd(p, _lib.current_stream(x.device)), "norm_residual_bwd")
    dw = sums[0].to(weight.dtype)
    db = sums[ib].to(bias.dtype) if bias is not None else None
    dw1 = sums[iw1].to(weight1.dtype) if weight1 is not None else None
    db1 = sums[ib1].to(bias1.dtype) if bias1 is not None else None
    if has_residual and dresidual_in is None:
        dresidual_in = dx
    return dx, dw, db, dresidual_in, dx1, dw1, db1


class LayerNormFn(torch.autograd.Function):
    """Same argument order and return forms as the reference's LayerNormFn (layer_norm.py:728)."""

    @staticmethod
    def forward(ctx, x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                rowscale=None, prenorm=False, residual_in_fp32=False, is_rms_norm=False, return_dropout_mask=False):
        x_shape_og = x.shape
        rows = lambda t: t.reshape(-1, t.shape[-1]) if t.stride(-1) == 1 else t.reshape(-1, t.shape[-1]).contiguous()
        x = rows(x)
        if x.stride(-1) != 1:
            x = x.contiguous()
        if residual is not None:
            assert residual.shape == x_shape_og
            residual = rows(residual)
            if residual.stride(-1) != 1:
                residual = residual.contiguous()
        if x1 is not None:
            assert x1.shape == x_shape_og
            assert rowscale is None, "rowscale is not supported with parallel LayerNorm"
            x1 = rows(x1)
            if x1.stride(-1) != 1:
                x1 = x1.contiguous()
        weight = weight.contiguous()
        bias = bias.contiguous() if bias is not None else None
        weight1 = weight1.contiguous() if weight1 is not None else None
        bias1 = bias1.contiguous() if bias1 is not None else None
        if rowscale is not None:
            rowscale = rowscale.reshape(-1).contiguous()
        residual_dtype = residual.dtype if residual is not None else (torch.float32 if residual_in_fp32 else None)
        y, y1, mean, rstd, residual_out, seeds, dropout_mask, dropout_mask1 = _layer_norm_fwd(
            x, weight, bias, eps, residual, x1, weight1, bias1, dropout_p=dropout_p, rowscale=rowscale,
            residual_dtype=residual_dtype, is_rms_norm=is_rms_norm, return_dropout_mask=return_dropout_mask)
        ctx.save_for_backward(residual_out, weight, bias, weight1, bias1, rowscale, seeds, mean, rstd)
        ctx.x_shape_og = x_shape_og
        ctx.eps, ctx.dropout_p, ctx.is_rms_norm = eps, dropout_p, is_rms_norm
        ctx.has_residual, ctx.has_x1, ctx.prenorm, ctx.x_dtype = residual is not None, x1 is not None, prenorm, x.dtype
        og = lambda t: t.reshape(x_shape_og) if t is not None else None
        y, y1, residual_out, dropout_mask, dropout_mask1 = map(og, (y, y1, residual_out, dropout_mask, dropout_mask1))
        outs = (y,) if weight1 is None else (y, y1)
        if prenorm:
            outs += (residual_out,)
        if return_dropout_mask:
            outs += (dropout_mask, dropout_mask1)
        return outs[0] if len(outs) == 1 else outs

    @staticmethod
    def backward(ctx, dy, *args):
        x, weight, bias, weight1, bias1, rowscale, seeds, mean, rstd = ctx.saved_tensors
        rows = lambda t: t.reshape(-1, t.shape[-1]) if t.stride(-1) == 1 else t.reshape(-1, t.shape[-1]).contiguous()
        dy = rows(dy)
        if dy.stride(-1) != 1:
            dy = dy.contiguous()
        assert dy.shape == x.shape
        dy1 = None
        if weight1 is not None:
            dy1, args = args[0], args[1:]
            dy1 = rows(dy1) if dy1 is not None else torch.zeros_like(dy)
            if dy1.stride(-1) != 1:
                dy1 = dy1.contiguous()
            assert dy1.shape == x.shape
        dresidual = None
        if ctx.prenorm and args[0] is not None:
            dresidual = rows(args[0])
            if dresidual.stride(-1) != 1:
                dresidual = dresidual.contiguous()
            assert dresidual.shape == x.shape
            dresidual = dresidual.to(x.dtype)
        dx, dw, db, dresidual_in, dx1, dw1, db1 = _layer_norm_bwd(
            dy, x, weight, bias, ctx.eps, mean, rstd, dresidual, dy1, weight1, bias1, seeds, ctx.dropout_p, rowscale,
            ctx.has_residual, ctx.has_x1, ctx.is_rms_norm, x_dtype=ctx.x_dtype)
        return (dx.reshape(ctx.x_shape_og), dw, db,
                dresidual_in.reshape(ctx.x_shape_og) if ctx.has_residual else None,
                dx1.reshape(ctx.x_shape_og) if dx1 is not None else None, dw1, db1,
                None, None, None, None, None, None, None)


def layer_norm_fn(x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                  rowscale=None, prenorm=False, residual_in_fp32=False, is_rms_norm=False, return_dropout_mask=False):
    return LayerNormFn.apply(x, weight, bias, residual, x1, weight1, bias1, eps, dropout_p, rowscale, prenorm,
                             residual_in_fp32, is_rms_norm, return_dropout_mask)


def rms_norm_fn(x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                rowscale=None, prenorm=False, residual_in_fp32=False, return_dropout_mask=False):
    return LayerNormFn.apply(x, weight, bias, residual, x1, weight1, bias1, eps, dropout_p, rowscale, prenorm,
                             residual_in_fp32, True, return_dropout_mask)


class RMSNorm(torch.nn.Module):
    """layer_norm.py:955: dropout (in training mode) on the input, then the residual add and RMSNorm."""

    def __init__(self, hidden_size, eps=1e-5, dropout_p=0.0, device=None, dtype=None):
        super().__init__()
        self.eps = eps
        self.drop = torch.nn.Dropout(dropout_p) if dropout_p > 0.0 else None
        self.weight = torch.nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)

    def forward(self, x, residual=None, prenorm=False, residual_in_fp32=False):
        return rms_norm_fn(x, self.weight, self.bias, residual=residual, eps=self.eps,
                           dropout_p=self.drop.p if self.drop is not None and self.training else 0.0,
                           prenorm=prenorm, residual_in_fp32=residual_in_fp32)


class LayerNormLinearFn:
    """Name of the reference's fused autograd function (layer_norm.py:985); `apply` takes its arguments in
    the same order and chains LayerNormFn with a torch GEMM."""

    @staticmethod
    def apply(x, norm_weight, norm_bias, linear_weight, linear_bias, residual=None, eps=1e-6, prenorm=False,
              residual_in_fp32=False, is_rms_norm=False):
        return layer_norm_linear_fn(x, norm_weight, norm_bias, linear_weight, linear_bias, residual, eps, prenorm,
                                    residual_in_fp32, is_rms_norm)


def layer_norm_linear_fn(x, norm_weight, norm_bias, linear_weight, linear_bias, residual=None, eps=1e-6,
                         prenorm=False, residual_in_fp32=False, is_rms_norm=False):
    """Norm on the HIP kernels followed by a torch GEMM (layer_norm.py:1092 keeps only the norm's input
    for the backward pass; here autograd also keeps the normalised activations)."""
    res = layer_norm_fn(x, norm_weight, norm_bias, residual=residual, eps=eps, prenorm=prenorm,
                        residual_in_fp32=residual_in_fp32, is_rms_norm=is_rms_norm)
    y, residual_out = res if prenorm else (res, None)
    if torch.is_autocast_enabled():
        ac = torch.get_autocast_dtype("cuda")
        y, linear_weight = y.to(ac), linear_weight.to(ac)
        linear_bias = linear_bias.to(ac) if linear_bias is not None else None
    out = F.linear(y.to(linear_weight.dtype), linear_weight, linear_bias)
    return out if not prenorm else (out, residual_out)
