"""LayerNorm / RMSNorm with the residual add fused in, on the HIP kernels: drop-in for the part of
mamba_ssm/ops/triton/layer_norm.py the reference's Block and models use (`layer_norm_fn` :888,
`rms_norm_fn` :922, `RMSNorm` :955, `layer_norm_linear_fn` :1092; call sites
mamba_ssm/modules/block.py:57-66, mamba_ssm/models/mixer_seq_simple.py:195-204).

Served: residual, prenorm, residual_in_fp32, LayerNorm or RMSNorm, bias or not.  Not served, and
raising NotImplementedError: dropout, rowscale, the second branch (x1 / weight1 / bias1) — the Mamba
blocks never pass them.  There is no CPU or PyTorch fallback: CPU tensors raise.  `layer_norm_ref` /
`rms_norm_ref` are the plain-torch statements of the arithmetic that tests import next to the
operators; no operator calls them.
"""
import torch
import torch.nn.functional as F

from mamba_amd import _lib


def _unsupported(x1, weight1, bias1, dropout_p, rowscale, return_dropout_mask=False):
    if x1 is not None or weight1 is not None or bias1 is not None:
        raise NotImplementedError("layer_norm: the second branch (x1 / weight1 / bias1) is not supported")
    if dropout_p != 0.0 or return_dropout_mask:
        raise NotImplementedError("layer_norm: dropout is not supported")
    if rowscale is not None:
        raise NotImplementedError("layer_norm: rowscale is not supported")


def layer_norm_ref(x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                   rowscale=None, prenorm=False, dropout_mask=None, dropout_mask1=None, upcast=False):
    _unsupported(x1, weight1, bias1, dropout_p, rowscale)
    dtype = x.dtype
    if upcast:
        x, weight = x.float(), weight.float()
        bias = bias.float() if bias is not None else None
        residual = residual.float() if residual is not None else None
    if residual is not None:
        x = (x + residual).to(x.dtype)
    out = F.layer_norm(x.to(weight.dtype), x.shape[-1:], weight=weight, bias=bias, eps=eps).to(dtype)
    return out if not prenorm else (out, x)


def rms_norm_ref(x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                 rowscale=None, prenorm=False, dropout_mask=None, dropout_mask1=None, upcast=False):
    _unsupported(x1, weight1, bias1, dropout_p, rowscale)
    dtype = x.dtype
    if upcast:
        x, weight = x.float(), weight.float()
        bias = bias.float() if bias is not None else None
        residual = residual.float() if residual is not None else None
    if residual is not None:
        x = (x + residual).to(x.dtype)
    rstd = torch.rsqrt(x.square().mean(dim=-1, keepdim=True) + eps)
    out = (x * rstd * weight + bias if bias is not None else x * rstd * weight).to(dtype)
    return out if not prenorm else (out, x)


def _rows(t, what):
    if t.dim() != 2 or t.stride(-1) != 1:
        raise RuntimeError(f"layer_norm: {what} must be (rows, dim) with unit channel stride")
    return t


def _layer_norm_fwd(x, weight, bias, eps, residual=None, residual_dtype=None, is_rms_norm=False):
    """x, residual: (rows, dim).  Returns (y, mean, rstd, residual_out): residual_out is x + residual
    in the residual's dtype (or residual_dtype), or x itself when no sum has to be written."""
    _lib.require_gpu(x, weight, bias, residual)
    M, N = _rows(x, "x").shape
    if x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError("layer_norm: x must be fp32, fp16 or bf16")
    if residual is not None:
        assert _rows(residual, "residual").shape == (M, N)
        residual_dtype = residual.dtype
    assert weight.shape == (N,)
    if bias is not None:
        assert bias.shape == (N,)
    if N > 65536 // x.element_size():
        raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
    res_dtype = residual_dtype if residual_dtype is not None else x.dtype
    if res_dtype not in (x.dtype, torch.float32):
        raise RuntimeError("layer_norm: the residual stream must be in x's dtype or fp32")
    y = torch.empty(M, N, dtype=x.dtype, device=x.device)
    write_sum = residual is not None or res_dtype != x.dtype
    residual_out = torch.empty(M, N, dtype=res_dtype, device=x.device) if write_sum else None
    mean = None if is_rms_norm else torch.empty(M, dtype=torch.float32, device=x.device)
    rstd = torch.empty(M, dtype=torch.float32, device=x.device)
    if M > 0:
        w32 = weight.float().contiguous()
        b32 = bias.float().contiguous() if bias is not None else None
        p = _lib.NormResidualParams()
        p.rows, p.dim, p.dtype, p.res_dtype = M, N, _lib.DTYPE_CODE[x.dtype], _lib.DTYPE_CODE[res_dtype]
        p.is_rms, p.eps = int(is_rms_norm), eps
        p.x, p.residual, p.weight, p.bias = x.data_ptr(), _lib.ptr(residual), w32.data_ptr(), _lib.ptr(b32)
        p.out, p.residual_out, p.mean, p.rstd = y.data_ptr(), _lib.ptr(residual_out), _lib.ptr(mean), rstd.data_ptr()
        p.x_rs, p.out_rs = x.stride(0), y.stride(0)
        p.residual_rs = residual.stride(0) if residual is not None else 0
        p.residual_out_rs = residual_out.stride(0) if residual_out is not None else 0
        with torch.cuda.device(x.device):
            _lib.check(_lib.load().norm_residual_fwd(p, _lib.current_stream(x.device)), "norm_residual_fwd")
    return y, mean, rstd, residual_out if residual_out is not None else x


def _layer_norm_bwd(dy, x, weight, bias, eps, mean, rstd, dresidual=None, has_residual=False, is_rms_norm=False,
                    x_dtype=None):
    """x is the summed input the forward call saved.  Returns (dx, dweight, dbias, dresidual_in):
    dx in x_dtype (default x.dtype); dresidual_in is dx itself when the dtypes agree."""
    _lib.require_gpu(dy, x, weight, bias, mean, rstd, dresidual)
    M, N = _rows(x, "x").shape
    assert _rows(dy, "dy").shape == (M, N)
    if dresidual is not None:
        assert _rows(dresidual, "dresidual").shape == (M, N) and dresidual.dtype == x.dtype
    x_dtype = x.dtype if x_dtype is None else x_dtype
    if dy.dtype != x_dtype:
        dy = dy.to(x_dtype)
    dx = torch.empty(M, N, dtype=x_dtype, device=x.device)
    dresidual_in = torch.empty(M, N, dtype=x.dtype, device=x.device) if has_residual and x_dtype != x.dtype else None
    if M == 0:
        return (dx, torch.zeros_like(weight), torch.zeros_like(bias) if bias is not None else None,
                dresidual_in if dresidual_in is not None else (dx if has_residual else None))
    team = 64 if N <= 1024 else 256 if N <= 4096 else 512 if N <= 8192 else 1024
    nparts = max(1, min(M, 4096 * 64 // team))
    nb = 2 if bias is not None else 1
    parts = torch.empty(nb, nparts, N, dtype=torch.float32, device=x.device)
    sums = torch.empty(nb, N, dtype=torch.float32, device=x.device)
    w32 = weight.float().contiguous()
    b32 = bias.float().contiguous() if bias is not None else None
    p = _lib.NormResidualParams()
    p.rows, p.dim, p.dtype, p.res_dtype = M, N, _lib.DTYPE_CODE[x_dtype], _lib.DTYPE_CODE[x.dtype]
    p.is_rms, p.eps, p.nparts = int(is_rms_norm), eps, nparts
    p.x, p.weight, p.bias, p.mean, p.rstd = x.data_ptr(), w32.data_ptr(), _lib.ptr(b32), _lib.ptr(mean), rstd.data_ptr()
    p.x_rs = x.stride(0)
    p.dy, p.dy_rs, p.dx, p.dx_rs = dy.data_ptr(), dy.stride(0), dx.data_ptr(), dx.stride(0)
    p.dresidual, p.dresidual_rs = _lib.ptr(dresidual), dresidual.stride(0) if dresidual is not None else 0
    p.dresidual_in = _lib.ptr(dresidual_in)
    p.dresidual_in_rs = dresidual_in.stride(0) if dresidual_in is not None else 0
    p.dweight, p.dw_part = sums[0].data_ptr(), parts[0].data_ptr()
    if bias is not None:
        p.dbias, p.db_part = sums[1].data_ptr(), parts[1].data_ptr()
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().norm_residual_bwd(p, _lib.current_stream(x.device)), "norm_residual_bwd")
    dw = sums[0].to(weight.dtype)
    db = sums[1].to(bias.dtype) if bias is not None else None
    if has_residual and dresidual_in is None:
        dresidual_in = dx
    return dx, dw, db, dresidual_in


class LayerNormFn(torch.autograd.Function):
    """Same argument order as the reference's LayerNormFn (layer_norm.py:728)."""

    @staticmethod
    def forward(ctx, x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                rowscale=None, prenorm=False, residual_in_fp32=False, is_rms_norm=False, return_dropout_mask=False):
        _unsupported(x1, weight1, bias1, dropout_p, rowscale, return_dropout_mask)
        x_shape_og = x.shape
        x = x.reshape(-1, x.shape[-1])
        if x.stride(-1) != 1:
            x = x.contiguous()
        if residual is not None:
            assert residual.shape == x_shape_og
            residual = residual.reshape(-1, residual.shape[-1])
            if residual.stride(-1) != 1:
                residual = residual.contiguous()
        weight = weight.contiguous()
        if bias is not None:
            bias = bias.contiguous()
        residual_dtype = residual.dtype if residual is not None else (torch.float32 if residual_in_fp32 else None)
        y, mean, rstd, residual_out = _layer_norm_fwd(x, weight, bias, eps, residual, residual_dtype=residual_dtype,
                                                       is_rms_norm=is_rms_norm)
        ctx.save_for_backward(residual_out, weight, bias, mean, rstd)
        ctx.x_shape_og = x_shape_og
        ctx.eps, ctx.is_rms_norm = eps, is_rms_norm
        ctx.has_residual, ctx.prenorm, ctx.x_dtype = residual is not None, prenorm, x.dtype
        y = y.reshape(x_shape_og)
        return y if not prenorm else (y, residual_out.reshape(x_shape_og))

    @staticmethod
    def backward(ctx, dy, *args):
        x, weight, bias, mean, rstd = ctx.saved_tensors
        dy = dy.reshape(-1, dy.shape[-1])
        if dy.stride(-1) != 1:
            dy = dy.contiguous()
        assert dy.shape == x.shape
        dresidual = None
        if ctx.prenorm and args[0] is not None:
            dresidual = args[0].reshape(-1, args[0].shape[-1])
            if dresidual.stride(-1) != 1:
                dresidual = dresidual.contiguous()
            assert dresidual.shape == x.shape
            dresidual = dresidual.to(x.dtype)
        dx, dw, db, dresidual_in = _layer_norm_bwd(dy, x, weight, bias, ctx.eps, mean, rstd, dresidual,
                                                   ctx.has_residual, ctx.is_rms_norm, x_dtype=ctx.x_dtype)
        return (dx.reshape(ctx.x_shape_og), dw, db,
                dresidual_in.reshape(ctx.x_shape_og) if ctx.has_residual else None,
                None, None, None, None, None, None, None, None, None, None)


def layer_norm_fn(x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                  rowscale=None, prenorm=False, residual_in_fp32=False, is_rms_norm=False, return_dropout_mask=False):
    return LayerNormFn.apply(x, weight, bias, residual, x1, weight1, bias1, eps, dropout_p, rowscale, prenorm,
                             residual_in_fp32, is_rms_norm, return_dropout_mask)


def rms_norm_fn(x, weight, bias, residual=None, x1=None, weight1=None, bias1=None, eps=1e-6, dropout_p=0.0,
                rowscale=None, prenorm=False, residual_in_fp32=False, return_dropout_mask=False):
    return LayerNormFn.apply(x, weight, bias, residual, x1, weight1, bias1, eps, dropout_p, rowscale, prenorm,
                             residual_in_fp32, True, return_dropout_mask)


class RMSNorm(torch.nn.Module):
    """layer_norm.py:955; dropout_p must stay 0."""

    def __init__(self, hidden_size, eps=1e-5, dropout_p=0.0, device=None, dtype=None):
        super().__init__()
        if dropout_p > 0.0:
            raise NotImplementedError("RMSNorm: dropout is not supported")
        self.eps = eps
        self.drop = None
        self.weight = torch.nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)

    def forward(self, x, residual=None, prenorm=False, residual_in_fp32=False):
        return rms_norm_fn(x, self.weight, self.bias, residual=residual, eps=self.eps, prenorm=prenorm,
                           residual_in_fp32=residual_in_fp32)


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
