"""Gated LayerNorm / RMSNorm over channel groups on the HIP kernels: drop-in for
mamba_ssm/ops/triton/layernorm_gated.py (`layernorm_fn` :380, `rmsnorm_fn` :384, `LayerNorm` :388,
`RMSNorm` :415), the norm between the chunked scan and the output projection of the Mamba-2 block
(mamba_ssm/modules/mamba2.py:242).

There is no CPU or PyTorch fallback: CPU tensors raise.  `rms_norm_ref` is the plain-torch
statement of the arithmetic that tests import next to the operator; no operator calls it.
"""
import torch
import torch.nn.functional as F

from mamba_amd import _lib


def rms_norm_ref(x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True, upcast=True):
    """RMSNorm(x) * silu(z) (norm_before_gate) or RMSNorm(x * silu(z)), per group of channels."""
    dtype = x.dtype
    weight = weight.float()
    bias = bias.float() if bias is not None else None
    if upcast:
        x = x.float()
        z = z.float() if z is not None else None
    if z is not None and not norm_before_gate:
        x = x * F.silu(z)
    gs = x.shape[-1] if group_size is None else group_size
    xg = x.reshape(*x.shape[:-1], x.shape[-1] // gs, gs)
    rstd = torch.rsqrt(xg.square().mean(dim=-1, keepdim=True) + eps)
    out = (xg * rstd).reshape(x.shape) * weight
    if bias is not None:
        out = out + bias
    if z is not None and norm_before_gate:
        out = out * F.silu(z)
    return out.to(dtype)


def _rows(t, what):
    if t.dim() != 2 or t.stride(-1) != 1:
        raise RuntimeError(f"layernorm_gated: {what} must be (rows, dim) with unit channel stride")
    return t


def _common(p, x, weight32, bias32, z, eps, group_size, norm_before_gate, is_rms_norm):
    M, N = x.shape
    p.rows, p.dim, p.group_size = M, N, group_size
    p.dtype = _lib.DTYPE_CODE[x.dtype]
    p.is_rms, p.norm_before_gate, p.eps = int(is_rms_norm), int(norm_before_gate), eps
    p.x, p.z, p.weight, p.bias = x.data_ptr(), _lib.ptr(z), weight32.data_ptr(), _lib.ptr(bias32)
    p.x_rs = x.stride(0)
    p.z_rs = z.stride(0) if z is not None else 0


def _check(x, weight, bias, z, group_size):
    _lib.require_gpu(x, weight, bias, z)
    if x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError("layernorm_gated: x must be fp32, fp16 or bf16")
    M, N = _rows(x, "x").shape
    group_size = N if group_size is None else group_size
    assert N % group_size == 0
    if z is not None:
        assert _rows(z, "z").shape == (M, N) and z.dtype == x.dtype
    assert weight.shape == (N,)
    if bias is not None:
        assert bias.shape == (N,)
    if group_size > 65536 // x.element_size():
        raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
    return group_size


def _layer_norm_fwd(x, weight, bias, eps, z=None, out=None, group_size=None, norm_before_gate=True,
                    is_rms_norm=False):
    """x, z: (rows, dim).  Returns (out, mean, rstd); mean (None for RMSNorm) and rstd are fp32
    (rows, ngroups)."""
    group_size = _check(x, weight, bias, z, group_size)
    M, N = x.shape
    if out is not None:
        assert out.shape == x.shape and out.dtype == x.dtype and out.stride(-1) == 1
    else:
        out = torch.empty_like(x)
        if out.stride(-1) != 1:
            out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    ngroups = N // group_size
    mean = None if is_rms_norm else torch.empty(M, ngroups, dtype=torch.float32, device=x.device)
    rstd = torch.empty(M, ngroups, dtype=torch.float32, device=x.device)
    if M == 0:
        return out, mean, rstd
    w32 = weight.float().contiguous()
    b32 = bias.float().contiguous() if bias is not None else None
    p = _lib.NormGatedParams()
    _common(p, x, w32, b32, z, eps, group_size, norm_before_gate, is_rms_norm)
    p.out, p.out_rs, p.mean, p.rstd = out.data_ptr(), out.stride(0), _lib.ptr(mean), rstd.data_ptr()
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().norm_gated_fwd(p, _lib.current_stream(x.device)), "norm_gated_fwd")
    return out, mean, rstd


def _layer_norm_bwd(dy, x, weight, bias, eps, mean, rstd, z=None, group_size=None, norm_before_gate=True,
                    is_rms_norm=False, recompute_output=False, dz=None, out=None):
    """Returns (dx, dweight, dbias, dz), plus the forward output with recompute_output (a second launch of the
    forward kernel here; the reference's backward kernel writes it on the side, layernorm_gated.py:271);
    dweight / dbias in the dtype of weight / bias."""
    if recompute_output:
        y = _layer_norm_fwd(x, weight, bias, eps, z=z, out=out, group_size=group_size,
                            norm_before_gate=norm_before_gate, is_rms_norm=is_rms_norm)[0]
        return (*_layer_norm_bwd(dy, x, weight, bias, eps, mean, rstd, z, group_size, norm_before_gate, is_rms_norm,
                                 False, dz), y)
    group_size = _check(x, weight, bias, z, group_size)
    _lib.require_gpu(dy, rstd, mean)
    M, N = x.shape
    assert _rows(dy, "dy").shape == (M, N) and dy.dtype == x.dtype
    ngroups = N // group_size
    dx = torch.empty(M, N, dtype=x.dtype, device=x.device)
    if dz is not None:
        assert z is not None and dz.shape == z.shape and dz.stride(-1) == 1 and dz.dtype == x.dtype
    elif z is not None:
        dz = torch.empty(M, N, dtype=x.dtype, device=x.device)
    if M == 0:
        return dx, torch.zeros_like(weight), torch.zeros_like(bias) if bias is not None else None, dz
    # enough teams of threads to fill the GPU several times over, never more parts than rows
    # the threads per (row, group) norm_gated.hip picks
    team = next((t for t in (8, 16, 32, 64, 256) if group_size <= 16 * t), 1024)
    if group_size % 512 == 0 and 2048 < group_size <= 4096:
        team = 512
    nparts = max(1, min(M, (4096 * 64 // team) // ngroups, 65536))
    nb = 2 if bias is not None else 1
    parts = torch.empty(nb, nparts, N, dtype=torch.float32, device=x.device)
    sums = torch.empty(nb, N, dtype=torch.float32, device=x.device)
    w32 = weight.float().contiguous()
    b32 = bias.float().contiguous() if bias is not None else None
    p = _lib.NormGatedParams()
    _common(p, x, w32, b32, z, eps, group_size, norm_before_gate, is_rms_norm)
    p.nparts = nparts
    p.mean, p.rstd = _lib.ptr(mean), rstd.data_ptr()
    p.dy, p.dy_rs, p.dx, p.dx_rs = dy.data_ptr(), dy.stride(0), dx.data_ptr(), dx.stride(0)
    p.dz, p.dz_rs = _lib.ptr(dz), dz.stride(0) if dz is not None else 0
    p.dweight, p.dw_part = sums[0].data_ptr(), parts[0].data_ptr()
    if bias is not None:
        p.dbias, p.db_part = sums[1].data_ptr(), parts[1].data_ptr()
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().norm_gated_bwd(p, _lib.current_stream(x.device)), "norm_gated_bwd")
    dw = sums[0].to(weight.dtype)
    db = sums[1].to(bias.dtype) if bias is not None else None
    return dx, dw, db, dz


class LayerNormFn(torch.autograd.Function):
    """Same argument order as the reference's LayerNormFn (layernorm_gated.py:338)."""

    @staticmethod
    def forward(ctx, x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True, is_rms_norm=False):
        x_shape_og = x.shape
        x = x.reshape(-1, x.shape[-1])
        if x.stride(-1) != 1:
            x = x.contiguous()
        if z is not None:
            assert z.shape == x_shape_og
            z = z.reshape(-1, z.shape[-1])
            if z.stride(-1) != 1:
                z = z.contiguous()
        weight = weight.contiguous()
        if bias is not None:
            bias = bias.contiguous()
        y, mean, rstd = _layer_norm_fwd(x, weight, bias, eps, z=z, group_size=group_size,
                                        norm_before_gate=norm_before_gate, is_rms_norm=is_rms_norm)
        ctx.save_for_backward(x, weight, bias, mean, rstd, z)
        ctx.x_shape_og = x_shape_og
        ctx.eps, ctx.group_size = eps, group_size
        ctx.norm_before_gate, ctx.is_rms_norm = norm_before_gate, is_rms_norm
        return y.reshape(x_shape_og)

    @staticmethod
    def backward(ctx, dy):
        x, weight, bias, mean, rstd, z = ctx.saved_tensors
        dy = dy.reshape(-1, dy.shape[-1])
        if dy.stride(-1) != 1:
            dy = dy.contiguous()
        assert dy.shape == x.shape
        dx, dw, db, dz = _layer_norm_bwd(dy.to(x.dtype), x, weight, bias, ctx.eps, mean, rstd, z, ctx.group_size,
                                         ctx.norm_before_gate, ctx.is_rms_norm)
        return (dx.reshape(ctx.x_shape_og), dw, db, dz.reshape(ctx.x_shape_og) if dz is not None else None,
                None, None, None, None)


def layernorm_fn(x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True, is_rms_norm=False):
    return LayerNormFn.apply(x, weight, bias, z, eps, group_size, norm_before_gate, is_rms_norm)


def rmsnorm_fn(x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True):
    return LayerNormFn.apply(x, weight, bias, z, eps, group_size, norm_before_gate, True)


class LayerNorm(torch.nn.Module):
    """group_size=None is one group of hidden_size channels (layernorm_gated.py:388)."""

    def __init__(self, hidden_size, eps=1e-5, group_size=None, norm_before_gate=True, device=None, dtype=None):
        super().__init__()
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.bias = torch.nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.group_size = group_size
        self.norm_before_gate = norm_before_gate
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)
        torch.nn.init.zeros_(self.bias)

    def forward(self, x, z=None):
        """norm(x) * silu(z) if norm_before_gate, else norm(x * silu(z))."""
        return layernorm_fn(x, self.weight, self.bias, z=z, group_size=self.group_size, eps=self.eps,
                            norm_before_gate=self.norm_before_gate)


class RMSNorm(torch.nn.Module):
    """group_size=None is one group of hidden_size channels (layernorm_gated.py:415)."""

    def __init__(self, hidden_size, eps=1e-5, group_size=None, norm_before_gate=True, device=None, dtype=None):
        super().__init__()
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.register_parameter("bias", None)
        self.group_size = group_size
        self.norm_before_gate = norm_before_gate
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)

    def forward(self, x, z=None):
        """norm(x) * silu(z) if norm_before_gate, else norm(x * silu(z))."""
        return rmsnorm_fn(x, self.weight, self.bias, z=z, eps=self.eps, group_size=self.group_size,
                          norm_before_gate=self.norm_before_gate)
