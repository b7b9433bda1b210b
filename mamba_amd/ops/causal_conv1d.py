"""Depthwise causal conv1d (+ SiLU) on the HIP kernels: the operator the reference takes from the
separate causal_conv1d package (`causal_conv1d_fn`; call sites
mamba_ssm/ops/selective_scan_interface.py:224, mamba_ssm/ops/triton/ssd_combined.py:845,
mamba_ssm/modules/mamba2.py:236) and otherwise spells as
nn.Conv1d(groups=channels, padding=width - 1)[..., :L] (mamba_ssm/modules/mamba_simple.py:168-169).

There is no CPU or PyTorch fallback: CPU tensors raise.
"""
import torch

from mamba_amd import _lib


def _strides_bcl(t):
    return t.stride(0), t.stride(1), t.stride(2)


def _usable(t):
    """(batch, channels, positions) view whose position stride or channel stride is 1."""
    return t.stride(2) == 1 or t.stride(1) == 1


def _like_layout(x):
    """A fresh (batch, dim, seqlen) tensor that is dense in x's layout: positions or channels contiguous."""
    b, d, L = x.shape
    if x.stride(2) == 1:
        return torch.empty(b, d, L, dtype=x.dtype, device=x.device)
    return torch.empty(b, L, d, dtype=x.dtype, device=x.device).transpose(1, 2)


def _fill(p, x, weight32, bias32, seq_idx, activation):
    batch, dim, seqlen = x.shape
    p.batch, p.dim, p.seqlen, p.width = batch, dim, seqlen, weight32.shape[1]
    p.dtype = _lib.DTYPE_CODE[x.dtype]
    p.silu = int(activation in ("silu", "swish"))
    p.x, p.weight, p.bias, p.seq_idx = x.data_ptr(), weight32.data_ptr(), _lib.ptr(bias32), _lib.ptr(seq_idx)
    p.x_bs, p.x_cs, p.x_ls = _strides_bcl(x)


def _check(x, weight, bias, seq_idx, activation):
    _lib.require_gpu(x, weight, bias, seq_idx)
    if activation not in (None, "silu", "swish"):
        raise NotImplementedError("activation must be None, silu, or swish")
    if x.dim() != 3 or x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError("causal_conv1d: x must be (batch, dim, seqlen) in fp32, fp16 or bf16")
    dim = x.shape[1]
    if weight.dim() != 2 or weight.shape[0] != dim or not 2 <= weight.shape[1] <= 4:
        raise RuntimeError("causal_conv1d: weight must be (dim, width) with width between 2 and 4")
    if bias is not None and tuple(bias.shape) != (dim,):
        raise RuntimeError("causal_conv1d: bias must be (dim,)")
    if seq_idx is not None and (tuple(seq_idx.shape) != (x.shape[0], x.shape[2]) or seq_idx.dtype != torch.int32):
        raise RuntimeError("causal_conv1d: seq_idx must be (batch, seqlen) int32")


def causal_conv1d_fwd(x, weight, bias=None, seq_idx=None, activation=None):
    """One call of the C ABI's causal_conv1d_fwd; out is dense in x's layout."""
    _check(x, weight, bias, seq_idx, activation)
    if not _usable(x):
        x = x.contiguous()
    seq_idx = seq_idx.contiguous() if seq_idx is not None else None
    w32 = weight.detach().float().contiguous()
    b32 = bias.detach().float().contiguous() if bias is not None else None
    out = _like_layout(x)
    p = _lib.CausalConvParams()
    _fill(p, x, w32, b32, seq_idx, activation)
    p.out = out.data_ptr()
    p.out_bs, p.out_cs, p.out_ls = _strides_bcl(out)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().causal_conv1d_fwd(p, _lib.current_stream(x.device)), "causal_conv1d_fwd")
    return out


def causal_conv1d_bwd(x, weight, bias, dout, seq_idx=None, activation=None, dx=None):
    """One call of the C ABI's causal_conv1d_bwd.  `dx` may be a caller-owned view in x's layout
    (unit stride on the same axis).  Returns (dx, dweight, dbias) in the dtypes of x, weight, bias."""
    _check(x, weight, bias, seq_idx, activation)
    _lib.require_gpu(dout, dx)
    if not _usable(x):
        x = x.contiguous()
    rows = x.stride(2) == 1
    if dout.shape != x.shape or dout.dtype != x.dtype:
        raise RuntimeError("causal_conv1d: dout must match x in shape and dtype")
    if rows:
        dout = dout if dout.stride(2) == 1 else dout.contiguous()
    else:
        dout = dout if dout.stride(1) == 1 else dout.transpose(1, 2).contiguous().transpose(1, 2)
    if dx is None:
        dx = _like_layout(x)
    elif dx.shape != x.shape or dx.dtype != x.dtype or dx.stride(2 if rows else 1) != 1:
        raise RuntimeError("causal_conv1d: dx must match x in shape, dtype and layout")
    seq_idx = seq_idx.contiguous() if seq_idx is not None else None
    w32 = weight.detach().float().contiguous()
    b32 = bias.detach().float().contiguous() if bias is not None else None
    dw32 = torch.zeros_like(w32)
    db32 = torch.zeros_like(b32) if b32 is not None else None
    p = _lib.CausalConvParams()
    _fill(p, x, w32, b32, seq_idx, activation)
    p.dout, p.dx, p.dweight, p.dbias = dout.data_ptr(), dx.data_ptr(), dw32.data_ptr(), _lib.ptr(db32)
    p.dout_bs, p.dout_cs, p.dout_ls = _strides_bcl(dout)
    p.dx_bs, p.dx_cs, p.dx_ls = _strides_bcl(dx)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().causal_conv1d_bwd(p, _lib.current_stream(x.device)), "causal_conv1d_bwd")
    return dx, dw32.to(weight.dtype), (db32.to(bias.dtype) if bias is not None else None)


class CausalConv1dFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias=None, seq_idx=None, activation=None):
        out = causal_conv1d_fwd(x, weight, bias, seq_idx, activation)
        ctx.save_for_backward(x, weight, bias, seq_idx)
        ctx.activation = activation
        return out

    @staticmethod
    def backward(ctx, dout):
        x, weight, bias, seq_idx = ctx.saved_tensors
        dx, dweight, dbias = causal_conv1d_bwd(x, weight, bias, dout, seq_idx, ctx.activation)
        return dx, dweight, dbias, None, None


def causal_conv1d_fn(x, weight, bias=None, seq_idx=None, initial_states=None, return_final_states=False,
                     final_states_out=None, activation=None):
    """x: (batch, dim, seqlen), position- or channel-contiguous; weight: (dim, width); bias: (dim,);
    seq_idx: (batch, seqlen) int32; activation: None, "silu" or "swish".  out: (batch, dim, seqlen) in
    x's layout.  Streaming states (initial_states / return_final_states) belong to the decode path of
    the separate package and are not served here."""
    if initial_states is not None or return_final_states or final_states_out is not None:
        raise NotImplementedError("causal_conv1d_fn: streaming conv states are not supported")
    return CausalConv1dFn.apply(x, weight, bias, seq_idx, activation)
