"""Depthwise causal conv1d (+ SiLU) on the HIP kernels: the operator the reference takes from the
separate causal_conv1d package (`causal_conv1d_fn`; call sites
mamba_ssm/ops/selective_scan_interface.py:224, mamba_ssm/ops/triton/ssd_combined.py:845,
mamba_ssm/modules/mamba2.py:236) and otherwise spells as
nn.Conv1d(groups=channels, padding=width - 1)[..., :L] (mamba_ssm/modules/mamba_simple.py:168-169).

There is no CPU or PyTorch fallback: CPU tensors raise.
"""
import torch

from mamba_amd import _lib
from mamba_amd.utils.determinism import fixed_point_scale, use_deterministic_mode


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


def causal_conv1d_fwd(x, weight, bias=None, seq_idx=None, activation=None, out=None):
    """One call of the C ABI's causal_conv1d_fwd; out is dense in x's layout unless the caller brings
    one (same shape and dtype, unit stride on the axis where x has it)."""
    _check(x, weight, bias, seq_idx, activation)
    if not _usable(x):
        x = x.contiguous()
    seq_idx = seq_idx.contiguous() if seq_idx is not None else None
    w32 = weight.detach().float().contiguous()
    b32 = bias.detach().float().contiguous() if bias is not None else None
    if out is None:
        out = _like_layout(x)
    elif out.shape != x.shape or out.dtype != x.dtype or out.stride(2 if x.stride(2) == 1 else 1) != 1:
        raise RuntimeError("causal_conv1d: out must match x in shape, dtype and layout")
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
    det = use_deterministic_mode()
    if det:
        # integer shadows of the two shared sums and the call's fixed-point scale (mamba_amd/utils/determinism.py)
        sw = torch.zeros(w32.numel(), dtype=torch.int64, device=x.device)
        sb = torch.zeros(b32.numel(), dtype=torch.int64, device=x.device) if b32 is not None else None
        scale = fixed_point_scale(dout)
        p.det_scale, p.det_dweight, p.det_dbias = scale.data_ptr(), sw.data_ptr(), _lib.ptr(sb)
    with torch.cuda.device(x.device):
        lib, stream = _lib.load(), _lib.current_stream(x.device)
        _lib.check(lib.causal_conv1d_bwd(p, stream), "causal_conv1d_bwd")
        if det:
            _lib.check(lib.ssd_det_convert(sw.data_ptr(), dw32.data_ptr(), sw.numel(), scale.data_ptr(), stream), "ssd_det_convert")
            if sb is not None:
                _lib.check(lib.ssd_det_convert(sb.data_ptr(), db32.data_ptr(), sb.numel(), scale.data_ptr(), stream),
                           "ssd_det_convert")
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
    x's layout.
    Streaming (the causal_conv1d package's arguments of the same names):
        initial_states: (batch, dim, width - 1), the positions in front of x; the output is that of the
            convolution over [initial_states, x], cut to x's positions; with seq_idx they belong to the row's
            first sequence
        return_final_states: also return (batch, dim, width - 1), the last width - 1 positions of
            [initial_states, x] (zero-filled on the left when there are fewer); no gradient flows through them
        final_states_out: a tensor to receive them
    The streaming form runs the same kernel over the joined row (one extra copy of x)."""
    if initial_states is None and not return_final_states and final_states_out is None:
        return CausalConv1dFn.apply(x, weight, bias, seq_idx, activation)
    width = weight.shape[1]
    batch, dim, seqlen = x.shape
    joined = x
    if initial_states is not None:
        if tuple(initial_states.shape) != (batch, dim, width - 1):
            raise RuntimeError("causal_conv1d_fn: initial_states must be (batch, dim, width - 1)")
        _lib.require_gpu(x, initial_states)
        if x.stride(1) == 1 and x.stride(2) != 1:   # keep a channel-contiguous row channel-contiguous
            joined = torch.cat([initial_states.to(x.dtype).transpose(1, 2), x.transpose(1, 2)], dim=1).transpose(1, 2)
        else:
            joined = torch.cat([initial_states.to(x.dtype), x], dim=2)
        joined_idx = None
        if seq_idx is not None:
            # the carried positions continue the row's first sequence (a prefill cut into pieces hands them on):
            # they take that sequence's id, so its first positions see them and no other sequence does
            joined_idx = torch.cat([seq_idx[:, :1].expand(batch, width - 1), seq_idx], dim=1).to(torch.int32).contiguous()
        out = CausalConv1dFn.apply(joined, weight, bias, joined_idx, activation)[:, :, width - 1:]
    else:
        out = CausalConv1dFn.apply(x, weight, bias, seq_idx, activation)
    if not return_final_states and final_states_out is None:
        return out
    with torch.no_grad():
        tail = joined[:, :, max(joined.shape[2] - (width - 1), 0):]
        if tail.shape[2] < width - 1:
            tail = torch.nn.functional.pad(tail, (width - 1 - tail.shape[2], 0))
        if final_states_out is not None:
            final_states_out.copy_(tail)
            final = final_states_out
        else:
            final = tail.clone()
    return out, final


def causal_conv1d_update(x, conv_state, weight, bias=None, activation=None, cache_seqlens=None,
                         conv_state_indices=None):
    """Decode step (the package's causal_conv1d_update as called at mamba_ssm/modules/mamba2.py:298,
    mamba_ssm/modules/mamba_simple.py:223).
        x: (batch, dim) or (batch, dim, seqlen): the new position(s)
        conv_state: (rows, dim, state_len), state_len >= width - 1, updated in place to the last
            state_len positions of [conv_state, x]
        weight: (dim, width); bias: (dim,)
        conv_state_indices: (batch,) int32, row of conv_state per batch entry (negative: padding)
        cache_seqlens: (batch,) int32; when given, conv_state is a circular buffer: entry b has seen
            cache_seqlens[b] positions, position t lives in slot t % state_len, the new ones are written to
            their slots and nothing is shifted (the causal_conv1d package's argument of the same name)
    Returns out with x's shape and dtype."""
    if activation not in (None, "silu", "swish"):
        raise NotImplementedError("activation must be None, silu, or swish")
    ext = _lib.torch_ext()
    if ext is not None:
        # the same checks and launch in C++; None = it declined, and the code below handles the call
        out = ext.causal_conv1d_update(x, conv_state, weight.detach(), None if bias is None else bias.detach(),
                                       activation is not None, cache_seqlens, conv_state_indices)
        if out is not None:
            return out
    _lib.require_gpu(x, conv_state, weight, bias, conv_state_indices)
    squeeze = x.dim() == 2
    if squeeze:
        x = x.unsqueeze(-1)
    batch, dim, seqlen = x.shape
    width = weight.shape[1]
    if x.dtype not in _lib.DTYPE_CODE or conv_state.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError("causal_conv1d_update: x and conv_state must be fp32, fp16 or bf16")
    if weight.shape[0] != dim or not 2 <= width <= 4:
        raise RuntimeError("causal_conv1d_update: weight must be (dim, width) with width between 2 and 4")
    if conv_state.dim() != 3 or conv_state.shape[1] != dim or conv_state.shape[2] < width - 1:
        raise RuntimeError("causal_conv1d_update: conv_state must be (rows, dim, state_len >= width - 1)")
    if conv_state_indices is None:
        if conv_state.shape[0] != batch:
            raise RuntimeError("causal_conv1d_update: conv_state must have one row per batch entry")
    else:
        if tuple(conv_state_indices.shape) != (batch,) or conv_state_indices.dtype != torch.int32:
            raise RuntimeError("causal_conv1d_update: conv_state_indices must be (batch,) int32")
        conv_state_indices = conv_state_indices.contiguous()
    if cache_seqlens is not None:
        _lib.require_gpu(cache_seqlens)
        if tuple(cache_seqlens.shape) != (batch,) or cache_seqlens.dtype != torch.int32:
            raise RuntimeError("causal_conv1d_update: cache_seqlens must be (batch,) int32")
        cache_seqlens = cache_seqlens.contiguous()
    if bias is not None and tuple(bias.shape) != (dim,):
        raise RuntimeError("causal_conv1d_update: bias must be (dim,)")
    out = torch.empty_like(x)
    if batch == 0:
        return out.squeeze(-1) if squeeze else out
    # the kernel reads the filter in fp32, bf16 or fp16 as it is (weight and bias in one dtype)
    w, bv = weight.detach(), bias.detach() if bias is not None else None
    if w.dtype not in _lib.DTYPE_CODE or (bv is not None and bv.dtype != w.dtype):
        w, bv = w.float(), bv.float() if bv is not None else None
    w, bv = w.contiguous(), bv.contiguous() if bv is not None else None
    p = _lib.CausalConvUpdateParams()
    p.batch, p.dim, p.seqlen, p.width, p.state_len = batch, dim, seqlen, width, conv_state.shape[2]
    p.dtype, p.state_dtype = _lib.DTYPE_CODE[x.dtype], _lib.DTYPE_CODE[conv_state.dtype]
    p.weight_dtype = _lib.DTYPE_CODE[w.dtype]
    p.silu, p.state_rows = int(activation in ("silu", "swish")), conv_state.shape[0]
    p.x, p.conv_state, p.weight, p.bias, p.out = x.data_ptr(), conv_state.data_ptr(), w.data_ptr(), _lib.ptr(bv), out.data_ptr()
    p.conv_state_indices = _lib.ptr(conv_state_indices)
    p.cache_seqlens = _lib.ptr(cache_seqlens)
    p.x_bs, p.x_cs, p.x_ls = _strides_bcl(x)
    p.out_bs, p.out_cs, p.out_ls = _strides_bcl(out)
    p.state_bs, p.state_cs, p.state_ls = _strides_bcl(conv_state)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().causal_conv1d_update(p, _lib.current_stream(x.device)), "causal_conv1d_update")
    return out.squeeze(-1) if squeeze else out


def causal_conv1d_varlen_states(x, cu_seqlens, state_len):
    """Convolution state left by each sequence of a packed row (the package's
    causal_conv1d_varlen_states as called at mamba_ssm/modules/mamba2.py:225).
        x: (total, dim); cu_seqlens: (nseq + 1,) int32 starting at 0
    Returns (nseq, dim, state_len), channel-contiguous: the last state_len positions of each
    sequence, zero-filled on the left where the sequence is shorter."""
    _lib.require_gpu(x, cu_seqlens)
    if x.dim() != 2 or x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError("causal_conv1d_varlen_states: x must be (total, dim) in fp32, fp16 or bf16")
    if cu_seqlens.dim() != 1 or cu_seqlens.dtype != torch.int32 or cu_seqlens.numel() < 1:
        raise RuntimeError("causal_conv1d_varlen_states: cu_seqlens must be (nseq + 1,) int32")
    total, dim = x.shape
    nseq = cu_seqlens.numel() - 1
    states = torch.empty(nseq, state_len, dim, dtype=x.dtype, device=x.device).transpose(1, 2)
    if nseq == 0 or state_len == 0:
        return states
    cu_seqlens = cu_seqlens.contiguous()
    p = _lib.CausalConvVarlenParams()
    p.nseq, p.dim, p.total, p.state_len, p.dtype = nseq, dim, total, state_len, _lib.DTYPE_CODE[x.dtype]
    p.x, p.cu_seqlens, p.states = x.data_ptr(), cu_seqlens.data_ptr(), states.data_ptr()
    p.x_ls, p.x_cs = x.stride(0), x.stride(1)
    p.states_bs, p.states_cs, p.states_ls = _strides_bcl(states)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().causal_conv1d_varlen_states(p, _lib.current_stream(x.device)), "causal_conv1d_varlen_states")
    return states
