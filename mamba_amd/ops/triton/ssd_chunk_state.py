"""Stage-level drop-in for mamba_ssm.ops.triton.ssd_chunk_state: the dt pipeline + per-chunk cumulative
sums, the chunk-local states and the per-sequence states of a packed batch, each one launch of the HIP
library (reference: ssd_chunk_state.py:718 _chunk_cumsum_fwd, :812 _chunk_state_fwd, :1018
chunk_state_varlen, :1081 chunk_state, :1094 chunk_state_ref)."""
import math

import torch
import torch.nn.functional as F

from mamba_amd import _lib
from mamba_amd.ops.triton import _ssd_stage as st


def _chunk_cumsum_fwd(dt, A, chunk_size, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """dt (batch, seqlen, nheads), A (nheads,) -> (dA_cumsum, dt_out), both (batch, nheads, nchunks, chunk_size)
    fp32; positions past seqlen hold dt = 0 (ssd_chunk_state.py:718-741)."""
    batch, seqlen, nheads = dt.shape
    assert A.shape == (nheads,)
    if dt_bias is not None:
        assert dt_bias.shape == (nheads,)
    _lib.require_gpu(dt, A, dt_bias)
    if dt.dtype not in _lib.DTYPE_CODE:
        dt = dt.float()
    A = st.f32c(A)
    dt_bias = st.f32c(dt_bias) if dt_bias is not None else None
    nchunks = math.ceil(seqlen / chunk_size)
    dt_out = torch.empty(batch, nheads, nchunks, chunk_size, device=dt.device, dtype=torch.float32)
    dA_cumsum = torch.empty_like(dt_out)
    p, _keep = st.stage_params(dt.device, batch=batch, seqlen=seqlen, nheads=nheads, headdim=1, dstate=1, ngroups=1,
                               chunk_size=chunk_size, dt_dtype=dt.dtype)
    p.dt, p.A, p.dt_bias = dt.data_ptr(), A.data_ptr(), _lib.ptr(dt_bias)
    p.dt_bs, p.dt_ls, p.dt_hs = dt.stride()
    p.dt_softplus = int(bool(dt_softplus))
    p.dt_min, p.dt_max = float(dt_limit[0]), float(min(dt_limit[1], 3.0e38))
    p.dt_out, p.dA_cumsum = dt_out.data_ptr(), dA_cumsum.data_ptr()
    st.run("ssd_chunk_cumsum_fwd", p, dt.device)
    return dA_cumsum, dt_out


def _chunk_cumsum_bwd(ddA, ddt_out, dt, A, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf")), ddt=None):
    """Backward of _chunk_cumsum_fwd (ssd_chunk_state.py:744): ddA, ddt_out (batch, nheads, nchunks, chunk_size) are the
    gradients with respect to dA_cumsum and the processed dt; dt (batch, seqlen, nheads) and A, dt_bias (nheads,) the
    forward inputs.  Returns (ddt like dt, dA (nheads,) fp32, ddt_bias (nheads,) fp32 or None)."""
    batch, seqlen, nheads = dt.shape
    _, _, nchunks, chunk_size = ddA.shape
    assert ddA.shape == (batch, nheads, nchunks, chunk_size) and ddt_out.shape == ddA.shape
    assert A.shape == (nheads,)
    _lib.require_gpu(ddA, ddt_out, dt, A, dt_bias, ddt)
    if dt.dtype not in _lib.DTYPE_CODE:
        dt = dt.float()
    A32 = st.f32c(A)
    bias32 = st.f32c(dt_bias) if dt_bias is not None else None
    _, dt_proc = _chunk_cumsum_fwd(dt, A32, chunk_size, dt_bias=bias32, dt_softplus=dt_softplus, dt_limit=dt_limit)
    ddA, ddt_out = st.f32c(ddA), st.f32c(ddt_out)
    out = torch.empty(batch, seqlen, nheads, device=dt.device, dtype=dt.dtype)
    sums = torch.zeros(2, nheads, device=dt.device, dtype=torch.float32)
    p, _keep = st.stage_params(dt.device, batch=batch, seqlen=seqlen, nheads=nheads, headdim=1, dstate=1, ngroups=1,
                               chunk_size=chunk_size, dt_dtype=dt.dtype, backward=True)
    p.dt, p.A, p.dt_bias = dt.data_ptr(), A32.data_ptr(), _lib.ptr(bias32)
    p.dt_bs, p.dt_ls, p.dt_hs = dt.stride()
    p.dt_softplus = int(bool(dt_softplus))
    p.dt_min, p.dt_max = float(dt_limit[0]), float(min(dt_limit[1], 3.0e38))
    p.dt_out, p.ddA_cumsum, p.ddt_out = dt_proc.data_ptr(), ddA.data_ptr(), ddt_out.data_ptr()
    p.ddt, p.dA = out.data_ptr(), sums[0].data_ptr()
    p.ddt_bias = sums[1].data_ptr() if dt_bias is not None else None
    st.run("ssd_chunk_cumsum_bwd", p, dt.device)
    if ddt is not None:
        ddt.copy_(out)
        out = ddt
    return out, sums[0], (sums[1] if dt_bias is not None else None)


def _chunk_state_fwd(B, x, dt, dA_cumsum, seq_idx=None, states=None, states_in_fp32=True):
    """Chunk-local states sum_l B[l] x[l] dt[l] exp(a_end - a_l): (batch, nchunks, nheads, headdim, dstate)
    (ssd_chunk_state.py:812-842).  The kernel writes fp32; another `states` dtype is a cast of that."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == dt.shape
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
    if states is not None:
        assert states.shape == (batch, nchunks, nheads, headdim, dstate)
    _lib.require_gpu(B, x, dt, dA_cumsum, seq_idx, states)
    if x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"_chunk_state_fwd: unsupported dtype {x.dtype}")
    assert nchunks == math.ceil(seqlen / chunk_size)
    x = x if x.stride(-1) == 1 else x.contiguous()
    B = B.to(x.dtype)
    B = B if B.stride(-1) == 1 else B.contiguous()
    dt, dA_cumsum, seq_idx = st.f32c(dt), st.f32c(dA_cumsum), st.seq_idx_i32(seq_idx)
    direct = states is not None and states.dtype == torch.float32 and states.is_contiguous()
    buf = states if direct else torch.empty(batch, nchunks, nheads, headdim, dstate, device=x.device,
                                             dtype=torch.float32)
    p, _keep = st.stage_params(x.device, batch=batch, seqlen=seqlen, nheads=nheads, headdim=headdim, dstate=dstate,
                               ngroups=ngroups, chunk_size=chunk_size, dtype=x.dtype)
    p.x, p.B, p.seq_idx = x.data_ptr(), B.data_ptr(), _lib.ptr(seq_idx)
    p.x_bs, p.x_ls, p.x_hs = x.stride(0), x.stride(1), x.stride(2)
    p.B_bs, p.B_ls, p.B_gs = B.stride(0), B.stride(1), B.stride(2)
    p.dt_out, p.dA_cumsum, p.states = dt.data_ptr(), dA_cumsum.data_ptr(), buf.data_ptr()
    st.run("ssd_chunk_state_fwd", p, x.device)
    if direct:
        return states
    if states is not None:
        states.copy_(buf)
        return states
    return buf if states_in_fp32 else buf.to(B.dtype)


def chunk_state_varlen(B, x, dt, dA_cumsum, cu_seqlens, chunk_states):
    """State at the end of every sequence of one packed row: B (L, ngroups, dstate), x (L, nheads, headdim),
    dt / dA_cumsum (nheads, nchunks, chunk_size), chunk_states (nchunks, nheads, headdim, dstate) = the state
    entering each chunk -> (nseq, nheads, headdim, dstate) in chunk_states' dtype (ssd_chunk_state.py:1018)."""
    total_seqlen, nheads, headdim = x.shape
    _, nchunks, chunk_size = dt.shape
    _, ngroups, dstate = B.shape
    nseq = cu_seqlens.shape[0] - 1
    assert nheads % ngroups == 0
    assert B.shape == (total_seqlen, ngroups, dstate)
    assert dt.shape == (nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == dt.shape
    assert chunk_states.shape == (nchunks, nheads, headdim, dstate)
    _lib.require_gpu(B, x, dt, dA_cumsum, cu_seqlens, chunk_states)
    if x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"chunk_state_varlen: unsupported dtype {x.dtype}")
    x = x if x.stride(-1) == 1 else x.contiguous()
    B = B.to(x.dtype)
    B = B if B.stride(-1) == 1 else B.contiguous()
    dt, dA_cumsum = st.f32c(dt), st.f32c(dA_cumsum)
    cu = cu_seqlens.to(torch.int32).contiguous()
    out = torch.empty(nseq, nheads, headdim, dstate, device=x.device, dtype=torch.float32)
    p, _keep = st.stage_params(x.device, batch=1, seqlen=total_seqlen, nheads=nheads, headdim=headdim, dstate=dstate,
                               ngroups=ngroups, chunk_size=chunk_size, dtype=x.dtype)
    p.x, p.B = x.data_ptr(), B.data_ptr()
    p.x_ls, p.x_hs = x.stride(0), x.stride(1)
    p.B_ls, p.B_gs = B.stride(0), B.stride(1)
    p.dt_out, p.dA_cumsum = dt.data_ptr(), dA_cumsum.data_ptr()
    _entering = st.set_carried(p, "states", chunk_states.unsqueeze(0), x.dtype)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().ssd_chunk_state_varlen(p, cu.data_ptr(), nseq, out.data_ptr(),
                                                      _lib.current_stream(x.device)), "ssd_chunk_state_varlen")
    return out.to(chunk_states.dtype)


class ChunkStateFn(torch.autograd.Function):
    """ssd_chunk_state.py:1047 ChunkStateFn."""

    @staticmethod
    def forward(ctx, B, x, dt, dA_cumsum, states_in_fp32=True):
        ctx.save_for_backward(B, x, dt, dA_cumsum)
        return _chunk_state_fwd(B, x, dt, dA_cumsum, states_in_fp32=states_in_fp32)

    @staticmethod
    def backward(ctx, dstates):
        from mamba_amd.ops.triton._ssd_stage_bwd import chunk_state_bwd
        B, x, dt, dA_cumsum = ctx.saved_tensors
        dB, dx, ddt, ddA_cumsum = chunk_state_bwd(B, x, dt, dA_cumsum, dstates)
        return dB, dx, ddt, ddA_cumsum, None


def chunk_state(B, x, dt, dA_cumsum, states_in_fp32=True):
    """B (batch, seqlen, ngroups, dstate), x (batch, seqlen, nheads, headdim), dt / dA_cumsum
    (batch, nheads, nchunks, chunk_size) -> states (batch, nchunks, nheads, headdim, dstate)."""
    return ChunkStateFn.apply(B, x, dt, dA_cumsum, states_in_fp32)


def chunk_state_ref(B, x, dt, dA_cumsum):
    """The same sum in plain torch (ssd_chunk_state.py:1094); seqlen is padded up to whole chunks."""
    batch, seqlen, nheads, headdim = x.shape
    ngroups, dstate = B.shape[2], B.shape[3]
    _, _, nchunks, chunk_size = dt.shape
    assert seqlen <= nchunks * chunk_size
    assert B.shape == (batch, seqlen, ngroups, dstate) and x.shape == (batch, seqlen, nheads, headdim)
    assert dA_cumsum.shape == dt.shape == (batch, nheads, nchunks, chunk_size)
    pad = nchunks * chunk_size - seqlen
    if pad:
        x, B = F.pad(x, (0, 0, 0, 0, 0, pad)), F.pad(B, (0, 0, 0, 0, 0, pad))
    Bh = B.repeat_interleave(nheads // ngroups, dim=2).reshape(batch, nchunks, chunk_size, nheads, dstate)
    xc = x.reshape(batch, nchunks, chunk_size, nheads, headdim)
    w = (torch.exp(dA_cumsum[..., -1:] - dA_cumsum) * dt).to(x.dtype)  # (b, h, c, l)
    return torch.einsum("bclhn,bhcl,bclhp->bchpn", Bh.to(x.dtype), w, xc)
