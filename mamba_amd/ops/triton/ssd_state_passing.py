"""Stage-level drop-in for mamba_ssm.ops.triton.ssd_state_passing: the recurrence over chunks that turns
chunk-local states into the state entering each chunk, and its adjoint (reference:
ssd_state_passing.py:196 _state_passing_fwd, :227 _state_passing_bwd, :314 state_passing, :327
state_passing_ref)."""
import torch

from mamba_amd import _lib
from mamba_amd.ops.triton import _ssd_stage as st


def _split_dim(dim):
    """dim = headdim * dstate with both factors within the library's limit of 256."""
    for d in range(min(dim, 256), 0, -1):
        if dim % d == 0 and dim // d <= 256:
            return dim // d, d
    raise RuntimeError(f"state_passing: dim {dim} has no factorisation into two factors <= 256")


def _per_chunk(dA_chunk_cumsum, seq_idx, chunk_size, nchunks):
    """The library's kernels read the decay at the last position of a chunk and compare the sequence index
    at the ends of neighbouring chunks: with one position per chunk both are the per-chunk arrays themselves."""
    dA = st.f32c(dA_chunk_cumsum)  # (batch, nheads, nchunks) = (batch, nheads, nchunks, 1)
    seq = None
    if seq_idx is not None:
        assert chunk_size is not None
        seqlen = seq_idx.shape[-1]
        ends = (torch.arange(1, nchunks + 1, device=seq_idx.device) * chunk_size).clamp(max=seqlen) - 1
        seq = seq_idx[:, ends].to(torch.int32).contiguous()
    return dA, seq


def _state_passing_fwd(states, dA_chunk_cumsum, initial_states=None, seq_idx=None, chunk_size=None, out_dtype=None):
    """states (batch, nchunks, nheads, dim) chunk-local, dA_chunk_cumsum (batch, nheads, nchunks) ->
    out[:, c] = state entering chunk c (out[:, 0] = initial_states or 0), final_states (batch, nheads, dim) fp32."""
    batch, nchunks, nheads, dim = states.shape
    assert dA_chunk_cumsum.shape == (batch, nheads, nchunks)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, dim)
    if seq_idx is not None:
        assert chunk_size is not None
        assert seq_idx.shape == (batch, seq_idx.shape[-1])
    _lib.require_gpu(states, dA_chunk_cumsum, initial_states, seq_idx)
    out_dtype = states.dtype if out_dtype is None else out_dtype
    dA, seq = _per_chunk(dA_chunk_cumsum, seq_idx, chunk_size, nchunks)
    work = states.float().contiguous()
    if work.data_ptr() == states.data_ptr():
        work = work.clone()  # the kernel works in place
    init = st.f32c(initial_states) if initial_states is not None else None
    final = torch.empty(batch, nheads, dim, device=states.device, dtype=torch.float32)
    hd, ds = _split_dim(dim)
    p, _keep = st.stage_params(states.device, batch=batch, seqlen=nchunks, nheads=nheads, headdim=hd, dstate=ds,
                               ngroups=1, chunk_size=1)
    p.states, p.final_states, p.dA_cumsum = work.data_ptr(), final.data_ptr(), dA.data_ptr()
    p.initial_states, p.seq_idx = _lib.ptr(init), _lib.ptr(seq)
    st.run("ssd_state_passing_fwd", p, states.device)
    return work.to(out_dtype), final


def _state_passing_bwd(states, dA_chunk_cumsum, dout, dfinal_states=None, seq_idx=None, has_initial_states=None,
                       dstates_dtype=None, states_dtype=None, chunk_size=None):
    """states = the forward pass's `out` (index 0 holds the initial states).  Returns (dstates,
    ddA_chunk_cumsum, dinitstates), plus states cast to states_dtype when that is asked for
    (ssd_state_passing.py:227-283)."""
    batch, nchunks, nheads, dim = states.shape
    assert dA_chunk_cumsum.shape == (batch, nheads, nchunks)
    assert dout.shape == (batch, nchunks, nheads, dim)
    if dfinal_states is not None:
        assert dfinal_states.shape == (batch, nheads, dim)
    _lib.require_gpu(states, dA_chunk_cumsum, dout, dfinal_states, seq_idx)
    dA, seq = _per_chunk(dA_chunk_cumsum, seq_idx, chunk_size, nchunks)
    entering = st.f32c(states)
    g = dout.float().contiguous()
    if g.data_ptr() == dout.data_ptr():
        g = g.clone()  # in: gradient of the state entering each chunk; out: gradient of the chunk-local states
    dfinal = st.f32c(dfinal_states) if dfinal_states is not None else None
    ddA = torch.zeros(batch, nheads, nchunks, device=states.device, dtype=torch.float32)
    dinit = torch.empty(batch, nheads, dim, device=states.device, dtype=torch.float32) if has_initial_states else None
    hd, ds = _split_dim(dim)
    p, _keep = st.stage_params(states.device, batch=batch, seqlen=nchunks, nheads=nheads, headdim=hd, dstate=ds,
                               ngroups=1, chunk_size=1, backward=True)
    p.states, p.dstates, p.dA_cumsum, p.ddA_cumsum = entering.data_ptr(), g.data_ptr(), dA.data_ptr(), ddA.data_ptr()
    p.dfinal_states, p.dinitial_states, p.seq_idx = _lib.ptr(dfinal), _lib.ptr(dinit), _lib.ptr(seq)
    st.run("ssd_state_passing_bwd", p, states.device)
    dstates = g.to(dstates_dtype if dstates_dtype is not None else dout.dtype)
    if dinit is not None:
        dinit = dinit.to(dstates.dtype)
    if states_dtype is not None and states_dtype != states.dtype:
        return dstates, ddA, dinit, states.to(states_dtype)
    return dstates, ddA, dinit


class StatePassingFn(torch.autograd.Function):
    """ssd_state_passing.py:286."""

    @staticmethod
    def forward(ctx, states, dA_chunk_cumsum, initial_states=None):
        out, final_states = _state_passing_fwd(states, dA_chunk_cumsum, initial_states)
        ctx.save_for_backward(out, dA_chunk_cumsum)
        ctx.has_initial_states = initial_states is not None
        return out, final_states

    @staticmethod
    def backward(ctx, dout, dfinal_states):
        out, dA_chunk_cumsum = ctx.saved_tensors
        dstates, ddA, dinit = _state_passing_bwd(out, dA_chunk_cumsum, dout, dfinal_states=dfinal_states,
                                                 has_initial_states=ctx.has_initial_states)
        return dstates, ddA.to(dA_chunk_cumsum.dtype), dinit


def state_passing(states, dA_chunk_cumsum, initial_states=None):
    """states (batch, nchunks, nheads, dim), dA_chunk_cumsum (batch, nheads, nchunks), initial_states
    (batch, nheads, dim) -> out (batch, nchunks, nheads, dim), final_states (batch, nheads, dim)."""
    return StatePassingFn.apply(states, dA_chunk_cumsum, initial_states)


def state_passing_ref(states, dA_chunk_cumsum, initial_states=None):
    """The recurrence step by step in plain torch (the reference, ssd_state_passing.py:327, writes it as one
    masked matrix product; the values are the same)."""
    batch, nchunks, nheads, dim = states.shape
    s = torch.zeros(batch, nheads, dim, device=states.device, dtype=states.dtype) if initial_states is None \
        else initial_states.to(states.dtype)
    out = []
    for c in range(nchunks):
        out.append(s)
        s = torch.exp(dA_chunk_cumsum[:, :, c]).to(states.dtype)[..., None] * s + states[:, c]
    return torch.stack(out, dim=1), s
