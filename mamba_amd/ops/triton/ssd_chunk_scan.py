"""Stage-level drop-in for mamba_ssm.ops.triton.ssd_chunk_scan: the output of every chunk from the
in-chunk C B^T products and the state entering the chunk (reference: ssd_chunk_scan.py:1259
_chunk_scan_fwd, :1828 chunk_scan, :1846 chunk_scan_ref)."""
import math

import torch
import torch.nn.functional as F

from mamba_amd import _lib
from mamba_amd.ops.triton import _ssd_stage as st
from mamba_amd.ops.triton.ssd_bmm import _bmm_chunk_fwd


def _chunk_scan_fwd(cb, x, dt, dA_cumsum, C, states, D=None, z=None, seq_idx=None):
    """cb (batch, nchunks, ngroups, chunk_size, chunk_size) = C B^T (triangle i >= j read), x
    (batch, seqlen, nheads, headdim), dt / dA_cumsum (batch, nheads, nchunks, chunk_size), C
    (batch, seqlen, ngroups, dstate), states (batch, nchunks, nheads, headdim, dstate) entering each chunk ->
    (out, out_x): out gated by silu(z) when z is given, out_x then the output before the gate, else None."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = C.shape
    assert nheads % ngroups == 0
    assert C.shape == (batch, seqlen, ngroups, dstate)
    assert cb.shape == (batch, nchunks, ngroups, chunk_size, chunk_size)
    if z is not None:
        assert z.shape == x.shape
    if D is not None:
        assert D.shape == (nheads, headdim) or D.shape == (nheads,)
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == (batch, nheads, nchunks, chunk_size)
    assert states.shape == (batch, nchunks, nheads, headdim, dstate)
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
    _lib.require_gpu(cb, x, dt, dA_cumsum, C, states, D, z, seq_idx)
    if x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"_chunk_scan_fwd: unsupported dtype {x.dtype}")
    assert nchunks == math.ceil(seqlen / chunk_size)
    x = x if x.stride(-1) == 1 else x.contiguous()
    C = C.to(x.dtype)
    C = C if C.stride(-1) == 1 else C.contiguous()
    if z is not None:
        z = z.to(x.dtype)
        z = z if z.stride(-1) == 1 else z.contiguous()
    cb, dt, dA_cumsum = st.f32c(cb), st.f32c(dt), st.f32c(dA_cumsum)
    D = st.f32c(D) if D is not None else None
    seq_idx = st.seq_idx_i32(seq_idx)
    out = torch.empty(batch, seqlen, nheads, headdim, device=x.device, dtype=x.dtype)
    out_x = torch.empty_like(out) if z is not None else None
    p, _keep = st.stage_params(x.device, batch=batch, seqlen=seqlen, nheads=nheads, headdim=headdim, dstate=dstate,
                               ngroups=ngroups, chunk_size=chunk_size, dtype=x.dtype)
    p.x, p.C, p.z, p.D, p.seq_idx = x.data_ptr(), C.data_ptr(), _lib.ptr(z), _lib.ptr(D), _lib.ptr(seq_idx)
    p.D_has_hdim = int(D is not None and D.dim() == 2)
    p.x_bs, p.x_ls, p.x_hs = x.stride(0), x.stride(1), x.stride(2)
    p.C_bs, p.C_ls, p.C_gs = C.stride(0), C.stride(1), C.stride(2)
    if z is not None:
        p.z_bs, p.z_ls, p.z_hs = z.stride(0), z.stride(1), z.stride(2)
    p.CB, p.dt_out, p.dA_cumsum = cb.data_ptr(), dt.data_ptr(), dA_cumsum.data_ptr()
    _states = st.set_carried(p, "states", states, x.dtype)
    p.out, p.out_x = out.data_ptr(), _lib.ptr(out_x)
    p.out_bs, p.out_ls, p.out_hs = out.stride(0), out.stride(1), out.stride(2)
    st.run("ssd_chunk_scan_fwd", p, x.device)
    return out, out_x


class ChunkScanFn(torch.autograd.Function):
    """ssd_chunk_scan.py:1764 ChunkScanFn."""

    @staticmethod
    def forward(ctx, B, C, x, dt, dA_cumsum, prev_states, D=None, z=None):
        batch, seqlen, nheads, headdim = x.shape
        _, _, nchunks, chunk_size = dt.shape
        assert B.shape == C.shape and B.shape[:2] == (batch, seqlen)
        assert seqlen == nchunks * chunk_size
        CB = _bmm_chunk_fwd(C, B, chunk_size, causal=True, output_dtype=torch.float32)
        out, out_x = _chunk_scan_fwd(CB, x, dt, dA_cumsum, C, prev_states, D=D, z=z)
        ctx.save_for_backward(out if z is None else out_x, B, C, x, dt, dA_cumsum, prev_states, D, z)
        return out

    @staticmethod
    def backward(ctx, dout):
        from mamba_amd.ops.triton._ssd_stage_bwd import chunk_scan_bwd
        y, B, C, x, dt, dA_cumsum, prev_states, D, z = ctx.saved_tensors
        return chunk_scan_bwd(B, C, x, dt, dA_cumsum, prev_states, D, z, y, dout)


def chunk_scan(B, C, x, dt, dA_cumsum, prev_states, D=None, z=None):
    """prev_states[:, c] is the state entering chunk c (index 0 = the initial states).  B, C
    (batch, seqlen, ngroups, dstate), x (batch, seqlen, nheads, headdim), dt / dA_cumsum
    (batch, nheads, nchunks, chunk_size), prev_states (batch, nchunks, nheads, headdim, dstate), D (nheads,) or
    (nheads, headdim), z like x -> out (batch, seqlen, nheads, headdim)."""
    return ChunkScanFn.apply(B, C, x, dt, dA_cumsum, prev_states, D, z)


def chunk_scan_ref(B, C, x, dt, dA_cumsum, prev_states, D=None, z=None):
    """The same output in plain torch (ssd_chunk_scan.py:1846), fp32 arithmetic."""
    batch, seqlen, nheads, headdim = x.shape
    ngroups, dstate = B.shape[2], B.shape[3]
    _, _, nchunks, Q = dt.shape
    assert seqlen == nchunks * Q
    rep = nheads // ngroups
    Bc = B.float().repeat_interleave(rep, dim=2).reshape(batch, nchunks, Q, nheads, dstate)
    Cc = C.float().repeat_interleave(rep, dim=2).reshape(batch, nchunks, Q, nheads, dstate)
    xc = x.float().reshape(batch, nchunks, Q, nheads, headdim)
    a = dA_cumsum.float()
    cb = torch.einsum("bclhn,bcshn->bhcls", Cc, Bc)
    mask = torch.tril(torch.ones(Q, Q, device=x.device, dtype=torch.bool))
    decay = torch.exp((a[..., :, None] - a[..., None, :]).masked_fill(~mask, float("-inf")))
    scores = cb * decay * dt.float()[..., None, :]
    out = torch.einsum("bhcls,bcshp->bclhp", scores, xc)
    out = out + torch.einsum("bclhn,bchpn->bclhp", Cc, prev_states.float()) * torch.exp(a).permute(0, 2, 3, 1)[..., None]
    out = out.reshape(batch, seqlen, nheads, headdim)
    if D is not None:
        Dv = D.float() if D.dim() == 2 else D.float()[:, None]
        out = out + x.float() * Dv
    if z is not None:
        out = out * F.silu(z.float())
    return out.to(x.dtype)
