"""Stage-level drop-in for mamba_ssm.ops.triton.ssd_bmm: per-chunk products a_chunk b_chunk^T
(reference: ssd_bmm.py:165 _bmm_chunk_fwd)."""
import math

import torch

from mamba_amd import _lib
from mamba_amd.ops.triton import _ssd_stage as st


def _lower(a, b, chunk_size, seq_idx):
    """One launch: out[..., i, j] = a_i . b_j for the tiles on and below the diagonal, fp32; the other tiles
    of the buffer are not written."""
    batch, seqlen, ngroups, k = a.shape
    nchunks = math.ceil(seqlen / chunk_size)
    out = torch.empty(batch, nchunks, ngroups, chunk_size, chunk_size, device=a.device, dtype=torch.float32)
    p, _keep = st.stage_params(a.device, batch=batch, seqlen=seqlen, nheads=ngroups, headdim=1, dstate=k,
                               ngroups=ngroups, chunk_size=chunk_size, dtype=a.dtype)
    p.C, p.B, p.CB, p.seq_idx = a.data_ptr(), b.data_ptr(), out.data_ptr(), _lib.ptr(seq_idx)
    p.C_bs, p.C_ls, p.C_gs = a.stride(0), a.stride(1), a.stride(2)
    p.B_bs, p.B_ls, p.B_gs = b.stride(0), b.stride(1), b.stride(2)
    st.run("ssd_bmm_chunk_fwd", p, a.device)
    return out


def _bmm_chunk_fwd(a, b, chunk_size, seq_idx=None, causal=False, output_dtype=None):
    """a, b: (batch, seqlen, k) or (batch, seqlen, ngroups, k) -> out (batch, nchunks, [ngroups,] chunk_size,
    chunk_size) with out[i, j] = a_i . b_j inside each chunk, zero where seq_idx[i] != seq_idx[j] and for
    positions past seqlen.  The library computes the triangle i >= j, the only part the scan reads (the one the
    reference keeps with causal=True, ssd_bmm.py:59-61); with causal=False the other triangle comes from a
    second launch with the operands exchanged.  With causal=True the entries above the diagonal are zero."""
    has_groups = a.dim() == 4
    if not has_groups:
        a, b = a.unsqueeze(2), b.unsqueeze(2)
    batch, seqlen, ngroups, k = a.shape
    assert b.shape == a.shape
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
    _lib.require_gpu(a, b, seq_idx)
    if a.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"_bmm_chunk_fwd: unsupported dtype {a.dtype}")
    if k > _lib.load().mamba_hip_query(3) or chunk_size > 256:
        raise RuntimeError("_bmm_chunk_fwd: k and chunk_size are limited to 256")
    b = b.to(a.dtype)
    a = a if a.stride(-1) == 1 else a.contiguous()
    b = b if b.stride(-1) == 1 else b.contiguous()
    seq_idx = st.seq_idx_i32(seq_idx)
    out = torch.tril(_lower(a, b, chunk_size, seq_idx))
    if not causal:
        out = out + torch.tril(_lower(b, a, chunk_size, seq_idx), diagonal=-1).transpose(-1, -2)
    out = out.to(a.dtype if output_dtype is None else output_dtype)
    return out if has_groups else out.squeeze(2)
