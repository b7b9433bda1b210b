"""Parameter block for calling ONE stage of the SSD pipeline through the C ABI.

The combined entry points fill every field of SsdParams; a single stage reads only a few of them,
but the library's argument check wants the always-present operands to be non-null.  `stage_params`
points every such field at a small placeholder tensor that no stage kernel reads through; the stage
wrappers then overwrite the fields their kernel really uses.
"""
import math

import torch

from mamba_amd import _lib

_ALWAYS = ("x", "dt", "A", "B", "C")
_ALWAYS_BWD = ("dout", "dt_out", "dA_cumsum", "states", "CB", "dstates", "ddA_cumsum", "ddt_out", "dCB", "dB32",
               "dC32", "dx", "ddt", "dA", "out")


def stage_params(device, *, batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, dtype=torch.float32,
                 dt_dtype=torch.float32, backward=False):
    """Returns (params, keepalive): SsdParams with the sizes set and placeholders in the mandatory pointers."""
    p = _lib.SsdParams()
    p.batch, p.seqlen, p.nheads, p.headdim, p.dstate, p.ngroups = batch, seqlen, nheads, headdim, dstate, ngroups
    p.chunk_size, p.nchunks = chunk_size, math.ceil(seqlen / chunk_size)
    p.dtype, p.dt_dtype = _lib.DTYPE_CODE[dtype], _lib.DTYPE_CODE[dt_dtype]
    p.dt_min, p.dt_max = 0.0, 3.0e38
    blank = torch.zeros(64, device=device, dtype=torch.float32)
    for name in _ALWAYS + (_ALWAYS_BWD if backward else ()):
        setattr(p, name, blank.data_ptr())
    if backward and dtype == torch.bfloat16:
        p.states_lp = p.dstates_lp = blank.data_ptr()
    return p, blank


def carried_dtype(x_dtype):
    """dtype in which the states carried between chunks, and their gradients, pass between the kernels: bf16 next to
    bf16 operands, fp32 otherwise."""
    return torch.bfloat16 if x_dtype == torch.bfloat16 else torch.float32


def set_carried(p, field, t, x_dtype):
    """Hands the kernels a (batch, nchunks, nheads, headdim, dstate) tensor of carried states (`field` = "states") or
    of their gradients ("dstates") in the dtype they take it in: bf16 through the *_lp field next to bf16 operands,
    fp32 through the field itself otherwise.  Returns the tensor handed over (a kernel that writes fills this one)."""
    want = carried_dtype(x_dtype)
    t = t if (t.dtype == want and t.is_contiguous()) else t.to(want).contiguous()
    setattr(p, field + "_lp" if want == torch.bfloat16 else field, t.data_ptr())
    return t


def f32c(t):
    """fp32, contiguous (the layout of every workspace the stages exchange)."""
    return t if (t.dtype == torch.float32 and t.is_contiguous()) else t.float().contiguous()


def seq_idx_i32(seq_idx):
    return None if seq_idx is None else seq_idx.to(torch.int32).contiguous()


def run(name, p, device):
    with torch.cuda.device(device):
        _lib.check(getattr(_lib.load(), name)(p, _lib.current_stream(device)), name)
