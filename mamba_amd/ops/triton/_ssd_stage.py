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
    return p, blank


def f32c(t):
    """fp32, contiguous (the layout of every workspace the stages exchange)."""
    return t if (t.dtype == torch.float32 and t.is_contiguous()) else t.float().contiguous()


def seq_idx_i32(seq_idx):
    return None if seq_idx is None else seq_idx.to(torch.int32).contiguous()


def run(name, p, device):
    with torch.cuda.device(device):
        _lib.check(getattr(_lib.load(), name)(p, _lib.current_stream(device)), name)


def forward_only(name):
    raise NotImplementedError(
        f"{name}: the stage-level function has no backward pass of its own here; gradients go through "
        "mamba_chunk_scan_combined, whose backward stages are fused across chunk_state and chunk_scan")
