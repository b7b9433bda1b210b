"""Switch of the deterministic mode, with the reference's names and rules
(mamba_ssm/utils/determinism.py:21-33): an explicit override, else the environment variable
MAMBA_DETERMINISTIC (first character '1' = on), else torch.are_deterministic_algorithms_enabled().

What the mode changes here: the backward passes of the SSD scan and of the causal convolution add the
sums that several workgroups share (dB, dC, the dt / decay gradients, dA, dD, dt_bias, the conv weight and
bias gradients) with 64-bit integer atomics on terms scaled to a fixed point, instead of float atomics;
integer addition does not depend on the order of the adds, so every gradient repeats bit for bit.  Every
other operator of the package is deterministic in either mode."""
import os

import torch

_deterministic_override = None


def use_deterministic_mode():
    if _deterministic_override is not None:
        return _deterministic_override
    env = os.environ.get("MAMBA_DETERMINISTIC")
    if env:
        return env[0] == "1"
    return torch.are_deterministic_algorithms_enabled()


def set_deterministic_mode(value):
    global _deterministic_override
    _deterministic_override = value


def fixed_point_scale(*grads):
    """{s, 1 / s} as a 2-element fp32 device tensor, s = 2^30 / 2^floor(log2(m)) with m the largest magnitude among
    the given upstream gradients (s = 1 when they are all zero).  Computed on the device: no host synchronisation."""
    m = None
    for g in grads:
        if g is None or g.numel() == 0:
            continue
        v = g.detach().abs().amax().float()
        m = v if m is None else torch.maximum(m, v)
    e = torch.floor(torch.log2(m))
    e = torch.where(torch.isfinite(e), e, torch.full_like(e, 30.0)).to(torch.int32)
    one = torch.ones_like(m)
    return torch.stack([torch.ldexp(one, 30 - e), torch.ldexp(one, e - 30)]).contiguous()
