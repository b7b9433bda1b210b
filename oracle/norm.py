"""Oracle for the gated LayerNorm / RMSNorm over channel groups (test infrastructure, CPU, plain PyTorch).

Restates the reference's own reference function mamba_ssm/ops/triton/layernorm_gated.py:18-39
(rms_norm_ref) and its LayerNorm counterpart (the kernel's `IS_RMS_NORM=False` branch, :75-88): the
gate silu(z) multiplies x before the statistics (norm_before_gate=False) or the normalised output
after them (:25-26, :37-38); statistics per group of `group_size` channels (:31-35).  Written as
explicit sums, not through F.layer_norm / F.rms_norm, so that tests/test_oracle_norm.py can pin it
against those library routines, against a per-element Python loop and by gradcheck.
"""
import torch
import torch.nn.functional as F


def gated_norm_oracle(x, weight, bias=None, z=None, eps=1e-6, group_size=None, norm_before_gate=True,
                      is_rms_norm=False, compute_dtype=torch.float64):
    """x, z: (..., dim); weight, bias: (dim,).  Returns the output in compute_dtype."""
    x = x.to(compute_dtype)
    weight = weight.to(compute_dtype)
    bias = bias.to(compute_dtype) if bias is not None else None
    z = z.to(compute_dtype) if z is not None else None
    dim = x.shape[-1]
    gs = dim if group_size is None else group_size
    assert dim % gs == 0
    if z is not None and not norm_before_gate:
        x = x * F.silu(z)
    xg = x.reshape(*x.shape[:-1], dim // gs, gs)
    if not is_rms_norm:
        xg = xg - xg.sum(dim=-1, keepdim=True) / gs
    var = (xg * xg).sum(dim=-1, keepdim=True) / gs
    y = (xg / torch.sqrt(var + eps)).reshape(x.shape) * weight
    if bias is not None:
        y = y + bias
    if z is not None and norm_before_gate:
        y = y * F.silu(z)
    return y
