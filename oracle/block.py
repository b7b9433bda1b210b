"""Oracle for mamba_split_conv1d_scan_combined (test infrastructure, CPU, plain PyTorch).

Restates the forward of MambaSplitConv1dScanCombinedFn (reference
mamba_ssm/ops/triton/ssd_combined.py:824-899): split of zxbcdt (:843), causal depthwise conv1d + SiLU
on xBC (:845-849; arithmetic of the un-vendored causal_conv1d package, restated with the library
routine the reference falls back to, mamba_ssm/modules/mamba2.py:230-234, and with taps across a
seq_idx boundary dropped as that package does for packed batches), the SSD scan (oracle.ssd), then
either the SiLU gate inside the scan (:855-861) or the gated group RMSNorm of
mamba_ssm/ops/triton/layernorm_gated.py:18-39 (:863-881), the SwiGLU of the non-SSM part
(mamba_ssm/ops/triton/k_activations.py:42) and out_proj (:884-891).
Pinned by tests/test_oracle_block.py.
"""
import torch
import torch.nn.functional as F

from oracle.ssd import ssd_oracle


def causal_conv1d_oracle(x, weight, bias=None, activation="silu", seq_idx=None):
    """x: (batch, seqlen, channels); weight: (channels, width).  Loop over taps."""
    batch, L, ch = x.shape
    width = weight.shape[1]
    y = torch.zeros_like(x)
    pos = torch.arange(L)
    for k in range(width):                         # tap k looks back k positions
        src = pos - k
        ok = src >= 0
        xs = x[:, src.clamp(min=0)]
        m = ok[None, :].expand(batch, L)
        if seq_idx is not None:
            m = m & (seq_idx[:, src.clamp(min=0)] == seq_idx)
        y = y + torch.where(m[..., None], xs, torch.zeros_like(xs)) * weight[:, width - 1 - k]
    if bias is not None:
        y = y + bias
    return F.silu(y) if activation in ("silu", "swish") else y


def causal_conv1d_update_oracle(x, conv_state, weight, bias=None, activation="silu"):
    """Decode step of the convolution: x (batch, dim, seqlen), conv_state (batch, dim, state_len),
    weight (dim, width).  Returns (out, new_state); generalises the roll + insert + dot of reference
    mamba_ssm/modules/mamba2.py:291-296 (one new position, state_len = width) to seqlen new positions
    and any state_len >= width - 1 by running the full convolution over [conv_state, x]."""
    batch, dim, seqlen = x.shape
    state_len, width = conv_state.shape[2], weight.shape[1]
    xn = torch.cat([conv_state.to(x.dtype), x], dim=-1)
    out = torch.zeros_like(x)
    for t in range(seqlen):
        for k in range(width):
            out[:, :, t] += weight[:, k] * xn[:, :, state_len + t - (width - 1) + k]
    if bias is not None:
        out = out + bias[None, :, None]
    if activation in ("silu", "swish"):
        out = F.silu(out)
    return out, xn[:, :, xn.shape[2] - state_len:]


def causal_conv1d_varlen_states_oracle(x, cu_seqlens, state_len):
    """x: (total, dim).  Per sequence the F.pad(x_seq^T, (state_len - len, 0)) of reference
    mamba_ssm/modules/mamba2.py:219-221: the last state_len positions, zero-filled on the left."""
    out = []
    for s in range(len(cu_seqlens) - 1):
        seq = x[int(cu_seqlens[s]):int(cu_seqlens[s + 1])].transpose(0, 1)
        out.append(F.pad(seq, (state_len - seq.shape[1], 0)))
    return torch.stack(out)


def gated_rms_norm_oracle(x, weight, z, eps, group_size, norm_before_gate):
    x, z, weight = x.double(), z.double(), weight.double()
    if not norm_before_gate:
        x = x * F.silu(z)
    g = x.reshape(*x.shape[:-1], -1, group_size)
    g = g / torch.sqrt(g.pow(2).mean(-1, keepdim=True) + eps)
    out = g.reshape(x.shape) * weight
    if norm_before_gate:
        out = out * F.silu(z)
    return out


def split_conv1d_scan_oracle(zxbcdt, conv1d_weight, conv1d_bias, dt_bias, A, D, initial_states=None, seq_idx=None,
                             dt_limit=(0.0, float("inf")), activation="silu", rmsnorm_weight=None, rmsnorm_eps=1e-6,
                             outproj_weight=None, outproj_bias=None, headdim=None, ngroups=1, norm_before_gate=True,
                             compute_dtype=torch.float32):
    """Returns (out, final_states)."""
    cd = compute_dtype
    nheads = D.shape[0]
    if D.dim() == 2:
        headdim = D.shape[1]
    batch, L, _ = zxbcdt.shape
    dim = nheads * headdim
    dstate = (conv1d_weight.shape[0] - dim) // ngroups // 2
    d_nonssm = (zxbcdt.shape[-1] - 2 * dim - 2 * ngroups * dstate - nheads) // 2
    zx0, z, xBC, dt = torch.split(zxbcdt.to(cd), [2 * d_nonssm, dim, dim + 2 * ngroups * dstate, nheads], dim=-1)
    xBC = causal_conv1d_oracle(xBC, conv1d_weight.to(cd), None if conv1d_bias is None else conv1d_bias.to(cd),
                               activation, seq_idx)
    x, B, C = torch.split(xBC, [dim, ngroups * dstate, ngroups * dstate], dim=-1)
    x = x.reshape(batch, L, nheads, headdim)
    B = B.reshape(batch, L, ngroups, dstate)
    C = C.reshape(batch, L, ngroups, dstate)
    z4 = z.reshape(batch, L, nheads, headdim)
    y, fin = ssd_oracle(x, dt, A.to(cd), B, C, D=D.to(cd), z=z4 if rmsnorm_weight is None else None,
                        dt_bias=dt_bias.to(cd), initial_states=initial_states, seq_idx=seq_idx, dt_softplus=True,
                        dt_limit=dt_limit, return_final_states=True, compute_dtype=cd)
    y = y.reshape(batch, L, dim)
    if rmsnorm_weight is not None:
        y = gated_rms_norm_oracle(y, rmsnorm_weight, z, rmsnorm_eps, dim // ngroups, norm_before_gate).to(cd)
    if d_nonssm > 0:
        a, b = zx0.chunk(2, dim=-1)
        y = torch.cat([F.silu(a) * b, y], dim=-1)
    if outproj_weight is not None:
        y = y @ outproj_weight.to(cd).t()
        if outproj_bias is not None:
            y = y + outproj_bias.to(cd)
    return y, fin
