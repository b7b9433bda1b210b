"""Oracle for mamba_inner_fn (test infrastructure, CPU, plain PyTorch).

Restates mamba_inner_ref (reference mamba_ssm/ops/selective_scan_interface.py:397-432): causal
depthwise conv1d + SiLU, x_proj, dt_proj, selective scan, out_proj.  The convolution is the library
routine the reference falls back to when the causal_conv1d package is missing
(mamba_ssm/modules/mamba_simple.py:168-169); the scan is oracle.mamba1.  The reference's own test of
this block compares two users of the same third-party conv package, so the conv boundary is pinned
here by the library routine instead (tests/test_oracle_mamba1.py pins the scan).
"""
import torch
import torch.nn.functional as F

from oracle.mamba1 import selective_scan_oracle


def mamba_inner_oracle(xz, conv1d_weight, conv1d_bias, x_proj_weight, delta_proj_weight, out_proj_weight,
                       out_proj_bias, A, D=None, delta_bias=None, B_proj_bias=None, C_proj_bias=None,
                       compute_dtype=torch.float32, B=None, C=None, b_rms_weight=None, c_rms_weight=None,
                       dt_rms_weight=None, b_c_dt_rms_eps=1e-6):
    """B / C given: input-independent (dim, dstate) matrices instead of the x_proj slices (:415-430);
    x_proj_weight then only carries the rows of the slices that are still projected.
    b / c / dt_rms_weight: RMSNorm of the projected B and C rows over the states and of delta over the
    channels before the scan (MambaInnerFn.forward, :263-274).  The reference's backward pass treats these
    norms as the identity (it hands the scan's dB / dC / ddelta straight to the projections and returns no
    gradient for the norm weights, :283-383), so they are written here with a straight-through gradient."""
    cd = compute_dtype
    batch, two_d, L = xz.shape
    d = two_d // 2
    R = delta_proj_weight.shape[1]
    N = A.shape[1] * (2 if A.is_complex() else 1)   # x_proj emits (re, im) pairs per state (:207, :255-258)

    def pack(m):  # (b l, N) -> (b, n, L) or, complex, (b, n, 2 L) with interleaved pairs
        if not A.is_complex():
            return m.reshape(batch, L, N).permute(0, 2, 1)
        return m.reshape(batch, L, N // 2, 2).permute(0, 2, 1, 3).reshape(batch, N // 2, 2 * L)

    x, z = xz.to(cd)[:, :d], xz.to(cd)[:, d:]
    w = conv1d_weight.to(cd)                                     # (d, 1, width)
    x = F.silu(F.conv1d(x, w, None if conv1d_bias is None else conv1d_bias.to(cd), padding=w.shape[-1] - 1,
                        groups=d)[..., :L])
    x_dbl = x.permute(0, 2, 1).reshape(batch * L, d) @ x_proj_weight.to(cd).t()           # (b l, R + 2N)
    delta = (delta_proj_weight.to(cd) @ x_dbl[:, :R].t()).reshape(d, batch, L).permute(1, 0, 2)
    if B is None:
        Bm = x_dbl[:, R:R + N]
        if B_proj_bias is not None:
            Bm = Bm + B_proj_bias.to(cd)
        Bm = pack(Bm)
    else:
        Bm = B if B.is_complex() else B.to(cd)
    if C is None:
        Cm = x_dbl[:, x_dbl.shape[1] - N:]
        if C_proj_bias is not None:
            Cm = Cm + C_proj_bias.to(cd)
        Cm = pack(Cm)
    else:
        Cm = C if C.is_complex() else C.to(cd)
    def rms_st(t, w, dim):  # value of the norm, gradient of the identity
        n = t * torch.rsqrt(t.pow(2).mean(dim, keepdim=True) + b_c_dt_rms_eps) * w
        return t + (n - t).detach()

    if b_rms_weight is not None:
        Bm = rms_st(Bm, b_rms_weight.to(cd)[None, :, None], 1)
    if c_rms_weight is not None:
        Cm = rms_st(Cm, c_rms_weight.to(cd)[None, :, None], 1)
    if dt_rms_weight is not None:
        delta = rms_st(delta, dt_rms_weight.to(cd)[None, :, None], 1)
    y = selective_scan_oracle(x, delta, A if A.is_complex() else A.to(cd), Bm, Cm, None if D is None else D.to(cd), z,
                              None if delta_bias is None else delta_bias.to(cd), True, compute_dtype=cd)
    out = y.permute(0, 2, 1) @ out_proj_weight.to(cd).t()
    if out_proj_bias is not None:
        out = out + out_proj_bias.to(cd)
    return out
