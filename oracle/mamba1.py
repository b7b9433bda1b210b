"""Oracle for the Mamba-1 selective scan (test infrastructure, CPU, plain PyTorch).

Restates selective_scan_ref (reference mamba_ssm/ops/selective_scan_interface.py:127-193):
    delta' = softplus(delta + delta_bias)              (:146-149)
    h_t = exp(delta'_t A) h_{t-1} + delta'_t B_t u_t    (:162-175)
    y_t = <h_t, C_t> + D u_t                            (:176-188)
    out = y * silu(z), cast back to the input dtype     (:189-192)
B, C of shape (batch, ngroups, dstate, L) are shared by the dim/ngroups channels of a
group (:169-172); an input-independent B or C is a (dim, dstate) matrix used at every
position (:163-166, :177-178).  With a complex A (:150-158) the state, A and the matrices B, C are
complex, per-position B, C carry (re, im) pairs interleaved along their last axis (length 2L,
:152-157), and the output is twice the real part of <h, C> (:186-187).  Gradients come from torch.autograd through this function, which is how
the reference's own test obtains them (tests/ops/test_selective_scan.py:119-121).
Pinned by tests/test_oracle_mamba1.py.
"""
import torch
import torch.nn.functional as F


def selective_scan_oracle(u, delta, A, B, C, D=None, z=None, delta_bias=None, delta_softplus=False,
                          return_last_state=False, compute_dtype=torch.float32):
    """u, delta, z: (b, d, L); A: (d, n); B, C: (b, n, L), (b, g, n, L) or (d, n); D, delta_bias: (d,)."""
    dtype_in = u.dtype
    cd = compute_dtype
    u = u.to(cd)
    delta = delta.to(cd)
    if delta_bias is not None:
        delta = delta + delta_bias.to(cd)[None, :, None]
    if delta_softplus:
        delta = F.softplus(delta)
    batch, dim, L = u.shape
    n = A.shape[1]
    is_complex = A.is_complex()
    if is_complex:
        ccd = torch.complex64 if cd == torch.float32 else torch.complex128
        A = A.to(ccd)

        def as_complex(t):  # per-position operands: (..., 2L) real pairs -> (..., L) complex
            if t.is_complex():
                return t.to(ccd)
            return torch.view_as_complex(t.to(cd).reshape(*t.shape[:-1], L, 2).contiguous())

        B, C = as_complex(B), as_complex(C)
    else:
        A = A.to(cd)
        B = B.to(cd)
        C = C.to(cd)
    def per_channel(t):  # -> (b or 1, d, n, L)
        if t.dim() == 2:
            return t[None, :, :, None].expand(1, dim, n, L)
        if t.dim() == 3:
            t = t[:, None]
        return t.repeat_interleave(dim // t.shape[1], dim=1)

    B = per_channel(B)
    C = per_channel(C)
    h = torch.zeros(batch, dim, n, dtype=A.dtype, device=u.device)
    ys = []
    # the time axis is taken apart once (unbind) rather than indexed per step: the same arithmetic, but autograd then
    # gathers the per-step gradients in one pass instead of writing a full-size tensor per step
    dts, us, Bts, Cts = delta.unbind(2), u.unbind(2), B.unbind(-1), C.unbind(-1)
    for t in range(L):
        dt = dts[t][:, :, None]                                # (b, d, 1)
        h = torch.exp(dt * A[None]) * h + (dt * us[t][:, :, None]) * Bts[t]
        yt = (h * Cts[t]).sum(-1)
        ys.append(2 * yt.real if is_complex else yt)
    y = torch.stack(ys, dim=2)
    if D is not None:
        y = y + u * D.to(cd)[None, :, None]
    if z is not None:
        y = y * F.silu(z.to(cd))
    out = y.to(dtype_in)
    return (out, h) if return_last_state else out


def scan_inputs(batch, dim, seqlen, dstate, ngroups=1, dtype=torch.float32, seed=0, device="cpu",
                has_z=True, has_D=True):
    """Seeded inputs with the distributions of the benchmark configurations: u, z, raw delta,
    B, C ~ N(0,1); delta_bias = softplus^-1(dt) with dt log-uniform in [1e-3, 1e-1];
    A[d, n] = -(n+1); D = 1 (initialisation of reference mamba_ssm/modules/mamba_simple.py:85-112)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g)
    u = rn(batch, dim, seqlen).to(dtype)
    delta = rn(batch, dim, seqlen).to(dtype)
    z = rn(batch, dim, seqlen).to(dtype) if has_z else None
    B = rn(batch, ngroups, dstate, seqlen).to(dtype)
    C = rn(batch, ngroups, dstate, seqlen).to(dtype)
    import math
    dt = torch.exp(torch.rand(dim, generator=g) * (math.log(1e-1) - math.log(1e-3)) + math.log(1e-3))
    delta_bias = dt + torch.log(-torch.expm1(-dt))
    A = -torch.arange(1, dstate + 1, dtype=torch.float32).repeat(dim, 1).contiguous()
    D = torch.ones(dim) if has_D else None
    dout = rn(batch, dim, seqlen).to(dtype)
    out = dict(u=u, delta=delta, A=A, B=B, C=C, D=D, z=z, delta_bias=delta_bias, dout=dout)
    return {k: (v.to(device) if v is not None else None) for k, v in out.items()}
