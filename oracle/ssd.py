"""Oracle for the Mamba-2 SSD scan (test infrastructure, CPU, plain PyTorch).

What it restates.  mamba_chunk_scan_combined (reference
mamba_ssm/ops/triton/ssd_combined.py:628) has these semantics, taken from its kernels and
reference functions:
  * step size: dt' = clamp(softplus(dt + dt_bias), dt_limit)       (ssd_chunk_state.py:72-81)
  * recurrence per head:  h_t = exp(dt'_t A_h) h_{t-1} + dt'_t x_t B_t^T,
    y_t = h_t C_t + D x_t,  out = y * silu(z)
    (ssd_combined.py:728-775 maps it onto selective_scan; ssd_minimal.py:34-78 is the chunked form;
    ssd_chunk_scan.py:1846-1887 the masked quadratic form)
  * initial_states seeds h before t = 0; final_states is h after the last position
    (ssd_state_passing.py:64-84)
  * seq_idx: a new sequence starts where seq_idx changes; the state is dropped there.  The id in
    force before t = 0 is 0, so initial_states reach only a first sequence whose id is 0
    (ssd_state_passing.py:71-79, ssd_chunk_scan.py:97-118, ssd_chunk_state.py:231-251).

Three independent formulations live here -- sequential (`ssd_oracle`), chunked
(`ssd_chunked`), quadratic (`ssd_quadratic`) -- and tests/test_oracle_ssd.py requires them to
agree, next to closed-form checks.  Gradients come from torch.autograd through `ssd_oracle`.
"""
import torch
import torch.nn.functional as F


def dt_pipeline(dt, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf")), compute_dtype=torch.float32):
    dt = dt.to(compute_dtype)
    if dt_bias is not None:
        dt = dt + dt_bias.to(compute_dtype)
    if dt_softplus:
        dt = F.softplus(dt)
    # The reference's kernel clamps even at the default limits (0, inf), so a negative dt without softplus
    # becomes 0 (ssd_chunk_state.py:80); its torch reference (ssd_combined.py:706-710) has no clamp.
    # The kernel's behaviour is the one restated here.
    return dt.clamp(min=dt_limit[0], max=dt_limit[1])


def ssd_oracle(x, dt, A, B, C, D=None, z=None, dt_bias=None, initial_states=None, seq_idx=None,
               dt_softplus=False, dt_limit=(0.0, float("inf")), return_final_states=False,
               compute_dtype=torch.float32):
    """x, z: (b, L, h, p); dt: (b, L, h); A: (h,); B, C: (b, L, g, n); D: (h,) or (h, p);
    initial_states: (b, h, p, n); seq_idx: (b, L) int.  Returns out (b, L, h, p) in x.dtype
    [, final_states (b, h, p, n) in compute_dtype]."""
    cd = compute_dtype
    batch, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    dtv = dt_pipeline(dt, dt_bias, dt_softplus, dt_limit, cd)          # (b, L, h)
    xf, Bf, Cf = x.to(cd), B.to(cd), C.to(cd)
    Bh = Bf.repeat_interleave(H // G, dim=2)                           # (b, L, h, n)
    Ch = Cf.repeat_interleave(H // G, dim=2)
    Af = A.to(cd)
    h = torch.zeros(batch, H, P, N, dtype=cd) if initial_states is None else initial_states.to(cd)
    prev_id = torch.zeros(batch, dtype=torch.long)
    ys = []
    for t in range(L):
        if seq_idx is not None:
            cur = seq_idx[:, t].long()
            keep = (cur == prev_id).to(cd)[:, None, None, None]
            h = h * keep
            prev_id = cur
        dA = torch.exp(dtv[:, t] * Af)                                 # (b, h)
        h = h * dA[:, :, None, None] + (dtv[:, t, :, None] * xf[:, t])[..., None] * Bh[:, t, :, None, :]
        ys.append(torch.einsum("bhpn,bhn->bhp", h, Ch[:, t]))
    y = torch.stack(ys, dim=1)
    if D is not None:
        Dv = D.to(cd)
        y = y + xf * (Dv[:, None] if Dv.dim() == 1 else Dv)
    if z is not None:
        y = y * F.silu(z.to(cd))
    out = y.to(x.dtype)
    return (out, h) if return_final_states else out


def ssd_chunked(x, dt, A, B, C, chunk_size, D=None, z=None, initial_states=None, return_final_states=False,
                compute_dtype=torch.float64):
    """The four-step chunked algorithm (ssd_minimal.py:47-78): diagonal blocks, chunk states, the
    recurrence over chunk states, state -> output.  dt is the final step size; no seq_idx."""
    cd = compute_dtype
    batch, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    Q = chunk_size
    pad = (Q - L % Q) % Q
    padL = lambda t: F.pad(t, [0, 0] * (t.dim() - 2) + [0, pad])
    xf, dtf = padL(x.to(cd)), padL(dt.to(cd))
    Bh = padL(B.to(cd).repeat_interleave(H // G, dim=2))
    Ch = padL(C.to(cd).repeat_interleave(H // G, dim=2))
    nc = (L + pad) // Q
    xf = xf.view(batch, nc, Q, H, P)
    dtf = dtf.view(batch, nc, Q, H)
    Bh, Ch = Bh.view(batch, nc, Q, H, N), Ch.view(batch, nc, Q, H, N)
    a = torch.cumsum(dtf * A.to(cd), dim=2)                            # (b, c, Q, h)
    # 1. inside each chunk
    seg = a[:, :, :, None, :] - a[:, :, None, :, :]                     # a_l - a_s: (b, c, l, s, h)
    causal = torch.tril(torch.ones(Q, Q, dtype=torch.bool))
    Lmat = torch.where(causal[None, None, :, :, None], torch.exp(seg), torch.zeros((), dtype=cd))
    CB = torch.einsum("bclhn,bcshn->bclsh", Ch, Bh)
    y_diag = torch.einsum("bclsh,bclsh,bcsh,bcshp->bclhp", CB, Lmat, dtf, xf)
    # 2. state contributed by each chunk
    decay_to_end = torch.exp(a[:, :, -1:, :] - a)                       # (b, c, s, h)
    S = torch.einsum("bcshn,bcsh,bcsh,bcshp->bchpn", Bh, decay_to_end, dtf, xf)
    # 3. recurrence over chunks
    Hc = torch.zeros(batch, H, P, N, dtype=cd) if initial_states is None else initial_states.to(cd)
    entering = []
    for c in range(nc):
        entering.append(Hc)
        Hc = Hc * torch.exp(a[:, c, -1, :])[:, :, None, None] + S[:, c]
    entering = torch.stack(entering, dim=1)                             # (b, c, h, p, n)
    # 4. carried state -> outputs
    y_off = torch.einsum("bclhn,bchpn,bclh->bclhp", Ch, entering, torch.exp(a))
    y = (y_diag + y_off).reshape(batch, nc * Q, H, P)[:, :L]
    xr = x.to(cd)
    if D is not None:
        Dv = D.to(cd)
        y = y + xr * (Dv[:, None] if Dv.dim() == 1 else Dv)
    if z is not None:
        y = y * F.silu(z.to(cd))
    return (y, Hc) if return_final_states else y


def ssd_quadratic(x, dt, A, B, C, compute_dtype=torch.float64):
    """y = (L o (C B^T)) (dt x) with L[l, s] = exp(sum_{s < r <= l} dt_r A) for l >= s: the masked
    attention form over the whole sequence.  No D, z, initial state."""
    cd = compute_dtype
    batch, L, H, P = x.shape
    G = B.shape[2]
    Bh = B.to(cd).repeat_interleave(H // G, dim=2)
    Ch = C.to(cd).repeat_interleave(H // G, dim=2)
    a = torch.cumsum(dt.to(cd) * A.to(cd), dim=1)                      # (b, L, h)
    seg = a[:, :, None, :] - a[:, None, :, :]
    causal = torch.tril(torch.ones(L, L, dtype=torch.bool))
    Lmat = torch.where(causal[None, :, :, None], torch.exp(seg), torch.zeros((), dtype=cd))
    CB = torch.einsum("blhn,bshn->blsh", Ch, Bh)
    return torch.einsum("blsh,blsh,bsh,bshp->blhp", CB, Lmat, dt.to(cd), x.to(cd))


def ssd_inputs(batch, seqlen, nheads, headdim, dstate, ngroups=1, dtype=torch.float32, seed=0, has_z=True,
               has_D=True, D_has_hdim=False, seq_lens=None, has_init=False):
    """Seeded inputs with the benchmark's distributions (initialisation of reference
    mamba_ssm/modules/mamba2.py:120-140): x, B, C, z ~ N(0,1); raw dt ~ N(0,1) with
    dt_bias = softplus^-1(log-uniform[1e-3, 1e-1]); A = -U(1,16); D ~ U(0,1)."""
    import math
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g)
    t = dict(
        x=rn(batch, seqlen, nheads, headdim).to(dtype),
        dt=rn(batch, seqlen, nheads).to(dtype),
        B=rn(batch, seqlen, ngroups, dstate).to(dtype),
        C=rn(batch, seqlen, ngroups, dstate).to(dtype),
        z=rn(batch, seqlen, nheads, headdim).to(dtype) if has_z else None,
        A=-(1.0 + 15.0 * torch.rand(nheads, generator=g)),
        D=(torch.rand(nheads, headdim, generator=g) if D_has_hdim else torch.rand(nheads, generator=g)) if has_D else None,
        dout=rn(batch, seqlen, nheads, headdim).to(dtype),
    )
    dtv = torch.exp(torch.rand(nheads, generator=g) * (math.log(1e-1) - math.log(1e-3)) + math.log(1e-3))
    t["dt_bias"] = dtv + torch.log(-torch.expm1(-dtv))
    t["initial_states"] = 0.1 * rn(batch, nheads, headdim, dstate) if has_init else None
    t["dfinal"] = rn(batch, nheads, headdim, dstate)
    if seq_lens is not None:
        assert sum(seq_lens) == seqlen
        ids = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(seq_lens)])
        t["seq_idx"] = ids[None].repeat(batch, 1).contiguous()
    else:
        t["seq_idx"] = None
    return t
