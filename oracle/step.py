"""Oracle for the single-token decode step (test infrastructure, CPU, plain PyTorch).

Restates selective_state_update_ref (reference
mamba_ssm/ops/triton/selective_state_update.py:224-285):
    dt' = softplus(dt + dt_bias)                                  (:266-268)
    state <- state * exp(dt' A) + (dt' B) x      in place          (:269-273)
    out = <state, C> + D x ;  out *= silu(z)                       (:274-278)
The arithmetic is done in `compute_dtype` and the new state is written back in the state's
own dtype; the output uses the unrounded new state, like the reference's kernel (:125-127).
Pinned by tests/test_oracle_step.py (T steps == a length-T Mamba-1 scan).
"""
import torch
import torch.nn.functional as F


def selective_state_update_oracle(state, x, dt, A, B, C, D=None, z=None, dt_bias=None, dt_softplus=False,
                                  state_batch_indices=None, compute_dtype=torch.float32):
    has_heads = state.dim() > 3
    cd = compute_dtype
    if state.dim() == 3:
        state = state.unsqueeze(1)
    un = lambda t, d: t.unsqueeze(1) if (t is not None and t.dim() == d) else t
    x, dt, z = un(x, 2), un(dt, 2), un(z, 2)
    B, C = un(B, 2), un(C, 2)
    if A.dim() == 2:
        A = A.unsqueeze(0)
    if D is not None and D.dim() == 1:
        D = D.unsqueeze(0)
    if dt_bias is not None and dt_bias.dim() == 1:
        dt_bias = dt_bias.unsqueeze(0)
    batch, nheads, dim = x.shape
    ngroups = B.shape[1]
    dtv = dt.to(cd)
    if dt_bias is not None:
        dtv = dtv + dt_bias.to(cd)
    if dt_softplus:
        dtv = F.softplus(dtv)
    Bh = B.to(cd).repeat_interleave(nheads // ngroups, dim=1)   # (b, h, n)
    Ch = C.to(cd).repeat_interleave(nheads // ngroups, dim=1)
    dA = torch.exp(dtv[..., None] * A.to(cd))                   # (b, h, p, n)
    rows = torch.arange(batch) if state_batch_indices is None else state_batch_indices.long()
    live = rows >= 0
    out = torch.zeros(batch, nheads, dim, dtype=cd)
    if live.any():
        r = rows[live]
        new = state[r].to(cd) * dA[live] + (dtv[live, ..., None] * Bh[live, :, None, :]) * x.to(cd)[live, ..., None]
        state[r] = new.to(state.dtype)
        o = (new * Ch[live, :, None, :]).sum(-1)
        if D is not None:
            o = o + x.to(cd)[live] * D.to(cd)
        if z is not None:
            o = o * F.silu(z.to(cd)[live])
        out[live] = o
    out = out.to(x.dtype)
    return out if has_heads else out.squeeze(1)
