"""Single-token decode step: drop-in for mamba_ssm.ops.triton.selective_state_update.

Same signature and shape rules as the reference host function
(mamba_ssm/ops/triton/selective_state_update.py:135-221); the Triton kernel (:24) is replaced
by the HIP kernel behind the C ABI's ssm_state_update.  The module path keeps the reference's
`triton` package name so that imports stay source compatible; no Triton is involved.
"""
import torch

from mamba_amd import _lib


def selective_state_update(state, x, dt, A, B, C, D=None, z=None, dt_bias=None, dt_softplus=False,
                           state_batch_indices=None):
    """
    Argument:
        state: (batch, dim, dstate) or (batch, nheads, dim, dstate)   -- updated in place
        x: (batch, dim) or (batch, nheads, dim)
        dt: (batch, dim) or (batch, nheads, dim)
        A: (dim, dstate) or (nheads, dim, dstate)
        B: (batch, dstate) or (batch, ngroups, dstate)
        C: (batch, dstate) or (batch, ngroups, dstate)
        D: (dim,) or (nheads, dim)
        z: (batch, dim) or (batch, nheads, dim)
        dt_bias: (dim,) or (nheads, dim)
        state_batch_indices: (batch,) int32, row of `state` per batch entry; an index outside
            [0, state.shape[0]) is a padding entry (state untouched, out = 0)
    Return:
        out: (batch, dim) or (batch, nheads, dim)
    """
    has_heads = state.dim() > 3
    if state.dim() == 3:
        state = state.unsqueeze(1)
    if x.dim() == 2:
        x = x.unsqueeze(1)
    if dt.dim() == 2:
        dt = dt.unsqueeze(1)
    if A.dim() == 2:
        A = A.unsqueeze(0)
    if B.dim() == 2:
        B = B.unsqueeze(1)
    if C.dim() == 2:
        C = C.unsqueeze(1)
    if D is not None and D.dim() == 1:
        D = D.unsqueeze(0)
    if z is not None and z.dim() == 2:
        z = z.unsqueeze(1)
    if dt_bias is not None and dt_bias.dim() == 1:
        dt_bias = dt_bias.unsqueeze(0)
    state_rows, nheads, dim, dstate = state.shape
    batch = x.shape[0]
    if state_batch_indices is None and state_rows < batch:
        raise RuntimeError(f"selective_state_update: state has {state_rows} rows for a batch of {batch} "
                           "and no state_batch_indices")
    assert x.shape == (batch, nheads, dim)
    assert dt.shape == x.shape
    assert A.shape == (nheads, dim, dstate)
    ngroups = B.shape[1]
    assert nheads % ngroups == 0, "nheads must be divisible by ngroups"
    assert B.shape == (batch, ngroups, dstate)
    assert C.shape == B.shape
    if D is not None:
        assert D.shape == (nheads, dim)
    if z is not None:
        assert z.shape == x.shape
    if dt_bias is not None:
        assert dt_bias.shape == (nheads, dim)
    if state_batch_indices is not None:
        assert state_batch_indices.shape == (batch,)
        if state_batch_indices.dtype != torch.int32:
            state_batch_indices = state_batch_indices.to(torch.int32)
        state_batch_indices = state_batch_indices.contiguous()
    _lib.require_gpu(state, x, dt, A, B, C, D, z, dt_bias, state_batch_indices)
    if z is not None and z.dtype != x.dtype:
        z = z.to(x.dtype)
    # The kernel takes A, D, dt_bias in fp32 and B, C, dt either in x's dtype or in fp32.
    # (.float() of an fp32 tensor is the tensor itself, so expanded stride-0 views stay views.)
    A = A.float()
    D = D.float() if D is not None else None
    dt_bias = dt_bias.float() if dt_bias is not None else None
    if B.dtype != x.dtype or C.dtype != x.dtype:
        B, C = B.float(), C.float()
    if dt.dtype != x.dtype:
        dt = dt.float()
    for t in (state, x, dt, A, B, D, dt_bias):
        if t is not None and t.dtype not in _lib.DTYPE_CODE:
            raise RuntimeError(f"selective_state_update: unsupported dtype {t.dtype}")
    out = torch.empty_like(x)

    p = _lib.MambaStepParams()
    p.batch, p.nheads, p.dim, p.dstate, p.ngroups = batch, nheads, dim, dstate, ngroups
    p.dt_softplus = int(bool(dt_softplus))
    p.state_rows = state_rows
    code = _lib.DTYPE_CODE
    p.state_dtype, p.x_dtype, p.dt_dtype = code[state.dtype], code[x.dtype], code[dt.dtype]
    p.A_dtype, p.bc_dtype = code[A.dtype], code[B.dtype]
    p.D_dtype = code[D.dtype] if D is not None else 0
    p.dt_bias_dtype = code[dt_bias.dtype] if dt_bias is not None else 0
    p.state, p.x, p.dt, p.A, p.B, p.C = (t.data_ptr() for t in (state, x, dt, A, B, C))
    p.D, p.z, p.dt_bias, p.out = _lib.ptr(D), _lib.ptr(z), _lib.ptr(dt_bias), out.data_ptr()
    p.state_batch_indices = _lib.ptr(state_batch_indices)
    p.state_bs, p.state_hs, p.state_ps, p.state_ns = state.stride()
    p.x_bs, p.x_hs, p.x_ps = x.stride()
    p.dt_bs, p.dt_hs, p.dt_ps = dt.stride()
    if dt_bias is not None:
        p.dt_bias_hs, p.dt_bias_ps = dt_bias.stride()
    p.A_hs, p.A_ps, p.A_ns = A.stride()
    p.B_bs, p.B_gs, p.B_ns = B.stride()
    p.C_bs, p.C_gs, p.C_ns = C.stride()
    if D is not None:
        p.D_hs, p.D_ps = D.stride()
    if z is not None:
        p.z_bs, p.z_hs, p.z_ps = z.stride()
    p.out_bs, p.out_hs, p.out_ps = out.stride()
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().ssm_state_update(p, _lib.current_stream(x.device)), "ssm_state_update")
    if not has_heads:
        out = out.squeeze(1)
    return out


def selective_state_update_ref(state, x, dt, A, B, C, D=None, z=None, dt_bias=None, dt_softplus=False):
    """One decode step from plain torch operators, in place on `state`, on whatever device the
    inputs live on (the role of the reference's selective_state_update_ref,
    selective_state_update.py:224).  A utility for users; no op of this package calls it.
    Shapes as selective_state_update, with or without the head dimension."""
    import torch.nn.functional as F
    has_heads = state.dim() > 3
    if not has_heads:
        state, x, dt, A, B, C = state[:, None], x[:, None], dt[:, None], A[None], B[:, None], C[:, None]
        D = D[None] if D is not None else None
        z = z[:, None] if z is not None else None
        dt_bias = dt_bias[None] if dt_bias is not None else None
    nheads, ngroups = state.shape[1], B.shape[1]
    step = dt.float() + (dt_bias.float() if dt_bias is not None else 0.0)
    if dt_softplus:
        step = F.softplus(step)
    Bh = B.float().repeat_interleave(nheads // ngroups, dim=1)       # (batch, nheads, dstate)
    Ch = C.float().repeat_interleave(nheads // ngroups, dim=1)
    decay = torch.exp(step[..., None] * A.float())                  # (batch, nheads, dim, dstate)
    new_state = state.float() * decay + (step * x.float())[..., None] * Bh[:, :, None, :]
    state.copy_(new_state)
    out = (new_state * Ch[:, :, None, :]).sum(-1)
    if D is not None:
        out = out + x.float() * D.float()
    if z is not None:
        out = out * F.silu(z.float())
    out = out.to(x.dtype)
    return out if has_heads else out.squeeze(1)
