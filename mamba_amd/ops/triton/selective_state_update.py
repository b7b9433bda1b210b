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
    ext = _lib.torch_ext()
    if ext is not None:
        # the same checks and launch in C++ (a few us of host time instead of ~15); it declines (None)
        # whatever needs a conversion or an error message, which the code below then handles
        out = ext.selective_state_update(state, x, dt, A, B, C, D, z, dt_bias, bool(dt_softplus), state_batch_indices)
        if out is not None:
            return out
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


# (device index, stream, size) -> zeroed int32 counters of mamba2_decode_step (every call leaves them zero).  One buffer per
# stream: calls on one stream run one after the other, calls on two streams may overlap and must not share counters.
_SYNC = {}

E_UNSUPPORTED = -2
FUSE_MAX_BATCH = 16  # largest batch for which mamba2_decode_step picks the fused kernel by itself


def mamba2_decode_step(ssm_state, conv_state, xBC, dt, A, conv_weight, conv_bias=None, D=None, z=None, dt_bias=None,
                       ngroups=1, activation="silu", dt_softplus=True, fuse=None):
    """One generated token of a Mamba-2 mixer core: the two calls of the reference's step()
    (mamba_ssm/modules/mamba2.py:298-336)

        xBC = causal_conv1d_update(xBC, conv_state, conv_weight, conv_bias, activation)
        x, B, C = split(xBC, [nheads * headdim, ngroups * dstate, ngroups * dstate])
        y = selective_state_update(ssm_state, x, dt, A, B, C, D, z, dt_bias, dt_softplus)

    as ONE kernel launch where the library serves the form (per-head dt / A / dt_bias / D, conv state of at most
    4 positions, no state indices), otherwise as those two calls.  Both give the same bits.
        ssm_state: (batch, nheads, headdim, dstate), updated in place
        conv_state: (batch, conv_dim, state_len), updated in place; conv_dim = nheads * headdim + 2 * ngroups * dstate
        xBC: (batch, conv_dim); dt: (batch, nheads); A, dt_bias, D: (nheads,); z: (batch, nheads, headdim)
        conv_weight: (conv_dim, width); conv_bias: (conv_dim,)
        fuse: None = one launch where served, False = always the two calls, True = one launch or an error
    The fused launch keeps a small zeroed counter buffer per (device, stream, size), allocated on the first such call:
    to capture `fuse=True` in a HIP graph, make one eager call on the capturing stream first.
    Returns y: (batch, nheads, headdim) in xBC's dtype."""
    from mamba_amd.ops.causal_conv1d import causal_conv1d_update
    _, nheads, headdim, dstate = ssm_state.shape
    batch = xBC.shape[0]
    conv_dim = nheads * headdim + 2 * ngroups * dstate
    if tuple(xBC.shape) != (batch, conv_dim):
        raise RuntimeError(f"mamba2_decode_step: xBC must be (batch, {conv_dim})")
    if ssm_state.shape[0] < batch:
        raise RuntimeError("mamba2_decode_step: ssm_state has fewer rows than the batch")
    if conv_state.dim() != 3 or conv_state.shape[0] < batch or conv_state.shape[1] != conv_dim:
        raise RuntimeError("mamba2_decode_step: conv_state must be (rows >= batch, conv_dim, state_len)")
    if tuple(dt.shape) != (batch, nheads) or tuple(A.shape) != (nheads,):
        raise RuntimeError("mamba2_decode_step: dt must be (batch, nheads) and A (nheads,)")
    _lib.require_gpu(ssm_state, conv_state, xBC, dt, A, conv_weight, conv_bias, D, z, dt_bias)

    def two_calls():
        xc = causal_conv1d_update(xBC, conv_state, conv_weight, conv_bias, activation)
        x, B, C = torch.split(xc, [nheads * headdim, ngroups * dstate, ngroups * dstate], dim=-1)
        ex = lambda t: None if t is None else t[:, None].expand(nheads, headdim)
        return selective_state_update(
            ssm_state, x.reshape(batch, nheads, headdim), dt[:, :, None].expand(batch, nheads, headdim),
            A[:, None, None].expand(nheads, headdim, dstate), B.reshape(batch, ngroups, dstate),
            C.reshape(batch, ngroups, dstate), D=ex(D), z=z, dt_bias=ex(dt_bias), dt_softplus=dt_softplus)

    width, state_len = conv_weight.shape[1], conv_state.shape[2]
    code = _lib.DTYPE_CODE
    fusable = (activation in (None, "silu", "swish") and xBC.dtype in code and conv_state.dtype == xBC.dtype
               and ssm_state.dtype in code and 2 <= width <= 4 and width - 1 <= state_len <= 4 and dstate % 4 == 0 and dstate >= 16
               and xBC.stride(1) == 1 and ssm_state.stride(3) == 1 and (z is None or z.dtype == xBC.dtype))
    explicit = fuse is True
    if fuse is None:
        # Measured (80 heads x 64, 128 states, bf16 filter, one MI355X), per token: replayed from a captured graph
        # the two launches take 8.7 us at batch 1 and the fused kernel 9.2 us (13.6 against 16.2 us at batch 8: its
        # ordered hand-over of the shared B / C conv state costs more than the second launch).  Called eagerly the
        # fused kernel saves one host call: 17.6 against 37.9 us through the Python + ctypes host side, but nothing
        # once the C++ host side (mamba_amd/_torch_ext.so) is there: 15.4 against 15.0 us.  So it is picked only for
        # eager calls at small batch without that extension.
        fuse = (fusable and batch <= FUSE_MAX_BATCH and _lib.torch_ext() is None
                and not torch.cuda.is_current_stream_capturing())
        if not fuse:
            return two_calls()
    if fuse is False:
        return two_calls()
    if not fusable:
        raise RuntimeError("mamba2_decode_step: this form is not served by the fused kernel")
    A32 = A.float()
    D32 = D.float() if D is not None else None
    dtb32 = dt_bias.float() if dt_bias is not None else None
    if dt.dtype != xBC.dtype:
        dt = dt.float()
    # the filter is read in fp32, bf16 or fp16 as it is (weight and bias in one dtype)
    w32, b32 = conv_weight.detach(), conv_bias.detach() if conv_bias is not None else None
    if w32.dtype not in code or (b32 is not None and b32.dtype != w32.dtype):
        w32, b32 = w32.float(), b32.float() if b32 is not None else None
    w32, b32 = w32.contiguous(), b32.contiguous() if b32 is not None else None
    out = torch.empty(batch, nheads, headdim, dtype=xBC.dtype, device=xBC.device)
    q = _lib.MambaDecodeStepParams()
    p = q.ssm
    p.batch, p.nheads, p.dim, p.dstate, p.ngroups = batch, nheads, headdim, dstate, ngroups
    nsync = int(_lib.load().mamba2_decode_step_sync_ints(q))
    if nsync <= 0:
        _lib.check(nsync or -1, "mamba2_decode_step_sync_ints")
    key = (xBC.device.index, _lib.current_stream(xBC.device), nsync)
    sync = _SYNC.get(key)
    if sync is None:
        sync = _SYNC[key] = torch.zeros(nsync, dtype=torch.int32, device=xBC.device)
    p.dt_softplus, p.state_rows = int(bool(dt_softplus)), ssm_state.shape[0]
    p.state_dtype, p.x_dtype, p.dt_dtype, p.bc_dtype = code[ssm_state.dtype], code[xBC.dtype], code[dt.dtype], code[xBC.dtype]
    p.A_dtype = code[A32.dtype]
    p.D_dtype = code[D32.dtype] if D32 is not None else 0
    p.dt_bias_dtype = code[dtb32.dtype] if dtb32 is not None else 0
    p.state, p.dt, p.A, p.out = ssm_state.data_ptr(), dt.data_ptr(), A32.data_ptr(), out.data_ptr()
    p.D, p.z, p.dt_bias = _lib.ptr(D32), _lib.ptr(z), _lib.ptr(dtb32)
    p.state_bs, p.state_hs, p.state_ps, p.state_ns = ssm_state.stride()
    p.dt_bs, p.dt_hs = dt.stride()
    p.A_hs = A32.stride(0)
    if dtb32 is not None:
        p.dt_bias_hs = dtb32.stride(0)
    if D32 is not None:
        p.D_hs = D32.stride(0)
    if z is not None:
        p.z_bs, p.z_hs, p.z_ps = z.stride()
    p.out_bs, p.out_hs, p.out_ps = out.stride()
    q.conv_dim, q.width, q.state_len = conv_dim, width, state_len
    q.conv_weight_dtype = code[w32.dtype]
    q.silu, q.conv_state_rows = int(activation in ("silu", "swish")), conv_state.shape[0]
    q.xBC, q.conv_state, q.conv_weight, q.conv_bias = xBC.data_ptr(), conv_state.data_ptr(), w32.data_ptr(), _lib.ptr(b32)
    q.sync = sync.data_ptr()
    q.xBC_bs = xBC.stride(0)
    q.cs_bs, q.cs_cs, q.cs_ls = conv_state.stride()
    with torch.cuda.device(xBC.device):
        rc = _lib.load().mamba2_decode_step(q, _lib.current_stream(xBC.device))
    if rc == E_UNSUPPORTED and not explicit:
        return two_calls()
    _lib.check(rc, "mamba2_decode_step")
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
