"""Backward passes of the two differentiable stage-level functions, chunk_state and chunk_scan
(reference ChunkStateFn.backward, ssd_chunk_state.py:1060-1078, and ChunkScanFn.backward,
ssd_chunk_scan.py:1786-1825), composed from the library's backward stage entry points.

The library cuts the backward pass differently from the reference (dx of the carried-state path and of the
in-chunk path in one kernel; the dB / dC state products in one family), so each function below runs the
stages it needs with the other path's operand set to zero:
  chunk_state:  ssd_bwd_dBC_state (forward states = 0: no dC term), ssd_bwd_dx (C = 0 and C B^T = 0: no in-chunk term)
  chunk_scan:   ssd_bwd_dz, ssd_bwd_dstates (-> dprev_states), then with dstates = 0: ssd_bwd_dBC_state,
                ssd_bwd_dx, ssd_bwd_dcb, ssd_bmm_chunk_bwd
"""
import math

import torch

from mamba_amd import _lib
from mamba_amd.ops.triton import _ssd_stage as st


def _common(p, x, B, C, dt, dA_cumsum):
    p.x, p.B, p.C = x.data_ptr(), B.data_ptr(), C.data_ptr()
    p.x_bs, p.x_ls, p.x_hs = x.stride(0), x.stride(1), x.stride(2)
    p.B_bs, p.B_ls, p.B_gs = B.stride(0), B.stride(1), B.stride(2)
    p.C_bs, p.C_ls, p.C_gs = C.stride(0), C.stride(1), C.stride(2)
    p.dt_out, p.dA_cumsum = dt.data_ptr(), dA_cumsum.data_ptr()


def _rows(t):
    return t if t.stride(-1) == 1 else t.contiguous()


def chunk_state_bwd(B, x, dt, dA_cumsum, dstates):
    """Gradients of chunk_state(B, x, dt, dA_cumsum) for the upstream gradient dstates
    (batch, nchunks, nheads, headdim, dstate): (dB, dx, ddt, ddA_cumsum) in the shapes and dtypes of the inputs
    (ddt, ddA_cumsum fp32)."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, Q = dt.shape
    ngroups, dstate = B.shape[2], B.shape[3]
    assert nchunks == math.ceil(seqlen / Q)
    _lib.require_gpu(B, x, dt, dA_cumsum, dstates)
    dev, f32 = x.device, dict(device=x.device, dtype=torch.float32)
    xr, Br = _rows(x), _rows(B.to(x.dtype))
    dtf, daf = st.f32c(dt), st.f32c(dA_cumsum)
    zeros_states = torch.zeros(batch, nchunks, nheads, headdim, dstate, device=dev, dtype=st.carried_dtype(x.dtype))
    zeros_cb = torch.zeros(batch, nchunks, ngroups, Q, Q, **f32)
    acc = torch.zeros(2 * batch * nheads * nchunks * Q + 2 * batch * seqlen * ngroups * dstate, **f32)
    nrow, nbc = batch * nheads * nchunks * Q, batch * seqlen * ngroups * dstate
    ddA, ddt_out = acc[:nrow], acc[nrow:2 * nrow]
    dB32, dC32 = acc[2 * nrow:2 * nrow + nbc], acc[2 * nrow + nbc:]
    dx = torch.empty(batch, seqlen, nheads, headdim, device=dev, dtype=x.dtype)
    p, _keep = st.stage_params(dev, batch=batch, seqlen=seqlen, nheads=nheads, headdim=headdim, dstate=dstate,
                               ngroups=ngroups, chunk_size=Q, dtype=x.dtype, backward=True)
    Czero = torch.zeros_like(Br)  # C = 0: the dx stage forms C B^T itself on some shapes (kept alive to the end)
    _common(p, xr, Br, Czero, dtf, daf)
    p.dout = xr.data_ptr()  # stands in for g: it only meets the zero C B^T and the zero states
    p.dout_bs, p.dout_ls, p.dout_hs = xr.stride(0), xr.stride(1), xr.stride(2)
    p.CB = zeros_cb.data_ptr()
    _kept = (st.set_carried(p, "states", zeros_states, x.dtype), st.set_carried(p, "dstates", dstates, x.dtype))
    p.ddA_cumsum, p.ddt_out, p.dB32, p.dC32 = ddA.data_ptr(), ddt_out.data_ptr(), dB32.data_ptr(), dC32.data_ptr()
    p.dx = dx.data_ptr()
    p.dx_bs, p.dx_ls, p.dx_hs = dx.stride(0), dx.stride(1), dx.stride(2)
    st.run("ssd_bwd_dBC_state", p, dev)
    st.run("ssd_bwd_dx", p, dev)
    shape = (batch, nheads, nchunks, Q)
    return (dB32.view(batch, seqlen, ngroups, dstate).to(B.dtype), dx, ddt_out.view(shape).to(dt.dtype),
            ddA.view(shape).to(dA_cumsum.dtype))


def chunk_scan_bwd(B, C, x, dt, dA_cumsum, prev_states, D, z, y, dout):
    """Gradients of chunk_scan(B, C, x, dt, dA_cumsum, prev_states, D, z) for the upstream gradient dout; y is the
    forward output before the gate (z given) or the output itself.  Returns
    (dB, dC, dx, ddt, ddA_cumsum, dprev_states, dD, dz)."""
    from mamba_amd.ops.triton.ssd_bmm import _bmm_chunk_fwd
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, Q = dt.shape
    ngroups, dstate = B.shape[2], B.shape[3]
    _lib.require_gpu(B, C, x, dt, dA_cumsum, prev_states, D, z, y, dout)
    dev, f32 = x.device, dict(device=x.device, dtype=torch.float32)
    xr, Br, Cr = _rows(x), _rows(B.to(x.dtype)), _rows(C.to(x.dtype))
    zr = _rows(z.to(x.dtype)) if z is not None else None
    dor, yr = _rows(dout.to(x.dtype)), _rows(y.to(x.dtype))
    dtf, daf = st.f32c(dt), st.f32c(dA_cumsum)
    Df = st.f32c(D) if D is not None else None
    CB = _bmm_chunk_fwd(Cr, Br, Q, causal=True, output_dtype=torch.float32)
    nrow, nbc, ncb = batch * nheads * nchunks * Q, batch * seqlen * ngroups * dstate, batch * nchunks * ngroups * Q * Q
    nD = Df.numel() if Df is not None else 0
    acc = torch.zeros(2 * nrow + 2 * nbc + ncb + nD, **f32)
    ddA, ddt_out = acc[:nrow], acc[nrow:2 * nrow]
    dB32, dC32 = acc[2 * nrow:2 * nrow + nbc], acc[2 * nrow + nbc:2 * nrow + 2 * nbc]
    dCB = acc[2 * nrow + 2 * nbc:2 * nrow + 2 * nbc + ncb]
    dD = acc[2 * nrow + 2 * nbc + ncb:] if nD else None
    dprev = torch.empty(batch, nchunks, nheads, headdim, dstate, device=dev, dtype=st.carried_dtype(x.dtype))
    zeros_states = torch.zeros_like(dprev)
    dx = torch.empty(batch, seqlen, nheads, headdim, device=dev, dtype=x.dtype)
    dz = torch.empty_like(dx) if zr is not None else None
    gbuf = torch.empty_like(dx) if zr is not None else None
    p, _keep = st.stage_params(dev, batch=batch, seqlen=seqlen, nheads=nheads, headdim=headdim, dstate=dstate,
                               ngroups=ngroups, chunk_size=Q, dtype=x.dtype, backward=True)
    _common(p, xr, Br, Cr, dtf, daf)
    p.z, p.D = _lib.ptr(zr), _lib.ptr(Df)
    p.D_has_hdim = int(Df is not None and Df.dim() == 2)
    if zr is not None:
        p.z_bs, p.z_ls, p.z_hs = zr.stride(0), zr.stride(1), zr.stride(2)
        p.out_x = yr.data_ptr()
    else:
        p.out = yr.data_ptr()
    p.out_bs, p.out_ls, p.out_hs = yr.stride(0), yr.stride(1), yr.stride(2)
    p.dout = dor.data_ptr()
    p.dout_bs, p.dout_ls, p.dout_hs = dor.stride(0), dor.stride(1), dor.stride(2)
    p.CB = CB.data_ptr()
    _Hc = st.set_carried(p, "states", prev_states, x.dtype)
    p.ddA_cumsum, p.ddt_out, p.dB32, p.dC32, p.dCB = (t.data_ptr() for t in (ddA, ddt_out, dB32, dC32, dCB))
    p.dD = _lib.ptr(dD)
    p.dx, p.dz, p.gbuf = dx.data_ptr(), _lib.ptr(dz), _lib.ptr(gbuf)
    p.dx_bs, p.dx_ls, p.dx_hs = dx.stride(0), dx.stride(1), dx.stride(2)
    st.set_carried(p, "dstates", dprev, x.dtype)
    st.run("ssd_bwd_dz", p, dev)
    st.run("ssd_bwd_dstates", p, dev)          # the direct gradient of the state entering each chunk
    st.set_carried(p, "dstates", zeros_states, x.dtype)  # no chunk-state path in this function
    for stage in ("ssd_bwd_dBC_state", "ssd_bwd_dx", "ssd_bwd_dcb", "ssd_bmm_chunk_bwd"):
        st.run(stage, p, dev)
    shape = (batch, nheads, nchunks, Q)
    return (dB32.view(batch, seqlen, ngroups, dstate).to(B.dtype), dC32.view(batch, seqlen, ngroups, dstate).to(C.dtype),
            dx, ddt_out.view(shape).to(dt.dtype), ddA.view(shape).to(dA_cumsum.dtype), dprev.to(prev_states.dtype),
            (dD.view(D.shape).to(D.dtype) if D is not None else None), dz)
