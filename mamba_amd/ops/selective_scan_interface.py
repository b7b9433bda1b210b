"""Mamba-1 selective scan: drop-in for mamba_ssm.ops.selective_scan_interface.

Same names, argument meaning and error behaviour as the reference module
(mamba_ssm/ops/selective_scan_interface.py:34 SelectiveScanFn, :118
selective_scan_fn, :196 MambaInnerFn, :386 mamba_inner_fn).  The compute is
done by the HIP kernels of libmamba_gfx950.so through its C ABI; the functions
`selective_scan_fwd` / `selective_scan_bwd` below take the place of the
reference's pybind module `selective_scan_cuda`
(csrc/selective_scan/selective_scan.cpp:494-497).
"""
import math

import torch
import torch.nn.functional as F
from einops import rearrange

from mamba_amd import _lib
from mamba_amd.ops.causal_conv1d import causal_conv1d_bwd, causal_conv1d_fwd
from mamba_amd.utils.determinism import fixed_point_scale, use_deterministic_mode

_FLOAT_TYPES = (torch.float32, torch.bfloat16, torch.float16)


def scan_tile(complex_A=False):
    """Positions per checkpoint tile of the scan (MAMBA_Q_SCAN_TILE / MAMBA_Q_SCAN_TILE_COMPLEX)."""
    return _lib.load().mamba_hip_query(5 if complex_A else 1)


def _check_inputs(u, delta, A, B, C, D, z, delta_bias):
    """Argument checks of selective_scan.cpp:233-303, before any launch."""
    _lib.require_gpu(u, delta, A, B, C, D, z, delta_bias)
    if u.dtype not in _FLOAT_TYPES:
        raise RuntimeError(f"selective_scan: unsupported input dtype {u.dtype}")
    is_complex = A.is_complex()
    if A.dtype not in (torch.float32, torch.complex64):
        raise RuntimeError("selective_scan: A must be float32 or complex64")
    if u.dim() != 3:
        raise RuntimeError("selective_scan: u must be (batch, dim, seqlen)")
    batch, dim, seqlen = u.shape
    dstate = A.shape[1]
    if dstate > _lib.load().mamba_hip_query(2):
        raise RuntimeError("selective_scan only supports state dimension <= 256")
    if delta.dtype != u.dtype:
        raise RuntimeError("selective_scan: u and delta must share one dtype")
    for name, t in (("u", u), ("delta", delta), ("z", z)):
        if t is not None and t.stride(-1) != 1:
            raise RuntimeError(f"selective_scan: {name} must have stride 1 in the last dimension")
    # B / C: (batch, ngroups, dstate, seqlen) in u's dtype, or an input-independent (dim, dstate)
    # matrix in A's dtype (selective_scan.cpp:254-259, :268-277)
    ngroups = 1
    for name, t in (("B", B), ("C", C)):
        if t.dim() == 4:
            ngroups = t.shape[1]
    # with a complex A the matrices are complex64 and the per-position operands carry (re, im)
    # pairs along a last axis of length 2 * seqlen (selective_scan.cpp:258-259, :268-277)
    for name, t in (("B", B), ("C", C)):
        if t.dim() == 2:
            if t.dtype != A.dtype or tuple(t.shape) != (dim, dstate) or not t.is_contiguous():
                raise RuntimeError(f"selective_scan: input-independent {name} must be contiguous (dim, dstate) of A's dtype")
        elif t.dim() == 4:
            if t.dtype != u.dtype:
                raise RuntimeError(f"selective_scan: {name} must have u's dtype")
            if t.stride(-1) != 1:
                raise RuntimeError(f"selective_scan: {name} must have stride 1 in the last dimension")
            if tuple(t.shape) != (batch, ngroups, dstate, seqlen * (2 if is_complex else 1)):
                raise RuntimeError("selective_scan: B/C must be (batch, ngroups, dstate, seqlen), "
                                   "or (..., 2 * seqlen) with a complex A")
        else:
            raise RuntimeError(f"selective_scan: {name} must be (batch, ngroups, dstate, seqlen) or (dim, dstate)")
    if tuple(delta.shape) != (batch, dim, seqlen):
        raise RuntimeError("selective_scan: delta shape mismatch")
    if tuple(A.shape) != (dim, dstate):
        raise RuntimeError("selective_scan: A shape mismatch")
    if dim % ngroups != 0:
        raise RuntimeError("selective_scan: dim must be divisible by ngroups")
    if D is not None and (D.dtype != torch.float32 or tuple(D.shape) != (dim,) or D.stride(-1) != 1):
        raise RuntimeError("selective_scan: D must be contiguous float32 of shape (dim,)")
    if delta_bias is not None and (delta_bias.dtype != torch.float32 or tuple(delta_bias.shape) != (dim,)
                                   or delta_bias.stride(-1) != 1):
        raise RuntimeError("selective_scan: delta_bias must be contiguous float32 of shape (dim,)")
    if z is not None and (z.dtype != u.dtype or tuple(z.shape) != (batch, dim, seqlen)):
        raise RuntimeError("selective_scan: z must match u in dtype and shape")
    return batch, dim, seqlen, dstate, ngroups


def _fill_common(p, u, delta, A, B, C, D, z, delta_bias, delta_softplus, ckpt, dims):
    batch, dim, seqlen, dstate, ngroups = dims
    p.batch, p.dim, p.seqlen, p.dstate, p.ngroups = batch, dim, seqlen, dstate, ngroups
    p.dtype = _lib.DTYPE_CODE[u.dtype]
    p.delta_softplus = int(bool(delta_softplus))
    p.a_complex = int(A.is_complex())
    p.u, p.delta, p.A, p.B, p.C = u.data_ptr(), delta.data_ptr(), A.data_ptr(), B.data_ptr(), C.data_ptr()
    p.D, p.z, p.delta_bias = _lib.ptr(D), _lib.ptr(z), _lib.ptr(delta_bias)
    p.ckpt = ckpt.data_ptr()
    p.u_bs, p.u_ds = u.stride(0), u.stride(1)
    p.delta_bs, p.delta_ds = delta.stride(0), delta.stride(1)
    if z is not None:
        p.z_bs, p.z_ds = z.stride(0), z.stride(1)
    p.bc_const = (1 if B.dim() == 2 else 0) | (2 if C.dim() == 2 else 0)
    if B.dim() == 4:
        p.B_bs, p.B_gs, p.B_ns = B.stride(0), B.stride(1), B.stride(2)
    if C.dim() == 4:
        p.C_bs, p.C_gs, p.C_ns = C.stride(0), C.stride(1), C.stride(2)


def selective_scan_fwd(u, delta, A, B, C, D=None, z=None, delta_bias=None, delta_softplus=False):
    """Counterpart of selective_scan_cuda.fwd (selective_scan.cpp:226).

    Returns (out, ckpt): `out` is the gated output y*silu(z) when z is given, else y, in u's dtype;
    `ckpt` is (batch, dim, ntiles, dstate) fp32, the state after each tile of `scan_tile()` positions
    (ckpt[:, :, -1] is the last state).  The ungated y is not stored: the backward pass re-computes it.
    """
    ext = _lib.torch_ext()
    if ext is not None and not A.is_complex():
        # the same checks, allocations and launch in C++ (csrc/torch_ext.cpp); None = a case for the code below
        r = ext.scan_fwd(u, delta, A, B, C, D, z, delta_bias, bool(delta_softplus))
        if r is not None:
            return r
    dims = _check_inputs(u, delta, A, B, C, D, z, delta_bias)
    batch, dim, seqlen, dstate, _ = dims
    A = A.contiguous()
    tile = scan_tile(A.is_complex())
    ntiles = (seqlen + tile - 1) // tile
    out = torch.empty_like(delta)
    ckpt = torch.empty((batch, dim, ntiles, dstate) + ((2,) if A.is_complex() else ()), device=u.device,
                       dtype=torch.float32)
    p = _lib.MambaScanParams()
    _fill_common(p, u, delta, A, B, C, D, z, delta_bias, delta_softplus, ckpt, dims)
    p.out = out.data_ptr()
    p.out_bs, p.out_ds = out.stride(0), out.stride(1)
    with torch.cuda.device(u.device):
        _lib.check(_lib.load().mamba1_scan_fwd(p, _lib.current_stream(u.device)), "mamba1_scan_fwd")
    return out, ckpt


class ScanBwdBuffers:
    """Outputs and fp32 workspaces of one backward launch (all caller-owned).  `nparts` is
    mamba1_scan_bwd_nparts for the launch's sizes."""

    def __init__(self, u, delta, B, z, dims, dz=None, recompute_out_z=False, C=None, complex_A=False, nparts=1):
        batch, dim, seqlen, dstate, ngroups = dims
        dev = u.device
        self.du = torch.empty_like(u)
        self.ddelta = torch.empty_like(delta)
        # per operand: (batch, ngroups, nparts, dstate, seqlen) partial sums, one per workgroup, which the
        # call adds up into dB / dC in the operand's dtype; or (batch, dim, dstate) per-batch partials
        # when the operand is an input-independent matrix; with a complex A every entry is a (re, im) pair
        two = 2 if complex_A else 1
        self.dB32, self.dB = self._operand(B, batch, dim, ngroups, nparts, dstate, seqlen, two, dev)
        self.dC32, self.dC = self._operand(C, batch, dim, ngroups, nparts, dstate, seqlen, two, dev)
        self.dA_part = torch.empty(batch, dim, dstate * two, device=dev, dtype=torch.float32)
        self.dD_part = torch.empty(batch, dim, device=dev, dtype=torch.float32)
        self.dbias_part = torch.empty(batch, dim, device=dev, dtype=torch.float32)
        self.dz = self.out_z = None
        if z is not None:
            self.dz = dz if dz is not None else torch.empty_like(z)
            if recompute_out_z:
                self.out_z = torch.empty_like(u)

    @staticmethod
    def _operand(t, batch, dim, ngroups, nparts, dstate, seqlen, two, dev):
        if t is not None and t.dim() == 2:
            return torch.empty(batch, dim, dstate * two, device=dev, dtype=torch.float32), None
        part = torch.empty(batch, ngroups, nparts, dstate, seqlen * two, device=dev, dtype=torch.float32)
        return part, torch.empty(batch, ngroups, dstate, seqlen * two, device=dev, dtype=t.dtype)


def scan_bwd_launch(u, delta, A, B, C, D, z, delta_bias, dout, ckpt, delta_softplus, dims, dz=None,
                    recompute_out_z=False, bufs=None):
    """One call of the C ABI's mamba1_scan_bwd on the current stream; returns its buffers (allocated
    here unless the ScanBwdBuffers of an earlier call with the same sizes are passed in)."""
    p = _lib.MambaScanParams()
    _fill_common(p, u, delta, A, B, C, D, z, delta_bias, delta_softplus, ckpt, dims)
    lib = _lib.load()
    if bufs is None:
        with torch.cuda.device(u.device):
            nparts = lib.mamba1_scan_bwd_nparts(p)
        if nparts <= 0:
            _lib.check(nparts or -1, "mamba1_scan_bwd_nparts")
        bufs = ScanBwdBuffers(u, delta, B, z, dims, dz, recompute_out_z, C=C, complex_A=A.is_complex(), nparts=nparts)
    dz, out_z = bufs.dz, bufs.out_z
    p.dout, p.du, p.ddelta = dout.data_ptr(), bufs.du.data_ptr(), bufs.ddelta.data_ptr()
    p.dz, p.out_z = _lib.ptr(dz), _lib.ptr(out_z)
    p.dB32, p.dC32 = bufs.dB32.data_ptr(), bufs.dC32.data_ptr()
    p.dB, p.dC = _lib.ptr(bufs.dB), _lib.ptr(bufs.dC)
    p.dA_part, p.dD_part = bufs.dA_part.data_ptr(), bufs.dD_part.data_ptr()
    p.ddelta_bias_part = bufs.dbias_part.data_ptr()
    keep = None
    if A.is_complex() and use_deterministic_mode():
        # the complex kernels add every channel's dB / dC terms into one sum: as 64-bit integers of fixed-point terms
        # the sum does not depend on the order of the adds (a real A's backward pass has no such sums)
        scale = fixed_point_scale(dout)
        shadows = [torch.zeros_like(t, dtype=torch.int64) if o.dim() == 4 else None
                   for t, o in ((bufs.dB32, B), (bufs.dC32, C))]
        p.det_scale, p.det_dB, p.det_dC = scale.data_ptr(), _lib.ptr(shadows[0]), _lib.ptr(shadows[1])
        keep = (scale, shadows)
    p.dout_bs, p.dout_ds = dout.stride(0), dout.stride(1)
    p.du_bs, p.du_ds = bufs.du.stride(0), bufs.du.stride(1)
    p.ddelta_bs, p.ddelta_ds = bufs.ddelta.stride(0), bufs.ddelta.stride(1)
    if dz is not None:
        p.dz_bs, p.dz_ds = dz.stride(0), dz.stride(1)
    if out_z is not None:
        p.outz_bs, p.outz_ds = out_z.stride(0), out_z.stride(1)
    with torch.cuda.device(u.device):
        _lib.check(lib.mamba1_scan_bwd(p, _lib.current_stream(u.device)), "mamba1_scan_bwd")
    del keep  # (stream-ordered allocator: the buffers stay valid for the launches already queued)
    return bufs


def selective_scan_bwd(u, delta, A, B, C, D, z, delta_bias, dout, ckpt, dz=None, delta_softplus=False,
                       recompute_out_z=False):
    """Counterpart of selective_scan_cuda.bwd (selective_scan.cpp:338).

    `dz` may be a caller-owned strided view (last stride 1) that receives the gate gradient,
    as MambaInnerFn passes it (selective_scan_interface.py:333-338).
    Returns (du, ddelta, dA, dB, dC, dD, ddelta_bias, dz, out_z).  No float atomics are involved: the
    same inputs give the same bits every time.
    """
    ext = _lib.torch_ext()
    if ext is not None and not A.is_complex():
        r = ext.scan_bwd(u, delta, A, B, C, D, z, delta_bias, dout, ckpt, dz, bool(delta_softplus), bool(recompute_out_z))
        if r is not None:
            return tuple(r)
    dims = _check_inputs(u, delta, A, B, C, D, z, delta_bias)
    batch, dim, seqlen, dstate, ngroups = dims
    _lib.require_gpu(dout, ckpt, dz)
    if dout.dtype != u.dtype or tuple(dout.shape) != (batch, dim, seqlen) or dout.stride(-1) != 1:
        raise RuntimeError("selective_scan: dout must match u in dtype/shape with stride 1 in the last dimension")
    if z is not None and dz is not None and (dz.dtype != u.dtype or tuple(dz.shape) != (batch, dim, seqlen)
                                             or dz.stride(-1) != 1):
        raise RuntimeError("selective_scan: dz must match z in dtype/shape with stride 1 in the last dimension")
    A = A.contiguous()
    cplx = A.is_complex()
    tile = scan_tile(cplx)
    want = (batch, dim, (seqlen + tile - 1) // tile, dstate) + ((2,) if cplx else ())
    if ckpt.dtype != torch.float32 or tuple(ckpt.shape) != want or not ckpt.is_contiguous():
        raise RuntimeError(f"selective_scan: ckpt must be the contiguous fp32 {want} tensor of the forward call")
    bufs = scan_bwd_launch(u, delta, A, B, C, D, z, delta_bias, dout, ckpt, delta_softplus, dims, dz, recompute_out_z)
    as_A = (lambda t: torch.view_as_complex(t.reshape(dim, dstate, 2))) if cplx else (lambda t: t)
    dA = as_A(bufs.dA_part.sum(0))
    dD = bufs.dD_part.sum(0) if D is not None else None
    ddelta_bias = bufs.dbias_part.sum(0) if delta_bias is not None else None
    dB = as_A(bufs.dB32.sum(0)) if B.dim() == 2 else bufs.dB
    dC = as_A(bufs.dC32.sum(0)) if C.dim() == 2 else bufs.dC
    return (bufs.du, bufs.ddelta, dA, dB, dC, dD, ddelta_bias, bufs.dz, bufs.out_z)


class SelectiveScanFn(torch.autograd.Function):
    """autograd wrapper, as the reference's SelectiveScanFn (selective_scan_interface.py:34-93)."""

    @staticmethod
    def forward(ctx, u, delta, A, B, C, D=None, z=None, delta_bias=None, delta_softplus=False,
                return_last_state=False):
        if u.stride(-1) != 1:
            u = u.contiguous()
        if delta.stride(-1) != 1:
            delta = delta.contiguous()
        if D is not None:
            D = D.contiguous()
        if B.stride(-1) != 1 or B.dim() == 2:
            B = B.contiguous()
        if C.stride(-1) != 1 or C.dim() == 2:
            C = C.contiguous()
        if z is not None and z.stride(-1) != 1:
            z = z.contiguous()
        ctx.squeeze_B = ctx.squeeze_C = False
        if B.dim() == 3:
            B = rearrange(B, "b dstate l -> b 1 dstate l")
            ctx.squeeze_B = True
        if C.dim() == 3:
            C = rearrange(C, "b dstate l -> b 1 dstate l")
            ctx.squeeze_C = True
        out, ckpt = selective_scan_fwd(u, delta, A, B, C, D, z, delta_bias, delta_softplus)
        ctx.delta_softplus = delta_softplus
        ctx.has_z = z is not None
        ctx.has_D = D is not None
        ctx.has_bias = delta_bias is not None
        last_state = ckpt[:, :, -1]  # (batch, dim, dstate)
        if A.is_complex():
            last_state = torch.view_as_complex(last_state)
        ctx.save_for_backward(u, delta, A, B, C, D, z, delta_bias, ckpt)
        return out if not return_last_state else (out, last_state)

    @staticmethod
    def backward(ctx, dout, *args):
        u, delta, A, B, C, D, z, delta_bias, ckpt = ctx.saved_tensors
        if dout.stride(-1) != 1:
            dout = dout.contiguous()
        du, ddelta, dA, dB, dC, dD, ddelta_bias, dz, _ = selective_scan_bwd(
            u, delta, A, B, C, D, z, delta_bias, dout, ckpt, None, ctx.delta_softplus, False)
        dB = dB.squeeze(1) if ctx.squeeze_B else dB
        dC = dC.squeeze(1) if ctx.squeeze_C else dC
        return (du, ddelta, dA, dB, dC, dD, dz, ddelta_bias, None, None)


def selective_scan_fn(u, delta, A, B, C, D=None, z=None, delta_bias=None, delta_softplus=False,
                      return_last_state=False):
    """if return_last_state is True, returns (out, last_state)
    last_state has shape (batch, dim, dstate). The gradient of the last state is not
    considered in the backward pass (as in the reference, selective_scan_interface.py:118-124).
    """
    # (batches beyond the 65535 rows one launch's grid can index are served in slices inside the C entry points)
    return SelectiveScanFn.apply(u, delta, A, B, C, D, z, delta_bias, delta_softplus, return_last_state)


def selective_scan_ref(u, delta, A, B, C, D=None, z=None, delta_bias=None, delta_softplus=False,
                       return_last_state=False):
    """Plain-PyTorch evaluation of the same recurrence on whatever device the inputs live on (the
    role of the reference's selective_scan_ref, selective_scan_interface.py:127).  It is a utility
    for users and is not used by any op of this package."""
    dtype_in = u.dtype
    u, delta = u.float(), delta.float()
    if delta_bias is not None:
        delta = delta + delta_bias[..., None].float()
    if delta_softplus:
        delta = F.softplus(delta)
    dim, L = A.shape[0], u.shape[2]
    cplx = A.is_complex()

    def per_channel(t):  # -> (batch or 1, dim, dstate, L), complex when A is
        if t.dim() == 2:
            return (t if cplx else t.float())[None, :, :, None].expand(1, dim, A.shape[1], L)
        t = t.float() if t.dim() == 4 else t.float()[:, None]
        if cplx:  # (re, im) pairs interleaved along the last axis
            t = torch.view_as_complex(t.reshape(*t.shape[:-1], L, 2).contiguous())
        return t.repeat_interleave(dim // t.shape[1], dim=1)

    Bf, Cf = per_channel(B), per_channel(C)
    state = torch.zeros(u.shape[0], dim, A.shape[1], device=u.device, dtype=A.dtype)
    ys = []
    for t in range(L):
        step = delta[:, :, t, None]
        state = torch.exp(step * A) * state + step * u[:, :, t, None] * Bf[..., t]
        yt = (state * Cf[..., t]).sum(-1)
        ys.append(2 * yt.real if cplx else yt)
    y = torch.stack(ys, dim=2)
    if D is not None:
        y = y + u * D[None, :, None]
    if z is not None:
        y = y * F.silu(z.float())
    y = y.to(dtype_in)
    return y if not return_last_state else (y, state)


# --------------------------------------------------------------------------- mamba_inner_fn
def _causal_conv1d_silu(x, weight, bias):
    """Depthwise causal convolution (left padding width-1) followed by SiLU: the arithmetic of the
    un-vendored causal_conv1d package as the reference itself spells it when that package is missing
    (mamba_ssm/modules/mamba_simple.py:168-169).  x: (b, d, L), weight: (d, w)."""
    L = x.shape[-1]
    y = F.conv1d(x, weight.unsqueeze(1), bias, padding=weight.shape[-1] - 1, groups=weight.shape[0])[..., :L]
    return F.silu(y)


def rms_norm_forward(x, weight, bias, eps=1e-6, is_rms_norm=True):
    """RMSNorm (or LayerNorm) of the rows of x, (rows, dim), on the HIP norm kernel; no autograd
    (selective_scan_interface.py:98-115)."""
    from mamba_amd.ops.triton.layer_norm import _layer_norm_fwd
    if x.stride(-1) != 1:
        x = x.contiguous()
    return _layer_norm_fwd(x, weight.contiguous(), bias.contiguous() if bias is not None else None, eps,
                           is_rms_norm=is_rms_norm)[0]


def _rms_norm(x, weight, eps):
    return rms_norm_forward(x, weight, None, eps)


def _norm_over_state(t, weight, eps, L):
    # (b, 1, n, l) -> rows of n -> back, as selective_scan_interface.py:263-270
    rows = rearrange(t, "b 1 dstate l -> (b l) dstate", l=L).contiguous()
    return rearrange(_rms_norm(rows, weight, eps), "(b l) dstate -> b 1 dstate l", l=L).contiguous()


def _channel_major(x):
    """An empty (batch, dim, seqlen) tensor like x whose memory order is (dim, batch, seqlen)."""
    b, d, L = x.shape
    return torch.empty(d, b, L, dtype=x.dtype, device=x.device).permute(1, 0, 2)


def _as_matrix(t):
    """(batch, dim, seqlen) -> (dim, batch * seqlen): a view when t is channel-major, else a copy."""
    return t.permute(1, 0, 2).reshape(t.shape[1], -1)


def _from_matrix(m, L):
    """(dim, batch * seqlen) -> the (batch, dim, seqlen) view of the same memory."""
    return m.view(m.shape[0], -1, L).permute(1, 0, 2)


class MambaInnerFn(torch.autograd.Function):
    """conv1d+SiLU -> x_proj -> dt_proj -> selective scan -> out_proj with the reference's layout
    choreography and recompute-in-backward (selective_scan_interface.py:196-383).  The scan runs on
    the HIP kernels; the convolution and the projections are torch operators."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, xz, conv1d_weight, conv1d_bias, x_proj_weight, delta_proj_weight, out_proj_weight,
                out_proj_bias, A, B=None, C=None, D=None, delta_bias=None, B_proj_bias=None, C_proj_bias=None,
                delta_softplus=True, checkpoint_lvl=1, b_rms_weight=None, c_rms_weight=None, dt_rms_weight=None,
                b_c_dt_rms_eps=1e-6):
        assert checkpoint_lvl in [0, 1]
        L = xz.shape[-1]
        delta_rank = delta_proj_weight.shape[1]
        # x_proj emits (re, im) pairs per state when A is complex (selective_scan_interface.py:207)
        d_state = A.shape[-1] * (1 if not A.is_complex() else 2)
        pack = ("(b l) dstate -> b 1 dstate l" if not A.is_complex()
                else "(b l) (dstate two) -> b 1 dstate (l two)")
        pack_kw = dict(l=L) if not A.is_complex() else dict(l=L, two=2)
        if torch.is_autocast_enabled():
            ac = torch.get_autocast_dtype("cuda")
            x_proj_weight, delta_proj_weight = x_proj_weight.to(ac), delta_proj_weight.to(ac)
            out_proj_weight = out_proj_weight.to(ac)
            out_proj_bias = out_proj_bias.to(ac) if out_proj_bias is not None else None
        if xz.stride(-1) != 1:
            xz = xz.contiguous()
        conv1d_weight = rearrange(conv1d_weight, "d 1 w -> d w")
        x, z = xz.chunk(2, dim=1)
        conv1d_bias = conv1d_bias.contiguous() if conv1d_bias is not None else None
        # Every (batch, dim, seqlen) intermediate lives in memory as (dim, batch, seqlen): the kernels take
        # batch and channel strides as they come, and the projections then see (dim, batch * seqlen)
        # matrices and their transposes without a copy.
        conv1d_out = causal_conv1d_fwd(x, conv1d_weight, conv1d_bias, activation="silu", out=_channel_major(x))
        x_dbl = F.linear(_as_matrix(conv1d_out).t(), x_proj_weight)        # (b l) x (rank + 2 n)
        delta = _from_matrix(delta_proj_weight @ x_dbl[:, :delta_rank].t(), L)
        ctx.is_variable_B, ctx.is_variable_C = B is None, C is None
        ctx.B_proj_bias_is_None, ctx.C_proj_bias_is_None = B_proj_bias is None, C_proj_bias is None
        if B is None:
            B = x_dbl[:, delta_rank:delta_rank + d_state]
            if B_proj_bias is not None:
                B = B + B_proj_bias.to(dtype=B.dtype)
            B = rearrange(B, pack, **pack_kw).contiguous()
        elif B.stride(-1) != 1:
            B = B.contiguous()
        if C is None:
            C = x_dbl[:, -d_state:]
            if C_proj_bias is not None:
                C = C + C_proj_bias.to(dtype=C.dtype)
            C = rearrange(C, pack, **pack_kw).contiguous()
        elif C.stride(-1) != 1:
            C = C.contiguous()
        if D is not None:
            D = D.contiguous()
        if b_rms_weight is not None:
            B = _norm_over_state(B, b_rms_weight, b_c_dt_rms_eps, L)
        if c_rms_weight is not None:
            C = _norm_over_state(C, c_rms_weight, b_c_dt_rms_eps, L)
        if dt_rms_weight is not None:
            delta = rearrange(_rms_norm(rearrange(delta, "b d l -> (b l) d").contiguous(), dt_rms_weight,
                                        b_c_dt_rms_eps), "(b l) d -> b d l", l=L).contiguous()
        out_z, ckpt = selective_scan_fwd(conv1d_out, delta, A, B, C, D, z, delta_bias, delta_softplus)
        ctx.delta_softplus = delta_softplus
        ctx.out_proj_bias_is_None = out_proj_bias is None
        ctx.checkpoint_lvl = checkpoint_lvl
        ctx.dt_rms_weight, ctx.rms_eps = dt_rms_weight, b_c_dt_rms_eps
        if checkpoint_lvl >= 1:  # conv1d_out and delta are recomputed in the backward pass
            conv1d_out, delta = None, None
        ctx.save_for_backward(xz, conv1d_weight, conv1d_bias, x_dbl, x_proj_weight, delta_proj_weight,
                              out_proj_weight, conv1d_out, delta, A, B, C, D, delta_bias, ckpt)
        out = F.linear(_as_matrix(out_z).t(), out_proj_weight, out_proj_bias)   # out_z has delta's layout
        return out.view(xz.shape[0], L, -1)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dout):
        (xz, conv1d_weight, conv1d_bias, x_dbl, x_proj_weight, delta_proj_weight, out_proj_weight, conv1d_out,
         delta, A, B, C, D, delta_bias, ckpt) = ctx.saved_tensors
        L = xz.shape[-1]
        delta_rank = delta_proj_weight.shape[1]
        d_state = A.shape[-1] * (1 if not A.is_complex() else 2)
        unpack = ("b 1 dstate l -> (b l) dstate" if not A.is_complex()
                  else "b 1 dstate (l two) -> (b l) (dstate two)")
        unpack_kw = dict() if not A.is_complex() else dict(two=2)
        x, z = xz.chunk(2, dim=1)
        if dout.stride(-1) != 1:
            dout = dout.contiguous()
        if ctx.checkpoint_lvl == 1:  # the convolution output and delta are re-computed
            conv1d_out = causal_conv1d_fwd(x, conv1d_weight, conv1d_bias, activation="silu", out=_channel_major(x))
            delta = _from_matrix(delta_proj_weight @ x_dbl[:, :delta_rank].t(), L)
            if ctx.dt_rms_weight is not None:
                delta = rearrange(_rms_norm(rearrange(delta, "b d l -> (b l) d").contiguous(), ctx.dt_rms_weight,
                                            ctx.rms_eps), "(b l) d -> b d l", l=L).contiguous()
        dxz = torch.empty_like(xz)
        dx, dz = dxz.chunk(2, dim=1)
        dout = dout.reshape(-1, dout.shape[-1]).t()                                  # e x (b l)
        dout_y = _from_matrix(out_proj_weight.t() @ dout, L)
        # du, ddelta and out_z come back in the layouts of u and delta
        dconv1d_out, ddelta, dA, dB, dC, dD, ddelta_bias, dz, out_z = selective_scan_bwd(
            conv1d_out, delta, A, B, C, D, z, delta_bias, dout_y, ckpt, dz, ctx.delta_softplus, True)
        dout_proj_weight = dout @ _as_matrix(out_z).t()
        dout_proj_bias = dout.sum(dim=1) if not ctx.out_proj_bias_is_None else None
        dx_dbl = torch.empty_like(x_dbl)
        dB_proj_bias = dC_proj_bias = None
        if ctx.is_variable_B:
            dB = rearrange(dB, unpack, **unpack_kw).contiguous()
            dB_proj_bias = dB.sum(0) if not ctx.B_proj_bias_is_None else None
            dx_dbl[:, delta_rank:delta_rank + d_state] = dB
            dB = None
        if ctx.is_variable_C:
            dC = rearrange(dC, unpack, **unpack_kw).contiguous()
            dC_proj_bias = dC.sum(0) if not ctx.C_proj_bias_is_None else None
            dx_dbl[:, -d_state:] = dC
            dC = None
        ddelta = _as_matrix(ddelta)
        ddelta_proj_weight = ddelta @ x_dbl[:, :delta_rank]
        dx_dbl[:, :delta_rank] = ddelta.t() @ delta_proj_weight
        dx_proj_weight = dx_dbl.t() @ _as_matrix(conv1d_out).t()
        dconv1d_mat = _as_matrix(dconv1d_out)            # the scan's own du buffer: add the x_proj path in place
        dconv1d_out = _from_matrix(dconv1d_mat.addmm_(x_proj_weight.t(), dx_dbl.t()), L)
        # the convolution's backward kernel re-computes the pre-activation from x and writes dx in place
        _, dconv1d_weight, dconv1d_bias = causal_conv1d_bwd(x, conv1d_weight, conv1d_bias, dconv1d_out.to(x.dtype),
                                                            activation="silu", dx=dx)
        dconv1d_weight = rearrange(dconv1d_weight, "d w -> d 1 w")
        return (dxz, dconv1d_weight, dconv1d_bias, dx_proj_weight, ddelta_proj_weight, dout_proj_weight,
                dout_proj_bias, dA, dB, dC, dD, ddelta_bias if delta_bias is not None else None,
                dB_proj_bias, dC_proj_bias, None, None, None, None, None, None)


def mamba_inner_fn(xz, conv1d_weight, conv1d_bias, x_proj_weight, delta_proj_weight, out_proj_weight, out_proj_bias,
                   A, B=None, C=None, D=None, delta_bias=None, B_proj_bias=None, C_proj_bias=None,
                   delta_softplus=True, checkpoint_lvl=1, b_rms_weight=None, c_rms_weight=None, dt_rms_weight=None,
                   b_c_dt_rms_eps=1e-6):
    return MambaInnerFn.apply(xz, conv1d_weight, conv1d_bias, x_proj_weight, delta_proj_weight, out_proj_weight,
                              out_proj_bias, A, B, C, D, delta_bias, B_proj_bias, C_proj_bias, delta_softplus,
                              checkpoint_lvl, b_rms_weight, c_rms_weight, dt_rms_weight, b_c_dt_rms_eps)


def mamba_inner_ref(xz, conv1d_weight, conv1d_bias, x_proj_weight, delta_proj_weight, out_proj_weight,
                    out_proj_bias, A, B=None, C=None, D=None, delta_bias=None, B_proj_bias=None, C_proj_bias=None,
                    delta_softplus=True):
    """The same block from plain torch operators and selective_scan_ref (the role of the reference's
    mamba_inner_ref, selective_scan_interface.py:397)."""
    L = xz.shape[-1]
    delta_rank = delta_proj_weight.shape[1]
    d_state = A.shape[-1] * (1 if not A.is_complex() else 2)
    pack = "(b l) dstate -> b dstate l" if not A.is_complex() else "(b l) (dstate two) -> b dstate (l two)"
    pack_kw = dict(l=L) if not A.is_complex() else dict(l=L, two=2)
    x, z = xz.chunk(2, dim=1)
    x = _causal_conv1d_silu(x, rearrange(conv1d_weight, "d 1 w -> d w"), conv1d_bias)
    x_dbl = F.linear(rearrange(x, "b d l -> (b l) d"), x_proj_weight)
    delta = rearrange(delta_proj_weight @ x_dbl[:, :delta_rank].t(), "d (b l) -> b d l", l=L)
    if B is None:
        B = x_dbl[:, delta_rank:delta_rank + d_state]
        if B_proj_bias is not None:
            B = B + B_proj_bias.to(dtype=B.dtype)
        B = rearrange(B, pack, **pack_kw).contiguous()
    if C is None:
        C = x_dbl[:, -d_state:]
        if C_proj_bias is not None:
            C = C + C_proj_bias.to(dtype=C.dtype)
        C = rearrange(C, pack, **pack_kw).contiguous()
    y = selective_scan_ref(x, delta, A, B, C, D, z=z, delta_bias=delta_bias, delta_softplus=True)
    return F.linear(rearrange(y, "b d l -> b l d"), out_proj_weight, out_proj_bias)
