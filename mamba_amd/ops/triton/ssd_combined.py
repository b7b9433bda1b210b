"""Mamba-2 SSD chunked scan: drop-in for mamba_ssm.ops.triton.ssd_combined.

Same entry point, argument meaning, return arity and error behaviour as the reference
(mamba_ssm/ops/triton/ssd_combined.py:628 mamba_chunk_scan_combined, :596
MambaChunkScanCombinedFn, :343/:397 the forward/backward orchestration).  The Triton kernels
are replaced by the HIP kernels behind the C ABI's ssd_* entry points.  The module path keeps
the reference's `triton` package name so that imports stay source compatible.
"""
import math

import torch

from mamba_amd import _lib
from mamba_amd.ops.causal_conv1d import causal_conv1d_fn
from mamba_amd.ops.triton.layernorm_gated import rmsnorm_fn
from mamba_amd.utils.determinism import fixed_point_scale, use_deterministic_mode


def _fill_fwd(p, x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx, dt_softplus, dt_limit, ws):
    batch, seqlen, nheads, headdim = x.shape
    _, _, ngroups, dstate = B.shape
    p.batch, p.seqlen, p.nheads, p.headdim, p.dstate, p.ngroups = batch, seqlen, nheads, headdim, dstate, ngroups
    p.chunk_size, p.nchunks = chunk_size, ws["nchunks"]
    p.dtype, p.dt_dtype = _lib.DTYPE_CODE[x.dtype], _lib.DTYPE_CODE[dt.dtype]
    p.dt_softplus = int(bool(dt_softplus))
    p.D_has_hdim = int(D is not None and D.dim() == 2)
    p.dt_min, p.dt_max = float(dt_limit[0]), float(min(dt_limit[1], 3.0e38))
    p.x, p.dt, p.A, p.B, p.C = x.data_ptr(), dt.data_ptr(), A.data_ptr(), B.data_ptr(), C.data_ptr()
    p.D, p.z, p.dt_bias = _lib.ptr(D), _lib.ptr(z), _lib.ptr(dt_bias)
    p.initial_states, p.seq_idx = _lib.ptr(initial_states), _lib.ptr(seq_idx)
    p.dt_out, p.dA_cumsum = ws["dt_out"].data_ptr(), ws["dA_cumsum"].data_ptr()
    p.states, p.final_states, p.CB = _lib.ptr(ws["states"]), ws["final_states"].data_ptr(), ws["CB"].data_ptr()
    p.states_lp = _lib.ptr(ws["states_lp"])
    p.x_bs, p.x_ls, p.x_hs = x.stride(0), x.stride(1), x.stride(2)
    if z is not None:
        p.z_bs, p.z_ls, p.z_hs = z.stride(0), z.stride(1), z.stride(2)
    p.B_bs, p.B_ls, p.B_gs = B.stride(0), B.stride(1), B.stride(2)
    p.C_bs, p.C_ls, p.C_gs = C.stride(0), C.stride(1), C.stride(2)
    p.dt_bs, p.dt_ls, p.dt_hs = dt.stride()


def _prepare(x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx):
    """Shape checks and layout fixes of ssd_combined.py:344-369, then dtype normalisation."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, seqlen, nheads)
    assert A.shape == (nheads,)
    assert C.shape == B.shape
    if z is not None:
        assert z.shape == x.shape
    if D is not None:
        assert D.shape == (nheads, headdim) or D.shape == (nheads,)
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, headdim, dstate)
    _lib.require_gpu(x, dt, A, B, C, D, z, dt_bias, initial_states, seq_idx)
    if x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"mamba_chunk_scan_combined: unsupported dtype {x.dtype}")
    lim = _lib.load().mamba_hip_query
    if chunk_size > 256 or dstate > lim(3) or headdim > lim(4):
        raise RuntimeError("mamba_chunk_scan_combined: chunk_size, dstate and headdim are limited to 256")
    if B.stride(-1) != 1:
        B = B.contiguous()
    if C.stride(-1) != 1:
        C = C.contiguous()
    if x.stride(-1) != 1:
        x = x.contiguous()
    if z is not None and z.stride(-1) != 1:
        z = z.contiguous()
    B, C = B.to(x.dtype), C.to(x.dtype)
    z = z.to(x.dtype) if z is not None else None
    if dt.dtype not in _lib.DTYPE_CODE:
        dt = dt.float()
    A = A.float().contiguous()
    D = D.float().contiguous() if D is not None else None
    dt_bias = dt_bias.float().contiguous() if dt_bias is not None else None
    initial_states = initial_states.float().contiguous() if initial_states is not None else None
    if seq_idx is not None:
        seq_idx = seq_idx.to(torch.int32).contiguous()
    return x, dt, A, B, C, D, z, dt_bias, initial_states, seq_idx


def _workspace(x, B, chunk_size, forward_state=None):
    """Workspaces of the forward stages.  `states` (fp32) receives the chunks' own states and, for fp32 / fp16
    operands, in place the state entering each chunk; next to bf16 operands the entering states go to `states_lp`
    in bf16 instead (the dtype the reference hands them on in, ssd_combined.py:384-386).  `carried` names whichever
    of the two holds the entering states.  forward_state = (dt_out, dA_cumsum, carried) re-uses what a forward
    pass has filled; `states` is then only allocated when the stages that fill it are run again."""
    batch, seqlen, nheads, headdim = x.shape
    ngroups, dstate = B.shape[2], B.shape[3]
    nchunks = math.ceil(seqlen / chunk_size)
    f32 = dict(device=x.device, dtype=torch.float32)
    lp = x.dtype == torch.bfloat16
    shape = (batch, nchunks, nheads, headdim, dstate)
    if forward_state is not None:
        dt_out, dA_cumsum, carried = forward_state
        assert dt_out.shape == (batch, nheads, nchunks, chunk_size) and dA_cumsum.shape == dt_out.shape
        assert carried.shape == shape and carried.is_contiguous()
        assert carried.dtype == (torch.bfloat16 if lp else torch.float32)
        assert all(t.dtype == torch.float32 and t.is_contiguous() for t in (dt_out, dA_cumsum))
        states = None if lp else carried
        states_lp = carried if lp else None
    else:
        dt_out = torch.empty(batch, nheads, nchunks, chunk_size, **f32)
        dA_cumsum = torch.empty(batch, nheads, nchunks, chunk_size, **f32)
        states = torch.empty(shape, **f32)
        states_lp = torch.empty(shape, device=x.device, dtype=torch.bfloat16) if lp else None
    return dict(
        nchunks=nchunks,
        dt_out=dt_out,
        dA_cumsum=dA_cumsum,
        states=states,
        states_lp=states_lp,
        carried=states_lp if lp else states,
        final_states=torch.empty(batch, nheads, headdim, dstate, **f32),
        CB=torch.empty(batch, nchunks, ngroups, chunk_size, chunk_size, **f32),
    )


def _mamba_chunk_scan_combined_fwd(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, initial_states=None,
                                   seq_idx=None, cu_seqlens=None, dt_softplus=False, dt_limit=(0.0, float("inf")),
                                   state_dtype=None, want_out_x=True):
    """Counterpart of ssd_combined.py:343.  Returns (out, out_x, dt_out, dA_cumsum, states, final_states)
    where `states[:, c]` is the state entering chunk c (bf16 next to bf16 operands, else fp32) and out_x the output
    before the gate (None without z, and with want_out_x=False: only the backward pass reads it); with cu_seqlens a
    seventh element,
    varlen_states (nseq, nheads, headdim, dstate): the state at the end of every packed sequence
    (ssd_combined.py:390-394), in state_dtype, else C's dtype, as the reference returns it."""
    ext = _lib.torch_ext()
    if ext is not None and cu_seqlens is None:
        # the same checks, allocations and launch in C++ (csrc/torch_ext.cpp); None = a case for the code below
        r = ext.ssd_fwd(x, dt, A, B, C, int(chunk_size), D, z, dt_bias, initial_states, seq_idx, bool(dt_softplus),
                        float(dt_limit[0]), float(dt_limit[1]), bool(want_out_x))
        if r is not None:
            return tuple(r)
    state_out_dtype = state_dtype if state_dtype is not None else C.dtype
    x, dt, A, B, C, D, z, dt_bias, initial_states, seq_idx = _prepare(
        x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx)
    if cu_seqlens is not None:
        assert x.shape[0] == 1, "passing cu_seqlens to get the varlen states is only supported if batch dimension is 1"
        assert cu_seqlens.dim() == 1 and cu_seqlens.numel() >= 1
        _lib.require_gpu(cu_seqlens)
        cu_seqlens = cu_seqlens.to(torch.int32).contiguous()
    ws = _workspace(x, B, chunk_size)
    out = torch.empty_like(x, memory_format=torch.contiguous_format)
    out_x = torch.empty_like(out) if z is not None and want_out_x else None
    p = _lib.SsdParams()
    _fill_fwd(p, x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx, dt_softplus, dt_limit, ws)
    p.out, p.out_x = out.data_ptr(), _lib.ptr(out_x)
    p.out_bs, p.out_ls, p.out_hs = out.stride(0), out.stride(1), out.stride(2)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().ssd_combined_fwd(p, _lib.current_stream(x.device)), "ssd_combined_fwd")
        if cu_seqlens is not None:
            nseq = cu_seqlens.numel() - 1
            varlen = torch.empty(nseq, x.shape[2], x.shape[3], B.shape[3], device=x.device, dtype=torch.float32)
            _lib.check(_lib.load().ssd_chunk_state_varlen(p, cu_seqlens.data_ptr(), nseq, varlen.data_ptr(),
                                                          _lib.current_stream(x.device)), "ssd_chunk_state_varlen")
            return (out, out_x, ws["dt_out"], ws["dA_cumsum"], ws["carried"], ws["final_states"],
                    varlen.to(state_out_dtype))
    return out, out_x, ws["dt_out"], ws["dA_cumsum"], ws["carried"], ws["final_states"]


def _mamba_chunk_scan_combined_bwd(dout, x, dt, A, B, C, out, chunk_size, D=None, z=None, dt_bias=None,
                                   initial_states=None, dfinal_states=None, seq_idx=None, dt_softplus=False,
                                   dt_limit=(0.0, float("inf")), saved=None, dx=None, ddt=None, dB=None, dC=None):
    """Counterpart of ssd_combined.py:397.  `out` is the saved pre-gate output (out_x) when z is given,
    else the forward output.  `saved` = (dt_out, dA_cumsum, states) of the forward pass skips their
    re-computation (the reference always re-computes them, ssd_combined.py:441-448).  dx, ddt, dB, dC may
    be caller-owned views (slices of a wider gradient buffer, unit stride in the last dimension), as the
    reference's fused block function passes them (ssd_combined.py:934-944).
    Returns (dx, ddt, dA, dB, dC, dD, dz, ddt_bias, dinitial_states)."""
    ext = _lib.torch_ext()
    if (ext is not None and saved is not None and dx is None and ddt is None and dB is None and dC is None
            and not use_deterministic_mode()):
        r = ext.ssd_bwd(dout, x, dt, A, B, C, out, int(chunk_size), D, z, dt_bias, initial_states, dfinal_states, seq_idx,
                        bool(dt_softplus), float(dt_limit[0]), float(dt_limit[1]), saved[0], saved[1], saved[2])
        if r is not None:
            return tuple(r)
    in_dtypes = (A.dtype, D.dtype if D is not None else None, dt_bias.dtype if dt_bias is not None else None,
                 initial_states.dtype if initial_states is not None else None, B.dtype, C.dtype)
    D_shape = D.shape if D is not None else None
    x, dt, A, B, C, D, z, dt_bias, initial_states, seq_idx = _prepare(
        x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx)
    batch, seqlen, nheads, headdim = x.shape
    ngroups, dstate = B.shape[2], B.shape[3]
    _lib.require_gpu(dout, out, dfinal_states)
    if dout.stride(-1) != 1:
        dout = dout.contiguous()
    dout = dout.to(x.dtype)
    out = out.to(x.dtype)
    if out.stride(-1) != 1:
        out = out.contiguous()
    dev = x.device
    ws = _workspace(x, B, chunk_size, forward_state=saved)
    nchunks = ws["nchunks"]
    f32 = dict(device=dev, dtype=torch.float32)
    if dx is None:
        dx = torch.empty(batch, seqlen, nheads, headdim, device=dev, dtype=x.dtype)
    else:
        assert dx.shape == x.shape and dx.dtype == x.dtype and dx.stride(-1) == 1 and dx.is_cuda
    dz = torch.empty(batch, seqlen, nheads, headdim, device=dev, dtype=x.dtype) if z is not None else None
    gbuf = torch.empty_like(dz) if z is not None else None
    ddt_out_view = ddt
    ddt = torch.empty(batch, seqlen, nheads, device=dev, dtype=dt.dtype)
    # one zeroed arena for the small accumulators the kernels add into; the three large ones (dCB, dB32, dC32) are
    # cleared further down, and only where the library does not write them whole (ssd_bwd_overwrites)
    sizes = dict(dA=nheads, ddt_bias=nheads, dD=(D.numel() if D is not None else 0),
                 ddA_cumsum=batch * nheads * nchunks * chunk_size, ddt_out=batch * nheads * nchunks * chunk_size,
                 dCB=batch * nchunks * ngroups * chunk_size * chunk_size,
                 dB32=batch * seqlen * ngroups * dstate, dC32=batch * seqlen * ngroups * dstate)
    large = ("dCB", "dB32", "dC32")
    n_small = -(-sum(n for k, n in sizes.items() if k not in large) // 64) * 64  # the large ones start on 256 bytes
    arena = torch.empty(n_small + sum(sizes[k] for k in large), **f32)  # the small accumulators first
    acc, off = {}, 0
    for k in sizes:
        if k == large[0]:
            off = n_small
        acc[k] = arena[off:off + sizes[k]]
        off += sizes[k]
    lp = x.dtype == torch.bfloat16  # the carried states' gradients pass between the stages in bf16 too
    dstates = torch.empty(batch, nchunks, nheads, headdim, dstate, device=dev, dtype=torch.bfloat16 if lp else torch.float32)
    dinit = torch.empty(batch, nheads, headdim, dstate, **f32) if initial_states is not None else None
    dfinal = dfinal_states.float().contiguous() if dfinal_states is not None else None

    p = _lib.SsdParams()
    _fill_fwd(p, x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx, dt_softplus, dt_limit, ws)
    if z is not None:
        p.out_x = out.data_ptr()
    else:
        p.out = out.data_ptr()
    p.out_bs, p.out_ls, p.out_hs = out.stride(0), out.stride(1), out.stride(2)
    p.dout, p.dfinal_states = dout.data_ptr(), _lib.ptr(dfinal)
    p.dout_bs, p.dout_ls, p.dout_hs = dout.stride(0), dout.stride(1), dout.stride(2)
    p.dx, p.dz, p.ddt, p.gbuf = dx.data_ptr(), _lib.ptr(dz), ddt.data_ptr(), _lib.ptr(gbuf)
    p.dx_bs, p.dx_ls, p.dx_hs = dx.stride(0), dx.stride(1), dx.stride(2)
    p.dA, p.ddt_bias = acc["dA"].data_ptr(), acc["ddt_bias"].data_ptr()
    p.dD = acc["dD"].data_ptr() if D is not None else None
    p.dinitial_states = _lib.ptr(dinit)
    if lp:
        p.dstates_lp = dstates.data_ptr()
    else:
        p.dstates = dstates.data_ptr()
    p.ddA_cumsum, p.ddt_out, p.dCB = acc["ddA_cumsum"].data_ptr(), acc["ddt_out"].data_ptr(), acc["dCB"].data_ptr()
    p.dB32, p.dC32 = acc["dB32"].data_ptr(), acc["dC32"].data_ptr()
    # dB / dC in the operands' dtype are written by the call's last stage; a caller's own (strided) views are filled
    # from the fp32 sums afterwards instead
    dB_own = torch.empty(batch, seqlen, ngroups, dstate, device=dev, dtype=x.dtype) if dB is None and in_dtypes[4] == x.dtype else None
    dC_own = torch.empty(batch, seqlen, ngroups, dstate, device=dev, dtype=x.dtype) if dC is None and in_dtypes[5] == x.dtype else None
    p.dB, p.dC = _lib.ptr(dB_own), _lib.ptr(dC_own)
    if use_deterministic_mode():
        # integer shadows of the shared sums, laid out like the float arena, and the call's fixed-point scale
        shadow = torch.zeros(sum(sizes.values()), device=dev, dtype=torch.int64)
        det_scale = fixed_point_scale(dout, dfinal)
        p.det_scale = det_scale.data_ptr()
        off = 0
        for k, n in sizes.items():
            field = {"dB32": "det_dB", "dC32": "det_dC"}.get(k, "det_" + k)
            setattr(p, field, shadow[off:off + n].data_ptr() if n else None)
            off += n
    lib = _lib.load()
    with torch.cuda.device(dev):
        owned = lib.ssd_bwd_overwrites(p)  # which of the large sum buffers the kernels store rather than add into
        if owned == 0:
            arena.zero_()  # one fill
        else:
            arena[:n_small].zero_()
            if not owned & 1:
                acc["dCB"].zero_()
            if not owned & 2:
                arena[n_small + sizes["dCB"]:].zero_()  # dB32 and dC32 are neighbours
        stream = _lib.current_stream(dev)
        # forward workspaces: kept from the forward pass, or re-computed as the reference does
        # (ssd_combined.py:441-448); CB is re-computed (the fused forward never forms it) unless the library says
        # that its backward kernels do not read it (flag 4: the dCB stage then forms its tiles of C B^T itself)
        stages = () if saved is not None else ("ssd_chunk_cumsum_fwd", "ssd_chunk_state_fwd", "ssd_state_passing_fwd")
        if owned & 4:
            p.CB = None
        else:
            stages += ("ssd_bmm_chunk_fwd",)
        for stage in stages:
            _lib.check(getattr(lib, stage)(p, stream), stage)
        _lib.check(lib.ssd_combined_bwd(p, stream), "ssd_combined_bwd")
    dA = acc["dA"].to(in_dtypes[0])
    dD = acc["dD"].view(D_shape).to(in_dtypes[1]) if D is not None else None
    ddt_bias = acc["ddt_bias"].to(in_dtypes[2]) if dt_bias is not None else None
    dinit_out = dinit.to(in_dtypes[3]) if dinit is not None else None
    dB32 = acc["dB32"].view(batch, seqlen, ngroups, dstate)
    dC32 = acc["dC32"].view(batch, seqlen, ngroups, dstate)
    if dB_own is not None:
        dB = dB_own
    else:
        dB = dB32.to(in_dtypes[4]) if dB is None else dB.copy_(dB32)     # the copy is the cast
    if dC_own is not None:
        dC = dC_own
    else:
        dC = dC32.to(in_dtypes[5]) if dC is None else dC.copy_(dC32)
    if ddt_out_view is not None:
        ddt = ddt_out_view.copy_(ddt)
    return dx, ddt, dA, dB, dC, dD, dz, ddt_bias, dinit_out


# Keep the forward pass's fp32 workspaces for the backward pass (288 GB of HBM make the memory cheap;
# the re-computation costs ~7 % of a forward + backward step).  False restores the reference's behaviour.
KEEP_FORWARD_STATE = True


class MambaChunkScanCombinedFn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, initial_states=None, seq_idx=None,
                cu_seqlens=None, dt_softplus=False, dt_limit=(0.0, float("inf")), return_final_states=False,
                return_varlen_states=False, state_dtype=None):
        ctx.dt_dtype = dt.dtype
        if not return_varlen_states:
            cu_seqlens = None
        else:
            assert cu_seqlens is not None, "cu_seqlens must be provided if return_varlen_states is True"
        out, out_x, dt_out, dA_cumsum, states, final_states, *rest = _mamba_chunk_scan_combined_fwd(
            x, dt, A, B, C, chunk_size, D=D, z=z, dt_bias=dt_bias, initial_states=initial_states, seq_idx=seq_idx,
            cu_seqlens=cu_seqlens, dt_softplus=dt_softplus, dt_limit=dt_limit, state_dtype=state_dtype,
            want_out_x=any(ctx.needs_input_grad))  # no gradient asked for: the pre-gate copy is not written
        # with KEEP_FORWARD_STATE the fp32 dt, cumulative decay and chunk states of the forward pass
        # stay alive for the backward pass (batch*nchunks*nheads*headdim*dstate*4 bytes) instead of
        # being re-computed there as in the reference (ssd_combined.py:441-448)
        keep = (dt_out, states) if KEEP_FORWARD_STATE else ()
        ctx.kept = len(keep) > 0
        ctx.save_for_backward(out if z is None else out_x, x, dt, dA_cumsum, A, B, C, D, z, dt_bias, initial_states,
                              seq_idx, *keep)
        ctx.dt_softplus = dt_softplus
        ctx.chunk_size = chunk_size
        ctx.dt_limit = dt_limit
        ctx.return_final_states = return_final_states
        ctx.return_varlen_states = return_varlen_states
        if not return_varlen_states:
            return out if not return_final_states else (out, final_states)
        varlen_states = rest[0]
        return (out, varlen_states) if not return_final_states else (out, final_states, varlen_states)

    @staticmethod
    def backward(ctx, dout, *args):
        out, x, dt, dA_cumsum, A, B, C, D, z, dt_bias, initial_states, seq_idx, *kept = ctx.saved_tensors
        assert not ctx.return_varlen_states, "return_varlen_states is not supported in backward"
        dfinal_states = args[0] if ctx.return_final_states else None
        saved = (kept[0], dA_cumsum, kept[1]) if ctx.kept else None
        dx, ddt, dA, dB, dC, dD, dz, ddt_bias, dinitial_states = _mamba_chunk_scan_combined_bwd(
            dout, x, dt, A, B, C, out, ctx.chunk_size, D=D, z=z, dt_bias=dt_bias, initial_states=initial_states,
            dfinal_states=dfinal_states, seq_idx=seq_idx, dt_softplus=ctx.dt_softplus, dt_limit=ctx.dt_limit,
            saved=saved)
        return (dx, ddt, dA, dB, dC, None, dD, dz, ddt_bias, dinitial_states, None, None, None, None, None, None,
                None)


def mamba_chunk_scan_combined(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, initial_states=None,
                              seq_idx=None, cu_seqlens=None, dt_softplus=False, dt_limit=(0.0, float("inf")),
                              return_final_states=False, return_varlen_states=False, state_dtype=None):
    """
    Argument:
        x: (batch, seqlen, nheads, headdim)
        dt: (batch, seqlen, nheads)
        A: (nheads)
        B: (batch, seqlen, ngroups, dstate)
        C: (batch, seqlen, ngroups, dstate)
        chunk_size: int
        D: (nheads, headdim) or (nheads,)
        z: (batch, seqlen, nheads, headdim)
        dt_bias: (nheads,)
        initial_states: (batch, nheads, headdim, dstate)
        seq_idx: (batch, seqlen)
        cu_seqlens: (num_sequences + 1) or None, only used if return_varlen_states is True
        dt_softplus: Whether to apply softplus to dt
        state_dtype: accepted for compatibility; inter-chunk states are kept in fp32
    Return:
        out: (batch, seqlen, nheads, headdim) [, final_states (batch, nheads, headdim, dstate) fp32]
    """
    # (more than 65535 (batch, head) pairs are served in slices of batch rows inside the C entry points)
    return MambaChunkScanCombinedFn.apply(x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx,
                                          cu_seqlens, dt_softplus, dt_limit, return_final_states,
                                          return_varlen_states, state_dtype)


def mamba_chunk_scan(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False):
    """The stage-by-stage entry point of the reference (ssd_combined.py:651): same result as
    mamba_chunk_scan_combined with these arguments, and served by the same kernels here."""
    return mamba_chunk_scan_combined(x, dt, A, B, C, chunk_size, D=D, z=z, dt_bias=dt_bias, dt_softplus=dt_softplus)


def ssd_chunk_scan_combined_ref(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False):
    """The same operator from plain torch operators on whatever device the inputs live on (the role
    of the reference's ssd_chunk_scan_combined_ref, ssd_combined.py:687).  A utility for users; no op
    of this package calls it.  Evaluated as the per-position recurrence in fp32 (chunk_size does not
    change the result and is only accepted for signature compatibility)."""
    import torch.nn.functional as F
    batch, seqlen, nheads, headdim = x.shape
    ngroups = B.shape[2]
    step = dt.float() + (dt_bias.float() if dt_bias is not None else 0.0)
    if dt_softplus:
        step = F.softplus(step)
    decay = torch.exp(step * A.float())                                      # (batch, seqlen, nheads)
    Bh = B.float().repeat_interleave(nheads // ngroups, dim=2)
    Ch = C.float().repeat_interleave(nheads // ngroups, dim=2)
    xf = x.float()
    state = xf.new_zeros(batch, nheads, headdim, B.shape[3])
    ys = []
    for t in range(seqlen):
        state = state * decay[:, t, :, None, None] + (step[:, t, :, None] * xf[:, t])[..., None] * Bh[:, t, :, None, :]
        ys.append((state * Ch[:, t, :, None, :]).sum(-1))
    y = torch.stack(ys, dim=1)
    if D is not None:
        y = y + xf * (D.float()[..., None] if D.dim() == 1 else D.float())
    if z is not None:
        y = y * F.silu(z.float())
    return y.to(x.dtype)


def ssd_selective_scan(x, dt, A, B, C, D=None, z=None, dt_bias=None, dt_softplus=False,
                       dt_limit=(0.0, float("inf"))):
    """The SSD operator evaluated by the Mamba-1 selective scan kernels (ssd_combined.py:728): every
    (head, headdim) pair becomes a channel whose states all decay with the head's A.
    x, z: (batch, seqlen, nheads, headdim); dt: (batch, seqlen, nheads[, headdim]); A: (nheads) or
    (nheads * headdim, dstate); B, C: (batch, seqlen, ngroups, dstate); D: (nheads[, headdim])."""
    import torch.nn.functional as F
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    batch, seqlen, nheads, headdim = x.shape
    dstate = B.shape[3]
    chan = lambda t: t.reshape(batch, seqlen, nheads * headdim).transpose(1, 2)      # -> (b, h*p, l)
    dtc = dt if dt.dim() == 4 else dt[..., None].expand(batch, seqlen, nheads, headdim)
    u, delta = chan(x), chan(dtc)
    Af = (A.float()[:, None, None].expand(nheads, headdim, dstate).reshape(nheads * headdim, dstate)
          if A.dim() == 1 else A.float())
    Bc, Cc = B.permute(0, 2, 3, 1), C.permute(0, 2, 3, 1)                            # (b, g, n, l)
    Dc = None
    if D is not None:
        Dc = (D.reshape(-1) if D.dim() == 2 else D[:, None].expand(nheads, headdim).reshape(-1)).float().contiguous()
    zc = chan(z) if z is not None else None
    bias = None
    if dt_bias is not None:
        bias = (dt_bias if dt_bias.dim() == 2 else dt_bias[:, None].expand(nheads, headdim)).reshape(-1).float()
    if dt_limit != (0.0, float("inf")):
        if bias is not None:
            delta = delta + bias[:, None]
        if dt_softplus:
            delta = F.softplus(delta)
        delta = delta.clamp(min=dt_limit[0], max=dt_limit[1]).to(x.dtype)
        bias, dt_softplus = None, False
    out = selective_scan_fn(u.contiguous(), delta.to(x.dtype).contiguous(), Af.contiguous(), Bc.contiguous(),
                            Cc.contiguous(), D=Dc, z=zc.contiguous() if zc is not None else None,
                            delta_bias=bias.contiguous() if bias is not None else None,
                            delta_softplus=bool(dt_softplus))
    return out.transpose(1, 2).reshape(batch, seqlen, nheads, headdim)


def _causal_conv1d(xBC, weight, bias, activation, seq_idx=None):
    """Depthwise causal convolution over (batch, seqlen, channels) with optional SiLU: the arithmetic
    of the un-vendored causal_conv1d package as the reference spells it when the package is missing
    (mamba_ssm/modules/mamba2.py:230-234).  With seq_idx, taps that reach into another sequence of a
    packed batch contribute nothing."""
    import torch.nn.functional as F
    width = weight.shape[-1]
    if seq_idx is None:
        y = F.conv1d(xBC.transpose(1, 2), weight.unsqueeze(1), bias, padding=width - 1,
                     groups=weight.shape[0])[..., :xBC.shape[1]].transpose(1, 2)
    else:
        y = xBC * weight[:, width - 1]
        for k in range(1, width):
            shifted = F.pad(xBC, (0, 0, k, 0))[:, :xBC.shape[1]]
            same = F.pad(seq_idx, (k, 0), value=-1)[:, :xBC.shape[1]] == seq_idx
            y = y + torch.where(same[..., None], shifted, torch.zeros_like(shifted)) * weight[:, width - 1 - k]
        if bias is not None:
            y = y + bias
    return F.silu(y) if activation in ("silu", "swish") else y


def _gated_rms_norm(x, weight, z, eps, group_size, norm_before_gate):
    """RMSNorm over groups of `group_size` channels with the SiLU gate before or after it
    (mamba_ssm/ops/triton/layernorm_gated.py:18 with bias None), computed in fp32."""
    import torch.nn.functional as F
    dtype = x.dtype
    x, z = x.float(), z.float()
    if not norm_before_gate:
        x = x * F.silu(z)
    xg = x.reshape(*x.shape[:-1], x.shape[-1] // group_size, group_size)
    xg = xg * torch.rsqrt(xg.square().mean(dim=-1, keepdim=True) + eps)
    out = xg.reshape(x.shape) * weight.float()
    if norm_before_gate:
        out = out * F.silu(z)
    return out.to(dtype)


class MambaSplitConv1dScanCombinedFn(torch.autograd.Function):
    """The Mamba-2 block body as one autograd node (ssd_combined.py:822): the backward pass writes the
    gradients of z, xBC and dt straight into their slices of one dzxbcdt buffer (norm, convolution and
    scan kernels take the slices' strides), and the scan writes dx into its slice of the buffer the
    convolution's backward pass reads, so no concatenation is left."""

    @staticmethod
    def forward(ctx, zxbcdt, conv1d_weight, conv1d_bias, dt_bias, A, D, chunk_size, initial_states=None, seq_idx=None,
                dt_limit=(0.0, float("inf")), return_final_states=False, activation="silu", rmsnorm_weight=None,
                rmsnorm_eps=1e-6, outproj_weight=None, outproj_bias=None, headdim=None, ngroups=1,
                norm_before_gate=True, state_dtype=None):
        import torch.nn.functional as F
        from mamba_amd.ops.causal_conv1d import causal_conv1d_fwd
        from mamba_amd.ops.triton.layernorm_gated import _layer_norm_fwd
        assert activation in [None, "silu", "swish"]
        if D.dim() == 1:
            assert headdim is not None
            nheads, = D.shape
        else:
            nheads, headdim = D.shape
        batch, seqlen, _ = zxbcdt.shape
        dim = nheads * headdim
        assert nheads % ngroups == 0
        dstate = (conv1d_weight.shape[0] - dim) // ngroups // 2
        d_nonssm = (zxbcdt.shape[-1] - 2 * dim - 2 * ngroups * dstate - nheads) // 2
        assert d_nonssm >= 0
        assert zxbcdt.shape == (batch, seqlen, 2 * d_nonssm + 2 * dim + 2 * ngroups * dstate + nheads)
        assert dt_bias.shape == (nheads,) and A.shape == (nheads,)
        ctx.conv_w_3d = conv1d_weight.dim() == 3
        conv_w = conv1d_weight.squeeze(1) if ctx.conv_w_3d else conv1d_weight
        if zxbcdt.stride(-1) != 1:
            zxbcdt = zxbcdt.contiguous()
        zx0, z, xBC, dt = torch.split(zxbcdt, [2 * d_nonssm, dim, dim + 2 * ngroups * dstate, nheads], dim=-1)
        # the convolution reads the channel-contiguous slice as it lies and returns a dense (b, l, c) tensor
        xBC_conv = causal_conv1d_fwd(xBC.transpose(1, 2), conv_w, conv1d_bias, seq_idx=seq_idx,
                                     activation=activation).transpose(1, 2)
        x, B, C = torch.split(xBC_conv, [dim, ngroups * dstate, ngroups * dstate], dim=-1)
        x = x.reshape(batch, seqlen, nheads, headdim)
        B = B.reshape(batch, seqlen, ngroups, dstate)
        C = C.reshape(batch, seqlen, ngroups, dstate)
        z4 = z.reshape(batch, seqlen, nheads, headdim)
        gate_in_scan = rmsnorm_weight is None
        out, out_x, dt_out, dA_cumsum, states, final_states = _mamba_chunk_scan_combined_fwd(
            x, dt, A, B, C, chunk_size, D=D, z=z4 if gate_in_scan else None, dt_bias=dt_bias,
            initial_states=initial_states, seq_idx=seq_idx, dt_softplus=True, dt_limit=dt_limit, state_dtype=state_dtype)
        y = out.view(batch, seqlen, dim)
        rstd = None
        if not gate_in_scan:
            # reads z where it lies inside zxbcdt (unit channel stride, row stride of the whole projection)
            y, _, rstd = _layer_norm_fwd(out.view(batch * seqlen, dim), rmsnorm_weight, None, rmsnorm_eps,
                                         z=z.reshape(batch * seqlen, dim), group_size=dim // ngroups,
                                         norm_before_gate=norm_before_gate, is_rms_norm=True)
            y = y.view(batch, seqlen, dim)
        if d_nonssm > 0:
            gate, up = zx0.chunk(2, dim=-1)
            y = torch.cat([(F.silu(gate.float()) * up.float()).to(y.dtype), y], dim=-1)
        ctx.autocast = None
        if outproj_weight is not None:
            w, bias = outproj_weight, outproj_bias
            if torch.is_autocast_enabled():
                ctx.autocast = torch.get_autocast_dtype("cuda")
                y, w = y.to(ctx.autocast), w.to(ctx.autocast)
                bias = bias.to(ctx.autocast) if bias is not None else None
            res = F.linear(y, w, bias)
        else:
            assert outproj_bias is None
            res = y
        # the scan's backward pass wants its pre-gate output: out_x when the gate ran inside the scan
        ctx.save_for_backward(zxbcdt, conv_w, conv1d_bias, xBC_conv, out_x if gate_in_scan else out,
                              dt_out, dA_cumsum, states, A, D, dt_bias, initial_states, seq_idx, rmsnorm_weight, rstd,
                              outproj_weight, outproj_bias, y if outproj_weight is not None else None)
        ctx.dims = (batch, seqlen, nheads, headdim, ngroups, dstate, d_nonssm)
        ctx.chunk_size, ctx.dt_limit, ctx.activation = chunk_size, dt_limit, activation
        ctx.rmsnorm_eps, ctx.norm_before_gate = rmsnorm_eps, norm_before_gate
        ctx.return_final_states = return_final_states
        return res if not return_final_states else (res, final_states)

    @staticmethod
    def backward(ctx, dout, *args):
        import torch.nn.functional as F
        from mamba_amd.ops.causal_conv1d import causal_conv1d_bwd
        from mamba_amd.ops.triton.layernorm_gated import _layer_norm_bwd
        (zxbcdt, conv_w, conv_b, xBC_conv, scan_out, dt_out, dA_cumsum, states, A, D, dt_bias, initial_states, seq_idx,
         rmsnorm_weight, rstd, outproj_weight, outproj_bias, y_proj) = ctx.saved_tensors
        batch, seqlen, nheads, headdim, ngroups, dstate, d_nonssm = ctx.dims
        dim = nheads * headdim
        dfinal_states = args[0] if ctx.return_final_states else None
        gate_in_scan = rmsnorm_weight is None
        zx0, z, xBC, dt = torch.split(zxbcdt, [2 * d_nonssm, dim, dim + 2 * ngroups * dstate, nheads], dim=-1)
        dzxbcdt = torch.empty_like(zxbcdt)
        dzx0, dz, dxBC, ddt = torch.split(dzxbcdt, [2 * d_nonssm, dim, dim + 2 * ngroups * dstate, nheads], dim=-1)
        doutproj_weight = doutproj_bias = None
        if outproj_weight is not None:
            w = outproj_weight if ctx.autocast is None else outproj_weight.to(ctx.autocast)
            dout2 = dout.reshape(-1, dout.shape[-1]).to(w.dtype)
            dy_cat = (dout2 @ w).view(batch, seqlen, d_nonssm + dim)
            doutproj_weight = (dout2.t() @ y_proj.reshape(-1, d_nonssm + dim)).to(outproj_weight.dtype)
            doutproj_bias = dout2.sum(0).to(outproj_bias.dtype) if outproj_bias is not None else None
        else:
            dy_cat = dout
        if dy_cat.stride(-1) != 1:
            dy_cat = dy_cat.contiguous()
        dy_cat = dy_cat.to(zxbcdt.dtype)
        if d_nonssm > 0:  # SwiGLU of the part that bypasses the scan (k_activations.py:42)
            gate, up = (t.float() for t in zx0.chunk(2, dim=-1))
            d0 = dy_cat[..., :d_nonssm].float()
            sg = torch.sigmoid(gate)
            dzx0[..., :d_nonssm] = d0 * up * sg * (1 + gate * (1 - sg))
            dzx0[..., d_nonssm:] = d0 * gate * sg
        dy = dy_cat[..., d_nonssm:]
        drmsnorm_weight = None
        if not gate_in_scan:
            dy2, drmsnorm_weight, _, _ = _layer_norm_bwd(
                dy.reshape(batch * seqlen, dim), scan_out.view(batch * seqlen, dim), rmsnorm_weight, None,
                ctx.rmsnorm_eps, None, rstd, z=z.reshape(batch * seqlen, dim), group_size=dim // ngroups,
                norm_before_gate=ctx.norm_before_gate, is_rms_norm=True, dz=dz.view(batch * seqlen, dim))
            dy = dy2.view(batch, seqlen, dim)
        x, B, C = torch.split(xBC_conv, [dim, ngroups * dstate, ngroups * dstate], dim=-1)
        dxBC_conv = torch.empty_like(xBC_conv)
        dx, dB, dC = torch.split(dxBC_conv, [dim, ngroups * dstate, ngroups * dstate], dim=-1)
        _, _, dA, _, _, dD, dz_scan, ddt_bias, dinitial_states = _mamba_chunk_scan_combined_bwd(
            dy.reshape(batch, seqlen, nheads, headdim), x.reshape(batch, seqlen, nheads, headdim), dt, A,
            B.reshape(batch, seqlen, ngroups, dstate), C.reshape(batch, seqlen, ngroups, dstate), scan_out, ctx.chunk_size,
            D=D, z=z.reshape(batch, seqlen, nheads, headdim) if gate_in_scan else None, dt_bias=dt_bias,
            initial_states=initial_states, dfinal_states=dfinal_states, seq_idx=seq_idx, dt_softplus=True,
            dt_limit=ctx.dt_limit, saved=(dt_out, dA_cumsum, states),
            dx=dx.view(batch, seqlen, nheads, headdim), ddt=ddt, dB=dB.view(batch, seqlen, ngroups, dstate),
            dC=dC.view(batch, seqlen, ngroups, dstate))
        if gate_in_scan:
            dz.copy_(dz_scan.view(batch, seqlen, dim))
        # the convolution's backward kernel re-computes its pre-activation from xBC and writes into the xBC slice
        _, dconv_w, dconv_b = causal_conv1d_bwd(xBC.transpose(1, 2), conv_w, conv_b, dxBC_conv.transpose(1, 2),
                                                seq_idx=seq_idx, activation=ctx.activation, dx=dxBC.transpose(1, 2))
        if ctx.conv_w_3d:
            dconv_w = dconv_w.unsqueeze(1)
        return (dzxbcdt, dconv_w, dconv_b, ddt_bias, dA, dD, None, dinitial_states, None, None, None, None,
                drmsnorm_weight, None, doutproj_weight, doutproj_bias, None, None, None, None)


def mamba_split_conv1d_scan_combined(zxbcdt, conv1d_weight, conv1d_bias, dt_bias, A, D, chunk_size,
                                     initial_states=None, seq_idx=None, dt_limit=(0.0, float("inf")),
                                     return_final_states=False, activation="silu", rmsnorm_weight=None,
                                     rmsnorm_eps=1e-6, outproj_weight=None, outproj_bias=None, headdim=None,
                                     ngroups=1, norm_before_gate=True, state_dtype=None):
    """The Mamba-2 block body after in_proj (ssd_combined.py:983): split, causal conv1d + SiLU on xBC, the
    chunked scan and the gate or gated RMSNorm on the HIP kernels, SwiGLU of the non-SSM part and out_proj
    (torch GEMM), as one autograd node.
        zxbcdt: (batch, seqlen, 2 * d_nonssm + 2 * dim + 2 * ngroups * dstate + nheads), dim = nheads * headdim
        conv1d_weight: (dim + 2 * ngroups * dstate, width); conv1d_bias: (dim + 2 * ngroups * dstate,)
        dt_bias, A: (nheads,); D: (nheads, headdim) or (nheads,) (then headdim must be given)
        rmsnorm_weight: (dim,); outproj_weight: (out_dim, d_nonssm + dim); outproj_bias: (out_dim,)
        norm_before_gate: True computes RMSNorm(y) * silu(z), False RMSNorm(y * silu(z))
    Returns out, or (out, final_states) with return_final_states."""
    return MambaSplitConv1dScanCombinedFn.apply(zxbcdt, conv1d_weight, conv1d_bias, dt_bias, A, D, chunk_size,
                                                initial_states, seq_idx, dt_limit, return_final_states, activation,
                                                rmsnorm_weight, rmsnorm_eps, outproj_weight, outproj_bias, headdim,
                                                ngroups, norm_before_gate, state_dtype)


def mamba_conv1d_scan_ref(xBC, conv1d_weight, conv1d_bias, dt, A, chunk_size, D=None, z=None, dt_bias=None,
                          dt_softplus=False, dt_limit=(0.0, float("inf")), activation="silu", headdim=None, ngroups=1):
    """Convolution + scan through ssd_selective_scan (the role of ssd_combined.py:779).
    xBC: (batch, seqlen, dim + 2 * ngroups * dstate); returns (batch, seqlen, dim)."""
    batch, seqlen, nheads = dt.shape[:3]
    assert nheads % ngroups == 0
    if z is not None:
        dim = z.shape[-1]
        assert dim % nheads == 0
        headdim = dim // nheads
    else:
        if D.dim() == 1:
            assert headdim is not None
        else:
            headdim = D.shape[1]
        dim = nheads * headdim
    if conv1d_weight.dim() == 3:
        conv1d_weight = conv1d_weight.squeeze(1)
    xBC = _causal_conv1d(xBC, conv1d_weight, conv1d_bias, activation)
    dstate = (xBC.shape[-1] - dim) // ngroups // 2
    x, B, C = torch.split(xBC, [dim, ngroups * dstate, ngroups * dstate], dim=-1)
    out = ssd_selective_scan(x.reshape(batch, seqlen, nheads, headdim), dt.to(x.dtype), A,
                             B.reshape(batch, seqlen, ngroups, dstate), C.reshape(batch, seqlen, ngroups, dstate),
                             D=D.float() if D is not None else None,
                             z=z.reshape(batch, seqlen, nheads, headdim) if z is not None else None,
                             dt_bias=dt_bias, dt_softplus=dt_softplus, dt_limit=dt_limit)
    return out.reshape(batch, seqlen, dim)


def mamba_split_conv1d_scan_ref(zxbcdt, conv1d_weight, conv1d_bias, dt_bias, A, D, chunk_size,
                                dt_limit=(0.0, float("inf")), activation="silu", rmsnorm_weight=None, rmsnorm_eps=1e-6,
                                outproj_weight=None, outproj_bias=None, headdim=None, ngroups=1,
                                norm_before_gate=True):
    """mamba_split_conv1d_scan_combined with the scan routed through ssd_selective_scan (the role
    of ssd_combined.py:1006); no d_nonssm part, no packed sequences."""
    import torch.nn.functional as F
    if D.dim() == 1:
        assert headdim is not None
        nheads, = D.shape
    else:
        nheads, headdim = D.shape
    assert nheads % ngroups == 0
    batch, seqlen, _ = zxbcdt.shape
    dim = nheads * headdim
    dstate = (zxbcdt.shape[-1] - 2 * dim - nheads) // ngroups // 2
    assert zxbcdt.shape == (batch, seqlen, 2 * dim + 2 * ngroups * dstate + nheads)
    assert dt_bias.shape == (nheads,) and A.shape == (nheads,)
    if conv1d_weight.dim() == 3:
        conv1d_weight = conv1d_weight.squeeze(1)
    z, xBC, dt = torch.split(zxbcdt, [dim, dim + 2 * ngroups * dstate, nheads], dim=-1)
    xBC = _causal_conv1d(xBC, conv1d_weight, conv1d_bias, activation)
    x, B, C = torch.split(xBC, [dim, ngroups * dstate, ngroups * dstate], dim=-1)
    z4 = z.reshape(batch, seqlen, nheads, headdim)
    y = ssd_selective_scan(x.reshape(batch, seqlen, nheads, headdim), dt.to(x.dtype), A,
                           B.reshape(batch, seqlen, ngroups, dstate), C.reshape(batch, seqlen, ngroups, dstate),
                           D=D.float(), z=z4 if rmsnorm_weight is None else None, dt_bias=dt_bias, dt_softplus=True,
                           dt_limit=dt_limit).reshape(batch, seqlen, dim)
    if rmsnorm_weight is not None:
        y = _gated_rms_norm(y, rmsnorm_weight, z, rmsnorm_eps, dim // ngroups, norm_before_gate)
    if outproj_weight is not None:
        y = F.linear(y, outproj_weight, outproj_bias)
    return y
