"""The SSD stages one at a time, through the stage-level functions of the reference's modules
(ssd_chunk_state, ssd_state_passing, ssd_bmm, ssd_chunk_scan): each stage against a float64 restatement
of its formula on the CPU, and the five stages chained by hand against the sequential oracle."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle.ssd import dt_pipeline, ssd_inputs, ssd_oracle

pytestmark = pytest.mark.gpu


def _tol(dtype):
    return (6e-4, 2e-3) if dtype == torch.float32 else ((3e-3, 5e-3) if dtype == torch.float16 else (3e-2, 5e-2))


def _close(name, got, ref, rtol, atol):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    err = (got - ref).abs()
    bound = atol + rtol * ref.abs()
    assert bool((err <= bound).all()), (
        f"{name}: max err {err.max().item():.3e}, worst excess {(err - bound).max().item():.3e}, "
        f"ref max {ref.abs().max().item():.3e}")


def _cumsum_ref(dt, A, Q, dt_bias, dt_softplus, dt_limit):
    """dt_out and the in-chunk cumulative sums of dt * A, float64, zero dt past the end.  The kernel clamps to
    dt_limit even when that is the default (0, inf), so a negative dt without softplus becomes 0
    (ssd_chunk_state.py:80)."""
    b, L, H = dt.shape
    nc = math.ceil(L / Q)
    v = dt_pipeline(dt, dt_bias, dt_softplus, (0.0, float("inf")), torch.float64).clamp(min=dt_limit[0], max=dt_limit[1])
    v = F.pad(v, (0, 0, 0, nc * Q - L)).reshape(b, nc, Q, H).permute(0, 3, 1, 2)
    return torch.cumsum(v * A.double()[None, :, None, None], dim=-1), v


@pytest.mark.parametrize("dt_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seqlen,chunk", [(256, 64), (200, 64), (77, 128), (512, 256)])
def test_chunk_cumsum_fwd(seqlen, chunk, dt_dtype):
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_cumsum_fwd
    g = torch.Generator().manual_seed(seqlen + chunk)
    b, H = 2, 12
    dt = torch.randn(b, seqlen, H, generator=g).to(dt_dtype)
    A = -(1 + 15 * torch.rand(H, generator=g))
    bias = torch.rand(H, generator=g) - 4
    for kw in (dict(), dict(dt_bias=bias, dt_softplus=True), dict(dt_bias=bias, dt_softplus=True, dt_limit=(0.01, 0.05))):
        dA, dt_out = _chunk_cumsum_fwd(dt.cuda(), A.cuda(), chunk, **{k: (v.cuda() if torch.is_tensor(v) else v)
                                                                   for k, v in kw.items()})
        dA_ref, dt_ref = _cumsum_ref(dt, A, chunk, kw.get("dt_bias"), kw.get("dt_softplus", False),
                                     kw.get("dt_limit", (0.0, float("inf"))))
        assert dA.dtype == torch.float32 and dt_out.dtype == torch.float32
        _close("dt_out", dt_out, dt_ref, 1e-5, 1e-6)
        _close("dA_cumsum", dA, dA_ref, 1e-5, 1e-5)


def _chunk_state_ref64(B, x, dt, dA, seq_idx=None):
    b, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    nc, Q = dt.shape[2], dt.shape[3]
    pad = nc * Q - L
    xd, Bd = F.pad(x.double(), (0, 0, 0, 0, 0, pad)), F.pad(B.double(), (0, 0, 0, 0, 0, pad))
    Bh = Bd.repeat_interleave(H // G, dim=2).reshape(b, nc, Q, H, N)
    w = torch.exp(dA[..., -1:] - dA) * dt                      # (b, H, nc, Q)
    if seq_idx is not None:
        s = F.pad(seq_idx, (0, pad), value=-1).reshape(b, nc, Q)
        last = torch.stack([seq_idx[:, min((c + 1) * Q, L) - 1] for c in range(nc)], dim=1)  # (b, nc)
        w = w * (s == last[..., None]).double()[:, None]
    return torch.einsum("bclhn,bhcl,bclhp->bchpn", Bh, w, xd.reshape(b, nc, Q, H, P))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("seqlen,chunk,headdim,dstate,ngroups", [(256, 64, 64, 128, 1), (200, 64, 32, 16, 2),
                                                                 (384, 128, 64, 64, 4), (100, 256, 40, 24, 1)])
def test_chunk_state_fwd(seqlen, chunk, headdim, dstate, ngroups, dtype):
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_cumsum_fwd, _chunk_state_fwd, chunk_state, chunk_state_ref
    t = ssd_inputs(2, seqlen, 4, headdim, dstate, ngroups, dtype, seed=seqlen)
    dA, dtv = _cumsum_ref(t["dt"], t["A"], chunk, t["dt_bias"], True, (0.0, float("inf")))
    ref = _chunk_state_ref64(t["B"], t["x"], dtv, dA)
    rtol, atol = _tol(dtype)
    got = _chunk_state_fwd(t["B"].cuda(), t["x"].cuda(), dtv.float().cuda(), dA.float().cuda())
    assert got.dtype == torch.float32
    _close("states", got, ref, rtol, atol)
    low = _chunk_state_fwd(t["B"].cuda(), t["x"].cuda(), dtv.float().cuda(), dA.float().cuda(), states_in_fp32=False)
    assert low.dtype == dtype
    into = torch.empty_like(got)
    assert _chunk_state_fwd(t["B"].cuda(), t["x"].cuda(), dtv.float().cuda(), dA.float().cuda(), states=into) is into
    assert torch.equal(into, got)
    assert torch.equal(chunk_state(t["B"].cuda(), t["x"].cuda(), dtv.float().cuda(), dA.float().cuda()), got)
    if seqlen % chunk == 0 and dtype == torch.float32:
        _close("chunk_state_ref", chunk_state_ref(t["B"].cuda(), t["x"].cuda(), dtv.float().cuda(), dA.float().cuda()),
               ref, rtol, atol)


def test_chunk_state_fwd_packed_sequences():
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_state_fwd
    t = ssd_inputs(1, 320, 4, 32, 16, 2, torch.float32, seed=5, seq_lens=(70, 1, 129, 120))
    dA, dtv = _cumsum_ref(t["dt"], t["A"], 64, t["dt_bias"], True, (0.0, float("inf")))
    ref = _chunk_state_ref64(t["B"], t["x"], dtv, dA, t["seq_idx"].long())
    got = _chunk_state_fwd(t["B"].cuda(), t["x"].cuda(), dtv.float().cuda(), dA.float().cuda(), seq_idx=t["seq_idx"].cuda())
    _close("states", got, ref, *_tol(torch.float32))


def _passing_ref64(states, dAc, init, seq_chunk=None):
    b, nc, H, dim = states.shape
    s = torch.zeros(b, H, dim, dtype=torch.float64) if init is None else init.double()
    out, prev = [], torch.zeros(b, dtype=torch.long)
    for c in range(nc):
        out.append(s)
        scale = torch.exp(dAc[:, :, c].double())
        if seq_chunk is not None:
            scale = scale * (seq_chunk[:, c] == prev).double()[:, None]
            prev = seq_chunk[:, c]
        s = scale[..., None] * s + states[:, c].double()
    return torch.stack(out, dim=1), s


@pytest.mark.parametrize("has_init", [False, True])
# (2100 and 8300 chunks are beyond what the kernels keep as per-chunk tables in LDS: backward only, then both)
@pytest.mark.parametrize("nchunks,dim", [(1, 64), (7, 2048), (33, 1000), (16, 8192), (5, 77), (2100, 1024), (8300, 64)])
def test_state_passing_fwd_bwd(nchunks, dim, has_init):
    from mamba_amd.ops.triton.ssd_state_passing import state_passing, state_passing_ref
    g = torch.Generator().manual_seed(nchunks * 1000 + dim)
    b, H = 2, 3
    states = torch.randn(b, nchunks, H, dim, generator=g)
    dAc = -torch.rand(b, H, nchunks, generator=g) * 2
    init = torch.randn(b, H, dim, generator=g) if has_init else None
    dout, dfin = torch.randn(b, nchunks, H, dim, generator=g), torch.randn(b, H, dim, generator=g)
    leaves = [states.double().requires_grad_(), dAc.double().requires_grad_()] + ([init.double().requires_grad_()] if has_init else [])
    out_ref, fin_ref = _passing_ref64(leaves[0], leaves[1], leaves[2] if has_init else None)
    grads_ref = torch.autograd.grad((out_ref * dout.double()).sum() + (fin_ref * dfin.double()).sum(), leaves)
    dev = [states.cuda().requires_grad_(), dAc.cuda().requires_grad_()] + ([init.cuda().requires_grad_()] if has_init else [])
    out, fin = state_passing(dev[0], dev[1], dev[2] if has_init else None)
    grads = torch.autograd.grad([out, fin], dev, [dout.cuda(), dfin.cuda()])
    rtol, atol = 1e-4, 1e-4
    _close("out", out, out_ref, rtol, atol)
    _close("final_states", fin, fin_ref, rtol, atol)
    for name, a, r in zip(("dstates", "ddA_chunk_cumsum", "dinitial_states"), grads, grads_ref):
        _close(name, a, r, 2e-4, 2e-3 if name == "ddA_chunk_cumsum" else 1e-4)
    o2, f2 = state_passing_ref(states.cuda(), dAc.cuda(), init.cuda() if has_init else None)
    _close("state_passing_ref out", o2, out_ref, rtol, atol)
    _close("state_passing_ref final", f2, fin_ref, rtol, atol)


def test_state_passing_fwd_seq_idx_and_dtypes():
    from mamba_amd.ops.triton.ssd_state_passing import _state_passing_bwd, _state_passing_fwd
    g = torch.Generator().manual_seed(3)
    b, nc, H, dim, Q, L = 2, 6, 2, 256, 32, 180
    states = torch.randn(b, nc, H, dim, generator=g)
    dA_full = -torch.rand(b, H, nc, Q, generator=g)
    seq_idx = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate((40, 24, 64, 52))])[None].repeat(b, 1)
    ends = [min((c + 1) * Q, L) - 1 for c in range(nc)]
    out_ref, fin_ref = _passing_ref64(states, dA_full[..., -1], None, seq_idx[:, ends].long())
    out, fin = _state_passing_fwd(states.cuda(), dA_full.cuda()[:, :, :, -1], seq_idx=seq_idx.cuda(), chunk_size=Q,
                                  out_dtype=torch.bfloat16)
    assert out.dtype == torch.bfloat16 and fin.dtype == torch.float32
    _close("out", out, out_ref, 1e-2, 1e-2)
    _close("final_states", fin, fin_ref, 1e-4, 1e-4)
    dout = torch.randn(b, nc, H, dim, generator=g)
    res = _state_passing_bwd(out_ref.float().cuda(), dA_full.cuda()[:, :, :, -1], dout.cuda(), seq_idx=seq_idx.cuda(),
                             chunk_size=Q, has_initial_states=True, states_dtype=torch.bfloat16)
    assert len(res) == 4 and res[3].dtype == torch.bfloat16
    leaves = [states.double().requires_grad_(), dA_full[..., -1].double().requires_grad_()]
    o, f = _passing_ref64(leaves[0], leaves[1], None, seq_idx[:, ends].long())
    gs = torch.autograd.grad([o], leaves, [dout.double()])
    _close("dstates", res[0], gs[0], 2e-4, 1e-4)
    _close("ddA_chunk_cumsum", res[1], gs[1], 2e-4, 2e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seqlen,chunk,k,groups", [(256, 64, 128, 2), (200, 64, 16, 1), (300, 256, 64, None), (128, 128, 40, 3)])
def test_bmm_chunk_fwd(seqlen, chunk, k, groups, dtype):
    from mamba_amd.ops.triton.ssd_bmm import _bmm_chunk_fwd
    g = torch.Generator().manual_seed(seqlen + k)
    shape = (2, seqlen, k) if groups is None else (2, seqlen, groups, k)
    a, bb = torch.randn(*shape, generator=g).to(dtype), torch.randn(*shape, generator=g).to(dtype)
    seq_idx = (torch.arange(seqlen) >= seqlen // 3).to(torch.int32)[None].repeat(2, 1)
    nc = math.ceil(seqlen / chunk)
    pad = nc * chunk - seqlen
    a4 = (a if groups is not None else a[:, :, None]).double()
    b4 = (bb if groups is not None else bb[:, :, None]).double()
    a4, b4 = F.pad(a4, (0, 0, 0, 0, 0, pad)), F.pad(b4, (0, 0, 0, 0, 0, pad))
    G = a4.shape[2]
    ref = torch.einsum("bclgk,bcsgk->bcgls", a4.reshape(2, nc, chunk, G, k), b4.reshape(2, nc, chunk, G, k))
    s = F.pad(seq_idx, (0, pad), value=-1).reshape(2, nc, chunk)
    same = (s[:, :, :, None] == s[:, :, None, :])[:, :, None]
    rtol, atol = _tol(dtype)
    atol = atol * math.sqrt(k)
    for causal in (False, True):
        for sq in (None, seq_idx):
            got = _bmm_chunk_fwd(a.cuda(), bb.cuda(), chunk, seq_idx=None if sq is None else sq.cuda(), causal=causal,
                                 output_dtype=torch.float32)
            r = ref if sq is None else ref * same.double()
            if groups is None:
                assert got.shape == (2, nc, chunk, chunk)
                got = got[:, :, None]
            if causal:
                got, r = torch.tril(got), torch.tril(r)
            _close(f"cb causal={causal} seq={sq is not None}", got, r, rtol, atol)
    assert _bmm_chunk_fwd(a.cuda(), bb.cuda(), chunk).dtype == dtype


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seqlen,chunk,ngroups,seq_lens,has_init", [
    (256, 64, 1, None, False), (200, 64, 2, None, True), (320, 128, 4, (70, 1, 129, 120), False), (96, 256, 1, None, True)])
def test_stages_chained_match_sequential_oracle(seqlen, chunk, ngroups, seq_lens, has_init, dtype):
    """cumsum -> chunk_state -> state_passing -> bmm -> chunk_scan by hand, as ssd_combined.py:374-387 chains them."""
    from mamba_amd.ops.triton.ssd_bmm import _bmm_chunk_fwd
    from mamba_amd.ops.triton.ssd_chunk_scan import _chunk_scan_fwd
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_cumsum_fwd, _chunk_state_fwd
    from mamba_amd.ops.triton.ssd_state_passing import _state_passing_fwd
    H, P, N = 4, 32, 64
    t = ssd_inputs(2, seqlen, H, P, N, ngroups, dtype, seed=seqlen + chunk, seq_lens=seq_lens, has_init=has_init)
    out_ref, fin_ref = ssd_oracle(t["x"], t["dt"], t["A"], t["B"], t["C"], D=t["D"], z=t["z"], dt_bias=t["dt_bias"],
                                  initial_states=t["initial_states"], seq_idx=t["seq_idx"], dt_softplus=True,
                                  return_final_states=True)
    cu = lambda v: None if v is None else v.cuda()
    x, dt, A, B, C, D, z, bias, init, seq = (cu(t[k]) for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias",
                                                                "initial_states", "seq_idx"))
    dA_cumsum, dt_out = _chunk_cumsum_fwd(dt, A, chunk, dt_bias=bias, dt_softplus=True)
    states = _chunk_state_fwd(B, x, dt_out, dA_cumsum, seq_idx=seq)
    entering, final = _state_passing_fwd(states.flatten(-2), dA_cumsum[:, :, :, -1],
                                         initial_states=None if init is None else init.flatten(-2), seq_idx=seq,
                                         chunk_size=chunk)
    entering, final = entering.unflatten(-1, (P, N)), final.unflatten(-1, (P, N))
    CB = _bmm_chunk_fwd(C, B, chunk, seq_idx=seq, output_dtype=torch.float32)
    out, out_x = _chunk_scan_fwd(CB, x, dt_out, dA_cumsum, C, entering, D=D, z=z, seq_idx=seq)
    rtol, atol = _tol(dtype)
    assert out.dtype == dtype and out_x.dtype == dtype
    _close("out", out, out_ref, rtol, atol)
    _close("final_states", final, fin_ref, rtol, atol)
    _close("out_x * silu(z)", out_x.float() * F.silu(z.float()), out_ref, rtol, atol)
    out_noz, none = _chunk_scan_fwd(CB, x, dt_out, dA_cumsum, C, entering, D=D, seq_idx=seq)
    assert none is None
    _close("out without z", out_noz, out_x, rtol, atol)


def test_chunk_scan_function_and_ref():
    from mamba_amd.ops.triton.ssd_chunk_scan import chunk_scan, chunk_scan_ref
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_cumsum_fwd
    t = ssd_inputs(2, 256, 4, 32, 64, 2, torch.float32, seed=11, has_init=True)
    cu = lambda v: v.cuda()
    dA, dt_out = _chunk_cumsum_fwd(cu(t["dt"]), cu(t["A"]), 64, dt_bias=cu(t["dt_bias"]), dt_softplus=True)
    prev = 0.1 * torch.randn(2, 4, 4, 32, 64, generator=torch.Generator().manual_seed(1)).cuda()
    out = chunk_scan(cu(t["B"]), cu(t["C"]), cu(t["x"]), dt_out, dA, prev, D=cu(t["D"]), z=cu(t["z"]))
    ref = chunk_scan_ref(t["B"].double(), t["C"].double(), t["x"].double(), dt_out.cpu().double(), dA.cpu().double(),
                         prev.cpu().double(), D=t["D"].double(), z=t["z"].double())
    _close("chunk_scan", out, ref, *_tol(torch.float32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seqlen,chunk,headdim,dstate,ngroups", [(256, 64, 32, 64, 2), (512, 256, 64, 128, 1), (384, 128, 64, 16, 4)])
def test_chunk_state_backward(seqlen, chunk, headdim, dstate, ngroups, dtype):
    """chunk_state is differentiable (reference ChunkStateFn.backward, ssd_chunk_state.py:1060-1078): dB, dx, ddt,
    ddA_cumsum against autograd through the plain-torch form of the stage in float64."""
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_cumsum_fwd, chunk_state, chunk_state_ref
    t = ssd_inputs(2, seqlen, 4, headdim, dstate, ngroups, dtype, seed=21)
    cu = lambda v: v.cuda()
    dA, dt_out = _chunk_cumsum_fwd(cu(t["dt"]), cu(t["A"]), chunk, dt_bias=cu(t["dt_bias"]), dt_softplus=True)
    g = torch.Generator().manual_seed(2)
    dstates = torch.randn(2, seqlen // chunk, 4, headdim, dstate, generator=g)
    leaves = [cu(t["B"]).requires_grad_(), cu(t["x"]).requires_grad_(), dt_out.clone().requires_grad_(), dA.clone().requires_grad_()]
    (chunk_state(*leaves) * dstates.cuda()).sum().backward()
    ref_leaves = [t["B"].double().requires_grad_(), t["x"].double().requires_grad_(), dt_out.cpu().double().requires_grad_(),
                  dA.cpu().double().requires_grad_()]
    (chunk_state_ref(*ref_leaves) * dstates.double()).sum().backward()
    rtol, atol = _tol(dtype)
    for name, a, b in zip(("dB", "dx", "ddt", "ddA_cumsum"), leaves, ref_leaves):
        scale = max(1.0, float(b.grad.abs().max())) if name in ("ddt", "ddA_cumsum") else 1.0
        _close(name, a.grad, b.grad, 2 * rtol, 2 * atol * scale)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seqlen,chunk,headdim,dstate,ngroups,has_z,d_hdim", [
    (256, 64, 32, 64, 2, True, False), (512, 256, 64, 128, 1, True, False), (384, 128, 64, 16, 4, False, True)])
def test_chunk_scan_backward(seqlen, chunk, headdim, dstate, ngroups, has_z, d_hdim, dtype):
    """chunk_scan is differentiable (reference ChunkScanFn.backward, ssd_chunk_scan.py:1786-1825): dB, dC, dx, ddt,
    ddA_cumsum, dprev_states, dD, dz against autograd through the plain-torch form in float64."""
    from mamba_amd.ops.triton.ssd_chunk_scan import chunk_scan, chunk_scan_ref
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_cumsum_fwd
    H = 4
    t = ssd_inputs(2, seqlen, H, headdim, dstate, ngroups, dtype, seed=22, D_has_hdim=d_hdim)
    cu = lambda v: v.cuda()
    dA, dt_out = _chunk_cumsum_fwd(cu(t["dt"]), cu(t["A"]), chunk, dt_bias=cu(t["dt_bias"]), dt_softplus=True)
    prev = 0.1 * torch.randn(2, seqlen // chunk, H, headdim, dstate, generator=torch.Generator().manual_seed(3))
    names = ["B", "C", "x", "dt", "dA_cumsum", "prev_states", "D"] + (["z"] if has_z else [])
    gpu = dict(B=cu(t["B"]), C=cu(t["C"]), x=cu(t["x"]), dt=dt_out.clone(), dA_cumsum=dA.clone(), prev_states=prev.cuda(),
               D=cu(t["D"]), z=cu(t["z"]) if has_z else None)
    ref = dict(B=t["B"].double(), C=t["C"].double(), x=t["x"].double(), dt=dt_out.cpu().double(), dA_cumsum=dA.cpu().double(),
               prev_states=prev.double(), D=t["D"].double(), z=t["z"].double() if has_z else None)
    for d in (gpu, ref):
        for k in names:
            d[k].requires_grad_()
    call = lambda fn, d: fn(d["B"], d["C"], d["x"], d["dt"], d["dA_cumsum"], d["prev_states"], D=d["D"], z=d["z"])
    out = call(chunk_scan, gpu)
    out.backward(cu(t["dout"]))
    call(chunk_scan_ref, ref).backward(t["dout"].double())
    rtol, atol = _tol(dtype)
    for k in names:
        scale = max(1.0, float(ref[k].grad.abs().max())) if k in ("dt", "dA_cumsum", "D") else 1.0
        _close("d" + k, gpu[k].grad, ref[k].grad, 2 * rtol, 2 * atol * scale)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ngroups", [1, 2, "max"])
@pytest.mark.parametrize("chunk_size", [64, 128])
def test_chunk_state_varlen(chunk_size, ngroups, dtype):
    """The reference's own stage test (tests/ops/triton/test_ssd.py:30-80) at a smaller size: the states at the
    end of every packed sequence against the same stages run on each sequence alone."""
    from einops import rearrange
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_cumsum_fwd, _chunk_state_fwd, chunk_state, chunk_state_varlen
    from mamba_amd.ops.triton.ssd_state_passing import _state_passing_fwd
    device = "cuda"
    rtol, atol = (1e-2, 3e-3)
    torch.random.manual_seed(chunk_size + (ngroups if ngroups != "max" else 64))
    batch = 24
    seqlens = torch.randint(1, 200, (batch,), device=device)
    cu_seqlens = F.pad(seqlens.cumsum(0), (1, 0))
    total_seqlen = seqlens.sum().item()
    seq_idx = torch.cat([torch.full((s,), i, dtype=torch.int32, device=device) for i, s in enumerate(seqlens)], dim=0).unsqueeze(0)
    dim, headdim, dstate = 512, 64, 32
    nheads = dim // headdim
    if ngroups == "max":
        ngroups = nheads
    B = torch.randn(total_seqlen, ngroups, dstate, dtype=dtype, device=device) / 5
    x = torch.randn(total_seqlen, nheads, headdim, dtype=dtype, device=device)
    A = -0.1 * (torch.rand(nheads, device=device))
    dt = F.softplus(torch.randn(total_seqlen, nheads, device=device, dtype=torch.float32) - 4)
    dA_cumsum, dt_rounded = _chunk_cumsum_fwd(dt.unsqueeze(0), A, chunk_size)
    chunk_states = _chunk_state_fwd(B.unsqueeze(0), x.unsqueeze(0), dt_rounded, dA_cumsum, seq_idx=seq_idx)
    chunk_states, _ = _state_passing_fwd(rearrange(chunk_states, "... p n -> ... (p n)"), dA_cumsum[:, :, :, -1],
                                         seq_idx=seq_idx, chunk_size=chunk_size)
    chunk_states = rearrange(chunk_states, "... (p n) -> ... p n", n=dstate).squeeze(0)
    out = chunk_state_varlen(B, x, dt_rounded.squeeze(0), dA_cumsum.squeeze(0), cu_seqlens, chunk_states)
    out_ref = []
    for b in range(batch):
        sl = slice(cu_seqlens[b].item(), cu_seqlens[b + 1].item())
        dA_cumsum_s, dt_rounded_s = _chunk_cumsum_fwd(dt[sl].unsqueeze(0), A, chunk_size)
        states = chunk_state(B[sl].unsqueeze(0), x[sl].unsqueeze(0), dt_rounded_s, dA_cumsum_s)
        _, final_states = _state_passing_fwd(rearrange(states, "... p n -> ... (p n)"), dA_cumsum_s[:, :, :, -1],
                                             chunk_size=chunk_size)
        out_ref.append(rearrange(final_states, "... (p n) -> ... p n", n=dstate))
    out_ref = torch.cat(out_ref, dim=0)
    assert torch.allclose(out, out_ref, rtol=rtol, atol=atol), f"max diff {(out - out_ref).abs().max().item()}"


def test_stage_functions_reject_cpu_tensors():
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_cumsum_fwd
    with pytest.raises(RuntimeError):
        _chunk_cumsum_fwd(torch.randn(1, 64, 2), -torch.rand(2), 64)


@pytest.mark.parametrize("softplus,limit", [(True, (0.0, float("inf"))), (False, (0.0, float("inf"))), (True, (0.01, 0.5))])
def test_chunk_cumsum_backward(softplus, limit):
    """_chunk_cumsum_bwd (reference ssd_chunk_state.py:744) against autograd through the dt pipeline and the
    per-chunk running sum written out in float64."""
    import torch.nn.functional as F
    from mamba_amd.ops.triton.ssd_chunk_state import _chunk_cumsum_bwd
    batch, L, H, Q = 2, 320, 6, 128
    g = torch.Generator().manual_seed(5)
    dt = torch.randn(batch, L, H, generator=g)
    A, bias = -(1 + torch.rand(H, generator=g)), torch.randn(H, generator=g) - 2
    nc = (L + Q - 1) // Q
    ddA, ddt_out = torch.randn(batch, H, nc, Q, generator=g), torch.randn(batch, H, nc, Q, generator=g)
    got = _chunk_cumsum_bwd(ddA.cuda(), ddt_out.cuda(), dt.cuda(), A.cuda(), dt_bias=bias.cuda(), dt_softplus=softplus,
                            dt_limit=limit)
    dtr, Ar, br = dt.double().requires_grad_(), A.double().requires_grad_(), bias.double().requires_grad_()
    v = dtr + br
    v = F.softplus(v) if softplus else v
    v = v.clamp(limit[0], limit[1])
    v = F.pad(v, (0, 0, 0, nc * Q - L)).reshape(batch, nc, Q, H).permute(0, 3, 1, 2)        # (b, h, c, Q)
    dA_cs = torch.cumsum(v * Ar[None, :, None, None], dim=-1)
    ((dA_cs * ddA.double()).sum() + (v * ddt_out.double()).sum()).backward()
    for name, a, b in zip(("ddt", "dA", "ddt_bias"), got, (dtr.grad, Ar.grad, br.grad)):
        _close(name, a, b, 6e-4, 2e-3 * max(1.0, float(b.abs().max())))
