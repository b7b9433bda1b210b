"""GPU parity of the SSD chunked scan (mamba_chunk_scan_combined) against the CPU oracle.

The reference has no test that compares this op with a reference function (its test_ssd.py
imports the refs but never calls them); the cases below follow the shapes of its generation
and determinism tests and of the benchmark configurations, with the tolerances the benchmark
states: fp32 (6e-4, 2e-3), bf16 (3e-2, 5e-2).
"""
import pytest
import torch

from oracle.ssd import ssd_oracle, ssd_inputs

pytestmark = pytest.mark.gpu


def _tol(dtype):
    return (6e-4, 2e-3) if dtype == torch.float32 else ((3e-3, 5e-3) if dtype == torch.float16 else (3e-2, 5e-2))


def _close(name, got, ref, rtol, atol):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    err = (got - ref).abs()
    bound = atol + rtol * ref.abs()
    assert bool((err <= bound).all()), (
        f"{name}: max err {err.max().item():.3e}, worst excess {(err - bound).max().item():.3e}, "
        f"ref max {ref.abs().max().item():.3e}")


def _fwd_case(batch, seqlen, nheads, headdim, dstate, ngroups, chunk, dtype, seq_lens=None, has_init=False,
              has_z=True, has_D=True, D_has_hdim=False, dt_limit=(0.0, float("inf")), seed=0):
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    t = ssd_inputs(batch, seqlen, nheads, headdim, dstate, ngroups, dtype, seed, has_z=has_z, has_D=has_D,
                   D_has_hdim=D_has_hdim, seq_lens=seq_lens, has_init=has_init)
    rtol, atol = _tol(dtype)
    out_ref, fin_ref = ssd_oracle(t["x"], t["dt"], t["A"], t["B"], t["C"], D=t["D"], z=t["z"], dt_bias=t["dt_bias"],
                                  initial_states=t["initial_states"], seq_idx=t["seq_idx"], dt_softplus=True,
                                  dt_limit=dt_limit, return_final_states=True)
    cu = lambda v: None if v is None else v.cuda()
    out, fin = mamba_chunk_scan_combined(cu(t["x"]), cu(t["dt"]), cu(t["A"]), cu(t["B"]), cu(t["C"]), chunk,
                                         D=cu(t["D"]), z=cu(t["z"]), dt_bias=cu(t["dt_bias"]),
                                         initial_states=cu(t["initial_states"]), seq_idx=cu(t["seq_idx"]),
                                         dt_softplus=True, dt_limit=dt_limit, return_final_states=True)
    assert out.dtype == dtype and out.shape == out_ref.shape and fin.dtype == torch.float32
    _close("out", out, out_ref, rtol, atol)
    _close("final_states", fin, fin_ref, rtol, atol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("seqlen,chunk", [(256, 64), (300, 128), (1024, 256), (77, 256), (512, 32)])
def test_ssd_fwd_basic(seqlen, chunk, dtype):
    _fwd_case(2, seqlen, 4, 64, 32, 2, chunk, dtype)


@pytest.mark.parametrize("headdim,dstate,ngroups", [(64, 128, 1), (128, 64, 4), (32, 16, 1), (48, 40, 2), (64, 256, 1)])
def test_ssd_fwd_shapes(headdim, dstate, ngroups):
    _fwd_case(1, 384, 4, headdim, dstate, ngroups, 128, torch.float32)


@pytest.mark.parametrize("headdim,dstate,chunk,seqlen", [
    (64, 128, 256, 1024), (64, 64, 128, 300), (32, 128, 64, 200), (64, 128, 256, 77), (32, 64, 256, 513),
    (64, 128, 128, 640)])
def test_ssd_fwd_fused_scan_shapes(headdim, dstate, chunk, seqlen):
    # bf16 shapes served by the fused C B^T + scan kernel, full and partial last chunks
    _fwd_case(2, seqlen, 4, headdim, dstate, 2, chunk, torch.bfloat16, has_init=True)
    _fwd_case(1, seqlen, 4, headdim, dstate, 1, chunk, torch.bfloat16, has_z=False, D_has_hdim=True)


def test_ssd_fwd_fused_scan_packed():
    _fwd_case(1, 1024, 4, 64, 128, 2, 256, torch.bfloat16, seq_lens=[300, 212, 100, 156, 256], has_init=True)
    _fwd_case(1, 700, 4, 32, 64, 1, 128, torch.bfloat16, seq_lens=[1, 127, 129, 443])
    # chunk 256 (two tiles of the chunk per wave): a ragged last chunk with whole tiles past the end, no gate, no D
    _fwd_case(1, 900, 4, 64, 64, 2, 256, torch.bfloat16, seq_lens=[255, 257, 388], has_z=False, has_D=False)
    _fwd_case(2, 300, 4, 32, 128, 1, 256, torch.bfloat16, has_init=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ssd_fwd_options(dtype):
    _fwd_case(2, 320, 4, 64, 32, 1, 64, dtype, has_init=True)
    _fwd_case(2, 320, 4, 64, 32, 1, 64, dtype, has_z=False)
    _fwd_case(2, 320, 4, 64, 32, 1, 64, dtype, has_D=False)
    _fwd_case(2, 320, 4, 64, 32, 1, 64, dtype, D_has_hdim=True)
    _fwd_case(2, 320, 4, 64, 32, 1, 64, dtype, dt_limit=(0.01, 0.05))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ssd_fwd_packed_sequences(dtype):
    # sequence boundaries inside chunks, on chunk edges, and a first sequence seeded by initial_states
    _fwd_case(1, 1024, 8, 64, 64, 8, 256, dtype, seq_lens=[100, 156, 256, 300, 212], has_init=True)
    _fwd_case(2, 640, 4, 32, 32, 2, 128, dtype, seq_lens=[1, 127, 129, 383], has_init=False)


def _bwd_case(batch, seqlen, nheads, headdim, dstate, ngroups, chunk, dtype, seq_lens=None, has_init=False,
              has_z=True, has_D=True, D_has_hdim=False, dt_limit=(0.0, float("inf")), with_dfinal=True, seed=0,
              grad_scale=1.0):
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    t = ssd_inputs(batch, seqlen, nheads, headdim, dstate, ngroups, dtype, seed, has_z=has_z, has_D=has_D,
                   D_has_hdim=D_has_hdim, seq_lens=seq_lens, has_init=has_init)
    rtol, atol = _tol(dtype)
    names = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states"]
    ref_in = {k: (t[k].clone().requires_grad_() if t[k] is not None else None) for k in names}
    gpu_in = {k: (t[k].cuda().requires_grad_() if t[k] is not None else None) for k in names}
    # the oracle runs in float64 on the same (already rounded) inputs, so its own rounding is no part of the error
    out_ref, fin_ref = ssd_oracle(ref_in["x"], ref_in["dt"], ref_in["A"], ref_in["B"], ref_in["C"], D=ref_in["D"],
                                  z=ref_in["z"], dt_bias=ref_in["dt_bias"], initial_states=ref_in["initial_states"],
                                  seq_idx=t["seq_idx"], dt_softplus=True, dt_limit=dt_limit,
                                  return_final_states=True, compute_dtype=torch.float64)
    cu = lambda v: None if v is None else v.cuda()
    out, fin = mamba_chunk_scan_combined(gpu_in["x"], gpu_in["dt"], gpu_in["A"], gpu_in["B"], gpu_in["C"], chunk,
                                         D=gpu_in["D"], z=gpu_in["z"], dt_bias=gpu_in["dt_bias"],
                                         initial_states=gpu_in["initial_states"], seq_idx=cu(t["seq_idx"]),
                                         dt_softplus=True, dt_limit=dt_limit, return_final_states=True)
    _close("out", out, out_ref, rtol, atol)
    dfin = t["dfinal"] if with_dfinal else torch.zeros_like(t["dfinal"])
    (out_ref.double() * t["dout"].double()).sum().add((fin_ref * dfin.double()).sum()).backward()
    (out.float() * t["dout"].cuda().float()).sum().add((fin * dfin.cuda()).sum()).backward()
    # Every gradient at the base tolerance of its dtype, with these stated exceptions for 16-bit inputs:
    #  * ddt: x LOOSE_DDT.  The gate gradient g = dout * silu(z) reaches the matrix cores rounded to the inputs'
    #    dtype (the reference stores it the same way, ssd_chunk_scan.py:1386 `dout_x = torch.empty_like(dout)`),
    #    and ddt sums ~headdim * chunk products of it with mixed signs; with fp32 kernels on the same values, or
    #    without a gate, ddt holds the base tolerance (tests/test_ssd_rounding_sites_gpu.py).
    #  * dA, dD, ddt_bias: fp32 sums over every position of a head; the absolute part of the tolerance follows the
    #    largest entry of the reference (summation of 16-bit-rounded terms).
    #  * dinitial_states: the gradient of each chunk's entering state is stored in the inputs' dtype before state
    #    passing adds the chunks up in fp32 (the reference keeps it in fp32 until then, ssd_combined.py:455-466; half
    #    the bytes of the largest workspace of the backward pass): where a head hardly decays the sum carries those
    #    roundings, so the absolute part of the tolerance is at least one bf16 step (2^-8) of the largest entry.
    #  * fp16 inputs (no tolerance of their own in the benchmark; (3e-3, 5e-3) is the reference's fp16 setting for
    #    the Mamba-1 scan, tests/ops/test_selective_scan.py:43-47): every gradient x 2, measured 1.5 on dx.
    lowp = dtype != torch.float32
    if dtype == torch.float16:
        rtol, atol = 2 * rtol, 2 * atol
    for k in names:
        if ref_in[k] is None:
            continue
        gr, rr = gpu_in[k].grad, ref_in[k].grad
        assert gr is not None, f"no gradient for {k}"
        assert gr.dtype == gpu_in[k].dtype and gr.shape == gpu_in[k].shape
        f = LOOSE_DDT if (lowp and k == "dt") else 1.0
        scale = max(1.0, float(rr.abs().max())) if (lowp and k in ("A", "D", "dt_bias")) else 1.0
        if lowp and k == "initial_states":
            scale = max(1.0, float(rr.abs().max()) / 256 / atol)
        _close("d" + k, gr, rr, rtol * f, atol * f * scale * grad_scale)


LOOSE_DDT = 3.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seqlen,chunk", [(256, 64), (300, 128), (512, 256), (77, 256)])
def test_ssd_bwd_basic(seqlen, chunk, dtype):
    _bwd_case(2, seqlen, 4, 64, 32, 2, chunk, dtype)


@pytest.mark.parametrize("headdim,dstate,ngroups", [(64, 128, 1), (128, 64, 4), (32, 16, 1), (48, 40, 2)])
def test_ssd_bwd_shapes(headdim, dstate, ngroups):
    _bwd_case(1, 384, 4, headdim, dstate, ngroups, 128, torch.float32)


@pytest.mark.parametrize("headdim,dstate,ngroups,dtype", [
    (32, 128, 1, torch.bfloat16), (128, 256, 2, torch.float32), (16, 128, 1, torch.bfloat16), (96, 128, 1, torch.float32)])
def test_ssd_bwd_wide_tiles(headdim, dstate, ngroups, dtype):
    # whole 128-state blocks and whole 32-position steps: chunk states, their gradients and the
    # state part of dB run on 64 x 128 tiles, with head dimensions below, at and above one tile
    _bwd_case(2, 512, 4, headdim, dstate, ngroups, 128, dtype, has_init=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ssd_bwd_options(dtype):
    _bwd_case(2, 320, 4, 64, 32, 1, 64, dtype, has_init=True)
    _bwd_case(2, 320, 4, 64, 32, 1, 64, dtype, has_z=False)
    _bwd_case(2, 320, 4, 64, 32, 1, 64, dtype, has_D=False, with_dfinal=False)
    _bwd_case(2, 320, 4, 64, 32, 1, 64, dtype, D_has_hdim=True)
    _bwd_case(2, 320, 4, 64, 32, 1, 64, dtype, dt_limit=(0.01, 0.05))


@pytest.mark.parametrize("headdim,dstate,ngroups,chunk,seqlen", [
    (64, 128, 1, 256, 700), (32, 64, 2, 64, 300), (64, 64, 4, 128, 512)])
def test_ssd_bwd_no_gate_bf16(headdim, dstate, ngroups, chunk, seqlen):
    """Without z (the Mamba-2 block with its gated norm after the scan, modules/mamba2.py:226-242) g is dout itself:
    where the fused dx kernel runs and D is one value per head, dD comes out of that kernel; a D per (head, p), no D
    and packed sequences take their own branches.  dout is not damped by silu(z) here (rms 0.6 for z ~ N(0, 1)), so
    every sum is about 1.7 times larger at the same relative rounding of its 16-bit terms: the absolute part of the
    tolerance is doubled."""
    kw = dict(has_z=False, grad_scale=2.0)
    _bwd_case(2, seqlen, 8, headdim, dstate, ngroups, chunk, torch.bfloat16, has_init=True, **kw)
    _bwd_case(1, seqlen, 8, headdim, dstate, ngroups, chunk, torch.bfloat16,
              seq_lens=[seqlen // 3, 1, seqlen - seqlen // 3 - 1], seed=3, **kw)
    _bwd_case(2, seqlen, 8, headdim, dstate, ngroups, chunk, torch.bfloat16, D_has_hdim=True, seed=4, **kw)
    _bwd_case(2, seqlen, 8, headdim, dstate, ngroups, chunk, torch.bfloat16, has_D=False, seed=5, **kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ssd_bwd_packed_sequences(dtype):
    _bwd_case(1, 1024, 8, 64, 64, 8, 256, dtype, seq_lens=[100, 156, 256, 300, 212], has_init=True)
    _bwd_case(2, 640, 4, 32, 32, 2, 128, dtype, seq_lens=[1, 127, 129, 383], has_init=False)


def test_ssd_bwd_recompute_mode_matches_kept_state():
    """Backward from the kept forward workspaces and backward with the reference's re-computation
    (ssd_combined.py:441-448) give the same gradients, bit for bit."""
    from mamba_amd.ops.triton import ssd_combined as sc
    t = ssd_inputs(2, 600, 4, 64, 64, 2, torch.bfloat16, 5, seq_lens=None, has_init=True)
    names = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states"]
    grads = []
    for keep in (True, False):
        old, sc.KEEP_FORWARD_STATE = sc.KEEP_FORWARD_STATE, keep
        try:
            g = {k: t[k].cuda().requires_grad_() for k in names}
            out, fin = sc.mamba_chunk_scan_combined(g["x"], g["dt"], g["A"], g["B"], g["C"], 128, D=g["D"], z=g["z"],
                                                    dt_bias=g["dt_bias"], initial_states=g["initial_states"],
                                                    dt_softplus=True, return_final_states=True)
            (out.float().square().sum() + fin.sum()).backward()
            grads.append({k: g[k].grad.clone() for k in names})
        finally:
            sc.KEEP_FORWARD_STATE = old
    for k in ("x", "z", "initial_states"):  # written once per element: deterministic
        assert torch.equal(grads[0][k], grads[1][k]), k
    for k in ("dt", "A", "B", "C", "D", "dt_bias"):  # sums of float atomics: order-dependent rounding
        assert torch.allclose(grads[0][k].float(), grads[1][k].float(), rtol=2e-2, atol=1e-2), k


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seq_lens", [[100, 156, 256, 1, 299, 212], [300, 84, 128, 512]])
def test_ssd_varlen_states(seq_lens, dtype):
    """return_varlen_states: the state at the end of every packed sequence equals the final state of
    that sequence run alone through the oracle.  Boundaries inside chunks, on chunk edges, length 1.
    Only sequence 0 sees initial_states (ssd_state_passing.py:71-79), and, as in the reference
    (ssd_chunk_state.py:700-706 adds the carried state only when the sequence began before its last
    chunk), not when it ends inside the first chunk."""
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    chunk = 128
    total = sum(seq_lens)
    t = ssd_inputs(1, total, 4, 64, 32, 2, dtype, 3, seq_lens=seq_lens, has_init=True)
    rtol, atol = _tol(dtype)
    cu_seqlens = torch.tensor([0] + list(torch.tensor(seq_lens).cumsum(0)), dtype=torch.int32)
    refs, start = [], 0
    for i, n in enumerate(seq_lens):
        sl = slice(start, start + n)
        seeded = i == 0 and n > chunk
        _, fin = ssd_oracle(t["x"][:, sl], t["dt"][:, sl], t["A"], t["B"][:, sl], t["C"][:, sl], D=t["D"],
                            z=t["z"][:, sl], dt_bias=t["dt_bias"],
                            initial_states=t["initial_states"] if seeded else None, dt_softplus=True,
                            return_final_states=True)
        refs.append(fin[0])
        start += n
    ref = torch.stack(refs)
    cu = lambda v: None if v is None else v.cuda()
    out, fin, varlen = mamba_chunk_scan_combined(
        cu(t["x"]), cu(t["dt"]), cu(t["A"]), cu(t["B"]), cu(t["C"]), chunk, D=cu(t["D"]), z=cu(t["z"]),
        dt_bias=cu(t["dt_bias"]), initial_states=cu(t["initial_states"]), seq_idx=cu(t["seq_idx"]),
        cu_seqlens=cu_seqlens.cuda(), dt_softplus=True, return_final_states=True, return_varlen_states=True)
    assert varlen.shape == ref.shape and varlen.dtype == dtype
    _close("varlen_states", varlen, ref, rtol, atol)
    _close("final_states", fin, ref[-1:], rtol, atol)
    out2, varlen2 = mamba_chunk_scan_combined(
        cu(t["x"]), cu(t["dt"]), cu(t["A"]), cu(t["B"]), cu(t["C"]), chunk, D=cu(t["D"]), z=cu(t["z"]),
        dt_bias=cu(t["dt_bias"]), initial_states=cu(t["initial_states"]), seq_idx=cu(t["seq_idx"]),
        cu_seqlens=cu_seqlens.cuda(), dt_softplus=True, return_varlen_states=True, state_dtype=torch.float32)
    assert varlen2.dtype == torch.float32 and torch.equal(out, out2)
    _close("varlen_states fp32", varlen2, ref, rtol, atol)


@pytest.mark.parametrize("seqlen,chunk", [(300, 64), (512, 256)])
def test_ssd_bwd_fp16(seqlen, chunk):
    _bwd_case(2, seqlen, 4, 64, 64, 2, chunk, torch.float16, has_init=True, seed=12)
    _bwd_case(1, seqlen, 2, 32, 128, 1, chunk, torch.float16, seq_lens=[seqlen // 3, seqlen - seqlen // 3], seed=13)


def test_ssd_negative_dt_without_softplus_is_clamped():
    """Without softplus a raw dt can be negative; the reference's kernels clamp it to dt_limit's lower bound 0
    (ssd_chunk_state.py:80) and pass no gradient through the clamped positions (ssd_chunk_state.py:147-160)."""
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    t = ssd_inputs(2, 200, 4, 32, 64, 2, torch.float32, seed=21)
    t["dt"] = 0.05 * torch.randn(2, 200, 4, generator=torch.Generator().manual_seed(1))
    assert 0.3 < (t["dt"] < 0).float().mean() < 0.7
    names = ["x", "dt", "A", "B", "C", "D", "z"]
    ref_in = {k: t[k].clone().requires_grad_() for k in names}
    gpu_in = {k: t[k].cuda().requires_grad_() for k in names}
    out_ref = ssd_oracle(ref_in["x"], ref_in["dt"], ref_in["A"], ref_in["B"], ref_in["C"], D=ref_in["D"], z=ref_in["z"])
    out = mamba_chunk_scan_combined(gpu_in["x"], gpu_in["dt"], gpu_in["A"], gpu_in["B"], gpu_in["C"], 64,
                                    D=gpu_in["D"], z=gpu_in["z"])
    rtol, atol = _tol(torch.float32)
    _close("out", out, out_ref, rtol, atol)
    (out_ref * t["dout"]).sum().backward()
    (out * t["dout"].cuda()).sum().backward()
    assert bool((gpu_in["dt"].grad[gpu_in["dt"] < 0] == 0).all())
    for k in names:
        scale = max(1.0, float(ref_in[k].grad.abs().max())) if k in ("A", "D", "dt") else 1.0
        _close("d" + k, gpu_in[k].grad, ref_in[k].grad, rtol * 2, atol * 2 * scale)
