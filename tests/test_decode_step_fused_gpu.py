"""mamba2_decode_step: the convolution's decode step and the state update in one launch must give the
same bits as the two separate calls (causal_conv1d_update, then selective_state_update), for the output
and for both states, over consecutive steps; the two-call path itself is held to the oracle elsewhere
(tests/test_state_update_gpu.py, tests/test_causal_conv1d_gpu.py, tests/test_prefill_decode_gpu.py)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _setup(batch, H, P, N, G, W, SL, dtype, state_dtype, channel_last, has_z, has_D, has_bias, has_dtb, seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)
    conv_dim = H * P + 2 * G * N
    t = dict(
        ssm=(0.1 * r(batch, H, P, N)).to(state_dtype).cuda(),
        conv_w=(0.4 * r(conv_dim, W)).to(dtype).cuda(),
        conv_b=(0.1 * r(conv_dim)).to(dtype).cuda() if has_bias else None,
        A=-(0.5 + torch.rand(H, generator=g)).cuda(),
        D=torch.rand(H, generator=g).cuda() if has_D else None,
        dtb=(torch.rand(H, generator=g) - 2).cuda() if has_dtb else None,
    )
    cs = r(batch, conv_dim, SL).to(dtype)
    t["conv"] = (cs.transpose(1, 2).contiguous().transpose(1, 2) if channel_last else cs.contiguous()).cuda()
    steps = [dict(xBC=r(batch, conv_dim).to(dtype).cuda(), dt=r(batch, H).to(dtype).cuda(),
                  z=r(batch, H, P).to(dtype).cuda() if has_z else None) for _ in range(4)]
    return t, steps


def _run(t, steps, G, fuse):
    from mamba_amd.ops.triton.selective_state_update import mamba2_decode_step
    ssm, conv = t["ssm"].clone(), t["conv"].clone()
    outs = []
    for s in steps:
        outs.append(mamba2_decode_step(ssm, conv, s["xBC"], s["dt"], t["A"], t["conv_w"], t["conv_b"], D=t["D"], z=s["z"],
                                       dt_bias=t["dtb"], ngroups=G, fuse=fuse).clone())
    return outs, ssm, conv


@pytest.mark.parametrize("dtype,state_dtype", [(torch.bfloat16, torch.float32), (torch.float32, torch.float32),
                                               (torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("batch,H,P,N,G", [(1, 4, 64, 128, 1), (3, 6, 32, 64, 2), (2, 2, 48, 16, 1), (5, 8, 64, 96, 4)])
def test_fused_equals_two_calls(batch, H, P, N, G, dtype, state_dtype):
    t, steps = _setup(batch, H, P, N, G, 4, 4, dtype, state_dtype, True, True, True, True, True)
    want, ssm_w, conv_w = _run(t, steps, G, False)
    got, ssm_g, conv_g = _run(t, steps, G, True)
    for i, (a, b) in enumerate(zip(got, want)):
        assert torch.equal(a, b), f"step {i}: {(a.float() - b.float()).abs().max().item():.3e}"
    assert torch.equal(ssm_g, ssm_w) and torch.equal(conv_g, conv_w)


@pytest.mark.parametrize("W,SL", [(2, 1), (2, 4), (3, 2), (3, 3), (4, 3), (4, 4)])
@pytest.mark.parametrize("channel_last", [True, False])
def test_fused_filter_widths_and_state_layouts(W, SL, channel_last):
    t, steps = _setup(2, 4, 64, 64, 2, W, SL, torch.bfloat16, torch.float32, channel_last, True, True, True, True, seed=W * 10 + SL)
    want, ssm_w, conv_w = _run(t, steps, 2, False)
    got, ssm_g, conv_g = _run(t, steps, 2, True)
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    assert torch.equal(ssm_g, ssm_w) and torch.equal(conv_g, conv_w)


@pytest.mark.parametrize("has_z,has_D,has_bias,has_dtb", [(False, True, True, True), (True, False, True, True),
                                                          (True, True, False, True), (True, True, True, False),
                                                          (False, False, False, False)])
def test_fused_optional_operands(has_z, has_D, has_bias, has_dtb):
    t, steps = _setup(2, 4, 64, 128, 1, 4, 4, torch.bfloat16, torch.float32, True, has_z, has_D, has_bias, has_dtb)
    want, ssm_w, conv_w = _run(t, steps, 1, False)
    got, ssm_g, conv_g = _run(t, steps, 1, True)
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    assert torch.equal(ssm_g, ssm_w) and torch.equal(conv_g, conv_w)


@pytest.mark.parametrize("dtype,rtol,atol", [(torch.float32, 6e-4, 2e-3), (torch.bfloat16, 3e-2, 5e-2)])
@pytest.mark.parametrize("batch,H,P,N,G", [(2, 4, 64, 128, 1), (3, 8, 64, 64, 2)])
def test_fused_against_the_oracle(batch, H, P, N, G, dtype, rtol, atol):
    """The fused step alone against the CPU restatement: F.conv1d over [conv_state, x] + SiLU, then the
    oracle's state update (the oracle runs in fp32 on the same, already rounded, inputs; its conv output is
    rounded to the activations' dtype as the operator's is)."""
    import torch.nn.functional as F
    from oracle.step import selective_state_update_oracle
    W = 4
    t, steps = _setup(batch, H, P, N, G, W, W, dtype, torch.float32, True, True, True, True, True, seed=5)
    got, ssm_g, conv_g = _run(t, steps, G, True)
    ssm, conv = t["ssm"].cpu().clone(), t["conv"].cpu().float().clone()
    cw, cb = t["conv_w"].cpu().float(), t["conv_b"].cpu().float()
    for i, s in enumerate(steps):
        full = torch.cat([conv, s["xBC"].cpu().float()[:, :, None]], dim=2)      # (batch, conv_dim, W + 1)
        xc = F.silu(F.conv1d(full, cw[:, None, :], cb, groups=cw.shape[0])[:, :, -1]).to(dtype).float()
        conv = full[:, :, 1:].clone()
        x, B, C = torch.split(xc, [H * P, G * N, G * N], dim=-1)
        ref = selective_state_update_oracle(
            ssm, x.reshape(batch, H, P), s["dt"].cpu().float()[:, :, None].expand(batch, H, P),
            t["A"].cpu()[:, None, None].expand(H, P, N), B.reshape(batch, G, N), C.reshape(batch, G, N),
            D=t["D"].cpu()[:, None].expand(H, P), z=s["z"].cpu().float(), dt_bias=t["dtb"].cpu()[:, None].expand(H, P),
            dt_softplus=True)
        assert torch.allclose(got[i].cpu().float(), ref, rtol=rtol, atol=atol), f"step {i}"
    assert torch.allclose(ssm_g.cpu(), ssm, rtol=rtol, atol=atol)
    assert torch.equal(conv_g.cpu().float(), conv)


@pytest.mark.parametrize("N,P", [(8, 128), (4, 64), (8, 64)])
def test_few_states_take_the_two_calls(N, P):
    """Fewer than 16 states put more than 64 rows into a wave of the fused kernel, which it does not serve: the
    C entry point refuses, `fuse=True` raises, and `fuse=None` gives the two-call result."""
    t, steps = _setup(2, 2, P, N, 1, 4, 4, torch.bfloat16, torch.float32, True, True, True, True, True, seed=N + P)
    want, ssm_w, conv_w = _run(t, steps, 1, False)
    got, ssm_g, conv_g = _run(t, steps, 1, None)
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    assert torch.equal(ssm_g, ssm_w) and torch.equal(conv_g, conv_w)
    with pytest.raises(RuntimeError):
        _run(t, steps, 1, True)


def test_fused_in_a_captured_graph():
    from mamba_amd.ops.triton.selective_state_update import mamba2_decode_step
    batch, H, P, N, G = 2, 4, 64, 128, 1
    t, steps = _setup(batch, H, P, N, G, 4, 4, torch.bfloat16, torch.float32, True, True, True, True, True, seed=9)
    want, ssm_w, conv_w = _run(t, steps, G, False)
    ssm, conv = t["ssm"].clone(), t["conv"].clone()
    s_xBC, s_dt, s_z = (torch.zeros_like(steps[0][k]) for k in ("xBC", "dt", "z"))
    step = lambda: mamba2_decode_step(ssm, conv, s_xBC, s_dt, t["A"], t["conv_w"], t["conv_b"], D=t["D"], z=s_z,
                                      dt_bias=t["dtb"], ngroups=G, fuse=True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s_out = step()
    ssm.copy_(t["ssm"])
    conv.copy_(t["conv"])
    for i, s in enumerate(steps):
        s_xBC.copy_(s["xBC"]); s_dt.copy_(s["dt"]); s_z.copy_(s["z"])
        graph.replay()
        torch.cuda.synchronize()
        got = s_out.clone()
        _ = (got.float() * 2).sum().item()   # eager work and a synchronisation between the replays
        assert torch.equal(got, want[i]), f"replay {i}"
    assert torch.equal(ssm, ssm_w) and torch.equal(conv, conv_w)


@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("fuse", [False, True])
def test_filter_dtypes_same_bits_as_their_fp32_copies(wdtype, W, fuse):
    """The kernels read a bf16 / fp16 filter as it is: same bits as with its exact fp32 copy."""
    t, steps = _setup(2, 4, 64, 64, 2, W, 4, torch.bfloat16, torch.float32, True, True, True, True, True, seed=W)
    t["conv_w"], t["conv_b"] = t["conv_w"].to(wdtype), t["conv_b"].to(wdtype)
    got, ssm_g, conv_g = _run(t, steps, 2, fuse)
    t["conv_w"], t["conv_b"] = t["conv_w"].float(), t["conv_b"].float()
    want, ssm_w, conv_w = _run(t, steps, 2, fuse)
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    assert torch.equal(ssm_g, ssm_w) and torch.equal(conv_g, conv_w)
