"""GPU parity of selective_state_update against the CPU oracle.

Follows the reference's tests/ops/triton/test_selective_state_update.py (:22 plain, :66 heads /
groups / tie_hdim, :112 state_batch_indices, :161 both), with its tolerances (:24-28), and
adds the decode benchmark's shape and the T-steps == scan property.
"""
import pytest
import torch
import torch.nn.functional as F

from oracle.step import selective_state_update_oracle

pytestmark = pytest.mark.gpu


def _tol(itype):
    rtol, atol = (3e-4, 1e-3) if itype == torch.float32 else (5e-3, 1e-2)
    if itype == torch.bfloat16:
        rtol, atol = 1e-2, 5e-2
    return rtol, atol


def _check(got, ref, rtol, atol, name):
    got, ref = got.float().cpu(), ref.float()
    err = (got - ref).abs()
    assert bool((err <= atol + rtol * ref.abs()).all()), f"{name}: max err {err.max().item():.3e}"


@pytest.mark.parametrize("itype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("has_z", [False, True])
@pytest.mark.parametrize("dstate", [16, 32, 64])
@pytest.mark.parametrize("dim", [2048, 2048 + 16, 4096])
def test_selective_state_update(dim, dstate, has_z, itype):
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    rtol, atol = _tol(itype)
    g = torch.Generator().manual_seed(0)
    batch = 2
    state = torch.randn(batch, dim, dstate, generator=g).to(itype)
    x = torch.randn(batch, dim, generator=g).to(itype)
    dt = torch.randn(batch, dim, generator=g).to(itype)
    dt_bias = torch.rand(dim, generator=g) - 4.0
    A = -torch.rand(dim, dstate, generator=g) - 1.0
    B = torch.randn(batch, dstate, generator=g)
    C = torch.randn(batch, dstate, generator=g)
    D = torch.randn(dim, generator=g)
    z = torch.randn(batch, dim, generator=g).to(itype) if has_z else None
    state_ref = state.clone()
    out_ref = selective_state_update_oracle(state_ref, x, dt, A, B, C, D=D, z=z, dt_bias=dt_bias, dt_softplus=True)
    cu = lambda t: None if t is None else t.cuda()
    state_g = state.cuda()
    out = selective_state_update(state_g, cu(x), cu(dt), cu(A), cu(B), cu(C), D=cu(D), z=cu(z), dt_bias=cu(dt_bias),
                                 dt_softplus=True)
    assert out.dtype == itype and out.shape == out_ref.shape
    _check(state_g, state_ref, rtol, atol, "state")
    _check(out, out_ref, rtol, atol, "out")


@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("has_z", [True])
@pytest.mark.parametrize("tie_hdim", [False, True])
@pytest.mark.parametrize("ngroups", [1, 2, 4])
@pytest.mark.parametrize("dstate", [16, 64, 128, 20])
@pytest.mark.parametrize("dim", [64, 50])
@pytest.mark.parametrize("with_indices", [False, True])
def test_selective_state_update_with_heads(with_indices, dim, dstate, ngroups, has_z, tie_hdim, itype):
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    rtol, atol = _tol(itype)
    if itype == torch.bfloat16:
        atol = 1e-1
    g = torch.Generator().manual_seed(0)
    batch, headdim = 3, dim
    nheads = 8
    total = batch + 4 if with_indices else batch
    state = torch.randn(total, nheads, headdim, dstate, generator=g).to(itype)
    idx = None
    if with_indices:
        idx = torch.randperm(total, generator=g)[:batch].to(torch.int32)
        idx[1] = -1  # a padding entry
    x = torch.randn(batch, nheads, headdim, generator=g).to(itype)
    if not tie_hdim:
        dt = torch.randn(batch, nheads, headdim, generator=g).to(itype)
        dt_bias = torch.rand(nheads, headdim, generator=g) - 4.0
        A = -torch.rand(nheads, headdim, dstate, generator=g) - 1.0
        D = torch.randn(nheads, headdim, generator=g)
    else:  # expanded (stride-0) per-head operands, as Mamba2.step builds them (modules/mamba2.py:324-327)
        dt = torch.randn(batch, nheads, generator=g).to(itype)[:, :, None].expand(batch, nheads, headdim)
        dt_bias = (torch.rand(nheads, generator=g) - 4.0)[:, None].expand(nheads, headdim)
        A = (-torch.rand(nheads, generator=g) - 1.0)[:, None, None].expand(nheads, headdim, dstate)
        D = torch.randn(nheads, generator=g)[:, None].expand(nheads, headdim)
    B = torch.randn(batch, ngroups, dstate, generator=g).to(itype)
    C = torch.randn(batch, ngroups, dstate, generator=g).to(itype)
    z = torch.randn(batch, nheads, headdim, generator=g).to(itype) if has_z else None
    state_ref = state.clone()
    out_ref = selective_state_update_oracle(state_ref, x, dt, A, B, C, D=D, z=z, dt_bias=dt_bias, dt_softplus=True,
                                            state_batch_indices=idx)

    def cu(t):  # keep the stride-0 expansion on the device copy
        if t is None:
            return None
        if 0 in t.stride():
            keep = [1 if s == 0 else n for n, s in zip(t.shape, t.stride())]
            base = t[tuple(slice(0, k) for k in keep)].contiguous().cuda()
            return base.expand(*t.shape)
        return t.cuda()

    state_g = state.cuda()
    out = selective_state_update(state_g, cu(x), cu(dt), cu(A), cu(B), cu(C), D=cu(D), z=cu(z), dt_bias=cu(dt_bias),
                                 dt_softplus=True, state_batch_indices=cu(idx))
    _check(state_g, state_ref, rtol, atol, "state")
    _check(out, out_ref, rtol, atol, "out")
    if with_indices:
        assert float(out[1].abs().max()) == 0.0


def test_index_past_the_state_rows_is_a_padding_entry():
    """An index >= state.shape[0] must not be written through: the entry is skipped like a negative one."""
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    g = torch.Generator().manual_seed(5)
    rows, batch, nheads, headdim, dstate = 3, 4, 2, 64, 16
    state = torch.randn(rows, nheads, headdim, dstate, generator=g)
    guard = torch.zeros(8, nheads, headdim, dstate)           # memory behind the state, must stay zero
    buf = torch.cat([state, guard]).cuda()
    state_g = buf[:rows]
    x = torch.randn(batch, nheads, headdim, generator=g)
    dt = torch.rand(batch, nheads, headdim, generator=g)
    A = -torch.rand(nheads, headdim, dstate, generator=g)
    B = torch.randn(batch, 1, dstate, generator=g)
    C = torch.randn(batch, 1, dstate, generator=g)
    idx = torch.tensor([2, 3, -1, 0], dtype=torch.int32)     # 3 == rows: out of range
    state_ref = state.clone()
    ok = torch.tensor([0, 3])
    out_ref = selective_state_update_oracle(state_ref, x, dt, A, B, C, state_batch_indices=torch.where(idx >= rows, -1, idx))
    out = selective_state_update(state_g, x.cuda(), dt.cuda(), A.cuda(), B.cuda(), C.cuda(), state_batch_indices=idx.cuda())
    _check(state_g, state_ref, 1e-4, 1e-4, "state")
    _check(out[ok], out_ref[ok], 1e-4, 1e-4, "out")
    assert float(out[1].abs().max()) == 0.0 and float(out[2].abs().max()) == 0.0
    assert float(buf[rows:].abs().max()) == 0.0


def test_decode_steps_equal_scan():
    """T decode steps reproduce a length-T selective scan (the invariant of the reference's
    tests/test_generation.py:34-43), checked end to end on the GPU ops."""
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    g = torch.Generator().manual_seed(3)
    batch, dim, dstate, T = 2, 96, 16, 40
    u = torch.randn(batch, dim, T, generator=g).cuda()
    delta = torch.randn(batch, dim, T, generator=g).cuda()
    A = (-torch.rand(dim, dstate, generator=g) - 0.5).cuda()
    B = torch.randn(batch, dstate, T, generator=g).cuda()
    C = torch.randn(batch, dstate, T, generator=g).cuda()
    D = torch.randn(dim, generator=g).cuda()
    z = torch.randn(batch, dim, T, generator=g).cuda()
    bias = (torch.rand(dim, generator=g) - 3.0).cuda()
    y_scan, last = selective_scan_fn(u, delta, A, B, C, D, z=z, delta_bias=bias, delta_softplus=True,
                                     return_last_state=True)
    state = torch.zeros(batch, dim, dstate, device="cuda")
    ys = []
    for t in range(T):
        ys.append(selective_state_update(state, u[:, :, t].contiguous(), delta[:, :, t].contiguous(), A,
                                         B[:, :, t].contiguous(), C[:, :, t].contiguous(), D=D,
                                         z=z[:, :, t].contiguous(), dt_bias=bias, dt_softplus=True))
    y_step = torch.stack(ys, dim=2)
    assert torch.allclose(y_step, y_scan, rtol=3e-4, atol=1e-3)
    assert torch.allclose(state, last, rtol=3e-4, atol=1e-3)


def test_decode_benchmark_shape():
    """The decode benchmark's shape (batch 256 is cut to 8 here): bf16 x/B/C/z, fp32 state, expanded
    per-head dt/A/dt_bias/D."""
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    g = torch.Generator().manual_seed(5)
    batch, nheads, headdim, dstate = 8, 80, 64, 128
    state = 0.1 * torch.randn(batch, nheads, headdim, dstate, generator=g)
    bf = torch.bfloat16
    x = torch.randn(batch, nheads, headdim, generator=g).to(bf)
    z = torch.randn(batch, nheads, headdim, generator=g).to(bf)
    B = torch.randn(batch, 1, dstate, generator=g).to(bf)
    C = torch.randn(batch, 1, dstate, generator=g).to(bf)
    dt = torch.randn(batch, nheads, generator=g).to(bf)
    dt_bias = torch.rand(nheads, generator=g) - 4.0
    A = -(1.0 + 15.0 * torch.rand(nheads, generator=g))
    D = torch.rand(nheads, generator=g)
    ex = lambda t, *shape: t.expand(*shape)
    args_cpu = (ex(dt[:, :, None], batch, nheads, headdim), ex(A[:, None, None], nheads, headdim, dstate), B, C)
    kw_cpu = dict(D=ex(D[:, None], nheads, headdim), z=z, dt_bias=ex(dt_bias[:, None], nheads, headdim),
                  dt_softplus=True)
    state_ref = state.clone()
    out_ref = selective_state_update_oracle(state_ref, x, *args_cpu, **kw_cpu)
    dtg, Ag, Dg, bg = dt.cuda(), A.cuda(), D.cuda(), dt_bias.cuda()
    state_g = state.cuda()
    out = selective_state_update(state_g, x.cuda(), ex(dtg[:, :, None], batch, nheads, headdim),
                                 ex(Ag[:, None, None], nheads, headdim, dstate), B.cuda(), C.cuda(),
                                 D=ex(Dg[:, None], nheads, headdim), z=z.cuda(),
                                 dt_bias=ex(bg[:, None], nheads, headdim), dt_softplus=True)
    _check(state_g, state_ref, 3e-4, 1e-3, "state")
    _check(out, out_ref, 1e-2, 1e-1, "out")


def test_decode_step_inside_a_hip_graph():
    """The decode step is what mamba_ssm/utils/generation.py:342-379 captures in a graph: capture one
    step, replay it several times with eager work in between, and compare every replay with the same
    sequence of eager steps (the op allocates nothing the graph does not own and never synchronises)."""
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    g = torch.Generator().manual_seed(0)
    batch, H, P, N = 4, 8, 64, 64
    dev = "cuda"
    state0 = torch.randn(batch, H, P, N, generator=g).to(dev)
    A = (-torch.rand(H, generator=g) - 1.0).to(dev)[:, None, None].expand(H, P, N)
    D = torch.randn(H, generator=g).to(dev)[:, None].expand(H, P)
    dtb = torch.rand(H, generator=g).to(dev)[:, None].expand(H, P)
    steps = [dict(x=torch.randn(batch, H, P, generator=g).to(dev).bfloat16(),
                  z=torch.randn(batch, H, P, generator=g).to(dev).bfloat16(),
                  dt=torch.randn(batch, H, generator=g).to(dev).bfloat16(),
                  B=torch.randn(batch, 1, N, generator=g).to(dev).bfloat16(),
                  C=torch.randn(batch, 1, N, generator=g).to(dev).bfloat16()) for _ in range(4)]
    call = lambda st, s: selective_state_update(st, s["x"], s["dt"][:, :, None].expand(batch, H, P), A, s["B"], s["C"],
                                                D=D, z=s["z"], dt_bias=dtb, dt_softplus=True)
    eager_state, eager_out = state0.clone(), []
    for s in steps:
        eager_out.append(call(eager_state, s).clone())
    # static buffers of the captured step
    gstate = state0.clone()
    buf = {k: v.clone() for k, v in steps[0].items()}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(gstate, buf)                      # warm-up on the side stream
    torch.cuda.current_stream().wait_stream(side)
    gstate.copy_(state0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gout = call(gstate, buf)
    gstate.copy_(state0)
    for i, s in enumerate(steps):
        for k in buf:
            buf[k].copy_(s[k])
        graph.replay()
        torch.cuda.synchronize()
        scratch = torch.randn(1024, device=dev).sum().item()   # eager work between replays
        assert torch.equal(gout, eager_out[i]), f"replay {i}"
    assert torch.equal(gstate, eager_state)
