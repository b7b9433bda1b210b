"""The decode-step operators inside a captured HIP graph (the reference captures its decode step the same
way, mamba_ssm/utils/generation.py:342-379): causal_conv1d_update, selective_state_update and the gated norm
are captured once and replayed with new inputs; every replay must equal the eager result, with eager work and
synchronisations of the program in between."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_decode_step_replays_match_eager():
    from mamba_amd.ops.causal_conv1d import causal_conv1d_update
    from mamba_amd.ops.triton.layernorm_gated import rmsnorm_fn
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    g = torch.Generator().manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=g).cuda()
    batch, nheads, headdim, N, ngroups, W = 4, 4, 32, 16, 1, 4
    dim = nheads * headdim
    conv_dim = dim + 2 * ngroups * N
    conv_w, conv_b = 0.4 * r(conv_dim, W), 0.1 * r(conv_dim)
    dt_bias, A, D = r(nheads) * 0.5 - 1, -(0.5 + torch.rand(nheads, generator=g)).cuda(), torch.rand(nheads, generator=g).cuda()
    norm_w = 1 + 0.1 * r(dim)

    def step(xBC, z, dt, conv_state, ssm_state):
        xc = causal_conv1d_update(xBC, conv_state, conv_w, conv_b, "silu")
        xs, B, C = torch.split(xc, [dim, ngroups * N, ngroups * N], dim=-1)
        y = selective_state_update(
            ssm_state, xs.reshape(batch, nheads, headdim), dt[:, :, None].expand(batch, nheads, headdim),
            A[:, None, None].expand(nheads, headdim, N), B.reshape(batch, ngroups, N), C.reshape(batch, ngroups, N),
            D=D[:, None].expand(nheads, headdim), dt_bias=dt_bias[:, None].expand(nheads, headdim), dt_softplus=True)
        return rmsnorm_fn(y.reshape(batch, dim), norm_w, None, z=z, eps=1e-5, norm_before_gate=False)

    inputs = [(r(batch, conv_dim), r(batch, dim), r(batch, nheads)) for _ in range(5)]
    conv0, ssm0 = 0.5 * r(batch, conv_dim, W), 0.1 * r(batch, nheads, headdim, N)
    with torch.no_grad():
        # eager: five consecutive steps from the initial states
        conv_e, ssm_e = conv0.clone(), ssm0.clone()
        want = [step(*inp, conv_e, ssm_e).clone() for inp in inputs]
        # captured: static buffers, one capture after a warm-up on a side stream
        s_xBC, s_z, s_dt = (torch.zeros_like(t) for t in inputs[0])
        conv_g, ssm_g = conv0.clone(), ssm0.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(s_xBC, s_z, s_dt, conv_g.clone(), ssm_g.clone())
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            s_out = step(s_xBC, s_z, s_dt, conv_g, ssm_g)
        conv_g.copy_(conv0)   # the capture does not run the kernels, but be explicit about the start
        ssm_g.copy_(ssm0)
        for i, inp in enumerate(inputs):
            for dst, src in zip((s_xBC, s_z, s_dt), inp):
                dst.copy_(src)
            graph.replay()
            torch.cuda.synchronize()
            got = s_out.clone()
            _ = (got.float() * 2).sum().item()          # eager work and a synchronisation between replays
            assert torch.allclose(got, want[i], rtol=1e-5, atol=1e-6), f"replay {i}: {(got - want[i]).abs().max().item():.3e}"
        assert torch.allclose(conv_g, conv_e) and torch.allclose(ssm_g, ssm_e, rtol=1e-5, atol=1e-6)
