"""Prefill + token-by-token decode against one pass over the whole sequence, for a Mamba-2 layer and a
Mamba-1 layer built from this package's operators the way the reference's modules chain them
(mamba_ssm/modules/mamba2.py:183-330 forward / step, mamba_ssm/modules/mamba_simple.py:119-262): the block
operator with final states, the convolution states of the prefill, then causal_conv1d_update +
selective_state_update (+ gated norm) per token must reproduce the outputs of the one-pass call."""
import math

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def _close(name, got, ref, rtol, atol):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    err = (got - ref).abs()
    assert bool((err <= atol + rtol * ref.abs()).all()), f"{name}: max err {err.max().item():.3e}, ref max {ref.abs().max().item():.3e}"


@pytest.mark.parametrize("dtype,rtol,atol", [(torch.float32, 2e-3, 2e-3), (torch.bfloat16, 3e-2, 5e-2)])
@pytest.mark.parametrize("ngroups", [1, 2])
def test_mamba2_layer_prefill_then_decode(ngroups, dtype, rtol, atol):
    from mamba_amd.ops.causal_conv1d import causal_conv1d_update, causal_conv1d_varlen_states
    from mamba_amd.ops.triton.layernorm_gated import rmsnorm_fn
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    from mamba_amd.ops.triton.ssd_combined import mamba_split_conv1d_scan_combined
    g = torch.Generator().manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=g)
    batch, L, k, d_model, headdim, nheads, N, W, chunk = 2, 150, 9, 64, 32, 4, 16, 4, 64
    dim = nheads * headdim
    conv_dim = dim + 2 * ngroups * N
    w_in = (r(2 * dim + 2 * ngroups * N + nheads, d_model) / math.sqrt(d_model)).cuda().to(dtype)
    conv_w, conv_b = (0.4 * r(conv_dim, W)).cuda(), (0.1 * r(conv_dim)).cuda()
    dt_bias, A, D = (r(nheads) * 0.5 - 1).cuda(), (-(0.5 + torch.rand(nheads, generator=g))).cuda(), torch.rand(nheads, generator=g).cuda()
    norm_w = (1 + 0.1 * r(dim)).cuda()
    w_out = (r(d_model, dim) / math.sqrt(dim)).cuda().to(dtype)
    x = r(batch, L, d_model).cuda().to(dtype)
    kw = dict(rmsnorm_weight=norm_w, rmsnorm_eps=1e-5, outproj_weight=w_out, headdim=headdim, ngroups=ngroups,
              norm_before_gate=False)
    with torch.no_grad():
        zxbcdt = F.linear(x, w_in)
        full = mamba_split_conv1d_scan_combined(zxbcdt, conv_w, conv_b, dt_bias, A, D, chunk, **kw)
        L0 = L - k
        head, ssm_state = mamba_split_conv1d_scan_combined(zxbcdt[:, :L0], conv_w, conv_b, dt_bias, A, D, chunk,
                                                           return_final_states=True, **kw)
        _close("prefill", head, full[:, :L0], rtol, atol)
        # convolution state of the prefill: its last W inputs, per batch row (mamba2.py:216-221)
        xBC_pre = zxbcdt[:, :L0, dim:dim + conv_dim]
        cu = torch.tensor([0, L0], dtype=torch.int32, device="cuda")
        conv_state = torch.cat([causal_conv1d_varlen_states(xBC_pre[b], cu, W) for b in range(batch)])
        assert conv_state.shape == (batch, conv_dim, W)
        ssm_state = ssm_state.clone()
        outs = []
        for t in range(L0, L):
            z, xBC, dt = torch.split(zxbcdt[:, t], [dim, conv_dim, nheads], dim=-1)
            xBC = causal_conv1d_update(xBC, conv_state, conv_w, conv_b, "silu")
            xs, B, C = torch.split(xBC, [dim, ngroups * N, ngroups * N], dim=-1)
            y = selective_state_update(
                ssm_state, xs.reshape(batch, nheads, headdim), dt[:, :, None].expand(batch, nheads, headdim),
                A[:, None, None].expand(nheads, headdim, N), B.reshape(batch, ngroups, N), C.reshape(batch, ngroups, N),
                D=D[:, None].expand(nheads, headdim), z=None, dt_bias=dt_bias[:, None].expand(nheads, headdim),
                dt_softplus=True)
            y = rmsnorm_fn(y.reshape(batch, dim), norm_w, None, z=z.contiguous(), eps=1e-5, group_size=dim // ngroups,
                           norm_before_gate=False)
            outs.append(F.linear(y, w_out))
        _close("decode", torch.stack(outs, dim=1), full[:, L0:], rtol, atol)


@pytest.mark.parametrize("dtype,rtol,atol", [(torch.float32, 2e-3, 2e-3), (torch.bfloat16, 3e-2, 5e-2)])
def test_mamba1_layer_prefill_then_decode(dtype, rtol, atol):
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fn, causal_conv1d_update
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    g = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=g)
    batch, L, k, d_inner, N, R, W = 2, 90, 7, 96, 16, 6, 4
    conv_w, conv_b = (0.4 * r(d_inner, W)).cuda(), (0.1 * r(d_inner)).cuda()
    x_proj = (r(R + 2 * N, d_inner) / math.sqrt(d_inner)).cuda().to(dtype)
    dt_proj = (r(d_inner, R) / math.sqrt(R)).cuda().to(dtype)
    dt_bias = (r(d_inner) * 0.5 - 1).cuda()
    A = (-torch.arange(1, N + 1, dtype=torch.float32)[None].repeat(d_inner, 1)).cuda()
    D = torch.ones(d_inner).cuda()
    xz = r(batch, 2 * d_inner, L).cuda().to(dtype)

    def layer(xz_part, conv_state=None, ssm_state=None):
        """mamba_simple.py:144-196 without the in / out projections: returns y (b, d, l) and the last state."""
        xs, z = xz_part.chunk(2, dim=1)
        xc = causal_conv1d_fn(xs, conv_w, conv_b, activation="silu")
        x_dbl = F.linear(xc.transpose(1, 2), x_proj)
        dt = (dt_proj @ x_dbl[..., :R].transpose(1, 2))
        B = x_dbl[..., R:R + N].transpose(1, 2).contiguous()
        C = x_dbl[..., R + N:].transpose(1, 2).contiguous()
        return selective_scan_fn(xc, dt.to(dtype), A, B, C, D, z=z, delta_bias=dt_bias, delta_softplus=True,
                                 return_last_state=True)

    with torch.no_grad():
        full, _ = layer(xz)
        L0 = L - k
        head, ssm_state = layer(xz[:, :, :L0])
        _close("prefill", head, full[:, :, :L0], rtol, atol)
        conv_state = F.pad(xz[:, :d_inner, :L0], (W - L0, 0)).contiguous()          # mamba_simple.py:158
        ssm_state = ssm_state.clone()
        outs = []
        for t in range(L0, L):
            xs, z = xz[:, :, t].chunk(2, dim=1)
            xc = causal_conv1d_update(xs, conv_state, conv_w, conv_b, "silu")
            x_db = F.linear(xc, x_proj)
            dt = F.linear(x_db[:, :R], dt_proj)
            y = selective_state_update(ssm_state, xc, dt, A, x_db[:, R:R + N], x_db[:, R + N:], D, z=z,
                                       dt_bias=dt_bias, dt_softplus=True)
            outs.append(y)
        _close("decode", torch.stack(outs, dim=2), full[:, :, L0:], rtol, atol)


def test_mamba2_packed_prefill_then_one_decode_step_per_sequence():
    """Variable-length inference (mamba2.py:216-228, :255-262): three sequences packed into one row are prefilled
    with seq_idx / cu_seqlens, the per-sequence scan and convolution states land in a pool of state rows, and one
    more token per sequence is decoded as a batch through the pool indices; each must equal position len_i of a
    one-pass call on that sequence alone."""
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fn, causal_conv1d_update, causal_conv1d_varlen_states
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    g = torch.Generator().manual_seed(2)
    r = lambda *s: torch.randn(*s, generator=g)
    lens, nheads, headdim, N, ngroups, W, chunk = [70, 33, 129], 4, 32, 16, 1, 4, 64
    dim, total = nheads * headdim, sum(lens)
    conv_dim = dim + 2 * ngroups * N
    conv_w, conv_b = (0.4 * r(conv_dim, W)).cuda(), (0.1 * r(conv_dim)).cuda()
    dt_bias, A, D = (r(nheads) * 0.5 - 1).cuda(), (-(0.5 + torch.rand(nheads, generator=g))).cuda(), torch.rand(nheads, generator=g).cuda()
    # inputs after in_proj, one token more than the prefill per sequence
    seqs = [dict(xBC=r(n + 1, conv_dim).cuda(), dt=r(n + 1, nheads).cuda()) for n in lens]

    def scan(xBC, dt, **kw):
        xc = causal_conv1d_fn(xBC.transpose(0, 1)[None], conv_w, conv_b, activation="silu", seq_idx=kw.get("seq_idx"))[0].transpose(0, 1)
        xs, B, C = torch.split(xc, [dim, ngroups * N, ngroups * N], dim=-1)
        return mamba_chunk_scan_combined(xs.reshape(1, -1, nheads, headdim), dt[None], A, B.reshape(1, -1, ngroups, N),
                                         C.reshape(1, -1, ngroups, N), chunk, D=D, dt_bias=dt_bias, dt_softplus=True, **kw)

    with torch.no_grad():
        want = torch.stack([scan(s["xBC"], s["dt"])[0, -1] for s in seqs])                 # (nseq, h, p): the extra token
        xBC_pack = torch.cat([s["xBC"][:-1] for s in seqs])
        dt_pack = torch.cat([s["dt"][:-1] for s in seqs])
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device="cuda")
        seq_idx = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(lens)])[None].cuda()
        _, varlen_states = scan(xBC_pack, dt_pack, seq_idx=seq_idx, cu_seqlens=cu, return_varlen_states=True)
        assert varlen_states.shape == (3, nheads, headdim, N)
        # pools of 5 state rows; the three sequences live in rows 4, 0, 2
        rows = torch.tensor([4, 0, 2], dtype=torch.int32, device="cuda")
        ssm_pool = torch.zeros(5, nheads, headdim, N, device="cuda")
        conv_pool = torch.zeros(5, conv_dim, W, device="cuda")
        ssm_pool[rows.long()] = varlen_states.float()
        conv_pool[rows.long()] = causal_conv1d_varlen_states(xBC_pack, cu, W)
        xBC_new = torch.stack([s["xBC"][-1] for s in seqs])
        dt_new = torch.stack([s["dt"][-1] for s in seqs])
        xc = causal_conv1d_update(xBC_new, conv_pool, conv_w, conv_b, "silu", conv_state_indices=rows)
        xs, B, C = torch.split(xc, [dim, ngroups * N, ngroups * N], dim=-1)
        got = selective_state_update(
            ssm_pool, xs.reshape(3, nheads, headdim), dt_new[:, :, None].expand(3, nheads, headdim),
            A[:, None, None].expand(nheads, headdim, N), B.reshape(3, ngroups, N), C.reshape(3, ngroups, N),
            D=D[:, None].expand(nheads, headdim), dt_bias=dt_bias[:, None].expand(nheads, headdim), dt_softplus=True,
            state_batch_indices=rows)
        _close("decode after packed prefill", got, want, 2e-3, 2e-3)
        assert float(ssm_pool[[1, 3]].abs().max()) == 0.0 and float(conv_pool[[1, 3]].abs().max()) == 0.0
