"""GPU parity of the HIP causal conv1d against oracle/block.py:causal_conv1d_oracle (pinned on the CPU
by tests/test_oracle_block.py against F.conv1d), forward and every gradient, both memory layouts."""
import pytest
import torch

from oracle.block import causal_conv1d_oracle, causal_conv1d_update_oracle, causal_conv1d_varlen_states_oracle

pytestmark = pytest.mark.gpu


def _tol(dtype):
    return (6e-4, 2e-3) if dtype == torch.float32 else ((3e-3, 5e-3) if dtype == torch.float16 else (3e-2, 5e-2))


def _close(name, got, ref, rtol, atol):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    err = (got - ref).abs()
    assert bool((err <= atol + rtol * ref.abs()).all()), f"{name}: max err {err.max().item():.3e}, ref max {ref.abs().max().item():.3e}"


def _case(batch, dim, seqlen, width, dtype, channel_last, has_bias=True, activation="silu", seq_lens=None, seed=0):
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fn
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(batch, seqlen, dim, generator=g).to(dtype)           # (b, l, d)
    w = (torch.randn(dim, width, generator=g) * 0.5).to(dtype)
    bias = torch.randn(dim, generator=g).to(dtype) if has_bias else None
    dout = torch.randn(batch, seqlen, dim, generator=g).to(dtype)
    seq_idx = None
    if seq_lens is not None:
        seq_idx = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(seq_lens)])[None].repeat(batch, 1)
    rtol, atol = _tol(dtype)
    # oracle in fp32 on the same (rounded) inputs
    xr, wr = x.float().clone().requires_grad_(), w.float().clone().requires_grad_()
    br = bias.float().clone().requires_grad_() if has_bias else None
    ref = causal_conv1d_oracle(xr, wr, br, activation, seq_idx)
    (ref * dout.float()).sum().backward()
    xg = x.cuda()
    xg = (xg.transpose(1, 2) if channel_last else xg.transpose(1, 2).contiguous()).requires_grad_()  # (b, d, l)
    wg = w.cuda().requires_grad_()
    bg = bias.cuda().requires_grad_() if has_bias else None
    out = causal_conv1d_fn(xg, wg, bg, seq_idx=seq_idx.cuda() if seq_idx is not None else None, activation=activation)
    assert out.shape == (batch, dim, seqlen) and out.dtype == dtype
    assert (out.stride(1) == 1) == (xg.stride(1) == 1 and xg.stride(2) != 1) or seqlen == 1 or dim == 1
    _close("out", out.transpose(1, 2), ref, rtol, atol)
    dg = dout.cuda().transpose(1, 2)
    out.backward(dg if channel_last else dg.contiguous())
    scale = max(1.0, float(wr.grad.abs().max()))
    _close("dx", xg.grad.transpose(1, 2), xr.grad, rtol * 2, atol * 2)
    _close("dweight", wg.grad, wr.grad, rtol * 2, atol * 2 * scale)
    if has_bias:
        _close("dbias", bg.grad, br.grad, rtol * 2, atol * 2 * max(1.0, float(br.grad.abs().max())))


@pytest.mark.parametrize("channel_last", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("seqlen,dim", [(64, 16), (200, 24), (1, 8), (2048 + 24, 8), (333, 20)])
def test_causal_conv1d(seqlen, dim, dtype, channel_last):
    _case(2, dim, seqlen, 4, dtype, channel_last)


@pytest.mark.parametrize("channel_last", [False, True])
@pytest.mark.parametrize("width", [2, 3, 4])
@pytest.mark.parametrize("has_bias,activation", [(True, None), (False, "silu"), (False, None)])
def test_causal_conv1d_options(width, has_bias, activation, channel_last):
    _case(2, 40, 150, width, torch.float32, channel_last, has_bias=has_bias, activation=activation)


@pytest.mark.parametrize("channel_last", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_causal_conv1d_packed_sequences(dtype, channel_last):
    _case(1, 32, 256, 4, dtype, channel_last, seq_lens=[1, 2, 61, 64, 3, 125])
    _case(2, 24, 100, 3, dtype, channel_last, seq_lens=[50, 50])


def test_causal_conv1d_strided_view():
    # the xBC slice of a wider projection output: channel-contiguous rows with a larger position stride
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fn
    g = torch.Generator().manual_seed(3)
    full = torch.randn(2, 96, 80, generator=g).to(torch.bfloat16)
    w = (torch.randn(48, 4, generator=g) * 0.5).to(torch.bfloat16)
    ref = causal_conv1d_oracle(full[:, :, 16:64].float(), w.float(), None, "silu")
    out = causal_conv1d_fn(full.cuda()[:, :, 16:64].transpose(1, 2), w.cuda(), None, activation="silu")
    _close("out", out.transpose(1, 2), ref, 3e-2, 5e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("channel_last_state", [False, True])
@pytest.mark.parametrize("width,state_len,seqlen", [(4, 4, 1), (4, 3, 1), (3, 3, 1), (2, 1, 1), (4, 7, 3), (4, 4, 6), (2, 5, 2)])
def test_causal_conv1d_update(width, state_len, seqlen, channel_last_state, dtype):
    from mamba_amd.ops.causal_conv1d import causal_conv1d_update
    g = torch.Generator().manual_seed(width * 100 + state_len * 10 + seqlen)
    batch, dim = 3, 200
    x = torch.randn(batch, dim, seqlen, generator=g).to(dtype)
    state = torch.randn(batch, dim, state_len, generator=g).to(dtype)
    w = (torch.randn(dim, width, generator=g) * 0.5).to(dtype)
    bias = torch.randn(dim, generator=g).to(dtype)
    rtol, atol = _tol(dtype)
    ref, new_ref = causal_conv1d_update_oracle(x.float(), state.float(), w.float(), bias.float(), "silu")
    sg = state.cuda()
    if channel_last_state:  # the layout the Mamba-2 module allocates (mamba_ssm/modules/mamba2.py:333-335)
        sg = sg.transpose(1, 2).contiguous().transpose(1, 2)
    xg = x.cuda() if seqlen > 1 else x.cuda()[:, :, 0]
    out = causal_conv1d_update(xg, sg, w.cuda(), bias.cuda(), "silu")
    assert out.shape == xg.shape and out.dtype == dtype
    _close("out", out.reshape(batch, dim, seqlen), ref, rtol, atol)
    assert torch.equal(sg.cpu(), new_ref.to(dtype))  # the state only moves values


def test_causal_conv1d_update_steps_match_the_sequence_kernel_and_indices():
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fn, causal_conv1d_update
    g = torch.Generator().manual_seed(3)
    batch, dim, L, width = 4, 96, 9, 4
    x = torch.randn(batch, dim, L, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(dim, width, generator=g) * 0.5).cuda()
    bias = torch.randn(dim, generator=g).cuda()
    full = causal_conv1d_fn(x, w, bias, activation="silu")
    # states live in a pool of 7 rows; entry 2 of the batch is padding
    pool = torch.zeros(7, dim, width, dtype=torch.bfloat16, device="cuda")
    idx = torch.tensor([5, 0, -1, 3], dtype=torch.int32, device="cuda")
    untouched = pool.clone()
    for t in range(L):
        out = causal_conv1d_update(x[:, :, t], pool, w, bias, "silu", conv_state_indices=idx)
        keep = [0, 1, 3]
        _close(f"step {t}", out[keep], full[keep, :, t], 3e-2, 5e-2)
        assert float(out[2].abs().max()) == 0.0
    assert torch.equal(pool[[1, 2, 4, 6]], untouched[[1, 2, 4, 6]])
    assert torch.equal(pool[5], x[0, :, L - width:])
    with pytest.raises(NotImplementedError):
        causal_conv1d_update(x[:, :, 0], pool[:4], w, bias, "silu", cache_seqlens=idx)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_causal_conv1d_varlen_states(dtype):
    from mamba_amd.ops.causal_conv1d import causal_conv1d_varlen_states
    g = torch.Generator().manual_seed(4)
    lens = [5, 1, 2, 300, 4, 3]
    total, dim = sum(lens), 520
    x = torch.randn(total, dim + 8, generator=g).to(dtype)[:, :dim]          # rows of a wider buffer
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    for state_len in (3, 4):
        ref = causal_conv1d_varlen_states_oracle(x, cu, state_len)
        got = causal_conv1d_varlen_states(x.cuda(), cu.cuda(), state_len)
        assert got.shape == (len(lens), dim, state_len) and got.stride(1) == 1
        assert torch.equal(got.cpu(), ref)
