"""GPU parity of the HIP causal conv1d against oracle/block.py:causal_conv1d_oracle (pinned on the CPU
by tests/test_oracle_block.py against F.conv1d), forward and every gradient, both memory layouts."""
import pytest
import torch

from oracle.block import causal_conv1d_oracle

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
