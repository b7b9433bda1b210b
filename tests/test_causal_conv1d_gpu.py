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


@pytest.mark.parametrize("seq_lens", [None, [500, 574]])
def test_causal_conv1d_channel_last_long_runs(seq_lens):
    """A channel-last problem large enough for the backward kernel's long runs (128 positions per thread): a ragged
    length, so that the last run of every row is cut short, with and without packed sequences."""
    _case(11, 4096, 1074, 4, torch.bfloat16, True, seq_lens=seq_lens, seed=3)


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
    with pytest.raises(RuntimeError):   # cache_seqlens must be int32 of the batch's length
        causal_conv1d_update(x[:, :, 0], pool[:4], w, bias, "silu", cache_seqlens=idx[:2])


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


@pytest.mark.parametrize("channel_last", [False, True])
@pytest.mark.parametrize("width,seqlen", [(4, 64), (3, 17), (4, 2), (2, 1)])
def test_causal_conv1d_streaming_states(width, seqlen, channel_last):
    """initial_states / return_final_states: a row cut in two and convolved piece by piece, the second piece
    starting from the first one's final states, equals the row convolved whole (outputs and every gradient);
    checked against F.conv1d over the joined row."""
    import torch.nn.functional as F
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fn
    g = torch.Generator().manual_seed(width * 100 + seqlen)
    batch, dim = 2, 24
    x = torch.randn(batch, dim, seqlen, generator=g)
    init = torch.randn(batch, dim, width - 1, generator=g)
    w, bias = 0.5 * torch.randn(dim, width, generator=g), torch.randn(dim, generator=g)
    dout = torch.randn(batch, dim, seqlen, generator=g)
    xr, ir, wr, br = (t.clone().requires_grad_() for t in (x, init, w, bias))
    ref = F.silu(F.conv1d(torch.cat([ir, xr], dim=2), wr[:, None, :], br, groups=dim))
    (ref * dout).sum().backward()
    lay = (lambda t: t.cuda().transpose(1, 2).contiguous().transpose(1, 2)) if channel_last else (lambda t: t.cuda())
    xg, ig = lay(x).requires_grad_(), lay(init).requires_grad_()
    wg, bg = w.cuda().requires_grad_(), bias.cuda().requires_grad_()
    out, fin = causal_conv1d_fn(xg, wg, bg, initial_states=ig, return_final_states=True, activation="silu")
    (out * dout.cuda()).sum().backward()
    _close("out", out, ref, 6e-4, 2e-3)
    _close("final_states", fin, torch.cat([init, x], dim=2)[:, :, -(width - 1):], 0, 0)
    for name, a, b in (("dx", xg.grad, xr.grad), ("dinitial_states", ig.grad, ir.grad), ("dweight", wg.grad, wr.grad),
                       ("dbias", bg.grad, br.grad)):
        _close(name, a, b, 6e-4, 2e-3)
    # without initial states the final states are the row's own tail, zero-filled on the left
    out2, fin2 = causal_conv1d_fn(xg.detach(), wg.detach(), bg.detach(), return_final_states=True, activation="silu")
    want = F.pad(x, (max(width - 1 - seqlen, 0), 0))[:, :, -(width - 1):]
    _close("final_states without initial", fin2, want, 0, 0)
    buf = torch.empty(batch, dim, width - 1, device="cuda")
    causal_conv1d_fn(xg.detach(), wg.detach(), bg.detach(), final_states_out=buf, activation="silu")
    _close("final_states_out", buf, want, 0, 0)


@pytest.mark.parametrize("channel_last", [False, True])
def test_causal_conv1d_initial_states_with_seq_idx(channel_last):
    """A packed row that continues a sequence (a prefill cut into pieces): initial_states carry the last width - 1
    positions of the row's first sequence, seq_idx separates the sequences.  Checked against F.conv1d per
    sequence, the first one convolved behind the carried positions, with every gradient.  (No call site of the
    reference passes both arguments and the causal_conv1d package's own tests are not in it: this combination is
    pinned by that arithmetic, not by a reference vector.)"""
    import torch.nn.functional as F
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fn
    g = torch.Generator().manual_seed(11)
    batch, dim, width, lens = 2, 16, 4, [5, 2, 30, 11]
    L = sum(lens)
    x = torch.randn(batch, dim, L, generator=g)
    init = torch.randn(batch, dim, width - 1, generator=g)
    w, bias = 0.5 * torch.randn(dim, width, generator=g), torch.randn(dim, generator=g)
    dout = torch.randn(batch, dim, L, generator=g)
    seq_idx = torch.cat([torch.full((n,), i + 3, dtype=torch.int32) for i, n in enumerate(lens)])[None].expand(batch, L).contiguous()
    xr, ir, wr, br = (t.clone().requires_grad_() for t in (x, init, w, bias))
    pieces, start = [], 0
    for i, n in enumerate(lens):
        seg = xr[:, :, start:start + n]
        front = ir if i == 0 else torch.zeros(batch, dim, width - 1)
        pieces.append(F.silu(F.conv1d(torch.cat([front, seg], dim=2), wr[:, None, :], br, groups=dim)))
        start += n
    ref = torch.cat(pieces, dim=2)
    (ref * dout).sum().backward()
    lay = (lambda t: t.cuda().transpose(1, 2).contiguous().transpose(1, 2)) if channel_last else (lambda t: t.cuda())
    xg, ig = lay(x).requires_grad_(), lay(init).requires_grad_()
    wg, bg = w.cuda().requires_grad_(), bias.cuda().requires_grad_()
    out, fin = causal_conv1d_fn(xg, wg, bg, seq_idx=seq_idx.cuda(), initial_states=ig, return_final_states=True,
                                activation="silu")
    (out * dout.cuda()).sum().backward()
    _close("out", out, ref, 6e-4, 2e-3)
    _close("final_states", fin, x[:, :, -(width - 1):], 0, 0)
    for name, a, b in (("dx", xg.grad, xr.grad), ("dinitial_states", ig.grad, ir.grad), ("dweight", wg.grad, wr.grad),
                       ("dbias", bg.grad, br.grad)):
        _close(name, a, b, 6e-4, 2e-3)


@pytest.mark.parametrize("width,state_len", [(4, 4), (4, 7), (3, 2), (2, 5)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_causal_conv1d_update_circular_buffer(width, state_len, dtype):
    """cache_seqlens: the conv state as a circular buffer.  Tokens fed one at a time (and two at a time) through
    the circular form must equal the shifting form fed the same tokens, at every step and for batch entries
    that stand at different positions."""
    from mamba_amd.ops.causal_conv1d import causal_conv1d_update
    g = torch.Generator().manual_seed(width * 10 + state_len)
    batch, dim, steps = 3, 40, 11
    w, bias = (0.5 * torch.randn(dim, width, generator=g)).to(dtype).cuda(), torch.randn(dim, generator=g).to(dtype).cuda()
    xs = torch.randn(steps, batch, dim, generator=g).to(dtype).cuda()
    start = torch.tensor([0, 5, 9], dtype=torch.int32)       # positions the entries have already seen
    shift_state = torch.zeros(batch, dim, state_len, dtype=dtype, device="cuda")
    ring_state = torch.zeros(batch, dim, state_len, dtype=dtype, device="cuda")
    lens = start.clone().cuda()
    for t in range(steps):
        want = causal_conv1d_update(xs[t], shift_state, w, bias, "silu")
        got = causal_conv1d_update(xs[t], ring_state, w, bias, "silu", cache_seqlens=lens)
        assert torch.equal(got, want), f"step {t}"
        lens += 1
    # the ring holds the same last positions, rotated by each entry's own count
    for b in range(batch):
        n = int(lens[b])
        for k in range(min(state_len, steps)):
            assert torch.equal(ring_state[b, :, (n - 1 - k) % state_len], shift_state[b, :, state_len - 1 - k])
    # two tokens per call
    ring2 = torch.zeros_like(ring_state)
    shift2 = torch.zeros_like(shift_state)
    lens2 = start.clone().cuda()
    for t in range(0, steps - 1, 2):
        pair = xs[t:t + 2].permute(1, 2, 0).contiguous()      # (batch, dim, 2)
        want = causal_conv1d_update(pair, shift2, w, bias, "silu")
        got = causal_conv1d_update(pair, ring2, w, bias, "silu", cache_seqlens=lens2)
        assert torch.equal(got, want), f"pair at {t}"
        lens2 += 2
