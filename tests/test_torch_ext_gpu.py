"""The C++ host side of the decode-step operators (mamba_amd/_torch_ext.so) against the Python + ctypes
host side: both fill the same parameter structs for the same kernels, so outputs and updated states
must agree bit for bit, and whatever the C++ side declines must still be served by the Python side."""
import pytest
import torch

from mamba_amd import _lib

pytestmark = pytest.mark.gpu


@pytest.fixture
def ext():
    e = _lib.torch_ext()
    if e is None:
        pytest.fail("mamba_amd/_torch_ext.so is not built (python -m mamba_amd.build)")
    return e


def _python_path(fn, *a, **k):
    saved = _lib._torch_ext
    _lib._torch_ext = None
    try:
        return fn(*a, **k)
    finally:
        _lib._torch_ext = saved


@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("has_heads", [False, True])
@pytest.mark.parametrize("tie_hdim", [False, True])
@pytest.mark.parametrize("has_z", [False, True])
def test_state_update_same_bits(ext, itype, has_heads, tie_hdim, has_z):
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    torch.manual_seed(0)
    dev, batch, H, P, N, G = "cuda", 3, 4, 64, 16, 2
    if has_heads:
        state = torch.randn(batch, H, P, N, device=dev, dtype=itype)
        x = torch.randn(batch, H, P, device=dev, dtype=itype)
        if tie_hdim:
            dt = torch.randn(batch, H, device=dev, dtype=itype)[:, :, None].expand(batch, H, P)
            A = (-torch.rand(H, device=dev) - 1.0)[:, None, None].expand(H, P, N)
            dt_bias = (torch.rand(H, device=dev) - 4.0)[:, None].expand(H, P)
            D = torch.randn(H, device=dev)[:, None].expand(H, P)
        else:
            dt = torch.randn(batch, H, P, device=dev, dtype=itype)
            A = -torch.rand(H, P, N, device=dev) - 1.0
            dt_bias = torch.rand(H, P, device=dev) - 4.0
            D = torch.randn(H, P, device=dev)
        B = torch.randn(batch, G, N, device=dev, dtype=itype)
        C = torch.randn(batch, G, N, device=dev, dtype=itype)
    else:
        state = torch.randn(batch, P, N, device=dev, dtype=itype)
        x = torch.randn(batch, P, device=dev, dtype=itype)
        dt = torch.randn(batch, P, device=dev, dtype=itype)
        A = -torch.rand(P, N, device=dev) - 1.0
        dt_bias = torch.rand(P, device=dev) - 4.0
        D = torch.randn(P, device=dev)
        B = torch.randn(batch, N, device=dev, dtype=itype)
        C = torch.randn(batch, N, device=dev, dtype=itype)
    z = torch.randn_like(x) if has_z else None
    s1, s2 = state.clone(), state.clone()
    assert ext.selective_state_update(s1.clone(), x, dt, A, B, C, D, z, dt_bias, True, None) is not None, "declined"
    out1 = selective_state_update(s1, x, dt, A, B, C, D=D, z=z, dt_bias=dt_bias, dt_softplus=True)
    out2 = _python_path(selective_state_update, s2, x, dt, A, B, C, D=D, z=z, dt_bias=dt_bias, dt_softplus=True)
    assert out1.shape == out2.shape and out1.stride() == out2.stride()
    assert torch.equal(out1, out2) and torch.equal(s1, s2)


def test_state_update_indices_and_declines(ext):
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    torch.manual_seed(1)
    dev, batch, rows, H, P, N = "cuda", 4, 9, 2, 32, 16
    state = torch.randn(rows, H, P, N, device=dev)
    x = torch.randn(batch, H, P, device=dev)
    dt = torch.randn(batch, H, P, device=dev)
    A = -torch.rand(H, P, N, device=dev) - 1.0
    B = torch.randn(batch, 1, N, device=dev)
    C = torch.randn(batch, 1, N, device=dev)
    idx = torch.tensor([5, 0, 20, 7], device=dev, dtype=torch.int32)  # 20: a padding entry
    s1, s2 = state.clone(), state.clone()
    out1 = selective_state_update(s1, x, dt, A, B, C, state_batch_indices=idx)
    out2 = _python_path(selective_state_update, s2, x, dt, A, B, C, state_batch_indices=idx)
    assert torch.equal(out1, out2) and torch.equal(s1, s2)
    # declined by the C++ side, served by the Python side: int64 indices, fp64 A, CPU tensors, wrong shapes
    assert ext.selective_state_update(s1, x, dt, A, B, C, None, None, None, False, idx.long()) is None
    assert ext.selective_state_update(s1, x, dt, A.double(), B, C, None, None, None, False, idx) is None
    assert ext.selective_state_update(s1.cpu(), x.cpu(), dt.cpu(), A.cpu(), B.cpu(), C.cpu(), None, None, None, False,
                                      None) is None
    assert ext.selective_state_update(s1, x[:, :1], dt, A, B, C, None, None, None, False, idx) is None
    out3 = selective_state_update(s1.clone(), x, dt, A, B, C, state_batch_indices=idx.long())
    out4 = _python_path(selective_state_update, s2.clone(), x, dt, A, B, C, state_batch_indices=idx.long())
    assert torch.equal(out3, out4)
    with pytest.raises(AssertionError):
        selective_state_update(s1, x[:, :1], dt, A, B, C, state_batch_indices=idx)
    with pytest.raises(RuntimeError):
        selective_state_update(s1.cpu(), x.cpu(), dt.cpu(), A.cpu(), B.cpu(), C.cpu())


@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [2, 4])
@pytest.mark.parametrize("form", ["plain", "indices", "circular", "several_positions", "channel_last_state"])
def test_conv_update_same_bits(ext, itype, width, form):
    from mamba_amd.ops.causal_conv1d import causal_conv1d_update
    torch.manual_seed(2)
    dev, batch, dim, state_len = "cuda", 5, 96, 5
    weight = torch.randn(dim, width, device=dev)
    bias = torch.randn(dim, device=dev)
    rows = 11 if form == "indices" else batch
    if form == "channel_last_state":
        conv_state = torch.randn(rows, state_len, dim, device=dev, dtype=itype).transpose(1, 2)
    else:
        conv_state = torch.randn(rows, dim, state_len, device=dev, dtype=itype)
    x = torch.randn(batch, dim, 3, device=dev, dtype=itype) if form == "several_positions" else \
        torch.randn(batch, dim, device=dev, dtype=itype)
    kw = {}
    if form == "indices":
        kw["conv_state_indices"] = torch.tensor([3, 10, -1, 0, 7], device=dev, dtype=torch.int32)
    if form == "circular":
        kw["cache_seqlens"] = torch.tensor([0, 4, 9, 13, 2], device=dev, dtype=torch.int32)
    c1, c2 = conv_state.clone(), conv_state.clone()  # clone keeps the strides of a dense tensor
    assert c1.stride() == conv_state.stride()
    out1 = causal_conv1d_update(x, c1, weight, bias, "silu", **kw)
    out2 = _python_path(causal_conv1d_update, x, c2, weight, bias, "silu", **kw)
    assert out1.shape == out2.shape and torch.equal(out1, out2) and torch.equal(c1, c2)
    # weights that need a conversion go through the Python side and give the same result as their fp32 copies
    wh = weight.to(torch.bfloat16)
    c3, c4 = conv_state.clone(), conv_state.clone()
    out3 = causal_conv1d_update(x, c3, wh, bias, None, **kw)
    out4 = _python_path(causal_conv1d_update, x, c4, wh.float(), bias, None, **kw)
    assert torch.equal(out3, out4) and torch.equal(c3, c4)
