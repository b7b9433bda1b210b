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


# ------------------------------------------------------------------ training operators
@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("var_bc,has_z,groups", [(True, True, 1), (True, False, 2), (False, True, 1)])
def test_selective_scan_same_bits(ext, itype, var_bc, has_z, groups):
    """selective_scan fwd / bwd through the C++ host side and through Python + ctypes: same kernels on the same
    structs, so every output is the same bit for bit (the Mamba-1 backward pass has no atomics)."""
    from mamba_amd.ops.selective_scan_interface import selective_scan_fwd, selective_scan_bwd
    torch.manual_seed(2)
    dev, batch, dim, L, N = "cuda", 2, 96, 300, 16
    u, delta, dout = (torch.randn(batch, dim, L, device=dev).to(itype) for _ in range(3))
    z = torch.randn(batch, dim, L, device=dev).to(itype) if has_z else None
    A = -torch.rand(dim, N, device=dev) - 0.5
    mk = (lambda: torch.randn(batch, groups, N, L, device=dev).to(itype)) if var_bc else (lambda: torch.randn(dim, N, device=dev))
    B, C = mk(), mk()
    D, bias = torch.randn(dim, device=dev), torch.rand(dim, device=dev) - 4
    assert ext.scan_fwd(u, delta, A, B, C, D, z, bias, True) is not None, "declined"
    out1, ck1 = selective_scan_fwd(u, delta, A, B, C, D, z, bias, True)
    out2, ck2 = _python_path(selective_scan_fwd, u, delta, A, B, C, D, z, bias, True)
    assert torch.equal(out1, out2) and torch.equal(ck1, ck2)
    assert ext.scan_bwd(u, delta, A, B, C, D, z, bias, dout, ck1, None, True, has_z) is not None, "declined"
    r1 = selective_scan_bwd(u, delta, A, B, C, D, z, bias, dout, ck1, None, True, has_z)
    r2 = _python_path(selective_scan_bwd, u, delta, A, B, C, D, z, bias, dout, ck1, None, True, has_z)
    assert len(r1) == len(r2) == 9
    for i, (a, b) in enumerate(zip(r1, r2)):
        assert (a is None) == (b is None), i
        if a is not None:
            assert a.dtype == b.dtype and a.shape == b.shape and torch.equal(a, b), i


def test_selective_scan_declines_what_python_reports(ext):
    """A complex A, a mismatched dtype or a transposed row are not served in C++: the call returns None and the
    Python host side handles (or reports) the case."""
    dev, batch, dim, L, N = "cuda", 1, 32, 64, 8
    u, delta = (torch.randn(batch, dim, L, device=dev) for _ in range(2))
    A = -torch.rand(dim, N, device=dev)
    B, C = (torch.randn(batch, 1, N, L, device=dev) for _ in range(2))
    assert ext.scan_fwd(u, delta.bfloat16(), A, B, C, None, None, None, False) is None
    assert ext.scan_fwd(u.transpose(1, 2).contiguous().transpose(1, 2), delta, A, B, C, None, None, None, False) is None
    assert ext.scan_fwd(u, delta, A, B[:, :, :, :32], C, None, None, None, False) is None
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    with pytest.raises(RuntimeError):
        selective_scan_fn(u, delta.bfloat16(), A, B, C)


@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("packed,has_z,has_init", [(False, True, False), (True, True, True), (False, False, True)])
def test_ssd_same_bits_forward_close_backward(ext, itype, packed, has_z, has_init):
    """mamba_chunk_scan_combined through both host sides: the forward pass gives the same bits; the backward pass
    adds shared sums with float atomics, whose order moves the last bits from run to run, so its gradients are held
    to a few ulps of their size instead (the deterministic mode always takes the Python host side)."""
    from mamba_amd.ops.triton import ssd_combined as sc
    torch.manual_seed(3)
    dev, batch, L, H, P, N, G, Q = "cuda", 2, 640, 4, 64, 64, 2, 128
    x, z0 = (torch.randn(batch, L, H, P, device=dev).to(itype) for _ in range(2))
    z = z0 if has_z else None
    B, C = (torch.randn(batch, L, G, N, device=dev).to(itype) for _ in range(2))
    dt = torch.randn(batch, L, H, device=dev).to(itype)
    A, D, dtb = -torch.rand(H, device=dev) - 1, torch.rand(H, device=dev), torch.rand(H, device=dev) - 4
    init = 0.1 * torch.randn(batch, H, P, N, device=dev) if has_init else None
    seq_idx = None
    if packed:
        seq_idx = torch.cat([torch.zeros(300), torch.ones(340)]).to(torch.int32).to(dev)[None].expand(batch, L).contiguous()
    dout = torch.randn(batch, L, H, P, device=dev).to(itype)
    dfin = torch.randn(batch, H, P, N, device=dev)
    fwd = lambda: sc._mamba_chunk_scan_combined_fwd(x, dt, A, B, C, Q, D=D, z=z, dt_bias=dtb, initial_states=init,
                                                    seq_idx=seq_idx, dt_softplus=True)
    assert ext.ssd_fwd(x, dt, A, B, C, Q, D, z, dtb, init, seq_idx, True, 0.0, float("inf"), True) is not None, "declined"
    f1, f2 = fwd(), _python_path(fwd)
    for i, (a, b) in enumerate(zip(f1, f2)):
        assert (a is None) == (b is None), i
        if a is not None:
            assert a.dtype == b.dtype and a.shape == b.shape and torch.equal(a, b), i
    out, out_x, dt_out, dA_cumsum, states, final = f1
    saved = (dt_out, dA_cumsum, states)
    bwd = lambda: sc._mamba_chunk_scan_combined_bwd(dout, x, dt, A, B, C, out_x if has_z else out, Q, D=D, z=z, dt_bias=dtb,
                                                    initial_states=init, dfinal_states=dfin, seq_idx=seq_idx,
                                                    dt_softplus=True, saved=saved)
    assert ext.ssd_bwd(dout, x, dt, A, B, C, out_x if has_z else out, Q, D, z, dtb, init, dfin, seq_idx, True, 0.0,
                       float("inf"), dt_out, dA_cumsum, states) is not None, "declined"
    b1, b2 = bwd(), _python_path(bwd)
    assert len(b1) == len(b2) == 9
    for i, (a, b) in enumerate(zip(b1, b2)):
        assert (a is None) == (b is None), i
        if a is not None:
            assert a.dtype == b.dtype and a.shape == b.shape, i
            a32, b32 = a.float(), b.float()
            tol = (2e-2 if itype == torch.bfloat16 and a.dtype == torch.bfloat16 else 1e-4) * float(b32.abs().max()) + 1e-6
            assert float((a32 - b32).abs().max()) <= tol, (i, float((a32 - b32).abs().max()), tol)
