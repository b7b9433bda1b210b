"""Run-to-run reproducibility (the reference's tests/test_determinism.py:186-211 asks for bitwise equality in
its deterministic mode and 1e-2 agreement with the default mode).  Here: every forward operator, the decode step,
the norm backward passes and the Mamba-1 scan's backward pass (real A) use no float atomics and must repeat bit
for bit in the one mode there is; the SSD and conv backward passes still sum dB, dC, ddt, dA, dD and the conv
weight gradient with float atomics, so their repeats must agree to rounding noise of the sums (far inside the
reference's 1e-2) but not bit for bit."""
import pytest
import torch

from oracle.ssd import ssd_inputs

pytestmark = pytest.mark.gpu


def _mamba1_inputs(dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(0)
    b, d, L, n = 2, 256, 1024, 16
    u, delta, z = (torch.randn(b, d, L, generator=g).to(dtype).cuda() for _ in range(3))
    A = -(1 + 15 * torch.rand(d, n, generator=g)).cuda()
    B, C = (torch.randn(b, 1, n, L, generator=g).to(dtype).cuda() for _ in range(2))
    D, bias = torch.rand(d, generator=g).cuda(), (torch.rand(d, generator=g) - 4).cuda()
    return [u, delta, A, B, C, D, z, bias]


def _twice(fn):
    a = fn()
    torch.cuda.synchronize()
    b = fn()
    torch.cuda.synchronize()
    return a, b


def _noise(a, b):
    scale = max(float(a.float().abs().max()), 1e-30)
    return float((a.float() - b.float()).abs().max()) / scale


def test_forward_operators_repeat_bit_for_bit():
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fn
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    from mamba_amd.ops.triton.layernorm_gated import rmsnorm_fn
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    u, delta, A, B, C, D, z, bias = _mamba1_inputs()
    a, b = _twice(lambda: selective_scan_fn(u, delta, A, B, C, D, z=z, delta_bias=bias, delta_softplus=True))
    assert torch.equal(a, b)
    t = {k: (v.cuda() if torch.is_tensor(v) else v) for k, v in ssd_inputs(2, 512, 8, 64, 128, 1, torch.bfloat16).items()}
    for chunk in (64, 256):  # the plain and the fused scan kernels
        a, b = _twice(lambda: mamba_chunk_scan_combined(t["x"], t["dt"], t["A"], t["B"], t["C"], chunk, D=t["D"], z=t["z"],
                                                        dt_bias=t["dt_bias"], dt_softplus=True, return_final_states=True))
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    state = torch.randn(4, 8, 64, 128, device="cuda")
    args = (t["x"][:, 0][:, :, :][:2].repeat(2, 1, 1), torch.rand(4, 8, 64, device="cuda"), -torch.rand(8, 64, 128, device="cuda"),
            torch.randn(4, 1, 128, device="cuda"), torch.randn(4, 1, 128, device="cuda"))
    a, b = _twice(lambda: selective_state_update(state.clone(), *args))
    assert torch.equal(a, b)
    xc, w = torch.randn(2, 512, 1024, device="cuda", dtype=torch.bfloat16).transpose(1, 2), torch.randn(1024, 4, device="cuda")
    a, b = _twice(lambda: causal_conv1d_fn(xc, w, None, activation="silu"))
    assert torch.equal(a, b)
    xn, zn, wn = torch.randn(512, 2048, device="cuda", dtype=torch.bfloat16), torch.randn(512, 2048, device="cuda", dtype=torch.bfloat16), torch.rand(2048, device="cuda")
    a, b = _twice(lambda: rmsnorm_fn(xn, wn, None, z=zn, group_size=512, norm_before_gate=False))
    assert torch.equal(a, b)


def test_norm_backward_repeats_bit_for_bit():
    from mamba_amd.ops.triton.layer_norm import rms_norm_fn
    from mamba_amd.ops.triton.layernorm_gated import rmsnorm_fn
    x = torch.randn(1024, 2048, device="cuda", dtype=torch.bfloat16)
    z, dy = torch.randn_like(x), torch.randn_like(x)
    w = torch.rand(2048, device="cuda")

    def gated():
        leaves = [x.clone().requires_grad_(), w.clone().requires_grad_(), z.clone().requires_grad_()]
        rmsnorm_fn(leaves[0], leaves[1], None, z=leaves[2], group_size=512, norm_before_gate=False).backward(dy)
        return [t.grad for t in leaves]

    def residual():
        leaves = [x.clone().requires_grad_(), w.clone().requires_grad_(), z.clone().requires_grad_()]
        rms_norm_fn(leaves[0], leaves[1], None, residual=leaves[2]).backward(dy)
        return [t.grad for t in leaves]

    for fn in (gated, residual):
        a, b = _twice(fn)
        for ga, gb in zip(a, b):
            assert torch.equal(ga, gb)


def test_scan_backward_repeats_to_rounding_noise():
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    base = _mamba1_inputs()
    dout = torch.randn_like(base[0])

    def mamba1():
        leaves = [t.clone().requires_grad_() for t in base]
        u, delta, A, B, C, D, z, bias = leaves
        selective_scan_fn(u, delta, A, B, C, D, z=z, delta_bias=bias, delta_softplus=True).backward(dout)
        return [t.grad for t in leaves]

    t = {k: (v.cuda() if torch.is_tensor(v) else v) for k, v in ssd_inputs(2, 512, 16, 64, 128, 1, torch.bfloat16).items()}
    names = ("x", "dt", "A", "B", "C", "D", "z", "dt_bias")

    def ssd():
        leaves = {k: t[k].clone().requires_grad_() for k in names}
        mamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], 256, D=leaves["D"],
                                  z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True).backward(t["dout"])
        return [leaves[k].grad for k in names]

    a, b = _twice(mamba1)   # per-workgroup partial sums added up in a fixed order: every gradient repeats exactly
    for ga, gb in zip(a, b):
        assert torch.equal(ga, gb)
    for fn in (ssd,):
        a, b = _twice(fn)
        # a 16-bit gradient may flip its last bit (2^-8 of the element); fp32 sums differ by summation order only.
        # Both are inside the reference's det-vs-default bound of 1e-2.
        noise = [(_noise(ga, gb), ga.dtype) for ga, gb in zip(a, b)]
        assert all(n < (1e-2 if dt != torch.float32 else 1e-3) for n, dt in noise), (fn.__name__, noise)


@pytest.fixture
def deterministic_mode():
    from mamba_amd.utils.determinism import set_deterministic_mode
    set_deterministic_mode(True)
    yield
    set_deterministic_mode(None)


def _ssd_grads(t, names, chunk, **kw):
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    leaves = {k: t[k].clone().requires_grad_() for k in names if t.get(k) is not None}
    res = mamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], chunk,
                                    D=leaves.get("D"), z=leaves.get("z"), dt_bias=leaves.get("dt_bias"),
                                    initial_states=leaves.get("initial_states"), dt_softplus=True, **kw)
    if isinstance(res, tuple):
        (res[0].float() * t["dout"].float()).sum().add((res[1] * t["dfinal"]).sum()).backward()
    else:
        res.backward(t["dout"])
    return {k: v.grad for k, v in leaves.items()}


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("headdim,dstate,ngroups,d_hdim", [(64, 128, 1, False), (128, 64, 2, True), (64, 64, 8, False)])
def test_ssd_backward_deterministic_mode(deterministic_mode, headdim, dstate, ngroups, d_hdim, dtype):
    """The reference's requirement for its deterministic mode (tests/test_determinism.py:186-211): five runs give
    the same bits for every gradient, and the result is within 1e-2 of the default mode's."""
    from mamba_amd.utils.determinism import set_deterministic_mode
    names = ("x", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states")
    t = {k: (v.cuda() if torch.is_tensor(v) else v)
         for k, v in ssd_inputs(2, 640, 16, headdim, dstate, ngroups, dtype, 7, D_has_hdim=d_hdim, has_init=True).items()}
    runs = [_ssd_grads(t, names, 256, return_final_states=True) for _ in range(5)]
    for r in runs[1:]:
        for k in runs[0]:
            assert torch.equal(runs[0][k], r[k]), k
    set_deterministic_mode(False)
    default = _ssd_grads(t, names, 256, return_final_states=True)
    for k in default:
        assert torch.allclose(default[k].float(), runs[0][k].float(), rtol=1e-2, atol=1e-2), k


def test_ssd_backward_deterministic_mode_no_gate(deterministic_mode):
    """Without z, dD (one value per head) is summed by the dx kernel: the same requirement."""
    from mamba_amd.utils.determinism import set_deterministic_mode
    names = ("x", "dt", "A", "B", "C", "D", "dt_bias")
    t = {k: (v.cuda() if torch.is_tensor(v) else v)
         for k, v in ssd_inputs(2, 640, 16, 64, 128, 1, torch.bfloat16, 9, has_z=False).items()}
    runs = [_ssd_grads(t, names, 256, return_final_states=True) for _ in range(3)]
    for r in runs[1:]:
        for k in runs[0]:
            assert torch.equal(runs[0][k], r[k]), k
    set_deterministic_mode(False)
    default = _ssd_grads(t, names, 256, return_final_states=True)
    for k in default:
        assert torch.allclose(default[k].float(), runs[0][k].float(), rtol=1e-2, atol=1e-2), k


def test_ssd_backward_deterministic_mode_packed(deterministic_mode):
    names = ("x", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states")
    t = {k: (v.cuda() if torch.is_tensor(v) else v)
         for k, v in ssd_inputs(1, 1024, 8, 64, 128, 4, torch.bfloat16, 8, seq_lens=[300, 500, 224], has_init=True).items()}
    runs = [_ssd_grads(t, names, 128, seq_idx=t["seq_idx"], return_final_states=True) for _ in range(3)]
    for r in runs[1:]:
        for k in runs[0]:
            assert torch.equal(runs[0][k], r[k]), k


def test_conv_and_block_backward_deterministic_mode(deterministic_mode):
    from mamba_amd.ops.causal_conv1d import causal_conv1d_fn
    from mamba_amd.ops.triton.ssd_combined import mamba_split_conv1d_scan_combined
    g = torch.Generator().manual_seed(3)
    r = lambda *s: torch.randn(*s, generator=g).cuda()
    for channel_last in (False, True):
        x = r(2, 2048, 512).bfloat16()
        x = x.transpose(1, 2) if channel_last else x.transpose(1, 2).contiguous()
        w, bias, dout = 0.5 * r(512, 4), r(512), r(2, 512, 2048).bfloat16()

        def conv():
            leaves = [x.clone().requires_grad_(), w.clone().requires_grad_(), bias.clone().requires_grad_()]
            causal_conv1d_fn(*leaves, activation="silu").backward(dout if not channel_last else dout.transpose(1, 2).contiguous().transpose(1, 2))
            return [t.grad for t in leaves]
        a, b = _twice(conv)
        for ga, gb in zip(a, b):
            assert torch.equal(ga, gb)
    # the whole Mamba-2 block body
    batch, L, H, P, N, G, W, dm = 2, 512, 8, 64, 64, 1, 4, 256
    d_inner, conv_dim = H * P, H * P + 2 * G * N
    zxbcdt = r(batch, L, 2 * d_inner + 2 * G * N + H).bfloat16()
    params = dict(conv_w=0.4 * r(conv_dim, W), conv_b=0.1 * r(conv_dim), dt_bias=r(H) - 3, A=-(1 + torch.rand(H, generator=g)).cuda(),
                  D=torch.rand(H, generator=g).cuda(), norm_w=1 + 0.1 * r(d_inner), out_w=0.05 * r(dm, d_inner).bfloat16())
    dout = r(batch, L, dm).bfloat16()

    def block():
        lv = {k: v.clone().requires_grad_() for k, v in params.items()}
        zx = zxbcdt.clone().requires_grad_()
        out = mamba_split_conv1d_scan_combined(zx, lv["conv_w"], lv["conv_b"], lv["dt_bias"], lv["A"], lv["D"], 128,
                                               activation="silu", rmsnorm_weight=lv["norm_w"], rmsnorm_eps=1e-5,
                                               outproj_weight=lv["out_w"], headdim=P, ngroups=G, norm_before_gate=False)
        out.backward(dout)
        return [zx.grad] + [v.grad for v in lv.values()]
    a, b = _twice(block)
    for ga, gb in zip(a, b):
        assert torch.equal(ga, gb)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_complex_scan_backward_deterministic_mode(deterministic_mode, dtype):
    """A complex A (the S4D-style variant): its kernels add every channel's dB / dC terms into one sum per position.
    In the deterministic mode those adds are integer adds of fixed-point terms: every gradient repeats bit for bit,
    and agrees with the default mode's float sums to rounding noise."""
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    from mamba_amd.utils.determinism import set_deterministic_mode
    g = torch.Generator().manual_seed(7)
    b, d, L, n = 2, 96, 700, 8
    u, delta, z, dout = (torch.randn(b, d, L, generator=g).to(dtype).cuda() for _ in range(4))
    delta = (0.5 * torch.rand(b, d, L, generator=g)).to(dtype).cuda()
    A = torch.complex(-0.5 * torch.rand(d, n, generator=g), 2.0 * torch.randn(d, n, generator=g)).cuda()
    B, C = (torch.randn(b, 2, n, 2 * L, generator=g).to(dtype).cuda() for _ in range(2))
    D, bias = torch.rand(d, generator=g).cuda(), (0.5 * torch.rand(d, generator=g)).cuda()

    def grads():
        leaves = [t.clone().requires_grad_() for t in (u, delta, A, B, C, D, z, bias)]
        out = selective_scan_fn(leaves[0], leaves[1], leaves[2], leaves[3], leaves[4], leaves[5], z=leaves[6],
                                delta_bias=leaves[7], delta_softplus=True)
        out.backward(dout)
        return [torch.view_as_real(t.grad) if t.grad.is_complex() else t.grad for t in leaves]

    a, bb = _twice(grads)
    for i, (x, y) in enumerate(zip(a, bb)):
        assert torch.equal(x, y), f"gradient {i} does not repeat bit for bit in the deterministic mode"
    set_deterministic_mode(False)
    try:
        c = grads()
    finally:
        set_deterministic_mode(True)
    for i, (x, y) in enumerate(zip(a, c)):
        assert _noise(x, y) <= (1e-2 if dtype == torch.bfloat16 else 1e-4), (i, _noise(x, y))


def test_deterministic_mode_keeps_non_finite_gradients_visible(deterministic_mode):
    """A NaN in the upstream gradient must come out as NaN in the sums the deterministic mode keeps as integers
    (dB, dC, ddt, dA, dD, ddt_bias), as it does with float atomics, not as a finite number; and one large outlier in
    dout must not wipe out the other terms (the call's one fixed-point scale follows the largest |dout|: terms 2^-30
    of it and larger keep their value)."""
    t = {k: (v.cuda() if torch.is_tensor(v) else v) for k, v in ssd_inputs(1, 256, 4, 64, 64, 2, torch.bfloat16, 9).items()}
    names = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias"]
    bad = dict(t)
    bad["dout"] = t["dout"].clone()
    bad["dout"][0, 100, 1, 3] = float("nan")
    g = _ssd_grads(bad, names, 64)
    for k in ("B", "C", "dt", "A", "D", "dt_bias"):
        assert bool(torch.isnan(g[k].float()).any()), f"d{k} hides the NaN"
    out = dict(t)
    out["dout"] = t["dout"].clone()
    out["dout"][0, 10, 0, 0] = 3.0e4   # an outlier 4 orders above the rest
    from mamba_amd.utils.determinism import set_deterministic_mode
    ga = _ssd_grads(out, names, 64)
    set_deterministic_mode(False)
    try:
        gb = _ssd_grads(out, names, 64)
    finally:
        set_deterministic_mode(True)
    for k in names:
        assert _noise(ga[k], gb[k]) <= 1e-2, (k, _noise(ga[k], gb[k]))
    # positions far from the outlier (another chunk): their small gradients survive the coarse scale
    far = slice(128, 256)
    for k in ("B", "C", "x"):
        a, b = ga[k][:, far].float(), gb[k][:, far].float()
        assert float((a - b).abs().max()) <= 2e-2 * float(b.abs().max()) + 1e-3, k
