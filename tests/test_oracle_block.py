"""Pins oracle/block.py (conv1d + scan + gated RMSNorm block) and the plain-torch utilities the
host modules export next to the operators; none of this needs a GPU."""
import torch
import torch.nn.functional as F

from oracle.block import (causal_conv1d_oracle, causal_conv1d_update_oracle, causal_conv1d_varlen_states_oracle,
                          gated_rms_norm_oracle, split_conv1d_scan_oracle)
from oracle.ssd import ssd_oracle, ssd_inputs
from oracle.step import selective_state_update_oracle

f64 = torch.float64


def test_conv_equals_library_conv1d_and_brute_force():
    g = torch.Generator().manual_seed(0)
    b, L, ch, w = 2, 13, 5, 4
    x = torch.randn(b, L, ch, generator=g, dtype=f64)
    wt, bias = torch.randn(ch, w, generator=g, dtype=f64), torch.randn(ch, generator=g, dtype=f64)
    y = causal_conv1d_oracle(x, wt, bias, activation=None)
    lib = F.conv1d(x.transpose(1, 2), wt.unsqueeze(1), bias, padding=w - 1, groups=ch)[..., :L].transpose(1, 2)
    assert torch.allclose(y, lib, atol=1e-12)
    t, c = 7, 3   # one output by hand: taps reach back w-1 positions, last weight on the current one
    expect = bias[c] + sum(wt[c, w - 1 - k] * x[1, t - k, c] for k in range(w))
    assert abs(y[1, t, c] - expect) < 1e-12
    assert torch.allclose(causal_conv1d_oracle(x, wt, bias, "silu"), F.silu(lib), atol=1e-12)


def test_conv_on_packed_batch_equals_separate_sequences():
    g = torch.Generator().manual_seed(1)
    lens, ch, w = [5, 1, 9, 3], 4, 4
    x = torch.randn(1, sum(lens), ch, generator=g, dtype=f64)
    wt, bias = torch.randn(ch, w, generator=g, dtype=f64), torch.randn(ch, generator=g, dtype=f64)
    ids = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)])[None]
    packed = causal_conv1d_oracle(x, wt, bias, "silu", seq_idx=ids)
    start, parts = 0, []
    for n in lens:
        parts.append(causal_conv1d_oracle(x[:, start:start + n], wt, bias, "silu"))
        start += n
    assert torch.allclose(packed, torch.cat(parts, dim=1), atol=1e-12)


def test_rms_norm_against_library_and_gate_order():
    g = torch.Generator().manual_seed(2)
    x, z = torch.randn(3, 7, 24, generator=g, dtype=f64), torch.randn(3, 7, 24, generator=g, dtype=f64)
    wt = torch.randn(24, generator=g, dtype=f64)
    ones = torch.full_like(z, 1e4)  # silu(1e4) = 1e4: the gate becomes a plain factor
    full = gated_rms_norm_oracle(x, wt, ones, 1e-5, 24, True) / 1e4
    assert torch.allclose(full, F.rms_norm(x, (24,), wt, 1e-5), atol=1e-10)
    grouped = gated_rms_norm_oracle(x, wt, ones, 1e-5, 8, True) / 1e4
    lib = F.rms_norm(x.reshape(3, 7, 3, 8), (8,), None, 1e-5).reshape(3, 7, 24) * wt
    assert torch.allclose(grouped, lib, atol=1e-10)
    after = gated_rms_norm_oracle(x, wt, z, 1e-5, 8, True)
    before = gated_rms_norm_oracle(x, wt, z, 1e-5, 8, False)
    assert torch.allclose(after, F.rms_norm(x.reshape(3, 7, 3, 8), (8,), None, 1e-5).reshape(3, 7, 24) * wt * F.silu(z))
    assert torch.allclose(before, F.rms_norm((x * F.silu(z)).reshape(3, 7, 3, 8), (8,), None, 1e-5).reshape(3, 7, 24) * wt)


def _block_inputs(batch, L, nheads, headdim, dstate, ngroups, d_nonssm, d_out, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    dim, width = nheads * headdim, 4
    r = lambda *s: torch.randn(*s, generator=g)
    return dict(
        zxbcdt=r(batch, L, 2 * d_nonssm + 2 * dim + 2 * ngroups * dstate + nheads).to(dtype),
        conv1d_weight=0.5 * r(dim + 2 * ngroups * dstate, width), conv1d_bias=0.1 * r(dim + 2 * ngroups * dstate),
        dt_bias=torch.rand(nheads, generator=g) - 4.0, A=-(1.0 + 15.0 * torch.rand(nheads, generator=g)),
        D=torch.rand(nheads, generator=g), rmsnorm_weight=1.0 + 0.1 * r(dim),
        outproj_weight=0.2 * r(d_out, d_nonssm + dim), outproj_bias=0.1 * r(d_out))


def test_block_is_the_composition_of_its_parts():
    # no norm, no projection, no extra part: conv -> scan with the gate inside
    t = _block_inputs(2, 40, 4, 8, 6, 2, 0, 5, 3)
    out, fin = split_conv1d_scan_oracle(t["zxbcdt"], t["conv1d_weight"], t["conv1d_bias"], t["dt_bias"], t["A"], t["D"],
                                        headdim=8, ngroups=2)
    dim = 32
    z, xBC, dt = torch.split(t["zxbcdt"], [dim, dim + 24, 4], dim=-1)
    xBC = F.silu(F.conv1d(xBC.transpose(1, 2), t["conv1d_weight"].unsqueeze(1), t["conv1d_bias"], padding=3,
                          groups=dim + 24)[..., :40].transpose(1, 2))
    x, B, C = torch.split(xBC, [dim, 12, 12], dim=-1)
    ref, fin_ref = ssd_oracle(x.reshape(2, 40, 4, 8), dt, t["A"], B.reshape(2, 40, 2, 6), C.reshape(2, 40, 2, 6),
                              D=t["D"], z=z.reshape(2, 40, 4, 8), dt_bias=t["dt_bias"], dt_softplus=True,
                              return_final_states=True)
    assert torch.allclose(out, ref.reshape(2, 40, dim), atol=1e-6) and torch.allclose(fin, fin_ref, atol=1e-6)
    # the non-SSM part goes through silu(a) * b in front of the scan output, then the projection
    t = _block_inputs(1, 24, 2, 8, 4, 1, 3, 5, 4)
    out, _ = split_conv1d_scan_oracle(t["zxbcdt"], t["conv1d_weight"], t["conv1d_bias"], t["dt_bias"], t["A"], t["D"],
                                      headdim=8, rmsnorm_weight=t["rmsnorm_weight"], outproj_weight=t["outproj_weight"],
                                      outproj_bias=t["outproj_bias"])
    core, _ = split_conv1d_scan_oracle(t["zxbcdt"][..., 6:], t["conv1d_weight"], t["conv1d_bias"], t["dt_bias"], t["A"],
                                       t["D"], headdim=8, rmsnorm_weight=t["rmsnorm_weight"])
    a, b2 = t["zxbcdt"][..., :3], t["zxbcdt"][..., 3:6]
    expect = torch.cat([F.silu(a) * b2, core], dim=-1) @ t["outproj_weight"].t() + t["outproj_bias"]
    assert torch.allclose(out, expect, atol=1e-5)


def test_exported_torch_utilities_match_the_oracles():
    from mamba_amd.ops.triton.selective_state_update import selective_state_update_ref
    from mamba_amd.ops.triton.ssd_combined import ssd_chunk_scan_combined_ref, _causal_conv1d, _gated_rms_norm
    t = ssd_inputs(2, 50, 4, 8, 6, 2, torch.float32, 7)
    out = ssd_chunk_scan_combined_ref(t["x"], t["dt"], t["A"], t["B"], t["C"], 16, D=t["D"], z=t["z"], dt_bias=t["dt_bias"],
                                      dt_softplus=True)
    ref = ssd_oracle(t["x"], t["dt"], t["A"], t["B"], t["C"], D=t["D"], z=t["z"], dt_bias=t["dt_bias"], dt_softplus=True)
    assert torch.allclose(out, ref, atol=1e-5)
    g = torch.Generator().manual_seed(8)
    state = torch.randn(3, 4, 8, 6, generator=g)
    x, z = torch.randn(3, 4, 8, generator=g), torch.randn(3, 4, 8, generator=g)
    dt, dtb = torch.randn(3, 4, 8, generator=g), torch.randn(4, 8, generator=g)
    A, D = -torch.rand(4, 8, 6, generator=g), torch.randn(4, 8, generator=g)
    B, C = torch.randn(3, 2, 6, generator=g), torch.randn(3, 2, 6, generator=g)
    s1, s2 = state.clone(), state.clone()
    o1 = selective_state_update_ref(s1, x, dt, A, B, C, D=D, z=z, dt_bias=dtb, dt_softplus=True)
    o2 = selective_state_update_oracle(s2, x, dt, A, B, C, D=D, z=z, dt_bias=dtb, dt_softplus=True)
    assert torch.allclose(o1, o2, atol=1e-6) and torch.allclose(s1, s2, atol=1e-6)
    # headless form
    s1, s2 = state[:, 0].clone(), state[:, 0].clone()
    o1 = selective_state_update_ref(s1, x[:, 0], dt[:, 0], A[0], B[:, 0], C[:, 0], D=D[0], z=z[:, 0], dt_bias=dtb[0])
    o2 = selective_state_update_oracle(s2, x[:, 0], dt[:, 0], A[0], B[:, 0], C[:, 0], D=D[0], z=z[:, 0], dt_bias=dtb[0])
    assert torch.allclose(o1, o2, atol=1e-6) and torch.allclose(s1, s2, atol=1e-6)
    # conv (plain and packed) and norm used by the block's host code
    lens = [5, 1, 9, 3]
    xb = torch.randn(1, 18, 4, generator=g)
    wt, bias = torch.randn(4, 4, generator=g), torch.randn(4, generator=g)
    ids = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(lens)])[None]
    for sid in (None, ids):
        assert torch.allclose(_causal_conv1d(xb, wt, bias, "silu", sid), causal_conv1d_oracle(xb, wt, bias, "silu", sid),
                              atol=1e-6)
    xn, zn, wn = torch.randn(2, 5, 16, generator=g), torch.randn(2, 5, 16, generator=g), torch.randn(16, generator=g)
    for nbg in (True, False):
        assert torch.allclose(_gated_rms_norm(xn, wn, zn, 1e-5, 8, nbg),
                              gated_rms_norm_oracle(xn, wn, zn, 1e-5, 8, nbg).float(), atol=1e-5)


def test_selective_scan_ref_utility_matches_the_oracle_real_and_complex():
    from mamba_amd.ops.selective_scan_interface import selective_scan_ref
    from oracle.mamba1 import selective_scan_oracle
    g = torch.Generator().manual_seed(9)
    b, d, L, n = 2, 4, 30, 3
    u, delta, z = (torch.randn(b, d, L, generator=g) for _ in range(3))
    D, bias = torch.randn(d, generator=g), torch.rand(d, generator=g)
    for cplx in (False, True):
        A = -torch.rand(d, n, generator=g)
        if cplx:
            A = torch.complex(A, torch.randn(d, n, generator=g))
        Bv = torch.randn(b, 2, n, L * (2 if cplx else 1), generator=g)
        Cm = torch.complex(torch.randn(d, n, generator=g), torch.randn(d, n, generator=g)) if cplx else torch.randn(d, n, generator=g)
        got, st = selective_scan_ref(u, delta, A, Bv, Cm, D, z, bias, True, return_last_state=True)
        ref, st_ref = selective_scan_oracle(u, delta, A, Bv, Cm, D, z, bias, True, return_last_state=True)
        assert torch.allclose(got, ref, atol=1e-5) and torch.allclose(st, st_ref, atol=1e-5)


def test_conv_update_is_the_roll_insert_dot_and_continues_the_full_convolution():
    g = torch.Generator().manual_seed(5)
    batch, dim, width = 2, 6, 4
    wt = torch.randn(dim, width, generator=g, dtype=torch.float64)
    bias = torch.randn(dim, generator=g, dtype=torch.float64)
    state = torch.randn(batch, dim, width, generator=g, dtype=torch.float64)
    x = torch.randn(batch, dim, 1, generator=g, dtype=torch.float64)
    out, new = causal_conv1d_update_oracle(x, state, wt, bias, "silu")
    # the reference's own spelling for one new position (mamba_ssm/modules/mamba2.py:291-296)
    rolled = torch.roll(state, shifts=-1, dims=-1)
    rolled[:, :, -1] = x[:, :, 0]
    assert torch.allclose(new, rolled)
    assert torch.allclose(out[:, :, 0], F.silu((rolled * wt).sum(-1) + bias), atol=1e-12)
    # steps over a sequence == the full causal convolution of that sequence; state_len = width - 1 and longer
    seq = torch.randn(batch, 11, dim, generator=g, dtype=torch.float64)
    full = causal_conv1d_oracle(seq, wt, bias, "silu")
    for state_len, chunk in ((3, 1), (3, 4), (7, 2), (5, 11)):
        st = torch.zeros(batch, dim, state_len, dtype=torch.float64)
        outs = []
        for t0 in range(0, 11, chunk):
            o, st = causal_conv1d_update_oracle(seq[:, t0:t0 + chunk].transpose(1, 2), st, wt, bias, "silu")
            outs.append(o)
        assert torch.allclose(torch.cat(outs, dim=-1).transpose(1, 2), full, atol=1e-12)
        keep = min(state_len, 11)
        assert torch.allclose(st[:, :, state_len - keep:], seq[:, 11 - keep:].transpose(1, 2))


def test_varlen_states_are_the_tails_of_the_sequences():
    x = torch.arange(10 * 3, dtype=torch.float64).reshape(10, 3) + 1
    cu = torch.tensor([0, 2, 7, 10], dtype=torch.int32)
    st = causal_conv1d_varlen_states_oracle(x, cu, 4)
    assert st.shape == (3, 3, 4)
    assert torch.equal(st[0, 0], torch.tensor([0, 0, x[0, 0], x[1, 0]], dtype=torch.float64))
    assert torch.equal(st[1, 2], x[3:7, 2])
    assert torch.equal(st[2, 1], torch.tensor([0, x[7, 1], x[8, 1], x[9, 1]], dtype=torch.float64))
