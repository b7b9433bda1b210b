"""The benchmark configurations at their full sizes.  The CPU oracle cannot run them whole, so each
test checks (i) an oracle-sized slice that the operator treats independently of the rest (channels and
batch rows of the Mamba-1 scan, heads of the SSD scan, batch rows of the decode step) and (ii) a
size-independent property of the quantities that mix everything (dB / dC: additivity over a split of
the channels / heads)."""
import pytest
import torch

from oracle.mamba1 import selective_scan_oracle, scan_inputs
from oracle.ssd import ssd_oracle, ssd_inputs
from oracle.step import selective_state_update_oracle

pytestmark = pytest.mark.gpu


def _close(name, got, ref, rtol, atol, floor=0.0):
    """|got - ref| <= atol + rtol |ref| + floor * max |ref|; the floor (one bf16 ulp of the largest
    entry is 3.9e-3 of it) is for gradients whose entries are sums of many bf16-rounded products of
    mixed sign, where the error follows the size of the terms and not of the result."""
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    err = (got - ref).abs()
    bound = atol + rtol * ref.abs() + floor * ref.abs().max()
    assert bool((err <= bound).all()), f"{name}: max err {err.max().item():.3e}, ref max {ref.abs().max().item():.3e}"


def test_mamba1_plumbing_configuration_full_size():
    """Configuration 0 (batch 2, 1536 channels, 2048 steps, 16 states, fp32, forward only): small
    enough for the oracle to run whole, so every output entry and the last state are compared."""
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    t = scan_inputs(2, 1536, 2048, 16, 1, torch.float32, 0)
    names = ("u", "delta", "A", "B", "C", "D", "z", "delta_bias")
    out, last = selective_scan_fn(*[t[k].cuda() for k in names], True, True)
    ref, rlast = selective_scan_oracle(*[t[k] for k in names], True, True)
    _close("out", out, ref, 6e-4, 2e-3)
    _close("last_state", last, rlast, 6e-4, 2e-3)


def test_mamba1_benchmark_configuration_full_size():
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    batch, dim, L, N = 8, 5120, 4096, 16
    t = scan_inputs(batch, dim, L, N, 1, torch.bfloat16, 0)
    leaves = {k: t[k].cuda().requires_grad_() for k in ("u", "delta", "A", "B", "C", "D", "z", "delta_bias")}
    out = selective_scan_fn(*[leaves[k] for k in ("u", "delta", "A", "B", "C", "D", "z", "delta_bias")], True)
    dout = t["dout"].cuda()
    out.backward(dout)
    # (i) a few channels of two batch rows against the oracle (they do not see the other channels)
    rows, chans = [0, 7], [0, 1, 2559, 5119]
    sub = lambda x: x[rows][:, chans].clone()
    ins = dict(u=sub(t["u"]), delta=sub(t["delta"]), A=t["A"][chans].clone(), B=t["B"][rows].clone(),
               C=t["C"][rows].clone(), D=t["D"][chans].clone(), z=sub(t["z"]), delta_bias=t["delta_bias"][chans].clone())
    for k in ("u", "delta", "z"):
        ins[k].requires_grad_()
    ref = selective_scan_oracle(ins["u"], ins["delta"], ins["A"], ins["B"], ins["C"], ins["D"], ins["z"],
                                ins["delta_bias"], True)
    ref.backward(sub(t["dout"]))
    pick = lambda x: x[rows][:, chans]
    _close("out", pick(out), ref, 3e-2, 5e-2)
    _close("du", pick(leaves["u"].grad), ins["u"].grad, 6e-2, 1e-1)
    _close("ddelta", pick(leaves["delta"].grad), ins["delta"].grad, 1.5e-1, 5e-1)
    _close("dz", pick(leaves["z"].grad), ins["z"].grad, 3e-2, 5e-2)
    # (ii) dB, dC, dA-rows: the sum over all channels equals the sum of two calls on channel halves
    half = dim // 2
    dB_parts, dC_parts = [], []
    for sl in (slice(0, half), slice(half, dim)):
        lv = {k: t[k].cuda()[:, sl].contiguous() for k in ("u", "delta", "z")}
        lv.update(A=t["A"].cuda()[sl].contiguous(), D=t["D"].cuda()[sl].contiguous(),
                  delta_bias=t["delta_bias"].cuda()[sl].contiguous())
        Bc, Cc = t["B"].cuda().requires_grad_(), t["C"].cuda().requires_grad_()
        A_half = lv["A"].requires_grad_()
        o = selective_scan_fn(lv["u"], lv["delta"], A_half, Bc, Cc, lv["D"], lv["z"], lv["delta_bias"], True)
        o.backward(dout[:, sl].contiguous())
        dB_parts.append(Bc.grad.float())
        dC_parts.append(Cc.grad.float())
        _close("dA rows", leaves["A"].grad[sl], A_half.grad, 2e-2, 5e-1)
    _close("dB additivity", leaves["B"].grad, dB_parts[0] + dB_parts[1], 3e-2, 2.0)
    _close("dC additivity", leaves["C"].grad, dC_parts[0] + dC_parts[1], 3e-2, 2.0)


def test_ssd_benchmark_configuration_full_size():
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    batch, L, H, P, N, G, Q = 4, 4096, 80, 64, 128, 1, 256
    t = ssd_inputs(batch, L, H, P, N, G, torch.bfloat16, 0)
    names = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias"]
    g = {k: t[k].cuda().requires_grad_() for k in names}
    out = mamba_chunk_scan_combined(g["x"], g["dt"], g["A"], g["B"], g["C"], Q, D=g["D"], z=g["z"], dt_bias=g["dt_bias"],
                                    dt_softplus=True)
    dout = t["dout"].cuda()
    out.backward(dout)
    # (i) two heads of one batch row against the oracle (with one group, B and C are common to all heads)
    row, heads = 1, [0, 79]
    r = dict(x=t["x"][row:row + 1, :, heads].clone().requires_grad_(), dt=t["dt"][row:row + 1, :, heads].clone().requires_grad_(),
             A=t["A"][heads].clone(), B=t["B"][row:row + 1].clone(), C=t["C"][row:row + 1].clone(), D=t["D"][heads].clone(),
             z=t["z"][row:row + 1, :, heads].clone().requires_grad_(), dt_bias=t["dt_bias"][heads].clone())
    ref = ssd_oracle(r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"], dt_softplus=True)
    ref.backward(t["dout"][row:row + 1, :, heads])
    _close("out", out[row:row + 1, :, heads], ref, 3e-2, 5e-2)
    _close("dx", g["x"].grad[row:row + 1, :, heads], r["x"].grad, 3e-2, 5e-2, floor=4e-3)
    _close("dz", g["z"].grad[row:row + 1, :, heads], r["z"].grad, 3e-2, 5e-2, floor=4e-3)
    _close("ddt", g["dt"].grad[row:row + 1, :, heads], r["dt"].grad, 6e-2, 2e-1, floor=4e-3)
    # (ii) dB, dC: all heads == heads 0..39 + heads 40..79
    parts = []
    for sl in (slice(0, 40), slice(40, 80)):
        Bc, Cc = t["B"].cuda().requires_grad_(), t["C"].cuda().requires_grad_()
        o = mamba_chunk_scan_combined(t["x"].cuda()[:, :, sl], t["dt"].cuda()[:, :, sl], t["A"].cuda()[sl], Bc, Cc, Q,
                                      D=t["D"].cuda()[sl], z=t["z"].cuda()[:, :, sl], dt_bias=t["dt_bias"].cuda()[sl],
                                      dt_softplus=True)
        o.backward(dout[:, :, sl])
        parts.append((Bc.grad.float(), Cc.grad.float()))
    _close("dB additivity", g["B"].grad, parts[0][0] + parts[1][0], 3e-2, 1.0)
    _close("dC additivity", g["C"].grad, parts[0][1] + parts[1][1], 3e-2, 1.0)


def test_decode_benchmark_configuration_full_size():
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    batch, H, P, N = 256, 80, 64, 128
    gen = torch.Generator().manual_seed(0)
    state = 0.1 * torch.randn(batch, H, P, N, generator=gen)
    x, z = torch.randn(batch, H, P, generator=gen).bfloat16(), torch.randn(batch, H, P, generator=gen).bfloat16()
    dt = torch.randn(batch, H, generator=gen).bfloat16()[:, :, None].expand(batch, H, P)
    A = (-(1 + 15 * torch.rand(H, generator=gen)))[:, None, None].expand(H, P, N)
    D = torch.rand(H, generator=gen)[:, None].expand(H, P)
    dtb = (torch.rand(H, generator=gen) - 4)[:, None].expand(H, P)
    B, C = torch.randn(batch, 1, N, generator=gen).bfloat16(), torch.randn(batch, 1, N, generator=gen).bfloat16()
    gstate = state.cuda()
    out = selective_state_update(gstate, x.cuda(), dt.cuda(), A.cuda(), B.cuda(), C.cuda(), D=D.cuda(), z=z.cuda(),
                                 dt_bias=dtb.cuda(), dt_softplus=True)
    rows = [0, 100, 255]
    rstate = state[rows].clone()
    ref = selective_state_update_oracle(rstate, x[rows], dt[rows], A, B[rows], C[rows], D=D, z=z[rows], dt_bias=dtb,
                                        dt_softplus=True)
    _close("out", out[rows], ref, 3e-2, 5e-2)
    _close("state", gstate[rows], rstate, 6e-4, 2e-3)
    untouched = torch.ones(batch, dtype=torch.bool)
    assert gstate.shape == state.shape and bool(torch.isfinite(gstate).all())


def test_ssd_packed_long_configuration_full_size():
    """Benchmark configuration 4: one batch row of 32768 positions packing 16 sequences (lengths in
    [512, 4096]), 64 heads in 8 groups, initial states, final states.  A sequence in the middle of the
    pack and the last one are compared, for two heads of different groups, with the oracle run on
    that sequence alone (packed == separate is what the oracle's own tests pin)."""
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    L, H, P, N, G, Q = 32768, 64, 64, 128, 8, 256
    gen = torch.Generator().manual_seed(4)
    lens = torch.randint(512, 4097, (16,), generator=gen).float()
    lens = (lens / lens.sum() * L).long()
    lens[-1] += L - lens.sum()
    lens = [int(v) for v in lens]
    t = ssd_inputs(1, L, H, P, N, G, torch.bfloat16, 4, seq_lens=lens, has_init=True)
    names = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states"]
    g = {k: t[k].cuda().requires_grad_() for k in names}
    out, fin = mamba_chunk_scan_combined(g["x"], g["dt"], g["A"], g["B"], g["C"], Q, D=g["D"], z=g["z"],
                                         dt_bias=g["dt_bias"], initial_states=g["initial_states"],
                                         seq_idx=t["seq_idx"].cuda(), dt_softplus=True, return_final_states=True)
    dout, dfin = t["dout"].cuda(), t["dfinal"].cuda()
    (out.float() * dout.float()).sum().add((fin * dfin).sum()).backward()
    heads = [0, 63]
    groups = [h // (H // G) for h in heads]
    starts = [0]
    for n in lens:
        starts.append(starts[-1] + n)
    for which in (7, 15):
        sl = slice(starts[which], starts[which + 1])
        for h, grp in zip(heads, groups):
            r = dict(x=t["x"][:, sl, h:h + 1].clone().requires_grad_(), dt=t["dt"][:, sl, h:h + 1].clone().requires_grad_(),
                     z=t["z"][:, sl, h:h + 1].clone().requires_grad_())
            ref, rfin = ssd_oracle(r["x"], r["dt"], t["A"][h:h + 1], t["B"][:, sl, grp:grp + 1], t["C"][:, sl, grp:grp + 1],
                                   D=t["D"][h:h + 1], z=r["z"], dt_bias=t["dt_bias"][h:h + 1], dt_softplus=True,
                                   return_final_states=True)
            loss = (ref.float() * t["dout"][:, sl, h:h + 1].float()).sum()
            if which == 15:
                loss = loss + (rfin * t["dfinal"][:, h:h + 1]).sum()
                _close(f"final_states h{h}", fin[:, h:h + 1], rfin, 3e-2, 5e-2)
            loss.backward()
            _close(f"out seq{which} h{h}", out[:, sl, h:h + 1], ref, 3e-2, 5e-2)
            _close(f"dx seq{which} h{h}", g["x"].grad[:, sl, h:h + 1], r["x"].grad, 3e-2, 5e-2, floor=4e-3)
            _close(f"dz seq{which} h{h}", g["z"].grad[:, sl, h:h + 1], r["z"].grad, 3e-2, 5e-2, floor=4e-3)
            _close(f"ddt seq{which} h{h}", g["dt"].grad[:, sl, h:h + 1], r["dt"].grad, 6e-2, 2e-1, floor=4e-3)
