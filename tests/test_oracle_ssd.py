"""Pins the SSD oracle (oracle/ssd.py): three independent formulations, invariances, the link to the
Mamba-1 oracle, packed sequences, gradcheck."""
import pytest
import torch
import torch.nn.functional as F

from oracle.mamba1 import selective_scan_oracle
from oracle.ssd import ssd_oracle, ssd_chunked, ssd_quadratic, ssd_inputs, dt_pipeline

f64 = torch.float64


def _inputs(**kw):
    t = ssd_inputs(dtype=f64, **kw)
    t["dtv"] = dt_pipeline(t["dt"], t["dt_bias"], True, compute_dtype=f64)
    return t


def test_three_formulations_agree():
    t = _inputs(batch=2, seqlen=70, nheads=4, headdim=5, dstate=6, ngroups=2, has_init=False)
    seq = ssd_oracle(t["x"], t["dtv"], t["A"], t["B"], t["C"], compute_dtype=f64)
    quad = ssd_quadratic(t["x"], t["dtv"], t["A"], t["B"], t["C"])
    chk = ssd_chunked(t["x"], t["dtv"], t["A"], t["B"], t["C"], 16)
    assert torch.allclose(seq, quad, atol=1e-10) and torch.allclose(seq, chk, atol=1e-10)


@pytest.mark.parametrize("chunk", [8, 32, 64, 256])
def test_chunk_size_invariance_with_state_d_z(chunk):
    t = _inputs(batch=1, seqlen=100, nheads=2, headdim=4, dstate=8, has_init=True)
    y1, f1 = ssd_oracle(t["x"], t["dtv"], t["A"], t["B"], t["C"], D=t["D"], z=t["z"],
                        initial_states=t["initial_states"], return_final_states=True, compute_dtype=f64)
    y2, f2 = ssd_chunked(t["x"], t["dtv"], t["A"], t["B"], t["C"], chunk, D=t["D"], z=t["z"],
                         initial_states=t["initial_states"], return_final_states=True)
    assert torch.allclose(y1, y2, atol=1e-10) and torch.allclose(f1, f2, atol=1e-10)


def test_split_sequence_carries_state():
    t = _inputs(batch=2, seqlen=60, nheads=2, headdim=3, dstate=4)
    kw = dict(D=t["D"], compute_dtype=f64, return_final_states=True)
    y, f = ssd_oracle(t["x"], t["dtv"], t["A"], t["B"], t["C"], **kw)
    cut = 23
    sl = lambda v, a, b: v[:, a:b]
    y1, f1 = ssd_oracle(sl(t["x"], 0, cut), sl(t["dtv"], 0, cut), t["A"], sl(t["B"], 0, cut), sl(t["C"], 0, cut), **kw)
    y2, f2 = ssd_oracle(sl(t["x"], cut, 60), sl(t["dtv"], cut, 60), t["A"], sl(t["B"], cut, 60), sl(t["C"], cut, 60),
                        initial_states=f1, **kw)
    assert torch.allclose(torch.cat([y1, y2], 1), y, atol=1e-10) and torch.allclose(f2, f, atol=1e-10)


def test_equals_mamba1_oracle_with_broadcast_A():
    # mapping of the reference's ssd_selective_scan (ssd_combined.py:746-775)
    t = _inputs(batch=2, seqlen=33, nheads=3, headdim=4, dstate=5, ngroups=1)
    y = ssd_oracle(t["x"], t["dt"], t["A"], t["B"], t["C"], D=t["D"], z=t["z"], dt_bias=t["dt_bias"],
                   dt_softplus=True, compute_dtype=f64)
    b, L, H, P = t["x"].shape
    to_bdl = lambda v: v.permute(0, 2, 3, 1).reshape(b, H * P, L)
    u, z = to_bdl(t["x"]), to_bdl(t["z"])
    delta = to_bdl(t["dt"][..., None].expand(b, L, H, P))
    A = t["A"].double()[:, None, None].expand(H, P, 5).reshape(H * P, 5)
    y1 = selective_scan_oracle(u, delta, A, t["B"].permute(0, 2, 3, 1), t["C"].permute(0, 2, 3, 1),
                               t["D"].double().repeat_interleave(P), z, t["dt_bias"].double().repeat_interleave(P),
                               True, compute_dtype=f64)
    assert torch.allclose(y, y1.reshape(b, H, P, L).permute(0, 3, 1, 2), atol=1e-10)


def test_dt_limit_is_a_clamp():
    t = _inputs(batch=1, seqlen=20, nheads=2, headdim=2, dstate=3)
    a = ssd_oracle(t["x"], t["dt"], t["A"], t["B"], t["C"], dt_bias=t["dt_bias"], dt_softplus=True,
                   dt_limit=(0.01, 0.04), compute_dtype=f64)
    dtc = F.softplus(t["dt"] + t["dt_bias"].double()).clamp(0.01, 0.04)
    b = ssd_oracle(t["x"], dtc, t["A"], t["B"], t["C"], compute_dtype=f64)
    assert torch.allclose(a, b, atol=1e-12)


def test_packed_sequences_equal_separate_runs():
    lens = [7, 12, 1, 20]
    t = _inputs(batch=1, seqlen=sum(lens), nheads=2, headdim=3, dstate=4, seq_lens=lens, has_init=True)
    y, f = ssd_oracle(t["x"], t["dtv"], t["A"], t["B"], t["C"], D=t["D"], z=t["z"],
                      initial_states=t["initial_states"], seq_idx=t["seq_idx"], return_final_states=True,
                      compute_dtype=f64)
    pos, outs = 0, []
    for i, n in enumerate(lens):
        sl = lambda v: v[:, pos:pos + n]
        yi, fi = ssd_oracle(sl(t["x"]), sl(t["dtv"]), t["A"], sl(t["B"]), sl(t["C"]), D=t["D"], z=sl(t["z"]),
                            initial_states=t["initial_states"] if i == 0 else None, return_final_states=True,
                            compute_dtype=f64)
        outs.append(yi)
        pos += n
    assert torch.allclose(torch.cat(outs, 1), y, atol=1e-12)
    assert torch.allclose(fi, f, atol=1e-12)           # final state = state of the last sequence


def test_initial_state_ignored_when_first_id_is_not_zero():
    t = _inputs(batch=1, seqlen=10, nheads=1, headdim=2, dstate=2, has_init=True)
    ids = torch.ones(1, 10, dtype=torch.int32)
    a = ssd_oracle(t["x"], t["dtv"], t["A"], t["B"], t["C"], initial_states=t["initial_states"], seq_idx=ids,
                   compute_dtype=f64)
    b = ssd_oracle(t["x"], t["dtv"], t["A"], t["B"], t["C"], compute_dtype=f64)
    assert torch.allclose(a, b, atol=1e-12)


def test_gradcheck_including_initial_and_final_states():
    t = _inputs(batch=1, seqlen=5, nheads=2, headdim=2, dstate=2, has_init=True)
    names = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states"]
    ins = [t[k].double().clone().requires_grad_() for k in names]

    def fn(x, dt, A, B, C, D, z, dt_bias, init):
        return ssd_oracle(x, dt, A, B, C, D=D, z=z, dt_bias=dt_bias, initial_states=init, dt_softplus=True,
                          return_final_states=True, compute_dtype=f64)
    assert torch.autograd.gradcheck(fn, ins, eps=1e-6, atol=1e-6)
