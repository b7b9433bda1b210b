"""ssd_chunk_state_passing_fwd (chunk states and state passing in one launch: one workgroup per (batch, head) walks
the sequence with the carried state in registers) against the two stages it replaces, ssd_chunk_state_fwd +
ssd_state_passing_fwd (reference mamba_ssm/ops/triton/ssd_combined.py:375-382), through the C-ABI on the same
workspaces' worth of inputs; then the whole operator against the oracle on a shape whose batch x heads makes
ssd_combined_fwd take the one-launch form."""
import pytest
import torch

from oracle.ssd import ssd_inputs
from tests.test_ssd_gpu import _fwd_case

pytestmark = pytest.mark.gpu


def _entering_states(t, chunk, stages):
    from mamba_amd import _lib
    from mamba_amd.ops.triton import ssd_combined as sc
    cu = lambda v: None if v is None else v.cuda()
    x, dt, A, B, C, D, z, dt_bias, init, seq_idx = sc._prepare(
        cu(t["x"]), cu(t["dt"]), cu(t["A"]), cu(t["B"]), cu(t["C"]), chunk, cu(t["D"]), None, cu(t["dt_bias"]),
        cu(t["initial_states"]), cu(t["seq_idx"]))
    ws = sc._workspace(x, B, chunk)
    ws["carried"].fill_(float("nan"))
    ws["final_states"].fill_(float("nan"))
    p = _lib.SsdParams()
    sc._fill_fwd(p, x, dt, A, B, C, chunk, D, None, dt_bias, init, seq_idx, True, (0.0, float("inf")), ws)
    lib, stream = _lib.load(), _lib.current_stream(x.device)
    for name in ("ssd_chunk_cumsum_fwd",) + stages:
        _lib.check(getattr(lib, name)(p, stream), name)
    torch.cuda.synchronize()
    return ws["carried"].float().cpu(), ws["final_states"].cpu()


@pytest.mark.parametrize("batch,seqlen,nheads,ngroups,chunk,seq_lens,has_init", [
    (2, 1024, 8, 1, 256, None, False),
    (1, 2048, 6, 2, 256, None, True),
    (2, 512, 4, 4, 128, None, True),
    (1, 1536, 8, 8, 256, [100, 156, 256, 300, 212, 1, 511], True),   # boundaries inside chunks and on chunk edges
    (2, 768, 4, 1, 128, [128, 128, 300, 212], False),
    (1, 256, 3, 1, 256, None, True),                                    # a single chunk
])
def test_one_launch_matches_the_two_stages(batch, seqlen, nheads, ngroups, chunk, seq_lens, has_init):
    t = ssd_inputs(batch, seqlen, nheads, 64, 128, ngroups, torch.bfloat16, 17, seq_lens=seq_lens, has_init=has_init)
    c2, f2 = _entering_states(t, chunk, ("ssd_chunk_state_fwd", "ssd_state_passing_fwd"))
    c1, f1 = _entering_states(t, chunk, ("ssd_chunk_state_passing_fwd",))
    assert not torch.isnan(c1).any() and not torch.isnan(f1).any()
    # the same fp32 products and the same recurrence; the only freedom is whether decay * H + S is fused
    assert torch.allclose(f1, f2, rtol=1e-5, atol=1e-5), float((f1 - f2).abs().max())
    assert torch.allclose(c1, c2, rtol=2 ** -7, atol=1e-6), float((c1 - c2).abs().max())  # one bf16 step at most
    assert float((c1 == c2).float().mean()) > 0.999


def test_one_launch_declines_other_shapes():
    from mamba_amd import _lib
    from mamba_amd.ops.triton import ssd_combined as sc
    for headdim, dstate, seqlen, chunk in ((32, 128, 512, 256), (64, 64, 512, 256), (64, 128, 500, 256), (64, 128, 512, 64)):
        t = ssd_inputs(1, seqlen, 4, headdim, dstate, 1, torch.bfloat16, 3)
        cu = lambda v: None if v is None else v.cuda()
        x, dt, A, B, C, D, z, dt_bias, init, seq_idx = sc._prepare(
            cu(t["x"]), cu(t["dt"]), cu(t["A"]), cu(t["B"]), cu(t["C"]), chunk, cu(t["D"]), None, cu(t["dt_bias"]), None, None)
        ws = sc._workspace(x, B, chunk)
        p = _lib.SsdParams()
        sc._fill_fwd(p, x, dt, A, B, C, chunk, D, None, dt_bias, init, seq_idx, True, (0.0, float("inf")), ws)
        assert _lib.load().ssd_chunk_state_passing_fwd(p, _lib.current_stream(x.device)) == -2  # MAMBA_E_UNSUPPORTED


def test_operator_on_enough_heads_for_the_one_launch_form():
    """batch x heads >= three quarters of the compute units: ssd_combined_fwd forms the entering states in one launch."""
    _fwd_case(2, 512, 96, 64, 128, 1, 256, torch.bfloat16, has_init=True)
    _fwd_case(1, 768, 192, 64, 128, 8, 128, torch.bfloat16, seq_lens=[200, 56, 512], has_init=True)
    # (the backward pass reads the entering states from the same workspace, whichever launch filled it)
