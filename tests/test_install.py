"""install_as_mamba_ssm_ops(): the reference's import paths resolve to this package (host logic, no GPU)."""
import importlib
import sys


def test_reference_import_paths_resolve_here():
    import mamba_amd
    before = {k: v for k, v in sys.modules.items() if k.split(".")[0] in ("mamba_ssm", "causal_conv1d")}
    try:
        for k in before:
            del sys.modules[k]
        mamba_amd.install_as_mamba_ssm_ops()
        m = importlib.import_module("mamba_ssm.ops.selective_scan_interface")
        assert m.selective_scan_fn.__module__.startswith("mamba_amd")
        from mamba_ssm.ops.triton.ssd_combined import mamba_chunk_scan_combined, mamba_split_conv1d_scan_combined
        from mamba_ssm.ops.triton.selective_state_update import selective_state_update
        from mamba_ssm.ops.triton.layernorm_gated import RMSNorm as RMSNormGated, rmsnorm_fn
        from mamba_ssm.ops.triton.layer_norm import RMSNorm, layer_norm_fn, rms_norm_fn
        from causal_conv1d import causal_conv1d_fn, causal_conv1d_update
        from causal_conv1d.causal_conv1d_varlen import causal_conv1d_varlen_states
        # the imports of the reference's own tests/ops/triton/test_ssd.py:10-17
        from mamba_ssm.ops.triton.ssd_chunk_state import chunk_state, chunk_state_ref
        from mamba_ssm.ops.triton.ssd_chunk_state import _chunk_cumsum_fwd, _chunk_state_fwd
        from mamba_ssm.ops.triton.ssd_chunk_state import chunk_state_varlen
        from mamba_ssm.ops.triton.ssd_state_passing import state_passing, state_passing_ref
        from mamba_ssm.ops.triton.ssd_state_passing import _state_passing_fwd
        from mamba_ssm.ops.triton.ssd_chunk_scan import chunk_scan, chunk_scan_ref
        from mamba_ssm.ops.triton.ssd_combined import mamba_chunk_scan, ssd_chunk_scan_combined_ref, ssd_selective_scan
        from mamba_ssm.ops.triton.ssd_combined import mamba_split_conv1d_scan_ref
        from mamba_ssm.ops.triton.ssd_bmm import _bmm_chunk_fwd
        for f in (chunk_state, chunk_state_ref, _chunk_cumsum_fwd, _chunk_state_fwd, chunk_state_varlen, state_passing,
                  state_passing_ref, _state_passing_fwd, chunk_scan, chunk_scan_ref, mamba_chunk_scan,
                  ssd_chunk_scan_combined_ref, ssd_selective_scan, mamba_split_conv1d_scan_ref, _bmm_chunk_fwd):
            assert f.__module__.startswith("mamba_amd"), f
        for f in (mamba_chunk_scan_combined, mamba_split_conv1d_scan_combined, selective_state_update, RMSNormGated,
                  rmsnorm_fn, RMSNorm, layer_norm_fn, rms_norm_fn, causal_conv1d_fn, causal_conv1d_update,
                  causal_conv1d_varlen_states):
            assert f.__module__.startswith("mamba_amd"), f
    finally:
        for k in [k for k in sys.modules if k.split(".")[0] in ("mamba_ssm", "causal_conv1d")]:
            del sys.modules[k]
        sys.modules.update(before)


def test_an_installed_causal_conv1d_package_is_left_alone():
    import types
    import mamba_amd
    before = {k: v for k, v in sys.modules.items() if k.split(".")[0] in ("mamba_ssm", "causal_conv1d")}
    try:
        for k in before:
            del sys.modules[k]
        theirs = types.ModuleType("causal_conv1d")
        sys.modules["causal_conv1d"] = theirs
        mamba_amd.install_as_mamba_ssm_ops()
        assert sys.modules["causal_conv1d"] is theirs and not hasattr(theirs, "causal_conv1d_fn")
    finally:
        for k in [k for k in sys.modules if k.split(".")[0] in ("mamba_ssm", "causal_conv1d")]:
            del sys.modules[k]
        sys.modules.update(before)
