"""mamba_amd: MI355X-native (gfx950) kernels for Mamba's scan hot path behind the reference's
operator API.  See mamba_amd.ops.* for the drop-in entry points."""
import sys
import types

__version__ = "0.1.0"


def install_as_mamba_ssm_ops(causal_conv1d=True):
    """Registers the drop-in modules under the reference's module paths, so that
    `from mamba_ssm.ops.selective_scan_interface import selective_scan_fn` (and the SSD / decode /
    norm imports) resolve to this package.  Existing `mamba_ssm` packages are left in place; only the
    operator modules are replaced.  With causal_conv1d=True (and no such package imported yet) the
    `causal_conv1d` package the reference's modules look for (mamba_ssm/modules/mamba2.py:11-19,
    mamba_ssm/modules/mamba_simple.py:15-18) resolves to this package's convolution as well, so those
    modules take their fused paths instead of falling back to nn.Conv1d."""
    from mamba_amd.ops import selective_scan_interface
    from mamba_amd.ops.triton import (layer_norm, layernorm_gated, selective_state_update, ssd_bmm, ssd_chunk_scan,
                                      ssd_chunk_state, ssd_combined, ssd_state_passing)

    def ensure(name):
        if name not in sys.modules:
            mod = types.ModuleType(name)
            mod.__path__ = []
            sys.modules[name] = mod
        return sys.modules[name]

    for pkg in ("mamba_ssm", "mamba_ssm.ops", "mamba_ssm.ops.triton"):
        ensure(pkg)
    mapping = {
        "mamba_ssm.ops.selective_scan_interface": selective_scan_interface,
        "mamba_ssm.ops.triton.ssd_combined": ssd_combined,
        "mamba_ssm.ops.triton.ssd_chunk_state": ssd_chunk_state,
        "mamba_ssm.ops.triton.ssd_state_passing": ssd_state_passing,
        "mamba_ssm.ops.triton.ssd_bmm": ssd_bmm,
        "mamba_ssm.ops.triton.ssd_chunk_scan": ssd_chunk_scan,
        "mamba_ssm.ops.triton.selective_state_update": selective_state_update,
        "mamba_ssm.ops.triton.layernorm_gated": layernorm_gated,
        "mamba_ssm.ops.triton.layer_norm": layer_norm,
    }
    for name, mod in mapping.items():
        sys.modules[name] = mod
        parent, leaf = name.rsplit(".", 1)
        setattr(sys.modules[parent], leaf, mod)
    setattr(sys.modules["mamba_ssm"], "ops", sys.modules["mamba_ssm.ops"])
    setattr(sys.modules["mamba_ssm.ops"], "triton", sys.modules["mamba_ssm.ops.triton"])
    if causal_conv1d and "causal_conv1d" not in sys.modules:
        from mamba_amd.ops import causal_conv1d as conv
        pkg = ensure("causal_conv1d")
        pkg.causal_conv1d_fn, pkg.causal_conv1d_update = conv.causal_conv1d_fn, conv.causal_conv1d_update
        varlen = types.ModuleType("causal_conv1d.causal_conv1d_varlen")
        varlen.causal_conv1d_varlen_states = conv.causal_conv1d_varlen_states
        sys.modules["causal_conv1d.causal_conv1d_varlen"] = varlen
        pkg.causal_conv1d_varlen = varlen
