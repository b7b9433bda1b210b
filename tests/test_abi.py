"""The C ABI on a machine without a GPU: the library loads, exports every function declared in
include/mamba_hip.h, the ctypes mirrors of the parameter structs match the C layout, and the
argument checks that run before any launch reject bad requests."""
import ctypes
import os
import re
import subprocess
import tempfile

import pytest
import torch

from mamba_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mamba_hip.h")


def _declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"^\s*(?:const\s+char\s*\*|int64_t|int)\s*(\w+)\s*\(", src, flags=re.M)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_functions()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in mamba_hip.h but not exported"


def test_query_and_strerror():
    lib = _lib.load()
    assert lib.mamba_hip_query(0) >= 5 and lib.mamba_hip_query(1) == 128 and lib.mamba_hip_query(5) == 512
    assert lib.mamba_hip_query(999) < 0
    assert b"success" in lib.mamba_hip_strerror(0)
    assert b"unsupported" in lib.mamba_hip_strerror(-2)


@pytest.mark.parametrize("name", ["MambaScanParams", "MambaStepParams", "MambaDecodeStepParams", "SsdParams", "CausalConvParams", "CausalConvUpdateParams",
                                  "CausalConvVarlenParams", "NormGatedParams", "NormResidualParams"])
def test_ctypes_structs_match_c_layout(name):
    cls = getattr(_lib, name)
    fields = [f[0] for f in cls._fields_]
    prog = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void){",
            f'printf("%zu\\n", sizeof({name}));']
    prog += [f'printf("%zu\\n", offsetof({name}, {f}));' for f in fields]
    prog += ["return 0;}"]
    with tempfile.TemporaryDirectory() as d:
        src, exe = os.path.join(d, "t.c"), os.path.join(d, "t")
        open(src, "w").write("\n".join(prog))
        subprocess.run(["gcc", "-std=c99", src, "-o", exe], check=True)
        vals = [int(v) for v in subprocess.run([exe], capture_output=True, text=True, check=True).stdout.split()]
    assert vals[0] == ctypes.sizeof(cls)
    for f, off in zip(fields, vals[1:]):
        assert getattr(cls, f).offset == off, f"{name}.{f}"


def test_null_and_inconsistent_arguments_are_rejected_before_launch():
    lib = _lib.load()
    p = _lib.MambaScanParams()
    assert lib.mamba1_scan_fwd(ctypes.byref(p), None) == -1          # null pointers
    s = _lib.MambaStepParams()
    assert lib.ssm_state_update(ctypes.byref(s), None) == -1
    assert lib.mamba2_decode_step(ctypes.byref(_lib.MambaDecodeStepParams()), None) == -1
    q = _lib.SsdParams()
    assert lib.ssd_combined_fwd(ctypes.byref(q), None) == -1
    assert lib.ssd_combined_bwd(ctypes.byref(q), None) == -1
    assert lib.mamba_hip_zero(None, 16, None) == -1
    assert lib.causal_conv1d_fwd(ctypes.byref(_lib.CausalConvParams()), None) == -1
    assert lib.norm_gated_fwd(ctypes.byref(_lib.NormGatedParams()), None) == -1
    assert lib.norm_gated_bwd(ctypes.byref(_lib.NormGatedParams()), None) == -1


def test_host_ops_refuse_cpu_tensors():
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    u = torch.randn(1, 2, 8)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        selective_scan_fn(u, u, -torch.ones(2, 4), torch.randn(1, 4, 8), torch.randn(1, 4, 8))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        selective_state_update(torch.zeros(1, 2, 4), torch.randn(1, 2), torch.randn(1, 2), -torch.ones(2, 4),
                               torch.randn(1, 4), torch.randn(1, 4))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mamba_chunk_scan_combined(torch.randn(1, 8, 2, 4), torch.randn(1, 8, 2), -torch.ones(2),
                                  torch.randn(1, 8, 1, 4), torch.randn(1, 8, 1, 4), 4)


def test_decode_step_refuses_a_state_with_fewer_rows_than_the_batch():
    from mamba_amd.ops.triton.selective_state_update import selective_state_update
    with pytest.raises(RuntimeError, match="rows"):   # checked before anything touches a device
        selective_state_update(torch.zeros(2, 2, 4), torch.randn(3, 2), torch.randn(3, 2), -torch.ones(2, 4),
                               torch.randn(3, 4), torch.randn(3, 4))
    lib = _lib.load()
    s = _lib.MambaStepParams()
    for f in ("state", "x", "dt", "A", "B", "C", "out"):
        setattr(s, f, 256)            # non-null stand-ins: the size checks below run before any launch
    s.batch, s.nheads, s.dim, s.dstate, s.ngroups = 3, 1, 2, 4, 1
    s.state_rows = 2
    assert lib.ssm_state_update(ctypes.byref(s), None) == -1      # row b of a 2-row state for b = 2
    s.state_rows = 0
    assert lib.ssm_state_update(ctypes.byref(s), None) == -1


def test_shape_errors_match_the_reference_behaviour():
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    with pytest.raises(AssertionError):   # nheads % ngroups, ssd_combined.py:346
        mamba_chunk_scan_combined(torch.randn(1, 8, 3, 4), torch.randn(1, 8, 3), -torch.ones(3),
                                  torch.randn(1, 8, 2, 4), torch.randn(1, 8, 2, 4), 4)


def test_torch_extension_loads_and_declines_cpu_tensors():
    """mamba_amd/_torch_ext.so (C++ host side of the decode-step operators): imports without a GPU, reports
    the library's ABI version, and declines (None) instead of launching on CPU tensors."""
    import torch
    from mamba_amd import _lib
    ext = _lib.torch_ext()
    assert ext is not None, "mamba_amd/_torch_ext.so is not built (python -m mamba_amd.build)"
    assert ext.abi_version() == _lib.load().mamba_hip_query(0)
    s, x = torch.zeros(2, 4, 8), torch.zeros(2, 4)
    A, B = -torch.ones(4, 8), torch.zeros(2, 8)
    assert ext.selective_state_update(s, x, x, A, B, B, None, None, None, False, None) is None
    assert ext.causal_conv1d_update(x, torch.zeros(2, 4, 3), torch.zeros(4, 4), None, True, None, None) is None
