"""ctypes binding of libmamba_gfx950.so (the C ABI declared in include/mamba_hip.h).

The library is the only compute backend: when it is missing, or a call returns
an error code, a RuntimeError is raised.  There is no CPU or PyTorch fallback.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# MAMBA_AMD_LIB names another build of the same library (same C ABI) to load instead of the in-tree one
LIB_PATH = os.environ.get("MAMBA_AMD_LIB") or os.path.join(_HERE, "libmamba_gfx950.so")

MAMBA_F32, MAMBA_BF16, MAMBA_F16 = 0, 1, 2
DTYPE_CODE = {torch.float32: MAMBA_F32, torch.bfloat16: MAMBA_BF16, torch.float16: MAMBA_F16}

c_i32, c_i64, c_vp, c_f32 = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p, ctypes.c_float


class MambaScanParams(ctypes.Structure):
    _fields_ = (
        [(n, c_i32) for n in ("batch", "dim", "seqlen", "dstate", "ngroups", "dtype", "delta_softplus", "bc_const", "a_complex", "reserved0")]
        + [(n, c_vp) for n in ("u", "delta", "A", "B", "C", "D", "z", "delta_bias", "out", "ckpt")]
        + [(n, c_i64) for n in ("u_bs", "u_ds", "delta_bs", "delta_ds", "z_bs", "z_ds", "out_bs", "out_ds",
                                "B_bs", "B_gs", "B_ns", "C_bs", "C_gs", "C_ns")]
        + [(n, c_vp) for n in ("dout", "du", "ddelta", "dz", "out_z", "dB32", "dC32", "dA_part", "dD_part",
                               "ddelta_bias_part")]
        + [(n, c_i64) for n in ("dout_bs", "dout_ds", "du_bs", "du_ds", "ddelta_bs", "ddelta_ds", "dz_bs", "dz_ds",
                                "outz_bs", "outz_ds")]
        + [("dB", c_vp), ("dC", c_vp), ("det_scale", c_vp), ("det_dB", c_vp), ("det_dC", c_vp)]
    )


class MambaStepParams(ctypes.Structure):
    _fields_ = (
        [(n, c_i32) for n in ("batch", "nheads", "dim", "dstate", "ngroups", "dt_softplus", "state_dtype", "x_dtype",
                              "dt_dtype", "dt_bias_dtype", "A_dtype", "bc_dtype", "D_dtype", "state_rows")]
        + [(n, c_vp) for n in ("state", "x", "dt", "A", "B", "C", "D", "z", "dt_bias", "out", "state_batch_indices")]
        + [(n, c_i64) for n in ("state_bs", "state_hs", "state_ps", "state_ns", "x_bs", "x_hs", "x_ps",
                                "dt_bs", "dt_hs", "dt_ps", "dt_bias_hs", "dt_bias_ps", "A_hs", "A_ps", "A_ns",
                                "B_bs", "B_gs", "B_ns", "C_bs", "C_gs", "C_ns", "D_hs", "D_ps",
                                "z_bs", "z_hs", "z_ps", "out_bs", "out_hs", "out_ps")]
    )


class MambaDecodeStepParams(ctypes.Structure):
    _fields_ = (
        [("ssm", MambaStepParams)]
        + [(n, c_i32) for n in ("conv_dim", "width", "state_len", "silu", "conv_state_rows", "conv_weight_dtype")]
        + [(n, c_vp) for n in ("xBC", "conv_state", "conv_weight", "conv_bias", "sync")]
        + [(n, c_i64) for n in ("xBC_bs", "cs_bs", "cs_cs", "cs_ls")]
    )


class SsdParams(ctypes.Structure):
    _fields_ = (
        [(n, c_i32) for n in ("batch", "seqlen", "nheads", "headdim", "dstate", "ngroups", "chunk_size", "nchunks",
                              "dtype", "dt_dtype", "dt_softplus", "D_has_hdim")]
        + [("dt_min", c_f32), ("dt_max", c_f32)]
        + [(n, c_vp) for n in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states", "seq_idx",
                               "out", "out_x", "dt_out", "dA_cumsum", "states", "final_states", "CB")]
        + [(n, c_i64) for n in ("x_bs", "x_ls", "x_hs", "z_bs", "z_ls", "z_hs", "out_bs", "out_ls", "out_hs",
                                "B_bs", "B_ls", "B_gs", "C_bs", "C_ls", "C_gs", "dt_bs", "dt_ls", "dt_hs")]
        + [(n, c_vp) for n in ("dout", "dfinal_states", "dx", "dz", "ddt", "dB", "dC", "dA", "ddt_bias", "dD",
                               "dinitial_states", "dstates", "ddA_cumsum", "ddt_out", "dCB", "dB32", "dC32", "gbuf")]
        + [(n, c_i64) for n in ("dout_bs", "dout_ls", "dout_hs", "dx_bs", "dx_ls", "dx_hs")]
        + [(n, c_vp) for n in ("det_scale", "det_dD", "det_ddA_cumsum", "det_ddt_out", "det_dCB", "det_dB", "det_dC",
                               "det_dA", "det_ddt_bias", "states_lp", "dstates_lp")]
    )


class CausalConvParams(ctypes.Structure):
    _fields_ = (
        [(n, c_i32) for n in ("batch", "dim", "seqlen", "width", "dtype", "silu", "reserved0", "reserved1")]
        + [(n, c_vp) for n in ("x", "weight", "bias", "seq_idx", "out")]
        + [(n, c_i64) for n in ("x_bs", "x_cs", "x_ls", "out_bs", "out_cs", "out_ls")]
        + [(n, c_vp) for n in ("dout", "dx", "dweight", "dbias")]
        + [(n, c_i64) for n in ("dout_bs", "dout_cs", "dout_ls", "dx_bs", "dx_cs", "dx_ls")]
        + [(n, c_vp) for n in ("det_scale", "det_dweight", "det_dbias")]
    )


class CausalConvUpdateParams(ctypes.Structure):
    _fields_ = (
        [(n, c_i32) for n in ("batch", "dim", "seqlen", "width", "state_len", "dtype", "state_dtype", "silu",
                                "state_rows", "weight_dtype")]
        + [(n, c_vp) for n in ("x", "conv_state", "weight", "bias", "out", "conv_state_indices")]
        + [(n, c_i64) for n in ("x_bs", "x_cs", "x_ls", "out_bs", "out_cs", "out_ls", "state_bs", "state_cs", "state_ls")]
        + [("cache_seqlens", c_vp)]
    )


class CausalConvVarlenParams(ctypes.Structure):
    _fields_ = (
        [(n, c_i32) for n in ("nseq", "dim", "total", "state_len", "dtype", "reserved")]
        + [(n, c_vp) for n in ("x", "cu_seqlens", "states")]
        + [(n, c_i64) for n in ("x_ls", "x_cs", "states_bs", "states_cs", "states_ls")]
    )


class NormGatedParams(ctypes.Structure):
    _fields_ = (
        [(n, c_i32) for n in ("rows", "dim", "group_size", "dtype", "is_rms", "norm_before_gate", "nparts")]
        + [("eps", ctypes.c_float)]
        + [(n, c_vp) for n in ("x", "z", "weight", "bias", "out", "mean", "rstd")]
        + [(n, c_i64) for n in ("x_rs", "z_rs", "out_rs")]
        + [(n, c_vp) for n in ("dy", "dx", "dz", "dweight", "dbias", "dw_part", "db_part")]
        + [(n, c_i64) for n in ("dy_rs", "dx_rs", "dz_rs")]
    )


class NormResidualParams(ctypes.Structure):
    _fields_ = (
        [(n, c_i32) for n in ("rows", "dim", "dtype", "res_dtype", "is_rms", "nparts")]
        + [("eps", ctypes.c_float), ("reserved", c_i32)]
        + [(n, c_vp) for n in ("x", "residual", "weight", "bias", "out", "residual_out", "mean", "rstd")]
        + [(n, c_i64) for n in ("x_rs", "residual_rs", "out_rs", "residual_out_rs")]
        + [(n, c_vp) for n in ("dy", "dresidual", "dx", "dresidual_in", "dweight", "dbias", "dw_part", "db_part")]
        + [(n, c_i64) for n in ("dy_rs", "dresidual_rs", "dx_rs", "dresidual_in_rs")]
        + [(n, c_vp) for n in ("x1", "rowscale", "seeds", "mask", "mask1", "weight1", "bias1", "out1", "dy1", "dx1",
                               "dweight1", "dbias1", "dw1_part", "db1_part")]
        + [(n, c_i64) for n in ("x1_rs", "out1_rs", "dy1_rs", "dx1_rs")]
        + [("dropout_p", ctypes.c_float), ("reserved2", c_i32)]
    )


_lib = None


def load():
    """Loads the shared library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m mamba_amd.build` (hipcc, gfx950). "
            "mamba_amd has no fallback backend."
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.mamba_hip_query.argtypes = [ctypes.c_int]
    lib.mamba_hip_query.restype = ctypes.c_int
    lib.mamba_hip_strerror.argtypes = [ctypes.c_int]
    lib.mamba_hip_strerror.restype = ctypes.c_char_p
    lib.mamba_hip_zero.argtypes = [c_vp, c_i64, c_vp]
    lib.mamba_hip_zero.restype = ctypes.c_int
    lib.mamba_hip_copy.argtypes = [c_vp, c_vp, c_i64, c_vp]
    lib.mamba_hip_copy.restype = ctypes.c_int
    for name in ("mamba1_scan_fwd", "mamba1_scan_bwd"):
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(MambaScanParams), c_vp]
        fn.restype = ctypes.c_int
    lib.mamba1_scan_bwd_nparts.argtypes = [ctypes.POINTER(MambaScanParams)]
    lib.mamba1_scan_bwd_nparts.restype = ctypes.c_int
    lib.mamba1_scan_fwd_noalloc.argtypes = [ctypes.POINTER(MambaScanParams), c_vp, c_vp]
    lib.mamba1_scan_fwd_noalloc.restype = ctypes.c_int
    lib.mamba_hip_init.argtypes = []
    lib.mamba_hip_init.restype = ctypes.c_int
    for name in ("ssd_chunk_cumsum_fwd", "ssd_chunk_state_fwd", "ssd_state_passing_fwd", "ssd_chunk_state_passing_fwd",
                 "ssd_bmm_chunk_fwd",
                 "ssd_chunk_scan_fwd", "ssd_combined_fwd", "ssd_chunk_scan_fwd_fused", "ssd_bwd_dz", "ssd_bwd_dstates",
                 "ssd_state_passing_bwd", "ssd_bwd_dx", "ssd_bwd_dBC_state", "ssd_bwd_dcb", "ssd_bmm_chunk_bwd",
                 "ssd_chunk_cumsum_bwd", "ssd_combined_bwd"):
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(SsdParams), c_vp]
        fn.restype = ctypes.c_int
    lib.ssd_bwd_overwrites.argtypes = [ctypes.POINTER(SsdParams)]
    lib.ssd_bwd_overwrites.restype = ctypes.c_int
    lib.ssd_det_convert.argtypes = [c_vp, c_vp, c_i64, c_vp, c_vp]
    lib.ssd_det_convert.restype = ctypes.c_int
    lib.ssd_chunk_state_varlen.argtypes = [ctypes.POINTER(SsdParams), c_vp, ctypes.c_int, c_vp, c_vp]
    lib.ssd_chunk_state_varlen.restype = ctypes.c_int
    lib.ssd_chunk_scan_fwd_fused_supported.argtypes = [ctypes.POINTER(SsdParams)]
    lib.ssd_chunk_scan_fwd_fused_supported.restype = ctypes.c_int
    lib.ssm_state_update.argtypes = [ctypes.POINTER(MambaStepParams), c_vp]
    lib.ssm_state_update.restype = ctypes.c_int
    lib.mamba2_decode_step.argtypes = [ctypes.POINTER(MambaDecodeStepParams), c_vp]
    lib.mamba2_decode_step.restype = ctypes.c_int
    lib.mamba2_decode_step_sync_ints.argtypes = [ctypes.POINTER(MambaDecodeStepParams)]
    lib.mamba2_decode_step_sync_ints.restype = ctypes.c_int64
    for name in ("causal_conv1d_fwd", "causal_conv1d_bwd"):
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(CausalConvParams), c_vp]
        fn.restype = ctypes.c_int
    lib.causal_conv1d_update.argtypes = [ctypes.POINTER(CausalConvUpdateParams), c_vp]
    lib.causal_conv1d_update.restype = ctypes.c_int
    lib.causal_conv1d_varlen_states.argtypes = [ctypes.POINTER(CausalConvVarlenParams), c_vp]
    lib.causal_conv1d_varlen_states.restype = ctypes.c_int
    for name in ("norm_gated_fwd", "norm_gated_bwd"):
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(NormGatedParams), c_vp]
        fn.restype = ctypes.c_int
    lib.mamba_hip_mfma_probe.argtypes = [c_vp, ctypes.c_int, ctypes.c_int, c_vp]
    lib.mamba_hip_mfma_probe.restype = ctypes.c_int64
    lib.mamba_hip_valu_probe.argtypes = [c_vp, ctypes.c_int, ctypes.c_int, c_vp]
    lib.mamba_hip_valu_probe.restype = ctypes.c_int64
    lib.mamba_hip_rows_probe.argtypes = [ctypes.POINTER(c_vp), ctypes.c_int, ctypes.POINTER(c_vp), ctypes.c_int,
                                         ctypes.c_int, ctypes.c_int, c_vp]
    lib.mamba_hip_rows_probe.restype = ctypes.c_int64
    for name in ("norm_residual_fwd", "norm_residual_bwd"):
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(NormResidualParams), c_vp]
        fn.restype = ctypes.c_int
    _lib = lib
    return lib


def check(rc, what):
    if rc != 0:
        msg = load().mamba_hip_strerror(rc).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {rc})")


def ptr(t):
    return None if t is None else t.data_ptr()


_torch_ext = False  # False: not tried yet; None: not built or switched off


def torch_ext():
    """The C++ host side of the decode-step operators (mamba_amd/_torch_ext.so, built by
    `python -m mamba_amd.build` from csrc/torch_ext.cpp), or None when it has not been built or
    MAMBA_AMD_NO_TORCH_EXT=1 is set.  It only shortens the host time of a call: with or without it
    the same kernels of the same library run."""
    global _torch_ext
    if _torch_ext is False:
        _torch_ext = None
        # with MAMBA_AMD_LIB set the extension stays off: it is linked against the in-tree library and would run
        # that one's kernels beside the override's
        if os.environ.get("MAMBA_AMD_NO_TORCH_EXT", "0") != "1" and not os.environ.get("MAMBA_AMD_LIB"):
            load()  # the extension links against the kernel library: fail on that first, and loudly
            try:
                from mamba_amd import _torch_ext as ext
                if ext.abi_version() == _lib.mamba_hip_query(0):
                    _torch_ext = ext
            except ImportError:
                pass
    return _torch_ext


def current_stream(device):
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("mamba_amd kernels need GPU tensors; there is no CPU fallback")
