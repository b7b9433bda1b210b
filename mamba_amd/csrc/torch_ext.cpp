// Host-side fast path for the decode-step operators: the argument checks, the parameter struct and
// the launch through the C ABI (include/mamba_hip.h) done in C++ on at::Tensor, so that one call costs
// a few microseconds of host time instead of the ~15 us the same work takes in Python + ctypes.
// Built as the Python extension module mamba_amd._torch_ext (pybind11), linked against
// libmamba_gfx950.so; it contains no device code.
//
// Every function here serves the plain, valid case and DECLINES anything else by returning None
// (wrong shapes, dtypes that need a conversion first, CPU tensors): the Python host side then runs
// its own path, which does the conversions and raises the reference's errors
// (mamba_ssm/ops/triton/selective_state_update.py:151-188).  Both paths end in the same kernels.
#include <torch/extension.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <optional>
#include <string>

#include "mamba_hip.h"

namespace {

using OptTensor = std::optional<at::Tensor>;

int dtype_code(const at::Tensor &t) {
  switch (t.scalar_type()) {
    case at::kFloat: return MAMBA_F32;
    case at::kBFloat16: return MAMBA_BF16;
    case at::kHalf: return MAMBA_F16;
    default: return -1;
  }
}

bool on_device(const at::Tensor &t, const c10::Device &dev) { return t.is_cuda() && t.device() == dev; }
bool on_device(const OptTensor &t, const c10::Device &dev) { return !t.has_value() || on_device(*t, dev); }

void *stream_of(const c10::Device &dev) { return c10::hip::getCurrentHIPStream(dev.index()).stream(); }

void check_rc(int rc, const char *what) {
  TORCH_CHECK(rc == MAMBA_OK, what, " failed: ", mamba_hip_strerror(rc), " (code ", rc, ")");
}

// Shape and strides of a tensor that may come without its head axis (inserted at `axis` with stride 0).
struct View {
  int64_t size[4], stride[4];
  int nd;
};
View with_axis(const at::Tensor &t, int full_nd, int axis) {
  View v;
  v.nd = full_nd;
  const int nd = (int)t.dim();
  if (nd == full_nd) {
    for (int i = 0; i < nd; ++i) {
      v.size[i] = t.size(i);
      v.stride[i] = t.stride(i);
    }
  } else {  // one axis short: unsqueeze(axis)
    for (int i = 0, j = 0; i < full_nd; ++i) {
      if (i == axis) {
        v.size[i] = 1;
        v.stride[i] = 0;
      } else {
        v.size[i] = t.size(j);
        v.stride[i] = t.stride(j);
        ++j;
      }
    }
  }
  return v;
}

// selective_state_update (mamba_ssm/ops/triton/selective_state_update.py:135): same argument
// meaning as mamba_amd.ops.triton.selective_state_update.selective_state_update.
OptTensor state_update_fast(const at::Tensor &state, const at::Tensor &x, const at::Tensor &dt, const at::Tensor &A,
                                 const at::Tensor &B, const at::Tensor &C, const OptTensor &D, const OptTensor &z,
                                 const OptTensor &dt_bias, bool dt_softplus, const OptTensor &state_batch_indices) {
  const c10::Device dev = x.device();
  if (!on_device(state, dev) || !on_device(x, dev) || !on_device(dt, dev) || !on_device(A, dev) || !on_device(B, dev) ||
      !on_device(C, dev) || !on_device(D, dev) || !on_device(z, dev) || !on_device(dt_bias, dev) ||
      !on_device(state_batch_indices, dev))
    return std::nullopt;
  const bool has_heads = state.dim() == 4;
  if (!has_heads && state.dim() != 3) return std::nullopt;
  const int xd = has_heads ? 3 : 2;
  if (x.dim() != xd || dt.dim() != xd || A.dim() != xd || B.dim() != (has_heads ? 3 : 2) || C.dim() != B.dim())
    return std::nullopt;
  if (D && D->dim() != xd - 1) return std::nullopt;
  if (dt_bias && dt_bias->dim() != xd - 1) return std::nullopt;
  if (z && z->dim() != xd) return std::nullopt;
  const View s = with_axis(state, 4, 1), vx = with_axis(x, 3, 1), vdt = with_axis(dt, 3, 1), vA = with_axis(A, 3, 0),
             vB = with_axis(B, 3, 1), vC = with_axis(C, 3, 1);
  const int64_t rows = s.size[0], H = s.size[1], P = s.size[2], N = s.size[3], batch = vx.size[0], G = vB.size[1];
  if (batch <= 0 || vx.size[1] != H || vx.size[2] != P) return std::nullopt;
  for (int i = 0; i < 3; ++i)
    if (vdt.size[i] != vx.size[i]) return std::nullopt;
  if (vA.size[0] != H || vA.size[1] != P || vA.size[2] != N) return std::nullopt;
  if (G <= 0 || H % G != 0 || vB.size[0] != batch || vB.size[2] != N) return std::nullopt;
  for (int i = 0; i < 3; ++i)
    if (vC.size[i] != vB.size[i]) return std::nullopt;
  if (!state_batch_indices && rows < batch) return std::nullopt;
  // dtypes the kernel takes as they are; anything else is converted by the Python path
  const int sc = dtype_code(state), xc = dtype_code(x), dc = dtype_code(dt), bc = dtype_code(B);
  if (sc < 0 || xc < 0 || dc < 0 || bc < 0 || A.scalar_type() != at::kFloat) return std::nullopt;
  if (dc != xc && dc != MAMBA_F32) return std::nullopt;
  if (C.scalar_type() != B.scalar_type() || (bc != xc && bc != MAMBA_F32)) return std::nullopt;
  if (D && D->scalar_type() != at::kFloat) return std::nullopt;
  if (dt_bias && dt_bias->scalar_type() != at::kFloat) return std::nullopt;
  if (z && z->scalar_type() != x.scalar_type()) return std::nullopt;
  if (state_batch_indices && (state_batch_indices->scalar_type() != at::kInt || state_batch_indices->dim() != 1 ||
                              state_batch_indices->size(0) != batch || !state_batch_indices->is_contiguous()))
    return std::nullopt;

  MambaStepParams p{};
  p.batch = (int32_t)batch, p.nheads = (int32_t)H, p.dim = (int32_t)P, p.dstate = (int32_t)N, p.ngroups = (int32_t)G;
  p.dt_softplus = dt_softplus ? 1 : 0;
  p.state_rows = (int32_t)rows;
  p.state_dtype = sc, p.x_dtype = xc, p.dt_dtype = dc, p.A_dtype = MAMBA_F32, p.bc_dtype = bc;
  p.state = state.data_ptr(), p.x = x.data_ptr(), p.dt = dt.data_ptr(), p.A = A.data_ptr(), p.B = B.data_ptr(),
  p.C = C.data_ptr();
  p.state_bs = s.stride[0], p.state_hs = s.stride[1], p.state_ps = s.stride[2], p.state_ns = s.stride[3];
  p.x_bs = vx.stride[0], p.x_hs = vx.stride[1], p.x_ps = vx.stride[2];
  p.dt_bs = vdt.stride[0], p.dt_hs = vdt.stride[1], p.dt_ps = vdt.stride[2];
  p.A_hs = vA.stride[0], p.A_ps = vA.stride[1], p.A_ns = vA.stride[2];
  p.B_bs = vB.stride[0], p.B_gs = vB.stride[1], p.B_ns = vB.stride[2];
  p.C_bs = vC.stride[0], p.C_gs = vC.stride[1], p.C_ns = vC.stride[2];
  if (D) {
    const View v = with_axis(*D, 2, 0);
    if (v.size[0] != H || v.size[1] != P) return std::nullopt;
    p.D = D->data_ptr(), p.D_dtype = MAMBA_F32, p.D_hs = v.stride[0], p.D_ps = v.stride[1];
  }
  if (dt_bias) {
    const View v = with_axis(*dt_bias, 2, 0);
    if (v.size[0] != H || v.size[1] != P) return std::nullopt;
    p.dt_bias = dt_bias->data_ptr(), p.dt_bias_dtype = MAMBA_F32, p.dt_bias_hs = v.stride[0], p.dt_bias_ps = v.stride[1];
  }
  if (z) {
    const View v = with_axis(*z, 3, 1);
    for (int i = 0; i < 3; ++i)
      if (v.size[i] != vx.size[i]) return std::nullopt;
    p.z = z->data_ptr(), p.z_bs = v.stride[0], p.z_hs = v.stride[1], p.z_ps = v.stride[2];
  }
  if (state_batch_indices) p.state_batch_indices = state_batch_indices->data_ptr<int32_t>();
  at::Tensor out = at::empty_like(x);
  const View vo = with_axis(out, 3, 1);
  p.out = out.data_ptr(), p.out_bs = vo.stride[0], p.out_hs = vo.stride[1], p.out_ps = vo.stride[2];
  c10::DeviceGuard guard(dev);
  check_rc(ssm_state_update(&p, stream_of(dev)), "ssm_state_update");
  return out;
}

// Strides of a (batch, channel, position) tensor whose last axis may be missing (one position).
void strides_bcl(const at::Tensor &t, int64_t &bs, int64_t &cs, int64_t &ls) {
  bs = t.stride(0), cs = t.stride(1), ls = t.dim() == 3 ? t.stride(2) : 1;
}

// causal_conv1d_update (the causal_conv1d package's function as called at
// mamba_ssm/modules/mamba2.py:298 and mamba_ssm/modules/mamba_simple.py:223): same argument meaning as
// mamba_amd.ops.causal_conv1d.causal_conv1d_update.  weight and bias: one dtype (fp32, bf16 or fp16), contiguous.
OptTensor conv_update_fast(const at::Tensor &x, const at::Tensor &conv_state, const at::Tensor &weight,
                               const OptTensor &bias, bool silu, const OptTensor &cache_seqlens,
                               const OptTensor &conv_state_indices) {
  const c10::Device dev = x.device();
  if (!on_device(x, dev) || !on_device(conv_state, dev) || !on_device(weight, dev) || !on_device(bias, dev) ||
      !on_device(cache_seqlens, dev) || !on_device(conv_state_indices, dev))
    return std::nullopt;
  if ((x.dim() != 2 && x.dim() != 3) || conv_state.dim() != 3 || weight.dim() != 2) return std::nullopt;
  const int64_t batch = x.size(0), dim = x.size(1), seqlen = x.dim() == 3 ? x.size(2) : 1, width = weight.size(1);
  const int xc = dtype_code(x), stc = dtype_code(conv_state), wc = dtype_code(weight);
  if (batch <= 0 || xc < 0 || stc < 0 || wc < 0) return std::nullopt;
  if (!weight.is_contiguous() || weight.size(0) != dim || width < 2 || width > 4) return std::nullopt;
  if (conv_state.size(1) != dim || conv_state.size(2) < width - 1) return std::nullopt;
  if (bias && (bias->scalar_type() != weight.scalar_type() || bias->dim() != 1 || bias->size(0) != dim ||
               !bias->is_contiguous()))
    return std::nullopt;
  auto index_ok = [&](const OptTensor &t) {
    return !t || (t->scalar_type() == at::kInt && t->dim() == 1 && t->size(0) == batch && t->is_contiguous());
  };
  if (!index_ok(conv_state_indices) || !index_ok(cache_seqlens)) return std::nullopt;
  if (!conv_state_indices && conv_state.size(0) != batch) return std::nullopt;

  at::Tensor out = at::empty_like(x);
  CausalConvUpdateParams p{};
  p.batch = (int32_t)batch, p.dim = (int32_t)dim, p.seqlen = (int32_t)seqlen, p.width = (int32_t)width;
  p.state_len = (int32_t)conv_state.size(2);
  p.dtype = xc, p.state_dtype = stc, p.weight_dtype = wc, p.silu = silu ? 1 : 0;
  p.state_rows = (int32_t)conv_state.size(0);
  p.x = x.data_ptr(), p.conv_state = conv_state.data_ptr(), p.weight = weight.data_ptr();
  p.bias = bias ? bias->data_ptr() : nullptr;
  p.out = out.data_ptr();
  p.conv_state_indices = conv_state_indices ? conv_state_indices->data_ptr<int32_t>() : nullptr;
  p.cache_seqlens = cache_seqlens ? cache_seqlens->data_ptr<int32_t>() : nullptr;
  strides_bcl(x, p.x_bs, p.x_cs, p.x_ls);
  strides_bcl(out, p.out_bs, p.out_cs, p.out_ls);
  strides_bcl(conv_state, p.state_bs, p.state_cs, p.state_ls);
  c10::DeviceGuard guard(dev);
  check_rc(::causal_conv1d_update(&p, stream_of(dev)), "causal_conv1d_update");
  return out;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "C++ host side of the decode-step operators of mamba_amd (argument checks + launch through the C ABI)";
  m.def("abi_version", []() { return mamba_hip_query(MAMBA_Q_ABI_VERSION); });
  m.def("selective_state_update", &state_update_fast, py::arg("state"), py::arg("x"), py::arg("dt"), py::arg("A"),
        py::arg("B"), py::arg("C"), py::arg("D"), py::arg("z"), py::arg("dt_bias"), py::arg("dt_softplus"),
        py::arg("state_batch_indices"),
        "Returns out, or None when the arguments need the Python path (conversions, error reporting).");
  m.def("causal_conv1d_update", &conv_update_fast, py::arg("x"), py::arg("conv_state"), py::arg("weight"),
        py::arg("bias"), py::arg("silu"), py::arg("cache_seqlens"), py::arg("conv_state_indices"),
        "Returns out, or None when the arguments need the Python path.");
}
