// The C++ host side of the operators (the role of the reference's csrc/selective_scan/selective_scan.cpp:226-349 for
// its CUDA kernels): the argument checks, the allocation of outputs and workspaces with torch's caching allocator,
// the parameter struct and the launch through the C ABI (include/mamba_hip.h) on the current HIP stream under a
// device guard, done on at::Tensor, so that one call costs a few microseconds of host time instead of the ~15 us the
// same work takes in Python + ctypes.  Serves the decode-step operators and the training operators
// (selective_scan fwd / bwd, mamba_chunk_scan_combined fwd / bwd).
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

#include <algorithm>
#include <optional>
#include <string>
#include <tuple>
#include <vector>

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

// ------------------------------------------------------------------------------------------------
// Training operators.  What the reference's own binding does on at::Tensor before and after its kernels
// (csrc/selective_scan/selective_scan.cpp:226-349: shape checks, outputs and workspaces from torch's caching
// allocator, the parameter struct, the current stream under a device guard) and what its Python orchestration
// does around the Triton launches (mamba_ssm/ops/triton/ssd_combined.py:343-395, :397-516).  As above, anything
// but the plain valid case is declined with None and served by the Python host side.

using TensorList = std::vector<OptTensor>;

bool rows_ok(const at::Tensor &t, int64_t b, int64_t d, int64_t l, at::ScalarType ty) {
  return t.dim() == 3 && t.size(0) == b && t.size(1) == d && t.size(2) == l && t.scalar_type() == ty && t.stride(2) == 1;
}

// Fills the fields the forward and backward calls share; false = decline.
bool fill_scan(MambaScanParams &p, const at::Tensor &u, const at::Tensor &delta, const at::Tensor &A, const at::Tensor &B,
               const at::Tensor &C, const OptTensor &D, const OptTensor &z, const OptTensor &delta_bias,
               bool delta_softplus) {
  const c10::Device dev = u.device();
  if (!on_device(u, dev) || !on_device(delta, dev) || !on_device(A, dev) || !on_device(B, dev) || !on_device(C, dev) ||
      !on_device(D, dev) || !on_device(z, dev) || !on_device(delta_bias, dev))
    return false;
  const int code = dtype_code(u);
  if (code < 0 || u.dim() != 3 || A.dim() != 2 || A.scalar_type() != at::kFloat || !A.is_contiguous()) return false;
  const int64_t batch = u.size(0), dim = u.size(1), L = u.size(2), N = A.size(1);
  if (batch <= 0 || dim <= 0 || L <= 0 || N <= 0 || A.size(0) != dim || N > mamba_hip_query(MAMBA_Q_MAX_DSTATE)) return false;
  if (batch > INT32_MAX || dim > INT32_MAX || L > INT32_MAX) return false;
  if (!rows_ok(u, batch, dim, L, u.scalar_type()) || !rows_ok(delta, batch, dim, L, u.scalar_type())) return false;
  if (z && !rows_ok(*z, batch, dim, L, u.scalar_type())) return false;
  int64_t G = 1;
  for (const at::Tensor *t : {&B, &C})
    if (t->dim() == 4) G = t->size(1);
  for (const at::Tensor *t : {&B, &C}) {
    if (t->dim() == 2) {
      if (t->scalar_type() != at::kFloat || t->size(0) != dim || t->size(1) != N || !t->is_contiguous()) return false;
    } else if (t->dim() == 4) {
      if (t->scalar_type() != u.scalar_type() || t->stride(3) != 1 || t->size(0) != batch || t->size(1) != G ||
          t->size(2) != N || t->size(3) != L)
        return false;
    } else {
      return false;
    }
  }
  if (dim % G != 0) return false;
  auto vec_ok = [&](const OptTensor &t) {
    return !t || (t->scalar_type() == at::kFloat && t->dim() == 1 && t->size(0) == dim && t->stride(0) == 1);
  };
  if (!vec_ok(D) || !vec_ok(delta_bias)) return false;
  p.batch = (int32_t)batch, p.dim = (int32_t)dim, p.seqlen = (int32_t)L, p.dstate = (int32_t)N, p.ngroups = (int32_t)G;
  p.dtype = code, p.delta_softplus = delta_softplus ? 1 : 0, p.a_complex = 0;
  p.bc_const = (B.dim() == 2 ? 1 : 0) | (C.dim() == 2 ? 2 : 0);
  p.u = u.data_ptr(), p.delta = delta.data_ptr(), p.A = A.data_ptr(), p.B = B.data_ptr(), p.C = C.data_ptr();
  p.D = D ? D->data_ptr() : nullptr, p.z = z ? z->data_ptr() : nullptr;
  p.delta_bias = delta_bias ? delta_bias->data_ptr() : nullptr;
  p.u_bs = u.stride(0), p.u_ds = u.stride(1), p.delta_bs = delta.stride(0), p.delta_ds = delta.stride(1);
  if (z) p.z_bs = z->stride(0), p.z_ds = z->stride(1);
  if (B.dim() == 4) p.B_bs = B.stride(0), p.B_gs = B.stride(1), p.B_ns = B.stride(2);
  if (C.dim() == 4) p.C_bs = C.stride(0), p.C_gs = C.stride(1), p.C_ns = C.stride(2);
  return true;
}

// selective_scan_cuda.fwd (selective_scan.cpp:226) -> (out, ckpt); real A only.
std::optional<std::tuple<at::Tensor, at::Tensor>> scan_fwd_fast(const at::Tensor &u, const at::Tensor &delta,
                                                                const at::Tensor &A, const at::Tensor &B,
                                                                const at::Tensor &C, const OptTensor &D,
                                                                const OptTensor &z, const OptTensor &delta_bias,
                                                                bool delta_softplus) {
  MambaScanParams p{};
  if (!fill_scan(p, u, delta, A, B, C, D, z, delta_bias, delta_softplus)) return std::nullopt;
  const c10::Device dev = u.device();
  const int64_t tile = mamba_hip_query(MAMBA_Q_SCAN_TILE), ntiles = (p.seqlen + tile - 1) / tile;
  at::Tensor out = at::empty_like(delta);
  at::Tensor ckpt = at::empty({p.batch, p.dim, ntiles, p.dstate}, u.options().dtype(at::kFloat));
  p.out = out.data_ptr(), p.out_bs = out.stride(0), p.out_ds = out.stride(1);
  p.ckpt = ckpt.data_ptr<float>();
  c10::DeviceGuard guard(dev);
  check_rc(mamba1_scan_fwd(&p, stream_of(dev)), "mamba1_scan_fwd");
  return std::make_tuple(out, ckpt);
}

// selective_scan_cuda.bwd (selective_scan.cpp:338) -> [du, ddelta, dA, dB, dC, dD, ddelta_bias, dz, out_z]
std::optional<TensorList> scan_bwd_fast(const at::Tensor &u, const at::Tensor &delta, const at::Tensor &A,
                                        const at::Tensor &B, const at::Tensor &C, const OptTensor &D, const OptTensor &z,
                                        const OptTensor &delta_bias, const at::Tensor &dout, const at::Tensor &ckpt,
                                        const OptTensor &dz_in, bool delta_softplus, bool recompute_out_z) {
  MambaScanParams p{};
  if (!fill_scan(p, u, delta, A, B, C, D, z, delta_bias, delta_softplus)) return std::nullopt;
  const c10::Device dev = u.device();
  const int64_t batch = p.batch, dim = p.dim, L = p.seqlen, N = p.dstate, G = p.ngroups;
  if (!on_device(dout, dev) || !on_device(ckpt, dev) || !on_device(dz_in, dev)) return std::nullopt;
  if (!rows_ok(dout, batch, dim, L, u.scalar_type())) return std::nullopt;
  if (dz_in && (!z || !rows_ok(*dz_in, batch, dim, L, u.scalar_type()))) return std::nullopt;
  const int64_t tile = mamba_hip_query(MAMBA_Q_SCAN_TILE), ntiles = (L + tile - 1) / tile;
  if (ckpt.scalar_type() != at::kFloat || ckpt.dim() != 4 || ckpt.size(0) != batch || ckpt.size(1) != dim ||
      ckpt.size(2) != ntiles || ckpt.size(3) != N || !ckpt.is_contiguous())
    return std::nullopt;
  c10::DeviceGuard guard(dev);
  const int nparts = mamba1_scan_bwd_nparts(&p);
  if (nparts <= 0) return std::nullopt;
  const auto f32 = u.options().dtype(at::kFloat);
  at::Tensor du = at::empty_like(u), ddelta = at::empty_like(delta);
  auto operand = [&](const at::Tensor &t, at::Tensor &part, OptTensor &grad) {
    if (t.dim() == 2) {
      part = at::empty({batch, dim, N}, f32);
    } else {
      part = at::empty({batch, G, (int64_t)nparts, N, L}, f32);
      grad = at::empty({batch, G, N, L}, t.options());
    }
  };
  at::Tensor dB32, dC32;
  OptTensor dB, dC, dz, out_z;
  operand(B, dB32, dB);
  operand(C, dC32, dC);
  at::Tensor dA_part = at::empty({batch, dim, N}, f32), dD_part = at::empty({batch, dim}, f32),
             dbias_part = at::empty({batch, dim}, f32);
  if (z) {
    dz = dz_in ? *dz_in : at::empty_like(*z);
    if (recompute_out_z) out_z = at::empty_like(u);
  }
  p.ckpt = ckpt.data_ptr<float>();
  p.dout = dout.data_ptr(), p.du = du.data_ptr(), p.ddelta = ddelta.data_ptr();
  p.dz = dz ? dz->data_ptr() : nullptr, p.out_z = out_z ? out_z->data_ptr() : nullptr;
  p.dB32 = dB32.data_ptr<float>(), p.dC32 = dC32.data_ptr<float>();
  p.dB = dB ? dB->data_ptr() : nullptr, p.dC = dC ? dC->data_ptr() : nullptr;
  p.dA_part = dA_part.data_ptr<float>(), p.dD_part = dD_part.data_ptr<float>();
  p.ddelta_bias_part = dbias_part.data_ptr<float>();
  p.dout_bs = dout.stride(0), p.dout_ds = dout.stride(1), p.du_bs = du.stride(0), p.du_ds = du.stride(1);
  p.ddelta_bs = ddelta.stride(0), p.ddelta_ds = ddelta.stride(1);
  if (dz) p.dz_bs = dz->stride(0), p.dz_ds = dz->stride(1);
  if (out_z) p.outz_bs = out_z->stride(0), p.outz_ds = out_z->stride(1);
  check_rc(mamba1_scan_bwd(&p, stream_of(dev)), "mamba1_scan_bwd");
  TensorList r(9);
  r[0] = du, r[1] = ddelta, r[2] = dA_part.sum(0);
  r[3] = B.dim() == 2 ? OptTensor(dB32.sum(0)) : dB;
  r[4] = C.dim() == 2 ? OptTensor(dC32.sum(0)) : dC;
  if (D) r[5] = dD_part.sum(0);
  if (delta_bias) r[6] = dbias_part.sum(0);
  r[7] = dz, r[8] = out_z;
  return r;
}

// The checks of _prepare (mamba_amd/ops/triton/ssd_combined.py; reference ssd_combined.py:344-369) for operands that
// need no conversion, and the forward fields of SsdParams; false = decline.
struct SsdDims {
  int64_t batch, L, H, P, G, N, Q, nchunks;
  bool lp;
};
bool fill_ssd(SsdParams &p, SsdDims &d, const at::Tensor &x, const at::Tensor &dt, const at::Tensor &A, const at::Tensor &B,
              const at::Tensor &C, int64_t chunk_size, const OptTensor &D, const OptTensor &z, const OptTensor &dt_bias,
              const OptTensor &initial_states, const OptTensor &seq_idx, bool dt_softplus, double dt_min, double dt_max) {
  const c10::Device dev = x.device();
  if (!on_device(x, dev) || !on_device(dt, dev) || !on_device(A, dev) || !on_device(B, dev) || !on_device(C, dev) ||
      !on_device(D, dev) || !on_device(z, dev) || !on_device(dt_bias, dev) || !on_device(initial_states, dev) ||
      !on_device(seq_idx, dev))
    return false;
  const int code = dtype_code(x), dtc = dtype_code(dt);
  if (code < 0 || dtc < 0 || x.dim() != 4 || B.dim() != 4 || C.dim() != 4 || dt.dim() != 3 || A.dim() != 1) return false;
  d.batch = x.size(0), d.L = x.size(1), d.H = x.size(2), d.P = x.size(3), d.G = B.size(2), d.N = B.size(3), d.Q = chunk_size;
  if (d.batch <= 0 || d.L <= 0 || d.H <= 0 || d.G <= 0 || d.H % d.G != 0 || d.Q <= 0 || d.Q > 256) return false;
  if (d.N > mamba_hip_query(MAMBA_Q_SSD_MAX_DSTATE) || d.P > mamba_hip_query(MAMBA_Q_SSD_MAX_HEADDIM)) return false;
  if (B.size(0) != d.batch || B.size(1) != d.L || C.sizes() != B.sizes()) return false;
  if (dt.size(0) != d.batch || dt.size(1) != d.L || dt.size(2) != d.H || A.size(0) != d.H) return false;
  if (B.scalar_type() != x.scalar_type() || C.scalar_type() != x.scalar_type()) return false;
  if (x.stride(3) != 1 || B.stride(3) != 1 || C.stride(3) != 1) return false;
  if (A.scalar_type() != at::kFloat || !A.is_contiguous()) return false;
  if (z && (z->sizes() != x.sizes() || z->scalar_type() != x.scalar_type() || z->stride(3) != 1)) return false;
  if (D && (D->scalar_type() != at::kFloat || !D->is_contiguous() ||
            !((D->dim() == 1 && D->size(0) == d.H) || (D->dim() == 2 && D->size(0) == d.H && D->size(1) == d.P))))
    return false;
  if (dt_bias && (dt_bias->scalar_type() != at::kFloat || dt_bias->dim() != 1 || dt_bias->size(0) != d.H ||
                  !dt_bias->is_contiguous()))
    return false;
  if (initial_states && (initial_states->scalar_type() != at::kFloat || !initial_states->is_contiguous() ||
                         initial_states->dim() != 4 || initial_states->size(0) != d.batch ||
                         initial_states->size(1) != d.H || initial_states->size(2) != d.P || initial_states->size(3) != d.N))
    return false;
  if (seq_idx && (seq_idx->scalar_type() != at::kInt || !seq_idx->is_contiguous() || seq_idx->dim() != 2 ||
                  seq_idx->size(0) != d.batch || seq_idx->size(1) != d.L))
    return false;
  d.nchunks = (d.L + d.Q - 1) / d.Q;
  d.lp = x.scalar_type() == at::kBFloat16;
  p.batch = (int32_t)d.batch, p.seqlen = (int32_t)d.L, p.nheads = (int32_t)d.H, p.headdim = (int32_t)d.P;
  p.dstate = (int32_t)d.N, p.ngroups = (int32_t)d.G, p.chunk_size = (int32_t)d.Q, p.nchunks = (int32_t)d.nchunks;
  p.dtype = code, p.dt_dtype = dtc, p.dt_softplus = dt_softplus ? 1 : 0, p.D_has_hdim = (D && D->dim() == 2) ? 1 : 0;
  p.dt_min = (float)dt_min, p.dt_max = (float)std::min(dt_max, 3.0e38);
  p.x = x.data_ptr(), p.dt = dt.data_ptr(), p.A = A.data_ptr(), p.B = B.data_ptr(), p.C = C.data_ptr();
  p.D = D ? D->data_ptr() : nullptr, p.z = z ? z->data_ptr() : nullptr, p.dt_bias = dt_bias ? dt_bias->data_ptr() : nullptr;
  p.initial_states = initial_states ? initial_states->data_ptr<float>() : nullptr;
  p.seq_idx = seq_idx ? seq_idx->data_ptr<int32_t>() : nullptr;
  p.x_bs = x.stride(0), p.x_ls = x.stride(1), p.x_hs = x.stride(2);
  if (z) p.z_bs = z->stride(0), p.z_ls = z->stride(1), p.z_hs = z->stride(2);
  p.B_bs = B.stride(0), p.B_ls = B.stride(1), p.B_gs = B.stride(2);
  p.C_bs = C.stride(0), p.C_ls = C.stride(1), p.C_gs = C.stride(2);
  p.dt_bs = dt.stride(0), p.dt_ls = dt.stride(1), p.dt_hs = dt.stride(2);
  return true;
}

// _mamba_chunk_scan_combined_fwd (ssd_combined.py:343) without cu_seqlens
// -> [out, out_x, dt_out, dA_cumsum, carried states, final_states]
std::optional<TensorList> ssd_fwd_fast(const at::Tensor &x, const at::Tensor &dt, const at::Tensor &A, const at::Tensor &B,
                                       const at::Tensor &C, int64_t chunk_size, const OptTensor &D, const OptTensor &z,
                                       const OptTensor &dt_bias, const OptTensor &initial_states, const OptTensor &seq_idx,
                                       bool dt_softplus, double dt_min, double dt_max, bool want_out_x) {
  SsdParams p{};
  SsdDims d;
  if (!fill_ssd(p, d, x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx, dt_softplus, dt_min, dt_max))
    return std::nullopt;
  const c10::Device dev = x.device();
  const auto f32 = x.options().dtype(at::kFloat);
  at::Tensor dt_out = at::empty({d.batch, d.H, d.nchunks, d.Q}, f32), dA_cumsum = at::empty({d.batch, d.H, d.nchunks, d.Q}, f32);
  at::Tensor states = at::empty({d.batch, d.nchunks, d.H, d.P, d.N}, f32);
  OptTensor states_lp;
  if (d.lp) states_lp = at::empty({d.batch, d.nchunks, d.H, d.P, d.N}, x.options());
  at::Tensor final_states = at::empty({d.batch, d.H, d.P, d.N}, f32);
  at::Tensor CB = at::empty({d.batch, d.nchunks, d.G, d.Q, d.Q}, f32);
  at::Tensor out = at::empty(x.sizes(), x.options());
  OptTensor out_x;
  if (z && want_out_x) out_x = at::empty(x.sizes(), x.options());
  p.dt_out = dt_out.data_ptr<float>(), p.dA_cumsum = dA_cumsum.data_ptr<float>(), p.states = states.data_ptr<float>();
  p.final_states = final_states.data_ptr<float>(), p.CB = CB.data_ptr<float>();
  p.states_lp = states_lp ? states_lp->data_ptr() : nullptr;
  p.out = out.data_ptr(), p.out_x = out_x ? out_x->data_ptr() : nullptr;
  p.out_bs = out.stride(0), p.out_ls = out.stride(1), p.out_hs = out.stride(2);
  c10::DeviceGuard guard(dev);
  check_rc(ssd_combined_fwd(&p, stream_of(dev)), "ssd_combined_fwd");
  TensorList r(6);
  r[0] = out, r[1] = out_x, r[2] = dt_out, r[3] = dA_cumsum, r[4] = d.lp ? *states_lp : states, r[5] = final_states;
  return r;
}

// _mamba_chunk_scan_combined_bwd (ssd_combined.py:397) with the forward pass's dt_out / dA_cumsum / carried states
// kept, float atomics (the deterministic mode goes through the Python host side)
// -> [dx, ddt, dA, dB, dC, dD, dz, ddt_bias, dinitial_states]
std::optional<TensorList> ssd_bwd_fast(const at::Tensor &dout, const at::Tensor &x, const at::Tensor &dt, const at::Tensor &A,
                                       const at::Tensor &B, const at::Tensor &C, const at::Tensor &out, int64_t chunk_size,
                                       const OptTensor &D, const OptTensor &z, const OptTensor &dt_bias,
                                       const OptTensor &initial_states, const OptTensor &dfinal_states,
                                       const OptTensor &seq_idx, bool dt_softplus, double dt_min, double dt_max,
                                       const at::Tensor &dt_out, const at::Tensor &dA_cumsum, const at::Tensor &carried) {
  SsdParams p{};
  SsdDims d;
  if (!fill_ssd(p, d, x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx, dt_softplus, dt_min, dt_max))
    return std::nullopt;
  const c10::Device dev = x.device();
  if (!on_device(dout, dev) || !on_device(out, dev) || !on_device(dfinal_states, dev) || !on_device(dt_out, dev) ||
      !on_device(dA_cumsum, dev) || !on_device(carried, dev))
    return std::nullopt;
  auto like_x = [&](const at::Tensor &t) { return t.sizes() == x.sizes() && t.scalar_type() == x.scalar_type() && t.stride(3) == 1; };
  if (!like_x(dout) || !like_x(out)) return std::nullopt;
  const std::vector<int64_t> cs = {d.batch, d.H, d.nchunks, d.Q}, ss = {d.batch, d.nchunks, d.H, d.P, d.N};
  auto f32c = [](const at::Tensor &t, const std::vector<int64_t> &shape) {
    return t.scalar_type() == at::kFloat && t.is_contiguous() && t.sizes().vec() == shape;
  };
  if (!f32c(dt_out, cs) || !f32c(dA_cumsum, cs)) return std::nullopt;
  if (carried.sizes().vec() != ss || !carried.is_contiguous() ||
      carried.scalar_type() != (d.lp ? at::kBFloat16 : at::kFloat))
    return std::nullopt;
  if (dfinal_states && (!f32c(*dfinal_states, {d.batch, d.H, d.P, d.N}))) return std::nullopt;
  const auto f32 = x.options().dtype(at::kFloat);
  at::Tensor final_states = at::empty({d.batch, d.H, d.P, d.N}, f32);
  at::Tensor CB = at::empty({d.batch, d.nchunks, d.G, d.Q, d.Q}, f32);
  at::Tensor dx = at::empty(x.sizes(), x.options());
  OptTensor dz, gbuf, dinit;
  if (z) dz = at::empty(x.sizes(), x.options()), gbuf = at::empty(x.sizes(), x.options());
  at::Tensor ddt = at::empty({d.batch, d.L, d.H}, dt.options());
  // one zeroed arena for the small accumulators the kernels add into; the three large ones (dCB, dB32, dC32) are
  // cleared below, and only where the library does not write them whole (ssd_bwd_overwrites)
  const int64_t nD = D ? D->numel() : 0, nHcQ = d.batch * d.H * d.nchunks * d.Q;
  const int64_t nCB = d.batch * d.nchunks * d.G * d.Q * d.Q, nBC = d.batch * d.L * d.G * d.N;
  const int64_t sizes[8] = {d.H, d.H, nD, nHcQ, nHcQ, nCB, nBC, nBC};  // the five small ones first
  int64_t total = 0, off[8];
  for (int i = 0; i < 8; ++i) {
    if (i == 5) total = (total + 63) / 64 * 64;  // the large ones start on 256 bytes
    off[i] = total, total += sizes[i];
  }
  at::Tensor arena = at::empty({total}, f32);
  float *base = arena.data_ptr<float>();
  at::Tensor dstates = at::empty({d.batch, d.nchunks, d.H, d.P, d.N}, d.lp ? x.options() : f32);
  if (initial_states) dinit = at::empty({d.batch, d.H, d.P, d.N}, f32);
  p.dt_out = dt_out.data_ptr<float>(), p.dA_cumsum = dA_cumsum.data_ptr<float>();
  p.final_states = final_states.data_ptr<float>(), p.CB = CB.data_ptr<float>();
  if (d.lp) p.states_lp = carried.data_ptr(); else p.states = carried.data_ptr<float>();
  if (z) p.out_x = out.data_ptr(); else p.out = out.data_ptr();
  p.out_bs = out.stride(0), p.out_ls = out.stride(1), p.out_hs = out.stride(2);
  p.dout = dout.data_ptr(), p.dfinal_states = dfinal_states ? dfinal_states->data_ptr<float>() : nullptr;
  p.dout_bs = dout.stride(0), p.dout_ls = dout.stride(1), p.dout_hs = dout.stride(2);
  p.dx = dx.data_ptr(), p.dz = dz ? dz->data_ptr() : nullptr, p.ddt = ddt.data_ptr(), p.gbuf = gbuf ? gbuf->data_ptr() : nullptr;
  p.dx_bs = dx.stride(0), p.dx_ls = dx.stride(1), p.dx_hs = dx.stride(2);
  p.dA = base + off[0], p.ddt_bias = base + off[1], p.dD = D ? base + off[2] : nullptr;
  p.ddA_cumsum = base + off[3], p.ddt_out = base + off[4];
  p.dCB = base + off[5], p.dB32 = base + off[6], p.dC32 = base + off[7];
  p.dinitial_states = dinit ? dinit->data_ptr<float>() : nullptr;
  if (d.lp) p.dstates_lp = dstates.data_ptr(); else p.dstates = dstates.data_ptr<float>();
  // dB / dC in the operands' dtype: written by the call's last stage
  at::Tensor dB = at::empty({d.batch, d.L, d.G, d.N}, B.options()), dC = at::empty({d.batch, d.L, d.G, d.N}, C.options());
  p.dB = dB.data_ptr(), p.dC = dC.data_ptr();
  c10::DeviceGuard guard(dev);
  const int owned = ssd_bwd_overwrites(&p);
  if (owned == 0) {
    arena.zero_();  // one fill
  } else {
    arena.narrow(0, 0, off[5]).zero_();
    if (!(owned & SSD_OVERWRITES_DCB)) arena.narrow(0, off[5], nCB).zero_();
    if (!(owned & SSD_OVERWRITES_DBC)) arena.narrow(0, off[6], 2 * nBC).zero_();  // dB32 and dC32 are neighbours
  }
  void *stream = stream_of(dev);
  // CB: the fused forward never forms it; the backward kernels may not need it either
  if (owned & SSD_BWD_FORMS_CB) p.CB = nullptr;
  else check_rc(ssd_bmm_chunk_fwd(&p, stream), "ssd_bmm_chunk_fwd");
  check_rc(ssd_combined_bwd(&p, stream), "ssd_combined_bwd");
  auto piece = [&](int i, at::IntArrayRef shape) { return arena.narrow(0, off[i], sizes[i]).view(shape); };
  TensorList r(9);
  r[0] = dx, r[1] = ddt, r[2] = piece(0, {d.H});
  r[3] = dB, r[4] = dC;
  if (D) r[5] = piece(2, D->sizes());
  r[6] = dz;
  if (dt_bias) r[7] = piece(1, {d.H});
  r[8] = dinit;
  return r;
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
  m.def("scan_fwd", &scan_fwd_fast, py::arg("u"), py::arg("delta"), py::arg("A"), py::arg("B"), py::arg("C"), py::arg("D"),
        py::arg("z"), py::arg("delta_bias"), py::arg("delta_softplus"),
        "selective_scan_cuda.fwd: returns (out, ckpt), or None when the arguments need the Python path.");
  m.def("scan_bwd", &scan_bwd_fast, py::arg("u"), py::arg("delta"), py::arg("A"), py::arg("B"), py::arg("C"), py::arg("D"),
        py::arg("z"), py::arg("delta_bias"), py::arg("dout"), py::arg("ckpt"), py::arg("dz"), py::arg("delta_softplus"),
        py::arg("recompute_out_z"),
        "selective_scan_cuda.bwd: returns [du, ddelta, dA, dB, dC, dD, ddelta_bias, dz, out_z], or None.");
  m.def("ssd_fwd", &ssd_fwd_fast, py::arg("x"), py::arg("dt"), py::arg("A"), py::arg("B"), py::arg("C"), py::arg("chunk_size"),
        py::arg("D"), py::arg("z"), py::arg("dt_bias"), py::arg("initial_states"), py::arg("seq_idx"), py::arg("dt_softplus"),
        py::arg("dt_min"), py::arg("dt_max"), py::arg("want_out_x"),
        "Forward of mamba_chunk_scan_combined: [out, out_x, dt_out, dA_cumsum, carried states, final_states], or None.");
  m.def("ssd_bwd", &ssd_bwd_fast, py::arg("dout"), py::arg("x"), py::arg("dt"), py::arg("A"), py::arg("B"), py::arg("C"),
        py::arg("out"), py::arg("chunk_size"), py::arg("D"), py::arg("z"), py::arg("dt_bias"), py::arg("initial_states"),
        py::arg("dfinal_states"), py::arg("seq_idx"), py::arg("dt_softplus"), py::arg("dt_min"), py::arg("dt_max"),
        py::arg("dt_out"), py::arg("dA_cumsum"), py::arg("carried"),
        "Backward of mamba_chunk_scan_combined with the forward pass's workspaces kept: [dx, ddt, dA, dB, dC, dD, dz, "
        "ddt_bias, dinitial_states], or None.");
}
