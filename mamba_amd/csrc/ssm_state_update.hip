// Single-token decode (selective_state_update) for gfx950: a pure HBM-streaming
// kernel.  A wave owns a run of rows (b, h, p..p+rows) of the state; the lanes
// of a row group hold 4 consecutive states each, so a row of `dstate` fp32
// states moves with one 16-byte load and one 16-byte store per lane.  B and C
// of the (batch, group) are loaded once per wave and stay in registers.
#include "common.hpp"

namespace {

DEVI float ld_any(const void *base, int64_t idx, int dtype) {
  switch (dtype) {
    case MAMBA_F32: return static_cast<const float *>(base)[idx];
    case MAMBA_BF16: return ld1<bf16_t>(static_cast<const bf16_t *>(base) + idx);
    default: return ld1<f16_t>(static_cast<const f16_t *>(base) + idx);
  }
}
DEVI void st_any(void *base, int64_t idx, int dtype, float v) {
  switch (dtype) {
    case MAMBA_F32: static_cast<float *>(base)[idx] = v; break;
    case MAMBA_BF16: st1<bf16_t>(static_cast<bf16_t *>(base) + idx, v); break;
    default: st1<f16_t>(static_cast<f16_t *>(base) + idx, v); break;
  }
}

// 4 consecutive states; VEC requires stride 1 and alignment (checked by the host).
template <bool VEC> DEVI void ld_state4(const void *base, int64_t idx, int64_t ns, int dtype, int nvalid, float (&o)[4]) {
  if (VEC) {
    if (dtype == MAMBA_F32) {
      f32x4 v = *reinterpret_cast<const f32x4 *>(static_cast<const float *>(base) + idx);
      o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    } else {
      u32x2 v = *reinterpret_cast<const u32x2 *>(static_cast<const uint16_t *>(base) + idx);
      if (dtype == MAMBA_BF16) {
        o[0] = bf16_lo(v.x); o[1] = bf16_hi(v.x); o[2] = bf16_lo(v.y); o[3] = bf16_hi(v.y);
      } else {
        o[0] = f16_lo(v.x); o[1] = f16_hi(v.x); o[2] = f16_lo(v.y); o[3] = f16_hi(v.y);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = i < nvalid ? ld_any(base, idx + i * ns, dtype) : 0.f;
  }
}
template <bool VEC> DEVI void st_state4(void *base, int64_t idx, int64_t ns, int dtype, int nvalid, const float (&v)[4]) {
  if (VEC) {
    if (dtype == MAMBA_F32) {
      f32x4 o = {v[0], v[1], v[2], v[3]};
      *reinterpret_cast<f32x4 *>(static_cast<float *>(base) + idx) = o;
    } else {
      u32x2 o;
      if (dtype == MAMBA_BF16) {
        o.x = pack_bf16(v[0], v[1]); o.y = pack_bf16(v[2], v[3]);
      } else {
        o.x = pack_f16(v[0], v[1]); o.y = pack_f16(v[2], v[3]);
      }
      *reinterpret_cast<u32x2 *>(static_cast<uint16_t *>(base) + idx) = o;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < nvalid) st_any(base, idx + i * ns, dtype, v[i]);
  }
}

constexpr int ROWS_PER_WAVE_PASS_MAX = 64;

// LPR lanes per row (power of two, 1..64), each lane 4 states per pass over n.
template <bool VEC, int LPR>
__global__ __launch_bounds__(256) void state_update_kernel(const MambaStepParams p, int rows_per_wave) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = blockIdx.z, h = blockIdx.y;
  const int g = h / (p.nheads / p.ngroups);
  constexpr int RPP = 64 / LPR;  // rows per pass
  const int sub = lane % LPR, rsel = lane / LPR;
  const int p_begin = (blockIdx.x * 4 + wave) * rows_per_wave;
  if (p_begin >= p.dim) return;
  const int p_end = min(p_begin + rows_per_wave, p.dim);

  int64_t sb = b;
  if (p.state_batch_indices) {
    const int idx = p.state_batch_indices[b];
    if (idx < 0) {  // padding entry: no state update, zero output
      for (int pp = p_begin + lane; pp < p_end; pp += 64)
        st_any(p.out, b * p.out_bs + h * p.out_hs + pp * p.out_ps, p.x_dtype, 0.f);
      return;
    }
    sb = idx;
  }
  const int64_t state_base = sb * p.state_bs + h * p.state_hs;
  const int N = p.dstate;  // N <= 4 * LPR: one pass over the states of a row
  const int n0 = sub * 4;
  const int nlane = min(max(N - n0, 0), 4);

  // operands that do not depend on the row
  float Bv[4], Cv[4], Av[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bool ok = i < nlane;
    Bv[i] = ok ? ld_any(p.B, b * p.B_bs + g * p.B_gs + (n0 + i) * p.B_ns, p.bc_dtype) : 0.f;
    Cv[i] = ok ? ld_any(p.C, b * p.C_bs + g * p.C_gs + (n0 + i) * p.C_ns, p.bc_dtype) : 0.f;
    Av[i] = ok ? ld_any(p.A, h * p.A_hs + (n0 + i) * p.A_ns, p.A_dtype) : 0.f;
  }
  const bool A_per_row = p.A_ps != 0;
  const bool dt_per_row = p.dt_ps != 0 || (p.dt_bias && p.dt_bias_ps != 0);
  float dt_head = ld_any(p.dt, b * p.dt_bs + h * p.dt_hs, p.dt_dtype);
  if (p.dt_bias) dt_head += ld_any(p.dt_bias, h * p.dt_bias_hs, p.dt_bias_dtype);
  if (p.dt_softplus) dt_head = softplus_f(dt_head);
  float dA_head[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) dA_head[i] = fast_exp(Av[i] * dt_head);

#pragma unroll 2
  for (int pr = p_begin; pr < p_end; pr += RPP) {
    const int row = pr + rsel;
    const bool rvalid = row < p_end;
    const int nvalid = rvalid ? nlane : 0;
    float out = 0.f, x = 0.f;
    if (nvalid > 0) {
      x = ld_any(p.x, b * p.x_bs + h * p.x_hs + row * p.x_ps, p.x_dtype);
      float dt = dt_head;
      if (dt_per_row) {
        dt = ld_any(p.dt, b * p.dt_bs + h * p.dt_hs + row * p.dt_ps, p.dt_dtype);
        if (p.dt_bias) dt += ld_any(p.dt_bias, h * p.dt_bias_hs + row * p.dt_bias_ps, p.dt_bias_dtype);
        if (p.dt_softplus) dt = softplus_f(dt);
      }
      const float dtx = dt * x;
      float s[4], dA[4];
      const int64_t sidx = state_base + row * p.state_ps + n0 * p.state_ns;
      ld_state4<VEC>(p.state, sidx, p.state_ns, p.state_dtype, nvalid, s);
      if (A_per_row || dt_per_row) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float a = Av[i];
          if (A_per_row && i < nvalid) a = ld_any(p.A, h * p.A_hs + row * p.A_ps + (n0 + i) * p.A_ns, p.A_dtype);
          dA[i] = fast_exp(a * dt);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) dA[i] = dA_head[i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        s[i] = __builtin_fmaf(s[i], dA[i], Bv[i] * dtx);
        out = __builtin_fmaf(s[i], Cv[i], out);
      }
      st_state4<VEC>(p.state, sidx, p.state_ns, p.state_dtype, nvalid, s);
    }
    // sum over the LPR lanes of the row
#pragma unroll
    for (int off = LPR / 2; off >= 1; off >>= 1) out += __shfl_xor(out, off, 64);
    if (rvalid && sub == 0) {
      if (p.D) out = __builtin_fmaf(x, ld_any(p.D, h * p.D_hs + row * p.D_ps, p.D_dtype), out);
      if (p.z) {
        const float z = ld_any(p.z, b * p.z_bs + h * p.z_hs + row * p.z_ps, p.x_dtype);
        out *= z * sigmoid_f(z);
      }
      st_any(p.out, b * p.out_bs + h * p.out_hs + row * p.out_ps, p.x_dtype, out);
    }
  }
}

template <bool VEC, int LPR> int launch(const MambaStepParams &p, hipStream_t stream) {
  // rows per wave: enough rows to amortise the per-wave set-up, enough waves to fill 256 CUs
  constexpr int RPP = 64 / LPR;
  int rows_per_wave = RPP * 8;
  const int64_t heads = (int64_t)p.batch * p.nheads;
  while (rows_per_wave > RPP && heads * ((p.dim + rows_per_wave - 1) / rows_per_wave) < 16384) rows_per_wave /= 2;
  const int waves = (p.dim + rows_per_wave - 1) / rows_per_wave;
  dim3 grid((waves + 3) / 4, p.nheads, p.batch), block(256);
  hipLaunchKernelGGL((state_update_kernel<VEC, LPR>), grid, block, 0, stream, p, rows_per_wave);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

template <bool VEC> int dispatch_lpr(const MambaStepParams &p, hipStream_t stream) {
  const int need = (p.dstate + 3) / 4;
  if (need <= 1) return launch<VEC, 1>(p, stream);
  if (need <= 2) return launch<VEC, 2>(p, stream);
  if (need <= 4) return launch<VEC, 4>(p, stream);
  if (need <= 8) return launch<VEC, 8>(p, stream);
  if (need <= 16) return launch<VEC, 16>(p, stream);
  if (need <= 32) return launch<VEC, 32>(p, stream);
  return launch<VEC, 64>(p, stream);
}

bool dtype_ok(int d) { return d == MAMBA_F32 || d == MAMBA_BF16 || d == MAMBA_F16; }

}  // namespace

extern "C" int ssm_state_update(const MambaStepParams *p, mamba_stream_t stream) {
  if (!p || !p->state || !p->x || !p->dt || !p->A || !p->B || !p->C || !p->out) return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->nheads <= 0 || p->dim <= 0 || p->dstate <= 0 || p->ngroups <= 0) return MAMBA_E_BADARG;
  if (p->nheads % p->ngroups != 0) return MAMBA_E_BADARG;
  if (!dtype_ok(p->state_dtype) || !dtype_ok(p->x_dtype) || !dtype_ok(p->dt_dtype) || !dtype_ok(p->A_dtype) ||
      !dtype_ok(p->bc_dtype))
    return MAMBA_E_BADARG;
  if (p->D && !dtype_ok(p->D_dtype)) return MAMBA_E_BADARG;
  if (p->dt_bias && !dtype_ok(p->dt_bias_dtype)) return MAMBA_E_BADARG;
  if (p->batch > 65535 || p->nheads > 65535 || p->dstate > 256) return MAMBA_E_UNSUPPORTED;
  const int es = p->state_dtype == MAMBA_F32 ? 4 : 2;
  const int64_t vb = 4 * es;  // bytes of one 4-state access
  const bool vec = p->state_ns == 1 && p->dstate % 4 == 0 && (reinterpret_cast<uintptr_t>(p->state) % vb) == 0 &&
                   (p->state_bs * es) % vb == 0 && (p->state_hs * es) % vb == 0 && (p->state_ps * es) % vb == 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return vec ? dispatch_lpr<true>(*p, s) : dispatch_lpr<false>(*p, s);
}
