// Single-token decode (selective_state_update) for gfx950: a pure HBM-streaming
// kernel.  A wave owns a short run of rows (b, h, p..) of the state; the lanes
// of a row hold 4 consecutive states each, so a row of `dstate` fp32 states
// moves with one 16-byte load and one 16-byte store per lane.  All state loads
// of the wave are issued first; the per-head operands (dt, A, B, C) are fetched
// while they are in flight.  Many short waves keep more bytes in flight than a
// grid-stride loop, which is what the HBM3E channels want.
#include "common.hpp"

namespace {

// 4 consecutive states; VEC requires stride 1 and alignment (checked by the host).
template <typename TS, bool VEC> DEVI void ld_state4(const TS *p, int64_t ns, int nvalid, float (&o)[4]) {
  if constexpr (VEC) {
    if constexpr (sizeof(TS) == 4) {
      f32x4 v = *reinterpret_cast<const f32x4 *>(p);
      o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    } else {
      u32x2 v = *reinterpret_cast<const u32x2 *>(p);
      if constexpr (DT<TS>::id == MAMBA_BF16) {
        o[0] = bf16_lo(v.x); o[1] = bf16_hi(v.x); o[2] = bf16_lo(v.y); o[3] = bf16_hi(v.y);
      } else {
        o[0] = f16_lo(v.x); o[1] = f16_hi(v.x); o[2] = f16_lo(v.y); o[3] = f16_hi(v.y);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = i < nvalid ? ld1<TS>(p + i * ns) : 0.f;
  }
}
template <typename TS, bool VEC> DEVI void st_state4(TS *p, int64_t ns, int nvalid, const float (&v)[4]) {
  if constexpr (VEC) {
    if constexpr (sizeof(TS) == 4) {
      f32x4 o = {v[0], v[1], v[2], v[3]};
      *reinterpret_cast<f32x4 *>(p) = o;
    } else {
      u32x2 o;
      if constexpr (DT<TS>::id == MAMBA_BF16) {
        o.x = pack_bf16(v[0], v[1]); o.y = pack_bf16(v[2], v[3]);
      } else {
        o.x = pack_f16(v[0], v[1]); o.y = pack_f16(v[2], v[3]);
      }
      *reinterpret_cast<u32x2 *>(p) = o;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < nvalid) st1<TS>(p + i * ns, v[i]);
  }
}

#ifndef SSU_UNR
#define SSU_UNR 4
#endif
constexpr int UNR = SSU_UNR;  // row passes per wave

// TS: state dtype.  TX: dtype of x, z, out.  TB: dtype of B, C.  TD: dtype of dt.
// A, D and dt_bias are fp32.  lpr = lanes per row (power of two, dstate <= 4 * lpr).
// Addressing: the (batch, head) part of every address is wave-uniform 64-bit scalar math; the
// per-lane part is a 32-bit element offset, so the vector ALU does no 64-bit multiplies (they would
// cost more than the streaming itself).
// Every global load of the wave sits in one branch-free block ahead of the first use: rows and
// states past the end are read from clamped (valid) addresses and masked afterwards, and absent
// optional operands read a stand-in address with a zero weight.  A load under a branch would make
// the compiler wait for all earlier loads at that point, which serialises the memory round trips.
// SHARE (with VEC): B and C are contiguous and aligned, so a lane's 4 values are one load each, and
// the wave has at most 64 rows, so lane j loads the per-row scalars (x, dt, dt_bias, z, D) of row j
// once and the lanes of a row pick them up through the LDS crossbar: 15 vector-memory instructions
// per wave instead of 36 for the same 4 KB of state.
template <typename TS, typename TX, typename TB, typename TD, bool VEC, bool SHARE>
__global__ __launch_bounds__(256) void state_update_kernel(const MambaStepParams p, int lpr_log2) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = blockIdx.z, h = blockIdx.y;
  const int g = h / (p.nheads / p.ngroups);
  const int lpr = 1 << lpr_log2, rpp = 64 >> lpr_log2;  // rows per pass
  const int sub = lane & (lpr - 1), rsel = lane >> lpr_log2;
  const int p_begin = (blockIdx.x * 4 + wave) * rpp * UNR;
  if (p_begin >= p.dim) return;

  TX *outp = static_cast<TX *>(p.out) + b * p.out_bs + h * p.out_hs;
  int64_t sb = b;
  if (p.state_batch_indices) {
    const int idx = p.state_batch_indices[b];
    if (idx < 0 || idx >= p.state_rows) {  // padding entry: no state update, zero output
      const int row = p_begin + lane;
      if (lane < rpp * UNR && row < p.dim) st1<TX>(outp + row * (int)p.out_ps, 0.f);
      return;
    }
    sb = idx;
  }
  const int N = p.dstate;
  const int n0 = sub * 4;
  const int nlane = min(max(N - n0, 0), 4);
  const int n0c = VEC ? min(n0, N - 4) : n0;  // clamped start of this lane's 4 states (VEC: N % 4 == 0)
  const int row0 = p_begin + rsel;
  // wave-uniform bases
  TS *state = static_cast<TS *>(p.state) + sb * p.state_bs + h * p.state_hs;
  const TX *xp = static_cast<const TX *>(p.x) + b * p.x_bs + h * p.x_hs;
  const TD *dtp = static_cast<const TD *>(p.dt) + b * p.dt_bs + h * p.dt_hs;
  const float *Ap = static_cast<const float *>(p.A) + h * p.A_hs;
  const TB *Bp = static_cast<const TB *>(p.B) + b * p.B_bs + g * p.B_gs;
  const TB *Cp = static_cast<const TB *>(p.C) + b * p.C_bs + g * p.C_gs;
  // optional operands: a stand-in pointer of the right type, stride 0 and weight 0 when absent
  const bool has_z = p.z != nullptr, has_D = p.D != nullptr, has_dtb = p.dt_bias != nullptr;
  const TX *zp = has_z ? static_cast<const TX *>(p.z) + b * p.z_bs + h * p.z_hs : xp;
  const float *dtb = has_dtb ? static_cast<const float *>(p.dt_bias) + h * p.dt_bias_hs : Ap;
  const float *Dp = has_D ? static_cast<const float *>(p.D) + h * p.D_hs : Ap;
  // 32-bit strides (the host checks that the per-head extents fit)
  const int s_ps = (int)p.state_ps, s_ns = (int)p.state_ns, x_ps = (int)p.x_ps, dt_ps = (int)p.dt_ps;
  const int dtb_ps = has_dtb ? (int)p.dt_bias_ps : 0, A_ps = (int)p.A_ps, A_ns = (int)p.A_ns;
  const int B_ns = (int)p.B_ns, C_ns = (int)p.C_ns;
  const int z_ps = has_z ? (int)p.z_ps : 0, D_ps = has_D ? (int)p.D_ps : 0, out_ps = (int)p.out_ps;
  const bool A_per_row = A_ps != 0;
  const bool dt_per_row = dt_ps != 0 || dtb_ps != 0;

  // 1. all loads
  float s[UNR][4], xs[UNR], dts[UNR], dtbs[UNR], zs[UNR], Ds[UNR], Arow[UNR][4];
  bool live[UNR];
#pragma unroll
  for (int k = 0; k < UNR; ++k) {
    const int row = row0 + k * rpp;
    live[k] = row < p.dim && nlane > 0;
    const int rc = min(row, p.dim - 1);
    if constexpr (VEC) {
      ld_state4<TS, true>(state + rc * s_ps + n0c * s_ns, s_ns, 4, s[k]);
    } else {
      ld_state4<TS, false>(state + rc * s_ps + n0 * s_ns, s_ns, live[k] ? nlane : 0, s[k]);
    }
    if constexpr (!SHARE) {
      xs[k] = ld1<TX>(xp + rc * x_ps);
      dts[k] = ld1<TD>(dtp + rc * dt_ps);
      dtbs[k] = dtb[rc * dtb_ps];
      zs[k] = ld1<TX>(zp + rc * z_ps);
      Ds[k] = Dp[rc * D_ps];
    }
  }
  float Bv[4], Cv[4], Av[4];
  float x_j = 0.f, dt_j = 0.f, dtb_j = 0.f, z_j = 0.f, D_j = 0.f;  // SHARE: the scalars of row p_begin + lane
  if constexpr (SHARE) {
    const int rj = min(p_begin + lane, p.dim - 1);
    x_j = ld1<TX>(xp + rj * x_ps);
    dt_j = ld1<TD>(dtp + rj * dt_ps);
    dtb_j = dtb[rj * dtb_ps];
    z_j = ld1<TX>(zp + rj * z_ps);
    D_j = Dp[rj * D_ps];
    ld_state4<TB, true>(Bp + n0c, 1, 4, Bv);
    ld_state4<TB, true>(Cp + n0c, 1, 4, Cv);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int nc = min(n0 + i, N - 1);
    if constexpr (!SHARE) {
      Bv[i] = ld1<TB>(Bp + nc * B_ns);
      Cv[i] = ld1<TB>(Cp + nc * C_ns);
    }
    if (!SHARE || i == 0) Av[i] = Ap[nc * A_ns];
  }
  if constexpr (SHARE) {  // one A per head (stride 0 along the states) needs no further loads
    if (A_ns != 0) {
#pragma unroll
      for (int i = 1; i < 4; ++i) Av[i] = Ap[min(n0 + i, N - 1) * A_ns];
    } else {
      Av[1] = Av[2] = Av[3] = Av[0];
    }
  }
  if (A_per_row) {  // uniform; the block holds loads only
#pragma unroll
    for (int k = 0; k < UNR; ++k) {
      const int rc = min(row0 + k * rpp, p.dim - 1);
#pragma unroll
      for (int i = 0; i < 4; ++i) Arow[k][i] = Ap[rc * A_ps + min(n0 + i, N - 1) * A_ns];
    }
  }
  // 2. masks and per-head values
  if constexpr (SHARE) {
#pragma unroll
    for (int k = 0; k < UNR; ++k) {
      const int src = rsel + k * rpp;  // the lane that holds this row's scalars
      xs[k] = __shfl(x_j, src, 64);
      dts[k] = __shfl(dt_j, src, 64);
      dtbs[k] = __shfl(dtb_j, src, 64);
      zs[k] = __shfl(z_j, src, 64);
      Ds[k] = __shfl(D_j, src, 64);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bool ok = i < nlane;
    Bv[i] = ok ? Bv[i] : 0.f;
    Cv[i] = ok ? Cv[i] : 0.f;
    Av[i] *= kLog2e;
  }
  const float w_dtb = has_dtb ? 1.f : 0.f, w_D = has_D ? 1.f : 0.f;
  const bool per_row = A_per_row || dt_per_row;
  float dt_head = __builtin_fmaf(w_dtb, dtbs[0], dts[0]);
  if (p.dt_softplus) dt_head = softplus_f(dt_head);
  float dA_head[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) dA_head[i] = fast_exp2(Av[i] * dt_head);

  float outs[UNR];
#pragma unroll
  for (int k = 0; k < UNR; ++k) {
    float dt = dt_head;
    float dA[4];
    if (per_row) {
      dt = __builtin_fmaf(w_dtb, dtbs[k], dts[k]);
      if (p.dt_softplus) dt = softplus_f(dt);
#pragma unroll
      for (int i = 0; i < 4; ++i) dA[i] = fast_exp2((A_per_row ? Arow[k][i] * kLog2e : Av[i]) * dt);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) dA[i] = dA_head[i];
    }
    const float dtx = dt * xs[k];
    float out = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s[k][i] = __builtin_fmaf(s[k][i], dA[i], Bv[i] * dtx);
      out = __builtin_fmaf(s[k][i], Cv[i], out);
    }
    outs[k] = live[k] ? out : 0.f;
    if (live[k]) {
      const int row = row0 + k * rpp;
      st_state4<TS, VEC>(state + row * s_ps + n0 * s_ns, s_ns, nlane, s[k]);
    }
  }
  // 3. sum over the lanes of each row, then the skip connection and the gate
#pragma unroll
  for (int k = 0; k < UNR; ++k) {
    const int row = row0 + k * rpp;
    float out = outs[k];
    for (int off = lpr >> 1; off >= 1; off >>= 1) out += __shfl_xor(out, off, 64);
    if (row < p.dim && sub == 0) {
      out = __builtin_fmaf(xs[k] * w_D, Ds[k], out);
      if (has_z) out *= zs[k] * sigmoid_f(zs[k]);
      st1<TX>(outp + row * out_ps, out);
    }
  }
}

template <typename TS, typename TX, typename TB, typename TD, bool VEC>
int launch(const MambaStepParams &p, hipStream_t stream) {
  int lpr_log2 = 0;
  while ((4 << lpr_log2) < p.dstate) ++lpr_log2;  // dstate <= 256 -> lpr <= 64
  const int rows_per_block = 4 * (64 >> lpr_log2) * UNR;
  dim3 grid((p.dim + rows_per_block - 1) / rows_per_block, p.nheads, p.batch), block(256);
  if constexpr (VEC) {
    // the shared loads need contiguous, aligned B / C rows and at most 64 rows per wave
    const int64_t eb = sizeof(TB), ab = 4 * eb;
    const bool share = (64 >> lpr_log2) * UNR <= 64 && p.B_ns == 1 && p.C_ns == 1 &&
                       reinterpret_cast<uintptr_t>(p.B) % ab == 0 && reinterpret_cast<uintptr_t>(p.C) % ab == 0 &&
                       (p.B_bs * eb) % ab == 0 && (p.B_gs * eb) % ab == 0 && (p.C_bs * eb) % ab == 0 &&
                       (p.C_gs * eb) % ab == 0;
    if (share) {
      hipLaunchKernelGGL((state_update_kernel<TS, TX, TB, TD, true, true>), grid, block, 0, stream, p, lpr_log2);
      return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
    }
  }
  hipLaunchKernelGGL((state_update_kernel<TS, TX, TB, TD, VEC, false>), grid, block, 0, stream, p, lpr_log2);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

template <typename TS, typename TX, typename TB, typename TD> int launch_vec(const MambaStepParams &p, hipStream_t s) {
  const int es = sizeof(TS);
  const int64_t vb = 4 * es;  // bytes of one 4-state access
  const bool vec = p.state_ns == 1 && p.dstate % 4 == 0 && (reinterpret_cast<uintptr_t>(p.state) % vb) == 0 &&
                   (p.state_bs * es) % vb == 0 && (p.state_hs * es) % vb == 0 && (p.state_ps * es) % vb == 0;
  return vec ? launch<TS, TX, TB, TD, true>(p, s) : launch<TS, TX, TB, TD, false>(p, s);
}

// B/C and dt are either of x's dtype or fp32.
template <typename TS, typename TX> int dispatch_small(const MambaStepParams &p, hipStream_t s) {
  const bool bc32 = p.bc_dtype == MAMBA_F32, dt32 = p.dt_dtype == MAMBA_F32;
  if (!bc32 && p.bc_dtype != DT<TX>::id) return MAMBA_E_UNSUPPORTED;
  if (!dt32 && p.dt_dtype != DT<TX>::id) return MAMBA_E_UNSUPPORTED;
  if constexpr (DT<TX>::id == MAMBA_F32) {
    return launch_vec<TS, TX, float, float>(p, s);
  } else {
    if (bc32 && dt32) return launch_vec<TS, TX, float, float>(p, s);
    if (bc32) return launch_vec<TS, TX, float, TX>(p, s);
    if (dt32) return launch_vec<TS, TX, TX, float>(p, s);
    return launch_vec<TS, TX, TX, TX>(p, s);
  }
}

template <typename TS> int dispatch_x(const MambaStepParams &p, hipStream_t s) {
  switch (p.x_dtype) {
    case MAMBA_F32: return dispatch_small<TS, float>(p, s);
    case MAMBA_BF16: return dispatch_small<TS, bf16_t>(p, s);
    default: return dispatch_small<TS, f16_t>(p, s);
  }
}

bool dtype_ok(int d) { return d == MAMBA_F32 || d == MAMBA_BF16 || d == MAMBA_F16; }

// ------------------------------------------------------------------ fused decode step
// causal_conv1d_update over the x / B / C channels and the state update in one launch (the pair of calls
// of the reference's Mamba2.step, mamba_ssm/modules/mamba2.py:298-336).  Same decomposition as
// state_update_kernel; on top of it
//   * lane j of a wave convolves the x channel of the wave's row j, shifts that channel's conv state in
//     place (no other wave reads it) and hands the value to the lanes of the row;
//   * every workgroup convolves the B and C channels of its head's group from the OLD conv state (re-done
//     per workgroup: a few cached loads per thread, shared through LDS) -- so nobody may shift those shared
//     channels until every workgroup of the batch entry has read them.  Workgroups count themselves off in
//     `sync` when their loads are done; the one that arrives last shifts the B / C channels and puts the
//     counters back to zero.  Nobody waits.
// The convolution's outputs are rounded to the activation dtype as the separate kernel's stored output is,
// so the fused step and the two calls give the same bits.
DEVI float silu_act(float v) { return v * sigmoid_f(v); }
template <typename T> DEVI float round_to(float x) {
  if constexpr (DT<T>::id == MAMBA_F32) return x;
  else if constexpr (DT<T>::id == MAMBA_BF16) return __builtin_bit_cast(float, f32_to_bf16_bits(x) << 16);
  else return (float)(_Float16)x;
}

constexpr int CW = 4;  // widest filter, longest conv state
constexpr int SYNC_FAN = 16;  // arrivals per counter

// taps sv[0..2] = the conv state's last three positions (0 where the state is shorter), xn the new value,
// w[0..3] the filter right-aligned in 4 taps
DEVI float conv_tap(const float (&sv)[3], float xn, const float (&w)[4], float bias, bool silu) {
  float v = bias;
  v = __builtin_fmaf(w[0], sv[0], v);
  v = __builtin_fmaf(w[1], sv[1], v);
  v = __builtin_fmaf(w[2], sv[2], v);
  v = __builtin_fmaf(w[3], xn, v);
  return silu ? silu_act(v) : v;
}

// one filter tap or bias value of the dtype the caller's parameters have
DEVI float param_at(const void *base, int dtype, int64_t i) {
  switch (dtype) {
    case MAMBA_BF16: return ld1<bf16_t>(static_cast<const bf16_t *>(base) + i);
    case MAMBA_F16: return ld1<f16_t>(static_cast<const f16_t *>(base) + i);
    default: return static_cast<const float *>(base)[i];
  }
}

// this thread's conv state taps and filter of channel c (element loads from valid addresses)
template <typename TX>
DEVI void conv_loads(const MambaDecodeStepParams &q, const TX *cstate, const TX *xBC, int c, float (&sv)[3], float &xn,
                     float (&w)[4], float &bias) {
  const int SL = q.state_len, W = q.width, cs_cs = (int)q.cs_cs, cs_ls = (int)q.cs_ls;
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    const int j = SL - 3 + i;
    const float v = ld1<TX>(cstate + c * cs_cs + max(j, 0) * cs_ls);
    sv[i] = j >= 0 ? v : 0.f;
  }
  xn = ld1<TX>(xBC + c);
  const int wd = q.conv_weight_dtype;
  if (wd == MAMBA_F32 && W == CW) {
    const f32x4 wq = *reinterpret_cast<const f32x4 *>(static_cast<const float *>(q.conv_weight) + (int64_t)c * CW);
    w[0] = wq.x; w[1] = wq.y; w[2] = wq.z; w[3] = wq.w;
  } else if (wd != MAMBA_F32 && W == CW) {  // four 16-bit taps: one 8-byte load
    const u32x2 wq = *reinterpret_cast<const u32x2 *>(static_cast<const uint16_t *>(q.conv_weight) + (int64_t)c * CW);
    if (wd == MAMBA_BF16) {
      w[0] = bf16_lo(wq.x); w[1] = bf16_hi(wq.x); w[2] = bf16_lo(wq.y); w[3] = bf16_hi(wq.y);
    } else {
      w[0] = f16_lo(wq.x); w[1] = f16_hi(wq.x); w[2] = f16_lo(wq.y); w[3] = f16_hi(wq.y);
    }
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int j = k - (CW - W);
      const float v = param_at(q.conv_weight, wd, (int64_t)c * W + max(j, 0));
      w[k] = j >= 0 ? v : 0.f;
    }
  }
  bias = q.conv_bias ? param_at(q.conv_bias, wd, c) : 0.f;
}
// conv state of one channel after the step: the old positions moved down by one, the new value last
template <typename TX> DEVI void conv_shift(TX *st, int SL, int cs_ls, const float (&sv)[3], float xn) {
  st1<TX>(st + (SL - 1) * cs_ls, xn);
  if (SL > 1) st1<TX>(st + (SL - 2) * cs_ls, sv[2]);
  if (SL > 2) st1<TX>(st + (SL - 3) * cs_ls, sv[1]);
  if (SL > 3) st1<TX>(st + (SL - 4) * cs_ls, sv[0]);
}

template <typename TS, typename TX, typename TD>
__global__ __launch_bounds__(256) void decode_step_fused_kernel(const MambaDecodeStepParams q, int lpr_log2) {
  const MambaStepParams &p = q.ssm;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = blockIdx.z, h = blockIdx.y;
  const int G = p.ngroups, N = p.dstate, hpg = p.nheads / G;
  const int g = h / hpg;
  const int lpr = 1 << lpr_log2, rpp = 64 >> lpr_log2;
  const int sub = lane & (lpr - 1), rsel = lane >> lpr_log2;
  const int p_begin = (blockIdx.x * 4 + wave) * rpp * UNR;  // may lie past the head's rows: such a wave loads from
  const int SL = q.state_len;                               // clamped rows like any other and stores nothing
  const int cs_cs = (int)q.cs_cs, cs_ls = (int)q.cs_ls;
  TX *cstate = static_cast<TX *>(q.conv_state) + b * q.cs_bs;
  const TX *xBC = static_cast<const TX *>(q.xBC) + b * q.xBC_bs;
  const int c_B0 = p.nheads * p.dim + g * N, c_C0 = c_B0 + G * N;  // first B / C channel of this group
  __shared__ __align__(16) float bc_lds[2 * 256];
  __shared__ int s_last;

  const int n0 = sub * 4;
  const int nlane = min(max(N - n0, 0), 4);
  const int n0c = min(n0, N - 4);  // the host requires N % 4 == 0
  const int row0 = p_begin + rsel;
  TS *state = static_cast<TS *>(p.state) + (int64_t)b * p.state_bs + h * p.state_hs;
  const int s_ps = (int)p.state_ps;
  const bool has_z = p.z != nullptr, has_D = p.D != nullptr, has_dtb = p.dt_bias != nullptr;
  const TX *zp = has_z ? static_cast<const TX *>(p.z) + b * p.z_bs + h * p.z_hs : xBC;
  const int z_ps = has_z ? (int)p.z_ps : 0;

  // 1. every load of the thread, branch-free, from clamped addresses: the state rows first
  float s[UNR][4];
  bool live[UNR];
#pragma unroll
  for (int k = 0; k < UNR; ++k) {
    const int row = row0 + k * rpp;
    live[k] = row < p.dim && nlane > 0;
    ld_state4<TS, true>(state + min(row, p.dim - 1) * s_ps + n0c, 1, 4, s[k]);
  }
  // the x channel of row p_begin + lane
  const int rj = min(p_begin + lane, p.dim - 1);
  const bool mine = lane < rpp * UNR && p_begin + lane < p.dim;
  const int cx = h * p.dim + rj;
  float xsv[3], xw[4], xn, xbias;
  conv_loads<TX>(q, cstate, xBC, cx, xsv, xn, xw, xbias);
  const float z_j = ld1<TX>(zp + rj * z_ps);
  // the B / C channels of this head's group: thread t takes channels t and t + 256 of the 2 N (B first, then C)
  constexpr int BCI = 2;  // 2 N <= 512
  float bsv[BCI][3], bw[BCI][4], bxn[BCI], bbias[BCI];
  int bc_c[BCI];
#pragma unroll
  for (int it = 0; it < BCI; ++it) {
    const int t = min((int)threadIdx.x + it * 256, 2 * N - 1);
    bc_c[it] = t < N ? c_B0 + t : c_C0 + (t - N);
    conv_loads<TX>(q, cstate, xBC, bc_c[it], bsv[it], bxn[it], bw[it], bbias[it]);
  }
  // per head: dt, dt_bias, A, D
  const float dt_raw = ld1<TD>(static_cast<const TD *>(p.dt) + b * p.dt_bs + h * p.dt_hs);
  const float dtb = has_dtb ? static_cast<const float *>(p.dt_bias)[h * p.dt_bias_hs] : 0.f;
  const float A2 = static_cast<const float *>(p.A)[h * p.A_hs] * kLog2e;
  const float Dh = has_D ? static_cast<const float *>(p.D)[h * p.D_hs] : 0.f;

  // 2. convolutions: B / C once per workgroup, shared through LDS
#pragma unroll
  for (int it = 0; it < BCI; ++it) {
    const int t = (int)threadIdx.x + it * 256;
    if (t < 2 * N) bc_lds[t] = round_to<TX>(conv_tap(bsv[it], bxn[it], bw[it], bbias[it], q.silu));
  }
  const float x_j = round_to<TX>(conv_tap(xsv, xn, xw, xbias, q.silu));
  if (mine) conv_shift<TX>(cstate + cx * cs_cs, SL, cs_ls, xsv, xn);  // no other thread reads this channel
  __syncthreads();
  float Bv[4], Cv[4];
  {
    const f32x4 bq = *reinterpret_cast<const f32x4 *>(bc_lds + n0c), cq = *reinterpret_cast<const f32x4 *>(bc_lds + N + n0c);
    Bv[0] = bq.x; Bv[1] = bq.y; Bv[2] = bq.z; Bv[3] = bq.w;
    Cv[0] = cq.x; Cv[1] = cq.y; Cv[2] = cq.z; Cv[3] = cq.w;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = i < nlane;
      Bv[i] = ok ? Bv[i] : 0.f;
      Cv[i] = ok ? Cv[i] : 0.f;
    }
  }
  // 3. the state update
  float dt = dt_raw + dtb;
  if (p.dt_softplus) dt = softplus_f(dt);
  const float dA = fast_exp2(A2 * dt);
  float outs[UNR], xs[UNR], zs[UNR];
#pragma unroll
  for (int k = 0; k < UNR; ++k) {
    const int src = rsel + k * rpp;  // the lane that holds this row's scalars
    xs[k] = __shfl(x_j, src, 64);
    zs[k] = __shfl(z_j, src, 64);
    const float dtx = dt * xs[k];
    float out = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s[k][i] = __builtin_fmaf(s[k][i], dA, Bv[i] * dtx);
      out = __builtin_fmaf(s[k][i], Cv[i], out);
    }
    outs[k] = live[k] ? out : 0.f;
    if (live[k]) st_state4<TS, true>(state + (row0 + k * rpp) * s_ps + n0, 1, nlane, s[k]);
  }
  TX *outp = static_cast<TX *>(p.out) + b * p.out_bs + h * p.out_hs;
#pragma unroll
  for (int k = 0; k < UNR; ++k) {
    const int row = row0 + k * rpp;
    float out = outs[k];
    for (int off = lpr >> 1; off >= 1; off >>= 1) out += __shfl_xor(out, off, 64);
    if (row < p.dim && sub == 0) {
      out = __builtin_fmaf(xs[k], Dh, out);
      if (has_z) out *= zs[k] * sigmoid_f(zs[k]);
      st1<TX>(outp + row * (int)p.out_ps, out);
    }
  }
  // 4. count this workgroup off among those of its (batch entry, group), in two levels so that no counter sees
  // more than SYNC_FAN arrivals (atomics to one address serialise); the last one shifts the conv state of the
  // group's B / C channels, which it still holds in registers.  Relaxed atomics are enough: the loads of the old
  // conv state have returned (their values went into LDS before the barrier above), and the last workgroup's stores
  // follow its own arrival in program order; acquire / release at device scope would write back and invalidate
  // the L2 at every arrival.
  if (threadIdx.x == 0) {
    const int nwg = (int)gridDim.x * hpg, wg = (h - g * hpg) * (int)gridDim.x + (int)blockIdx.x;
    const int ngrp = (nwg + SYNC_FAN - 1) / SYNC_FAN, grp = wg / SYNC_FAN;
    const int in_grp = min(SYNC_FAN, nwg - grp * SYNC_FAN);
    int *cnt = q.sync + ((int64_t)b * G + g) * (ngrp + 1);
    int last = 0;
    if (__hip_atomic_fetch_add(cnt + 1 + grp, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == in_grp - 1) {
      __hip_atomic_store(cnt + 1 + grp, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (__hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ngrp - 1) {
        __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last = 1;
      }
    }
    s_last = last;
  }
  __syncthreads();
  if (!s_last) return;
#pragma unroll
  for (int it = 0; it < BCI; ++it) {
    if ((int)threadIdx.x + it * 256 < 2 * N) conv_shift<TX>(cstate + bc_c[it] * cs_cs, SL, cs_ls, bsv[it], bxn[it]);
  }
}

int fused_grid_x(const MambaStepParams &p, int *lpr_log2_out) {
  int lpr_log2 = 0;
  while ((4 << lpr_log2) < p.dstate) ++lpr_log2;
  if (lpr_log2_out) *lpr_log2_out = lpr_log2;
  const int rows_per_block = 4 * (64 >> lpr_log2) * UNR;
  return (p.dim + rows_per_block - 1) / rows_per_block;
}

template <typename TS, typename TX, typename TD> int launch_fused(const MambaDecodeStepParams &q, hipStream_t stream) {
  const MambaStepParams &p = q.ssm;
  int lpr_log2 = 0;
  dim3 grid(fused_grid_x(p, &lpr_log2), p.nheads, p.batch), block(256);
  hipLaunchKernelGGL((decode_step_fused_kernel<TS, TX, TD>), grid, block, 0, stream, q, lpr_log2);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

template <typename TS, typename TX> int fused_dt(const MambaDecodeStepParams &q, hipStream_t s) {
  if (q.ssm.dt_dtype == MAMBA_F32) return launch_fused<TS, TX, float>(q, s);
  if (q.ssm.dt_dtype != DT<TX>::id) return MAMBA_E_UNSUPPORTED;
  return launch_fused<TS, TX, TX>(q, s);
}
template <typename TS> int fused_x(const MambaDecodeStepParams &q, hipStream_t s) {
  switch (q.ssm.x_dtype) {
    case MAMBA_F32: return fused_dt<TS, float>(q, s);
    case MAMBA_BF16: return fused_dt<TS, bf16_t>(q, s);
    default: return fused_dt<TS, f16_t>(q, s);
  }
}

}  // namespace

extern "C" int ssm_state_update(const MambaStepParams *p, mamba_stream_t stream) {
  if (!p || !p->state || !p->x || !p->dt || !p->A || !p->B || !p->C || !p->out) return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->nheads <= 0 || p->dim <= 0 || p->dstate <= 0 || p->ngroups <= 0) return MAMBA_E_BADARG;
  if (p->nheads % p->ngroups != 0) return MAMBA_E_BADARG;
  // rows of `state`: without indices entry b uses row b; with them, an index outside [0, state_rows) is padding
  if (p->state_rows <= 0 || (!p->state_batch_indices && p->state_rows < p->batch)) return MAMBA_E_BADARG;
  if (!dtype_ok(p->state_dtype) || !dtype_ok(p->x_dtype) || !dtype_ok(p->dt_dtype) || !dtype_ok(p->bc_dtype))
    return MAMBA_E_BADARG;
  // the small per-head operands are fp32 (the host side converts them)
  if (p->A_dtype != MAMBA_F32 || (p->D && p->D_dtype != MAMBA_F32) || (p->dt_bias && p->dt_bias_dtype != MAMBA_F32))
    return MAMBA_E_UNSUPPORTED;
  if (p->batch > 65535 || p->nheads > 65535 || p->dstate > 256) return MAMBA_E_UNSUPPORTED;
  {  // per-(batch, head) extents are addressed with 32-bit element offsets
    auto big = [&](int64_t ps, int64_t ns) {
      const int64_t a = (ps < 0 ? -ps : ps) * p->dim + (ns < 0 ? -ns : ns) * p->dstate;
      return a >= (int64_t(1) << 30);
    };
    if (big(p->state_ps, p->state_ns) || big(p->x_ps, 0) || big(p->dt_ps, 0) || big(p->dt_bias_ps, 0) ||
        big(p->A_ps, p->A_ns) || big(0, p->B_ns) || big(0, p->C_ns) || big(p->D_ps, 0) || big(p->z_ps, 0) ||
        big(p->out_ps, 0))
      return MAMBA_E_UNSUPPORTED;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (p->state_dtype) {
    case MAMBA_F32: return dispatch_x<float>(*p, s);
    case MAMBA_BF16: return dispatch_x<bf16_t>(*p, s);
    default: return dispatch_x<f16_t>(*p, s);
  }
}

extern "C" int64_t mamba2_decode_step_sync_ints(const MambaDecodeStepParams *q) {
  if (!q || q->ssm.batch <= 0 || q->ssm.nheads <= 0 || q->ssm.dim <= 0 || q->ssm.dstate <= 0) return MAMBA_E_BADARG;
  if (q->ssm.ngroups <= 0 || q->ssm.nheads % q->ssm.ngroups != 0) return MAMBA_E_BADARG;
  const int nwg = fused_grid_x(q->ssm, nullptr) * (q->ssm.nheads / q->ssm.ngroups);  // per (batch entry, group)
  return (int64_t)q->ssm.batch * q->ssm.ngroups * ((nwg + SYNC_FAN - 1) / SYNC_FAN + 1);
}

extern "C" int mamba2_decode_step(const MambaDecodeStepParams *q, mamba_stream_t stream) {
  if (!q) return MAMBA_E_BADARG;
  const MambaStepParams *p = &q->ssm;
  if (!p->state || !p->dt || !p->A || !p->out || !q->xBC || !q->conv_state || !q->conv_weight || !q->sync)
    return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->nheads <= 0 || p->dim <= 0 || p->dstate <= 0 || p->ngroups <= 0) return MAMBA_E_BADARG;
  if (p->nheads % p->ngroups != 0) return MAMBA_E_BADARG;
  if (q->conv_dim != p->nheads * p->dim + 2 * p->ngroups * p->dstate) return MAMBA_E_BADARG;
  if (p->state_rows < p->batch || q->conv_state_rows < p->batch) return MAMBA_E_BADARG;
  if (!dtype_ok(p->state_dtype) || !dtype_ok(p->x_dtype) || !dtype_ok(p->dt_dtype) || !dtype_ok(q->conv_weight_dtype))
    return MAMBA_E_BADARG;
  // the form served here; anything else is for the two separate calls
  if (p->state_batch_indices) return MAMBA_E_UNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(q->conv_weight) % 16 != 0) return MAMBA_E_UNSUPPORTED;
  if (q->width < 2 || q->width > CW || q->state_len < q->width - 1 || q->state_len > CW) return MAMBA_E_UNSUPPORTED;
  if (p->A_dtype != MAMBA_F32 || (p->D && p->D_dtype != MAMBA_F32) || (p->dt_bias && p->dt_bias_dtype != MAMBA_F32))
    return MAMBA_E_UNSUPPORTED;
  if (p->dt_ps != 0 || p->A_ps != 0 || p->A_ns != 0 || (p->dt_bias && p->dt_bias_ps != 0) || (p->D && p->D_ps != 0))
    return MAMBA_E_UNSUPPORTED;
  if (p->batch > 65535 || p->nheads > 65535 || p->dstate > 256 || p->dstate % 4 != 0) return MAMBA_E_UNSUPPORTED;
  {
    // lane j of a wave convolves the x channel of the wave's row j, so a wave may hold at most 64 rows:
    // fewer than 16 states (more than 16 rows per pass) are for the two separate calls
    int lpr_log2 = 0;
    (void)fused_grid_x(*p, &lpr_log2);
    if ((64 >> lpr_log2) * UNR > 64) return MAMBA_E_UNSUPPORTED;
  }
  {
    const int es = p->state_dtype == MAMBA_F32 ? 4 : 2;
    const int64_t vb = 4 * es;
    if (p->state_ns != 1 || reinterpret_cast<uintptr_t>(p->state) % vb != 0 || (p->state_bs * es) % vb != 0 ||
        (p->state_hs * es) % vb != 0 || (p->state_ps * es) % vb != 0)
      return MAMBA_E_UNSUPPORTED;
    auto big = [&](int64_t a) { return (a < 0 ? -a : a) >= (int64_t(1) << 30); };
    if (big(p->state_ps * p->dim + p->dstate) || big(p->z_ps * p->dim) || big(p->out_ps * p->dim) ||
        big(q->cs_cs * q->conv_dim + q->cs_ls * q->state_len))
      return MAMBA_E_UNSUPPORTED;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (p->state_dtype) {
    case MAMBA_F32: return fused_x<float>(*q, s);
    case MAMBA_BF16: return fused_x<bf16_t>(*q, s);
    default: return fused_x<f16_t>(*q, s);
  }
}
