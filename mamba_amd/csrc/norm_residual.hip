// LayerNorm / RMSNorm of (x + residual) with the sum handed on, forward and backward, for gfx950:
// the norm in front of every mixer of the reference's Block (mamba_ssm/modules/block.py:57-66 calls
// mamba_ssm/ops/triton/layer_norm.py:888; Triton launches :291 forward, :589 backward).
//   s = x + residual (fp32);  residual_out = s (in the residual's dtype, fp32 for residual_in_fp32)
//   out = (s - mean) * rstd * w + b,  mean = 0 for RMSNorm, statistics per row
// backward:  dx = d_norm(dy) + dresidual  (the gradient reaching the handed-on sum), written in x's
// dtype and, where the residual stream has another dtype, in that one too.
// Same team / row-walk / partial-sum scheme as the gated group norm; x and the residual stream may
// differ in dtype (bf16 activations next to an fp32 stream).
// The rest of the reference's operator (layer_norm.py:130-237, :393-518) is compiled as a second form of both
// kernels (EXTRA), so that the form every Mamba block uses carries none of it:
//   s = drop(x * rowscale) + drop1(x1) + residual;  out1 = (s - mean) * rstd * w1 + b1
//   d = gradient of s (from dy and dy1, + dresidual) -> dresidual_in;  dx = drop'(d) * rowscale;  dx1 = drop1'(d)
// A dropout draw is a hash of (seed of the stream, row, channel), so the backward pass repeats it.
#include "norm_common.hpp"

namespace {

// keep / drop of element (row, channel) of a stream: a 32-bit mix of the three, uniform in [0, 1), kept when above p
DEVI bool keep_draw(uint64_t seed, int row, int ch, float p) {
  uint32_t h = (uint32_t)seed ^ ((uint32_t)(seed >> 32) * 0x9E3779B9u);
  h ^= (uint32_t)row * 0x85EBCA6Bu;
  h = (h ^ (h >> 16)) * 0x7FEB352Du;
  h ^= (uint32_t)ch * 0xC2B2AE35u;
  h = (h ^ (h >> 15)) * 0x846CA68Bu;
  h ^= h >> 16;
  return (float)(h >> 8) * (1.f / 16777216.f) > p;
}
// drops / scales the 8-channel steps of a row in place; writes the draws as bytes where asked
template <int TEAM, int K>
DEVI void drop_row(float (&x)[K][8], uint64_t seed, int row, int col, int n, float p, float scale, uint8_t *mask) {
#pragma unroll
  for (int k = 0; k < K; ++k)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int ch = col + k * TEAM * 8 + e;
      const bool keep = keep_draw(seed, row, ch, p);
      x[k][e] = keep ? x[k][e] * scale : 0.f;
      if (mask && ch < n) mask[(int64_t)row * n + ch] = keep ? 1 : 0;
    }
}

template <int TEAM> DEVI bool my_part(int nparts, int &part, int &col) {
  constexpr int WGT = TEAM < 256 ? 256 : TEAM;
  part = blockIdx.x * (WGT / TEAM) + threadIdx.x / TEAM;
  col = (threadIdx.x % TEAM) * 8;
  return part < nparts;
}

template <typename T, typename R, int TEAM, int K, bool VEC, bool EXTRA>
__global__ __launch_bounds__(TEAM < 256 ? 256 : TEAM) void norm_res_fwd_kernel(const NormResidualParams p, int nparts) {
  __shared__ float lds[TEAM >= 128 ? 2 * (TEAM / 64) * 2 : 1];
  TeamSum<TEAM> ts(lds);
  int part, col;
  if (!my_part<TEAM>(nparts, part, col)) return;
  const int n = p.dim;
  float w[K][8], b[K][8];
  load_row<float, VEC, K, TEAM>(p.weight, col, n, w);
  if (p.bias) load_row<float, VEC, K, TEAM>(p.bias, col, n, b);
  const T *xp = static_cast<const T *>(p.x);
  const R *rp = static_cast<const R *>(p.residual);
  T *op = static_cast<T *>(p.out);
  R *rop = static_cast<R *>(p.residual_out);
  const float inv_n = 1.f / (float)n;
  const T *x1p = EXTRA ? static_cast<const T *>(p.x1) : nullptr;
  const bool drop = EXTRA && p.dropout_p > 0.f;
  const float keep_scale = drop ? 1.f / (1.f - p.dropout_p) : 1.f;
  const uint64_t seed0 = drop ? (uint64_t)p.seeds[0] : 0, seed1 = drop ? (uint64_t)p.seeds[1] : 0;
  RowBuf<T, VEC, K, TEAM> bx;
  RowBuf<R, VEC, K, TEAM> br;
  if (part < p.rows) {
    bx.fetch(xp + part * p.x_rs, col, n);
    if (rp) br.fetch(rp + part * p.residual_rs, col, n);
  }
  for (int r = part; r < p.rows; r += nparts) {
    float x[K][8];
    bx.get(x);
    if constexpr (EXTRA) {
      if (p.rowscale) {
        const float rsc = p.rowscale[r];
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int e = 0; e < 8; ++e) x[k][e] *= rsc;
      }
      if (drop) drop_row<TEAM, K>(x, seed0, r, col, n, p.dropout_p, keep_scale, p.mask);
      if (x1p) {
        float x1[K][8];
        load_row<T, VEC, K, TEAM>(x1p + r * p.x1_rs, col, n, x1);
        if (drop) drop_row<TEAM, K>(x1, seed1, r, col, n, p.dropout_p, keep_scale, p.mask1);
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int e = 0; e < 8; ++e) x[k][e] += x1[k][e];
      }
    }
    if (rp) {
      float res[K][8];
      br.get(res);
#pragma unroll
      for (int k = 0; k < K; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) x[k][e] += res[k][e];
    }
    if (r + nparts < p.rows) {
      bx.fetch(xp + (r + nparts) * p.x_rs, col, n);
      if (rp) br.fetch(rp + (r + nparts) * p.residual_rs, col, n);
    }
    if (rop) store_row<R, VEC, K, TEAM>(rop + r * p.residual_out_rs, col, n, x);
    float mean = 0.f, dummy = 0.f;
    if (!p.is_rms) {
#pragma unroll
      for (int k = 0; k < K; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) mean += x[k][e];
      ts.sum2(mean, dummy);
      mean *= inv_n;
    }
    float var = 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const bool in = col + k * TEAM * 8 + e < n;
        const float d = in ? x[k][e] - mean : 0.f;
        x[k][e] = d;
        var = __builtin_fmaf(d, d, var);
      }
    dummy = 0.f;
    ts.sum2(var, dummy);
    const float rstd = 1.f / sqrtf(var * inv_n + p.eps);
    if constexpr (EXTRA) {
      if (p.weight1) {  // the second set of norm parameters on the same normalised row
        float w1[K][8], b1[K][8], y1[K][8];
        load_row<float, VEC, K, TEAM>(p.weight1, col, n, w1);
        if (p.bias1) load_row<float, VEC, K, TEAM>(p.bias1, col, n, b1);
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float y = x[k][e] * rstd * w1[k][e];
            if (p.bias1) y += b1[k][e];
            y1[k][e] = y;
          }
        store_row<T, VEC, K, TEAM>(static_cast<T *>(p.out1) + r * p.out1_rs, col, n, y1);
      }
    }
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float y = x[k][e] * rstd * w[k][e];
        if (p.bias) y += b[k][e];
        x[k][e] = y;
      }
    store_row<T, VEC, K, TEAM>(op + r * p.out_rs, col, n, x);
    if (threadIdx.x % TEAM == 0) {
      if (p.mean) p.mean[r] = mean;
      p.rstd[r] = rstd;
    }
  }
}

template <typename T, typename R, int TEAM, int K, bool VEC, bool EXTRA>
__global__ __launch_bounds__(TEAM < 256 ? 256 : TEAM) void norm_res_bwd_kernel(const NormResidualParams p) {
  __shared__ float lds[TEAM >= 128 ? 2 * (TEAM / 64) * 2 : 1];
  TeamSum<TEAM> ts(lds);
  const int nparts = p.nparts;
  int part, col;
  if (!my_part<TEAM>(nparts, part, col)) return;
  const int n = p.dim;
  float w[K][8], dw[K][8], db[K][8];
  load_row<float, VEC, K, TEAM>(p.weight, col, n, w);
#pragma unroll
  for (int k = 0; k < K; ++k)
#pragma unroll
    for (int e = 0; e < 8; ++e) dw[k][e] = db[k][e] = 0.f;
  const R *xp = static_cast<const R *>(p.x);
  const T *gp = static_cast<const T *>(p.dy);
  const R *drp = static_cast<const R *>(p.dresidual);
  T *dxp = static_cast<T *>(p.dx);
  R *drip = static_cast<R *>(p.dresidual_in);
  const float inv_n = 1.f / (float)n;
  // the second set of norm parameters: its weight, the gradients arriving at its output, its own partial sums
  const bool two = EXTRA && p.weight1 != nullptr;
  float w1[EXTRA ? K : 1][8], dw1[EXTRA ? K : 1][8], db1[EXTRA ? K : 1][8];
  if constexpr (EXTRA) {
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) w1[k][e] = dw1[k][e] = db1[k][e] = 0.f;
    if (two) load_row<float, VEC, K, TEAM>(p.weight1, col, n, w1);
  }
  const bool drop = EXTRA && p.dropout_p > 0.f;
  const float keep_scale = drop ? 1.f / (1.f - p.dropout_p) : 1.f;
  const uint64_t seed0 = drop ? (uint64_t)p.seeds[0] : 0, seed1 = drop ? (uint64_t)p.seeds[1] : 0;
  RowBuf<R, VEC, K, TEAM> bx, bd;
  RowBuf<T, VEC, K, TEAM> bg;
  if (part < p.rows) {
    bx.fetch(xp + part * p.x_rs, col, n);
    bg.fetch(gp + part * p.dy_rs, col, n);
    if (drp) bd.fetch(drp + part * p.dresidual_rs, col, n);
  }
  for (int r = part; r < p.rows; r += nparts) {
    float x[K][8], g[K][8], dres[K][8];
    bx.get(x);
    bg.get(g);
    if (drp) bd.get(dres);
    if (r + nparts < p.rows) {
      bx.fetch(xp + (r + nparts) * p.x_rs, col, n);
      bg.fetch(gp + (r + nparts) * p.dy_rs, col, n);
      if (drp) bd.fetch(drp + (r + nparts) * p.dresidual_rs, col, n);
    }
    const float mean = p.is_rms ? 0.f : p.mean[r];
    const float rstd = p.rstd[r];
    float g1[EXTRA ? K : 1][8];
    if constexpr (EXTRA) {
      if (two) load_row<T, VEC, K, TEAM>(static_cast<const T *>(p.dy1) + r * p.dy1_rs, col, n, g1);
    }
    float c1 = 0.f, c2 = 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const bool in = col + k * TEAM * 8 + e < n;
        const float xhat = in ? (x[k][e] - mean) * rstd : 0.f;
        const float gv = g[k][e];
        dw[k][e] = __builtin_fmaf(gv, xhat, dw[k][e]);
        db[k][e] += gv;
        float wdy = in ? w[k][e] * gv : 0.f;
        if constexpr (EXTRA) {
          if (two) {
            const float gv1 = g1[k][e];
            dw1[k][e] = __builtin_fmaf(gv1, xhat, dw1[k][e]);
            db1[k][e] += gv1;
            wdy = in ? __builtin_fmaf(w1[k][e], gv1, wdy) : 0.f;
          }
        }
        c1 = __builtin_fmaf(xhat, wdy, c1);
        c2 += wdy;
        x[k][e] = xhat;
        g[k][e] = wdy;
      }
    ts.sum2(c1, c2);
    c1 *= inv_n;
    c2 = p.is_rms ? 0.f : c2 * inv_n;
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float d = (g[k][e] - (x[k][e] * c1 + c2)) * rstd;
        if (drp) d += dres[k][e];
        x[k][e] = d;
      }
    if (drip) store_row<R, VEC, K, TEAM>(drip + r * p.dresidual_in_rs, col, n, x);  // the gradient of the sum
    if constexpr (EXTRA) {
      if (p.x1) {  // the second input saw only its own dropout
        float d1[K][8];
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int e = 0; e < 8; ++e) d1[k][e] = x[k][e];
        if (drop) drop_row<TEAM, K>(d1, seed1, r, col, n, p.dropout_p, keep_scale, nullptr);
        store_row<T, VEC, K, TEAM>(static_cast<T *>(p.dx1) + r * p.dx1_rs, col, n, d1);
      }
      if (drop) drop_row<TEAM, K>(x, seed0, r, col, n, p.dropout_p, keep_scale, nullptr);
      if (p.rowscale) {
        const float rsc = p.rowscale[r];
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int e = 0; e < 8; ++e) x[k][e] *= rsc;
      }
    }
    store_row<T, VEC, K, TEAM>(dxp + r * p.dx_rs, col, n, x);
  }
  store_row<float, VEC, K, TEAM>(p.dw_part + (int64_t)part * p.dim, col, n, dw);
  if (p.db_part) store_row<float, VEC, K, TEAM>(p.db_part + (int64_t)part * p.dim, col, n, db);
  if constexpr (EXTRA) {
    if (two) {
      store_row<float, VEC, K, TEAM>(p.dw1_part + (int64_t)part * p.dim, col, n, dw1);
      if (p.db1_part) store_row<float, VEC, K, TEAM>(p.db1_part + (int64_t)part * p.dim, col, n, db1);
    }
  }
}

bool vec_ok(const NormResidualParams &p, bool bwd) {
  auto ok = [](const void *q, int64_t rs) { return !q || (aligned16(q) && rs % 8 == 0); };
  bool v = p.dim % 8 == 0 && aligned16(p.weight) && aligned16(p.bias) && ok(p.x, p.x_rs);
  if (!bwd) v = v && ok(p.residual, p.residual_rs) && ok(p.out, p.out_rs) && ok(p.residual_out, p.residual_out_rs);
  else
    v = v && ok(p.dy, p.dy_rs) && ok(p.dresidual, p.dresidual_rs) && ok(p.dx, p.dx_rs) &&
        ok(p.dresidual_in, p.dresidual_in_rs) && aligned16(p.dw_part) && aligned16(p.db_part);
  v = v && aligned16(p.weight1) && aligned16(p.bias1) && ok(p.x1, p.x1_rs) && ok(p.out1, p.out1_rs) &&
      ok(p.dy1, p.dy1_rs) && ok(p.dx1, p.dx1_rs) && aligned16(p.dw1_part) && aligned16(p.db1_part);
  return v;
}

template <typename T, typename R, int TEAM, int K, bool VEC> int launch(const NormResidualParams &p, bool bwd, hipStream_t st) {
  constexpr int WGT = TEAM < 256 ? 256 : TEAM;
  const int nparts = bwd ? p.nparts : min(p.rows, 16384);
  const int wgs = (nparts + WGT / TEAM - 1) / (WGT / TEAM);
  const bool extra = p.x1 || p.rowscale || p.weight1 || p.dropout_p > 0.f;
  if (extra) {
    if (bwd) norm_res_bwd_kernel<T, R, TEAM, K, VEC, true><<<dim3(wgs), dim3(WGT), 0, st>>>(p);
    else norm_res_fwd_kernel<T, R, TEAM, K, VEC, true><<<dim3(wgs), dim3(WGT), 0, st>>>(p, nparts);
  } else {
    if (bwd) norm_res_bwd_kernel<T, R, TEAM, K, VEC, false><<<dim3(wgs), dim3(WGT), 0, st>>>(p);
    else norm_res_fwd_kernel<T, R, TEAM, K, VEC, false><<<dim3(wgs), dim3(WGT), 0, st>>>(p, nparts);
  }
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

template <typename T, typename R, int TEAM, bool VEC> int pick_k(const NormResidualParams &p, bool bwd, hipStream_t st) {
  const int k = (p.dim + TEAM * 8 - 1) / (TEAM * 8);
  if (k == 1) return launch<T, R, TEAM, 1, VEC>(p, bwd, st);
  if (k == 2) return launch<T, R, TEAM, 2, VEC>(p, bwd, st);
  if constexpr (TEAM == 1024) {
    if (k == 3) return launch<T, R, TEAM, 3, VEC>(p, bwd, st);
    if (k == 4) return launch<T, R, TEAM, 4, VEC>(p, bwd, st);
  }
  return MAMBA_E_UNSUPPORTED;
}

template <typename T, typename R, bool VEC> int pick_team(const NormResidualParams &p, bool bwd, hipStream_t st) {
  if (p.dim <= 1024) return pick_k<T, R, 64, VEC>(p, bwd, st);
  if (p.dim <= 4096) return pick_k<T, R, 256, VEC>(p, bwd, st);
  if (p.dim <= 8192) return pick_k<T, R, 512, VEC>(p, bwd, st);
  return pick_k<T, R, 1024, VEC>(p, bwd, st);
}

template <typename T> int run(const NormResidualParams &p, bool bwd, hipStream_t st) {
  const bool vec = vec_ok(p, bwd);
  if (p.res_dtype == p.dtype) return vec ? pick_team<T, T, true>(p, bwd, st) : pick_team<T, T, false>(p, bwd, st);
  if (p.res_dtype == MAMBA_F32) return vec ? pick_team<T, float, true>(p, bwd, st) : pick_team<T, float, false>(p, bwd, st);
  return MAMBA_E_UNSUPPORTED;  // the stream is either in the activations' dtype or in fp32
}

int dispatch(const NormResidualParams *p, bool bwd, hipStream_t st) {
  if (!p || !p->x || !p->weight || !p->rstd) return MAMBA_E_BADARG;
  if (p->rows <= 0 || p->dim <= 0) return MAMBA_E_BADARG;
  if (p->dim > 32768) return MAMBA_E_UNSUPPORTED;
  if (!p->is_rms && !p->mean) return MAMBA_E_BADARG;
  if (!bwd && !p->out) return MAMBA_E_BADARG;
  if (bwd) {
    if (!p->dy || !p->dx || !p->dweight || !p->dw_part) return MAMBA_E_BADARG;
    if (p->bias && (!p->dbias || !p->db_part)) return MAMBA_E_BADARG;
    if (p->nparts < 1 || p->nparts > 65536) return MAMBA_E_BADARG;
  }
  // the optional parts
  if (p->dropout_p < 0.f || p->dropout_p >= 1.f || (p->dropout_p > 0.f && !p->seeds)) return MAMBA_E_BADARG;
  if (p->x1 && p->rowscale) return MAMBA_E_BADARG;  // as in the reference: no rowscale with a second input
  if (p->bias1 && !p->weight1) return MAMBA_E_BADARG;
  if (!bwd && p->weight1 && !p->out1) return MAMBA_E_BADARG;
  if (bwd) {
    if (p->x1 && !p->dx1) return MAMBA_E_BADARG;
    if (p->weight1 && (!p->dy1 || !p->dweight1 || !p->dw1_part)) return MAMBA_E_BADARG;
    if (p->bias1 && (!p->dbias1 || !p->db1_part)) return MAMBA_E_BADARG;
    // dx is no longer the gradient of the sum then: the caller needs dresidual_in for that
  }
  int rc;
  switch (p->dtype) {
    case MAMBA_F32: rc = run<float>(*p, bwd, st); break;
    case MAMBA_BF16: rc = run<bf16_t>(*p, bwd, st); break;
    case MAMBA_F16: rc = run<f16_t>(*p, bwd, st); break;
    default: return MAMBA_E_BADARG;
  }
  if (rc != MAMBA_OK || !bwd) return rc;
  norm_reduce_kernel<<<dim3((p->dim + 63) / 64), dim3(1024), 0, st>>>(p->dw_part, p->bias ? p->db_part : nullptr,
                                                                       p->dweight, p->bias ? p->dbias : nullptr,
                                                                       p->nparts, p->dim);
  if (p->weight1)
    norm_reduce_kernel<<<dim3((p->dim + 63) / 64), dim3(1024), 0, st>>>(p->dw1_part, p->bias1 ? p->db1_part : nullptr,
                                                                         p->dweight1, p->bias1 ? p->dbias1 : nullptr,
                                                                         p->nparts, p->dim);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

}  // namespace

extern "C" int norm_residual_fwd(const NormResidualParams *p, mamba_stream_t stream) {
  return dispatch(p, false, static_cast<hipStream_t>(stream));
}
extern "C" int norm_residual_bwd(const NormResidualParams *p, mamba_stream_t stream) {
  return dispatch(p, true, static_cast<hipStream_t>(stream));
}
