// LayerNorm / RMSNorm of (x + residual) with the sum handed on, forward and backward, for gfx950:
// the norm in front of every mixer of the reference's Block (mamba_ssm/modules/block.py:57-66 calls
// mamba_ssm/ops/triton/layer_norm.py:888; Triton launches :291 forward, :589 backward).
//   s = x + residual (fp32);  residual_out = s (in the residual's dtype, fp32 for residual_in_fp32)
//   out = (s - mean) * rstd * w + b,  mean = 0 for RMSNorm, statistics per row
// backward:  dx = d_norm(dy) + dresidual  (the gradient reaching the handed-on sum), written in x's
// dtype and, where the residual stream has another dtype, in that one too.
// Same team / row-walk / partial-sum scheme as the gated group norm; x and the residual stream may
// differ in dtype (bf16 activations next to an fp32 stream).
#include "norm_common.hpp"

namespace {

template <int TEAM> DEVI bool my_part(int nparts, int &part, int &col) {
  constexpr int WGT = TEAM < 256 ? 256 : TEAM;
  part = blockIdx.x * (WGT / TEAM) + threadIdx.x / TEAM;
  col = (threadIdx.x % TEAM) * 8;
  return part < nparts;
}

template <typename T, typename R, int TEAM, int K, bool VEC>
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
  RowBuf<T, VEC, K, TEAM> bx;
  RowBuf<R, VEC, K, TEAM> br;
  if (part < p.rows) {
    bx.fetch(xp + part * p.x_rs, col, n);
    if (rp) br.fetch(rp + part * p.residual_rs, col, n);
  }
  for (int r = part; r < p.rows; r += nparts) {
    float x[K][8];
    bx.get(x);
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

template <typename T, typename R, int TEAM, int K, bool VEC>
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
        const float wdy = in ? w[k][e] * gv : 0.f;
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
    store_row<T, VEC, K, TEAM>(dxp + r * p.dx_rs, col, n, x);
    if (drip) store_row<R, VEC, K, TEAM>(drip + r * p.dresidual_in_rs, col, n, x);
  }
  store_row<float, VEC, K, TEAM>(p.dw_part + (int64_t)part * p.dim, col, n, dw);
  if (p.db_part) store_row<float, VEC, K, TEAM>(p.db_part + (int64_t)part * p.dim, col, n, db);
}

bool vec_ok(const NormResidualParams &p, bool bwd) {
  auto ok = [](const void *q, int64_t rs) { return !q || (aligned16(q) && rs % 8 == 0); };
  bool v = p.dim % 8 == 0 && aligned16(p.weight) && aligned16(p.bias) && ok(p.x, p.x_rs);
  if (!bwd) v = v && ok(p.residual, p.residual_rs) && ok(p.out, p.out_rs) && ok(p.residual_out, p.residual_out_rs);
  else
    v = v && ok(p.dy, p.dy_rs) && ok(p.dresidual, p.dresidual_rs) && ok(p.dx, p.dx_rs) &&
        ok(p.dresidual_in, p.dresidual_in_rs) && aligned16(p.dw_part) && aligned16(p.db_part);
  return v;
}

template <typename T, typename R, int TEAM, int K, bool VEC> int launch(const NormResidualParams &p, bool bwd, hipStream_t st) {
  constexpr int WGT = TEAM < 256 ? 256 : TEAM;
  const int nparts = bwd ? p.nparts : min(p.rows, 16384);
  const int wgs = (nparts + WGT / TEAM - 1) / (WGT / TEAM);
  if (bwd) norm_res_bwd_kernel<T, R, TEAM, K, VEC><<<dim3(wgs), dim3(WGT), 0, st>>>(p);
  else norm_res_fwd_kernel<T, R, TEAM, K, VEC><<<dim3(wgs), dim3(WGT), 0, st>>>(p, nparts);
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
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

}  // namespace

extern "C" int norm_residual_fwd(const NormResidualParams *p, mamba_stream_t stream) {
  return dispatch(p, false, static_cast<hipStream_t>(stream));
}
extern "C" int norm_residual_bwd(const NormResidualParams *p, mamba_stream_t stream) {
  return dispatch(p, true, static_cast<hipStream_t>(stream));
}
