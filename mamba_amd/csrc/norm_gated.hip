// Gated LayerNorm / RMSNorm over groups of channels, forward and backward, for gfx950: the epilogue
// of the Mamba-2 block between the chunked scan and the output projection (reference
// mamba_ssm/ops/triton/layernorm_gated.py:108 forward, :271 backward; called from
// mamba_ssm/modules/mamba2.py:242 and mamba_ssm/ops/triton/ssd_combined.py:872-874).
//   x' = norm_before_gate ? x : x * silu(z)
//   y  = (x' - mean) * rstd * w + b          mean = 0 for RMSNorm, statistics per (row, group)
//   out = norm_before_gate ? y * silu(z) : y
// A team of 8 to 1024 threads owns one (row, group) at a time and keeps it in registers, 8
// consecutive channels per thread and step, so x, z and dy are read once and out / dx / dz written
// once.  A team walks rows r = part, part + nparts, ... of one group; the backward pass keeps the
// team's sums for dweight / dbias in registers over that walk, stores one partial row per part, and
// a second kernel adds the parts.
#include "norm_common.hpp"

namespace {

DEVI float silu_g(float z, float &sig) {
  sig = sigmoid_f(z);
  return z * sig;
}

// Neighbouring teams take neighbouring groups of the same rows, so that a wave of small teams still
// reads one contiguous stretch of a row.
struct Item {
  int group, part, col;  // col: first channel of this thread's step 0 inside the group
  bool live;
};
template <int TEAM> DEVI Item my_item(const NormGatedParams &p, int nparts) {
  constexpr int WGT = TEAM < 256 ? 256 : TEAM;
  const int ngroups = p.dim / p.group_size;
  const int team = blockIdx.x * (WGT / TEAM) + threadIdx.x / TEAM;
  Item it;
  it.group = team % ngroups;
  it.part = team / ngroups;
  it.col = (threadIdx.x % TEAM) * 8;
  it.live = it.part < nparts;
  return it;
}

template <typename T, int TEAM, int K, bool VEC>
__global__ __launch_bounds__(TEAM < 256 ? 256 : TEAM) void norm_fwd_kernel(const NormGatedParams p, int nparts) {
  __shared__ float lds[TEAM >= 128 ? 2 * (TEAM / 64) * 2 : 1];
  TeamSum<TEAM> ts(lds);
  const Item it = my_item<TEAM>(p, nparts);
  if (!it.live) return;  // whole teams only; a team of more than one wave is a whole workgroup
  const int gs = p.group_size, ngroups = p.dim / gs;
  const int64_t g0 = (int64_t)it.group * gs;
  float w[K][8], b[K][8];
  load_row<float, VEC, K, TEAM>(p.weight + g0, it.col, gs, w);
  if (p.bias) load_row<float, VEC, K, TEAM>(p.bias + g0, it.col, gs, b);
  const T *xp = static_cast<const T *>(p.x) + g0;
  const T *zp = p.z ? static_cast<const T *>(p.z) + g0 : nullptr;
  T *op = static_cast<T *>(p.out) + g0;
  const float inv_n = 1.f / (float)gs;
  RowBuf<T, VEC, K, TEAM> bx, bz;
  if (it.part < p.rows) {
    bx.fetch(xp + it.part * p.x_rs, it.col, gs);
    if (zp) bz.fetch(zp + it.part * p.z_rs, it.col, gs);
  }
  for (int r = it.part; r < p.rows; r += nparts) {
    float x[K][8], sz[K][8];
    bx.get(x);
    if (zp) bz.get(sz);
    if (r + nparts < p.rows) {
      bx.fetch(xp + (r + nparts) * p.x_rs, it.col, gs);
      if (zp) bz.fetch(zp + (r + nparts) * p.z_rs, it.col, gs);
    }
    if (zp) {
#pragma unroll
      for (int k = 0; k < K; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float sig;
          sz[k][e] = silu_g(sz[k][e], sig);
          if (!p.norm_before_gate) x[k][e] *= sz[k][e];
        }
    }
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
        const bool in = it.col + k * TEAM * 8 + e < gs;
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
        if (zp && p.norm_before_gate) y *= sz[k][e];
        x[k][e] = y;
      }
    store_row<T, VEC, K, TEAM>(op + r * p.out_rs, it.col, gs, x);
    if (threadIdx.x % TEAM == 0) {
      if (p.mean) p.mean[(int64_t)r * ngroups + it.group] = mean;
      p.rstd[(int64_t)r * ngroups + it.group] = rstd;
    }
  }
}

template <typename T, int TEAM, int K, bool VEC>
__global__ __launch_bounds__(TEAM < 256 ? 256 : TEAM) void norm_bwd_kernel(const NormGatedParams p) {
  __shared__ float lds[TEAM >= 128 ? 2 * (TEAM / 64) * 2 : 1];
  TeamSum<TEAM> ts(lds);
  const int nparts = p.nparts;
  const Item it = my_item<TEAM>(p, nparts);
  if (!it.live) return;
  const int gs = p.group_size, ngroups = p.dim / gs;
  const int64_t g0 = (int64_t)it.group * gs;
  float w[K][8], b[K][8], dw[K][8], db[K][8];
  load_row<float, VEC, K, TEAM>(p.weight + g0, it.col, gs, w);
  if (p.bias) load_row<float, VEC, K, TEAM>(p.bias + g0, it.col, gs, b);
#pragma unroll
  for (int k = 0; k < K; ++k)
#pragma unroll
    for (int e = 0; e < 8; ++e) dw[k][e] = db[k][e] = 0.f;
  const T *xp = static_cast<const T *>(p.x) + g0;
  const T *zp = p.z ? static_cast<const T *>(p.z) + g0 : nullptr;
  const T *gp = static_cast<const T *>(p.dy) + g0;
  T *dxp = static_cast<T *>(p.dx) + g0;
  T *dzp = p.z ? static_cast<T *>(p.dz) + g0 : nullptr;
  const float inv_n = 1.f / (float)gs;
  const bool gate_after = zp && p.norm_before_gate, gate_before = zp && !p.norm_before_gate;
  RowBuf<T, VEC, K, TEAM> bx, bg, bz;
  if (it.part < p.rows) {
    bx.fetch(xp + it.part * p.x_rs, it.col, gs);
    bg.fetch(gp + it.part * p.dy_rs, it.col, gs);
    if (zp) bz.fetch(zp + it.part * p.z_rs, it.col, gs);
  }
  for (int r = it.part; r < p.rows; r += nparts) {
    float x[K][8], z[K][8], g[K][8];
    bx.get(x);
    bg.get(g);
    if (zp) bz.get(z);
    const RowBuf<T, VEC, K, TEAM> xkeep = bx;  // x itself is needed again when the gate comes first
    if (r + nparts < p.rows) {
      bx.fetch(xp + (r + nparts) * p.x_rs, it.col, gs);
      bg.fetch(gp + (r + nparts) * p.dy_rs, it.col, gs);
      if (zp) bz.fetch(zp + (r + nparts) * p.z_rs, it.col, gs);
    }
    const float mean = p.is_rms ? 0.f : p.mean[(int64_t)r * ngroups + it.group];
    const float rstd = p.rstd[(int64_t)r * ngroups + it.group];
    float c1 = 0.f, c2 = 0.f;
    // after this loop: x = xhat (0 outside the group), g = w * dy', z = dz (gate after the norm) or
    // kept as z (gate before it, finished below)
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const bool in = it.col + k * TEAM * 8 + e < gs;
        float xv = x[k][e], gv = g[k][e];
        float sig = 0.f, sz = 1.f;
        if (zp) sz = silu_g(z[k][e], sig);
        if (gate_before) xv *= sz;
        const float xhat = in ? (xv - mean) * rstd : 0.f;
        if (gate_after) {
          float y = xhat * w[k][e];
          if (p.bias) y += b[k][e];
          z[k][e] = gv * y * sig * (1.f + z[k][e] * (1.f - sig));
          gv *= sz;
        }
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
    if (gate_before) {
      float xr[K][8];  // dz = dx' * x * dsilu(z), dx = dx' * silu(z)
      xkeep.get(xr);
#pragma unroll
      for (int k = 0; k < K; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float d = (g[k][e] - (x[k][e] * c1 + c2)) * rstd;
          float sig;
          const float sz = silu_g(z[k][e], sig);
          z[k][e] = d * xr[k][e] * sig * (1.f + z[k][e] * (1.f - sig));
          x[k][e] = d * sz;
        }
    } else {
#pragma unroll
      for (int k = 0; k < K; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) x[k][e] = (g[k][e] - (x[k][e] * c1 + c2)) * rstd;
    }
    store_row<T, VEC, K, TEAM>(dxp + r * p.dx_rs, it.col, gs, x);
    if (zp) store_row<T, VEC, K, TEAM>(dzp + r * p.dz_rs, it.col, gs, z);
  }
  store_row<float, VEC, K, TEAM>(p.dw_part + (int64_t)it.part * p.dim + g0, it.col, gs, dw);
  if (p.db_part) store_row<float, VEC, K, TEAM>(p.db_part + (int64_t)it.part * p.dim + g0, it.col, gs, db);
}

template <typename T> bool vec_ok(const NormGatedParams &p, bool bwd) {
  constexpr int per16 = 16 / (int)sizeof(T);  // elements per 16 bytes: loads of 8 need 8-element alignment of fp32 too
  (void)per16;
  bool ok = p.group_size % 8 == 0 && p.x_rs % 8 == 0 && p.out_rs % 8 == 0 && aligned16(p.x) && aligned16(p.weight) &&
            (!p.bias || aligned16(p.bias));
  if (!bwd) ok = ok && aligned16(p.out);
  if (p.z) ok = ok && p.z_rs % 8 == 0 && aligned16(p.z);
  if (bwd) {
    ok = ok && p.dy_rs % 8 == 0 && p.dx_rs % 8 == 0 && aligned16(p.dy) && aligned16(p.dx) && aligned16(p.dw_part) &&
         (!p.db_part || aligned16(p.db_part)) && p.dim % 8 == 0;
    if (p.z) ok = ok && p.dz_rs % 8 == 0 && aligned16(p.dz);
  }
  return ok;
}

template <typename T, int TEAM, int K, bool VEC> int launch(const NormGatedParams &p, bool bwd, hipStream_t st) {
  constexpr int WGT = TEAM < 256 ? 256 : TEAM;
  const int ngroups = p.dim / p.group_size;
  const int nparts = bwd ? p.nparts : min(p.rows, 16384);
  const int64_t teams = (int64_t)ngroups * nparts;
  const int64_t wgs = (teams + WGT / TEAM - 1) / (WGT / TEAM);
  if (wgs > 0x7fffffff) return MAMBA_E_UNSUPPORTED;
  if (bwd) norm_bwd_kernel<T, TEAM, K, VEC><<<dim3((unsigned)wgs), dim3(WGT), 0, st>>>(p);
  else norm_fwd_kernel<T, TEAM, K, VEC><<<dim3((unsigned)wgs), dim3(WGT), 0, st>>>(p, nparts);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

// The smallest team that holds the group in at most two steps of 8 channels per thread (more steps
// cost registers, hence waves in flight); only groups beyond 16384 channels take 3 or 4 steps.
template <typename T, int TEAM, bool VEC> int pick_k(const NormGatedParams &p, bool bwd, hipStream_t st) {
  const int k = (p.group_size + TEAM * 8 - 1) / (TEAM * 8);
  if (k == 1) return launch<T, TEAM, 1, VEC>(p, bwd, st);
  if (k == 2) return launch<T, TEAM, 2, VEC>(p, bwd, st);
  if constexpr (TEAM == 1024) {
    if (k == 3) return launch<T, TEAM, 3, VEC>(p, bwd, st);
    if (k == 4) return launch<T, TEAM, 4, VEC>(p, bwd, st);
  }
  return MAMBA_E_UNSUPPORTED;
}

template <typename T, bool VEC> int pick_team(const NormGatedParams &p, bool bwd, hipStream_t st) {
  if (p.group_size <= 128) return pick_k<T, 8, VEC>(p, bwd, st);
  if (p.group_size <= 256) return pick_k<T, 16, VEC>(p, bwd, st);
  if (p.group_size <= 512) return pick_k<T, 32, VEC>(p, bwd, st);
  if (p.group_size <= 1024) return pick_k<T, 64, VEC>(p, bwd, st);
  if (p.group_size <= 4096) return pick_k<T, 256, VEC>(p, bwd, st);
  if (p.group_size <= 8192) return pick_k<T, 512, VEC>(p, bwd, st);
  return pick_k<T, 1024, VEC>(p, bwd, st);
}

template <typename T> int run(const NormGatedParams &p, bool bwd, hipStream_t st) {
  return vec_ok<T>(p, bwd) ? pick_team<T, true>(p, bwd, st) : pick_team<T, false>(p, bwd, st);
}

int check(const NormGatedParams *p, bool bwd) {
  if (!p) return MAMBA_E_BADARG;
  if (p->rows < 0 || p->dim <= 0 || p->group_size <= 0 || p->dim % p->group_size != 0) return MAMBA_E_BADARG;
  if (p->group_size > 32768) return MAMBA_E_UNSUPPORTED;
  if (!p->x || !p->weight || !p->rstd) return MAMBA_E_BADARG;
  if (!p->is_rms && !p->mean) return MAMBA_E_BADARG;
  if (!bwd && !p->out) return MAMBA_E_BADARG;
  if (bwd) {
    if (!p->dy || !p->dx || !p->dweight || !p->dw_part) return MAMBA_E_BADARG;
    if (p->z && !p->dz) return MAMBA_E_BADARG;
    if (p->bias && (!p->dbias || !p->db_part)) return MAMBA_E_BADARG;
    if (p->nparts < 1 || p->nparts > 65536) return MAMBA_E_BADARG;
  }
  return MAMBA_OK;
}

int dispatch(const NormGatedParams *p, bool bwd, hipStream_t st) {
  int rc = check(p, bwd);
  if (rc != MAMBA_OK) return rc;
  if (p->rows == 0) {
    if (!bwd) return MAMBA_OK;
  }
  if (p->rows > 0 || bwd) {
    switch (p->dtype) {
      case MAMBA_F32: rc = run<float>(*p, bwd, st); break;
      case MAMBA_BF16: rc = run<bf16_t>(*p, bwd, st); break;
      case MAMBA_F16: rc = run<f16_t>(*p, bwd, st); break;
      default: return MAMBA_E_BADARG;
    }
  }
  if (rc != MAMBA_OK || !bwd) return rc;
  norm_reduce_kernel<<<dim3((p->dim + 63) / 64), dim3(1024), 0, st>>>(p->dw_part, p->bias ? p->db_part : nullptr,
                                                                       p->dweight, p->bias ? p->dbias : nullptr,
                                                                       p->nparts, p->dim);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

}  // namespace

extern "C" int norm_gated_fwd(const NormGatedParams *p, mamba_stream_t stream) {
  return dispatch(p, false, static_cast<hipStream_t>(stream));
}
extern "C" int norm_gated_bwd(const NormGatedParams *p, mamba_stream_t stream) {
  return dispatch(p, true, static_cast<hipStream_t>(stream));
}
