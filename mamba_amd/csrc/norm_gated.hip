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
  // the row's statistics are requested with the row, and before it: a load issued after the next row's would make
  // its first use wait for that whole row as well
  float mean_n = 0.f, rstd_n = 0.f;
  if (it.part < p.rows) {
    if (!p.is_rms) mean_n = p.mean[(int64_t)it.part * ngroups + it.group];
    rstd_n = p.rstd[(int64_t)it.part * ngroups + it.group];
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
    const float mean = mean_n, rstd = rstd_n;
    float c1 = 0.f, c2 = 0.f;
    if (r + nparts < p.rows) {
      if (!p.is_rms) mean_n = p.mean[(int64_t)(r + nparts) * ngroups + it.group];
      rstd_n = p.rstd[(int64_t)(r + nparts) * ngroups + it.group];
      bx.fetch(xp + (r + nparts) * p.x_rs, it.col, gs);
      bg.fetch(gp + (r + nparts) * p.dy_rs, it.col, gs);
      if (zp) bz.fetch(zp + (r + nparts) * p.z_rs, it.col, gs);
    }
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

// The forward pass in the same form as norm_bwd_wide_kernel (below): a part of the rows per workgroup, the next
// row requested before the current one is used, no branch around a row's loads or stores.
template <typename T, int TEAM, bool HAS_Z>
__global__ __launch_bounds__(TEAM, 8) void norm_fwd_wide_kernel(const NormGatedParams p, int nparts) {
  __shared__ float lds[2 * (TEAM / 64) * 2];
  TeamSum<TEAM> ts(lds);
  const int gs = p.group_size, ngroups = p.dim / gs, rows = p.rows;
  const int group = blockIdx.x % ngroups, part = blockIdx.x / ngroups;
  const int col = threadIdx.x * 8;
  if (__builtin_amdgcn_readfirstlane(col) >= gs) {
    for (int r = part; r < rows; r += nparts) {
      float a = 0.f, b = 0.f;
      if (!p.is_rms) ts.sum2(a, b);
      a = b = 0.f;  // sum2 hands back the team's totals
      ts.sum2(a, b);
    }
    return;
  }
  if (part >= rows) return;
  const int64_t c0 = (int64_t)group * gs + col;
  float w[8], b[8];
  ld8<float>(p.weight + c0, w);
#pragma unroll
  for (int e = 0; e < 8; ++e) b[e] = 0.f;
  if (p.bias) ld8<float>(p.bias + c0, b);
  const T *xp = static_cast<const T *>(p.x) + c0;
  const T *zp = HAS_Z ? static_cast<const T *>(p.z) + c0 : xp;
  T *op = static_cast<T *>(p.out) + c0;
  const float inv_n = 1.f / (float)gs;
  const bool gate_after = HAS_Z && p.norm_before_gate, gate_before = HAS_Z && !p.norm_before_gate;
  const int last = part + (rows - 1 - part) / nparts * nparts;  // the last row of this part
  Pack8<T> cx, cz;
  cx.load_global(xp + (int64_t)part * p.x_rs);
  if (HAS_Z) cz.load_global(zp + (int64_t)part * p.z_rs);
  for (int r = part; r < rows; r += nparts) {
    const int rn = min(r + nparts, last);
    Pack8<T> nx, nz;
    nx.load_global(xp + (int64_t)rn * p.x_rs);
    if (HAS_Z) nz.load_global(zp + (int64_t)rn * p.z_rs);
    float x[8], sz[8];
    cx.unpack(x);
    if (HAS_Z) {
      cz.unpack(sz);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float sig;
        sz[e] = silu_g(sz[e], sig);
        if (gate_before) x[e] *= sz[e];
      }
    }
    float mean = 0.f, dummy = 0.f;
    if (!p.is_rms) {
#pragma unroll
      for (int e = 0; e < 8; ++e) mean += x[e];
      ts.sum2(mean, dummy);
      mean *= inv_n;
    }
    float var = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      x[e] -= mean;
      var = __builtin_fmaf(x[e], x[e], var);
    }
    dummy = 0.f;
    ts.sum2(var, dummy);
    const float rstd = 1.f / sqrtf(var * inv_n + p.eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float y = __builtin_fmaf(x[e] * rstd, w[e], b[e]);
      if (gate_after) y *= sz[e];
      x[e] = y;
    }
    Pack8<T> o;
    o.pack(x);
    o.store_global(op + (int64_t)r * p.out_rs);
    if (threadIdx.x == 0) {
      if (p.mean) p.mean[(int64_t)r * ngroups + group] = mean;
      p.rstd[(int64_t)r * ngroups + group] = rstd;
    }
    cx = nx;
    if (HAS_Z) cz = nz;
  }
}

// The backward pass for groups of 1024 < group_size <= 8192 channels in whole waves' worth (multiples of 512), rows
// of 16-byte pieces: a workgroup of 256 / 512 / 1024 threads per (part, group), one piece per thread, so that a
// wave holds either 512 channels or none (5120 channels on 1024 threads: 10 waves of 16 work, 6 only take part in the
// team's sums, in a loop of their own).  No branch surrounds a load or a store of the loop over the rows: the row
// after next's operands are requested (the last row again at the end) before the current row's are used, and the
// waits the compiler places then name exactly the loads they need.  With the guarded accesses of norm_bwd_kernel
// every wait was for everything in flight, the row just requested included, and a row cost its whole latency.
template <typename T, int TEAM, bool HAS_Z>
__global__ __launch_bounds__(TEAM) void norm_bwd_wide_kernel(const NormGatedParams p) {
  __shared__ float lds[2 * (TEAM / 64) * 2];
  TeamSum<TEAM> ts(lds);
  const int gs = p.group_size, ngroups = p.dim / gs, nparts = p.nparts, rows = p.rows;
  const int group = blockIdx.x % ngroups, part = blockIdx.x / ngroups;
  const int col = threadIdx.x * 8;
  if (__builtin_amdgcn_readfirstlane(col) >= gs) {
    for (int r = part; r < rows; r += nparts) {
      float a = 0.f, b = 0.f;
      ts.sum2(a, b);
    }
    return;
  }
  const int64_t c0 = (int64_t)group * gs + col;
  float w[8], b[8], dw[8], db[8];
  ld8<float>(p.weight + c0, w);
#pragma unroll
  for (int e = 0; e < 8; ++e) b[e] = dw[e] = db[e] = 0.f;
  if (p.bias) ld8<float>(p.bias + c0, b);
  const T *xp = static_cast<const T *>(p.x) + c0;
  const T *gp = static_cast<const T *>(p.dy) + c0;
  const T *zp = HAS_Z ? static_cast<const T *>(p.z) + c0 : xp;
  T *dxp = static_cast<T *>(p.dx) + c0;
  T *dzp = HAS_Z ? static_cast<T *>(p.dz) + c0 : dxp;
  const float *rstdp = p.rstd + group, *meanp = p.is_rms ? rstdp : p.mean + group;
  const float inv_n = 1.f / (float)gs;
  const bool gate_after = HAS_Z && p.norm_before_gate, gate_before = HAS_Z && !p.norm_before_gate;
  if (part < rows) {
    const int last = part + (rows - 1 - part) / nparts * nparts;  // the last row of this part
    Pack8<T> cx, cg, cz;
    float cmean = *(const GLOBAL_AS float *)(meanp + (int64_t)part * ngroups);
    float crstd = *(const GLOBAL_AS float *)(rstdp + (int64_t)part * ngroups);
    cx.load_global(xp + (int64_t)part * p.x_rs);
    cg.load_global(gp + (int64_t)part * p.dy_rs);
    if (HAS_Z) cz.load_global(zp + (int64_t)part * p.z_rs);
    for (int r = part; r < rows; r += nparts) {
      const int rn = min(r + nparts, last);
      Pack8<T> nx, ng, nz;
      const float nmean = *(const GLOBAL_AS float *)(meanp + (int64_t)rn * ngroups);
      const float nrstd = *(const GLOBAL_AS float *)(rstdp + (int64_t)rn * ngroups);
      nx.load_global(xp + (int64_t)rn * p.x_rs);
      ng.load_global(gp + (int64_t)rn * p.dy_rs);
      if (HAS_Z) nz.load_global(zp + (int64_t)rn * p.z_rs);
      float x[8], g[8], z[8], xr[8];
      cx.unpack(x);
      cg.unpack(g);
      if (HAS_Z) cz.unpack(z);
      const float mean = p.is_rms ? 0.f : cmean, rstd = crstd;
      float c1 = 0.f, c2 = 0.f;
      // after this loop: x = xhat, g = w * dy', z = dz (gate after the norm) or kept as z (gate before it), xr = x
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float xv = x[e], gv = g[e];
        float sig = 0.f, sz = 1.f;
        if (HAS_Z) sz = silu_g(z[e], sig);
        xr[e] = xv;
        if (gate_before) xv *= sz;
        const float xhat = (xv - mean) * rstd;
        if (gate_after) {
          const float y = __builtin_fmaf(xhat, w[e], b[e]);
          z[e] = gv * y * sig * (1.f + z[e] * (1.f - sig));
          gv *= sz;
        }
        dw[e] = __builtin_fmaf(gv, xhat, dw[e]);
        db[e] += gv;
        const float wdy = w[e] * gv;
        c1 = __builtin_fmaf(xhat, wdy, c1);
        c2 += wdy;
        x[e] = xhat;
        g[e] = wdy;
      }
      ts.sum2(c1, c2);
      c1 *= inv_n;
      c2 = p.is_rms ? 0.f : c2 * inv_n;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = (g[e] - (x[e] * c1 + c2)) * rstd;
        if (gate_before) {  // dz = dx' * x * dsilu(z), dx = dx' * silu(z)
          float sig;
          const float sz = silu_g(z[e], sig);
          z[e] = d * xr[e] * sig * (1.f + z[e] * (1.f - sig));
          x[e] = d * sz;
        } else {
          x[e] = d;
        }
      }
      Pack8<T> ox, oz;
      ox.pack(x);
      ox.store_global(dxp + (int64_t)r * p.dx_rs);
      if (HAS_Z) {
        oz.pack(z);
        oz.store_global(dzp + (int64_t)r * p.dz_rs);
      }
      cx = nx;
      cg = ng;
      if (HAS_Z) cz = nz;
      cmean = nmean;
      crstd = nrstd;
    }
  }
  float *dwp = p.dw_part + (int64_t)part * p.dim + c0;
  *(GLOBAL_AS f32x4 *)dwp = f32x4{dw[0], dw[1], dw[2], dw[3]};
  *(GLOBAL_AS f32x4 *)(dwp + 4) = f32x4{dw[4], dw[5], dw[6], dw[7]};
  if (p.db_part) {
    float *dbp = p.db_part + (int64_t)part * p.dim + c0;
    *(GLOBAL_AS f32x4 *)dbp = f32x4{db[0], db[1], db[2], db[3]};
    *(GLOBAL_AS f32x4 *)(dbp + 4) = f32x4{db[4], db[5], db[6], db[7]};
  }
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
// cost registers, hence waves in flight); only groups beyond 16384 channels take 3 or 4 steps.  Above 4096
// channels a whole workgroup of 1024 threads: one step up to 8192 channels keeps the backward pass at 114
// registers (a team of 512 with two steps needs 240 and measured 10 % slower on 5120 channels).
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
  return pick_k<T, 1024, VEC>(p, bwd, st);
}

template <typename T, int TEAM> int launch_wide(const NormGatedParams &p, bool bwd, hipStream_t st) {
  // forward: as many parts as workgroups the chip holds at once (2048 threads per CU), never more than rows
  const int ngroups = p.dim / p.group_size;
  const int nparts = bwd ? p.nparts : max(1, min(p.rows, cu_count() * (2048 / TEAM) / ngroups));
  const int64_t wgs = (int64_t)ngroups * nparts;
  if (wgs > 0x7fffffff) return MAMBA_E_UNSUPPORTED;
  const dim3 grid((unsigned)wgs), block(TEAM);
  if (bwd) {
    if (p.z) norm_bwd_wide_kernel<T, TEAM, true><<<grid, block, 0, st>>>(p);
    else norm_bwd_wide_kernel<T, TEAM, false><<<grid, block, 0, st>>>(p);
  } else {
    if (p.z) norm_fwd_wide_kernel<T, TEAM, true><<<grid, block, 0, st>>>(p, nparts);
    else norm_fwd_wide_kernel<T, TEAM, false><<<grid, block, 0, st>>>(p, nparts);
  }
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

template <typename T> int run(const NormGatedParams &p, bool bwd, hipStream_t st) {
  const bool vec = vec_ok<T>(p, bwd);
  if (vec && p.rows > 0 && p.group_size > 1024 && p.group_size <= 8192 && p.group_size % 512 == 0) {
    if (p.group_size <= 2048) return launch_wide<T, 256>(p, bwd, st);
    if (p.group_size <= 4096) return launch_wide<T, 512>(p, bwd, st);
    return launch_wide<T, 1024>(p, bwd, st);
  }
  return vec ? pick_team<T, true>(p, bwd, st) : pick_team<T, false>(p, bwd, st);
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
