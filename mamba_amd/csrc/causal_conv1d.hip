// Depthwise causal 1-D convolution (kernel width 2..4) with optional SiLU, forward and backward, for
// gfx950.  It is the convolution in front of both scans (the reference calls the separate
// causal_conv1d package for it: mamba_ssm/ops/selective_scan_interface.py:224,
// mamba_ssm/ops/triton/ssd_combined.py:845); the arithmetic is
//   out[b, c, l] = act(bias[c] + sum_k w[c, k] x[b, c, l - (W-1) + k]),  x = 0 before the sequence,
// and with seq_idx a tap that reaches into another sequence of a packed row contributes nothing.
// Both memory layouts of the callers are served without a transpose:
//   * position-contiguous rows (batch, channel, position): a thread owns 8 consecutive positions of
//     one row (16-byte accesses) and reads the 3-position halo from the neighbouring chunk;
//   * channel-contiguous rows (batch, position, channel): a thread owns 8 consecutive channels and
//     walks a run of positions with the previous taps in registers, so every element is read once.
// The backward pass re-computes the pre-activation from x instead of storing it.
#include "common.hpp"

namespace {

constexpr int MAXW = 4;

DEVI float dsilu(float pre) {  // d/dpre silu(pre)
  const float s = sigmoid_f(pre);
  return s * (1.f + pre * (1.f - s));
}
DEVI float silu_f(float v) { return v * sigmoid_f(v); }

// Shared sums (dweight, dbias): float atomics, or -- deterministic mode, p.det_scale set -- 64-bit integer atomics
// on terms scaled to a fixed point, whose result does not depend on the order of the adds (see SsdParams).
DEVI void conv_acc_add(const CausalConvParams &p, float *dst, int64_t *shadow, int64_t idx, float v) {
  if (p.det_scale) {
    det_add(shadow, idx, v, p.det_scale[0]);
  } else {
    unsafeAtomicAdd(dst + idx, v);
  }
}

// Taps right-aligned in 4 slots: slot 3 multiplies x[l], slot 0 multiplies x[l - 3].
DEVI void load_taps(const CausalConvParams &p, int c, float (&w)[MAXW], float &bias) {
#pragma unroll
  for (int k = 0; k < MAXW; ++k) {
    const int j = k - (MAXW - p.width);
    w[k] = j >= 0 ? p.weight[(int64_t)c * p.width + j] : 0.f;
  }
  bias = p.bias ? p.bias[c] : 0.f;
}

// ------------------------------------------------------------------ position-contiguous rows
// Element j of win[] is position l0 - 3 + j; positions outside [0, L) read as 0.
template <typename T, bool VEC, int NWIN> DEVI void load_window(const T *row, int l0, int L, float (&win)[NWIN]) {
  static_assert(NWIN == 11 || NWIN == 19, "3 halo positions, 8 own, optionally 8 following");
  if constexpr (VEC) {  // l0 is a multiple of 8, L a multiple of 8, the row 16-byte aligned
    Pack8<T> prev, cur, next;
    prev.load(row + max(l0 - 8, 0));
    cur.load(row + l0);
    if (NWIN == 19) next.load(row + min(l0 + 8, L - 8));
    float a[8], c[8];
    prev.unpack(a);
    cur.unpack(c);
#pragma unroll
    for (int j = 0; j < 3; ++j) win[j] = l0 >= 8 ? a[5 + j] : 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) win[3 + j] = c[j];
    if constexpr (NWIN == 19) {
      float n[8];
      next.unpack(n);
#pragma unroll
      for (int j = 0; j < 8; ++j) win[11 + j] = l0 + 8 < L ? n[j] : 0.f;
    }
  } else {
#pragma unroll
    for (int j = 0; j < NWIN; ++j) {
      const int l = l0 - 3 + j;
      win[j] = (l >= 0 && l < L) ? ld1<T>(row + l) : 0.f;
    }
  }
}
template <int NWIN> DEVI void load_ids(const int32_t *seq, int l0, int L, int (&ids)[NWIN]) {
#pragma unroll
  for (int j = 0; j < NWIN; ++j) {
    const int l = l0 - 3 + j;
    ids[j] = (l >= 0 && l < L) ? seq[l] : -0x7fffffff;
  }
}

template <typename T, bool VEC> __global__ __launch_bounds__(256) void conv_rows_fwd_kernel(const CausalConvParams p) {
  const int L = p.seqlen, c = blockIdx.y, b = blockIdx.z;
  const int l0 = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (l0 >= L) return;
  float w[MAXW], bias;
  load_taps(p, c, w, bias);
  float win[11];
  load_window<T, VEC, 11>(static_cast<const T *>(p.x) + b * p.x_bs + c * p.x_cs, l0, L, win);
  int ids[11];
  if (p.seq_idx) load_ids<11>(p.seq_idx + (int64_t)b * L, l0, L, ids);
  float o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float v = bias;
#pragma unroll
    for (int k = 0; k < MAXW; ++k) {
      float t = win[i + k];
      if (p.seq_idx && ids[i + k] != ids[i + 3]) t = 0.f;
      v = __builtin_fmaf(w[k], t, v);
    }
    o[i] = p.silu ? silu_f(v) : v;
  }
  st8_guard<T, VEC>(static_cast<T *>(p.out) + b * p.out_bs + c * p.out_cs + l0, min(8, L - l0), o);
}

template <typename T, bool VEC> __global__ __launch_bounds__(256) void conv_rows_bwd_kernel(const CausalConvParams p) {
  const int L = p.seqlen, c = blockIdx.y, b = blockIdx.z;
  const int l0 = (blockIdx.x * 256 + threadIdx.x) * 8;
  float dw[MAXW] = {0.f, 0.f, 0.f, 0.f}, db = 0.f;
  if (l0 < L) {
    float w[MAXW], bias;
    load_taps(p, c, w, bias);
    float xw[19], gw[19];  // x and dout at positions l0 - 3 .. l0 + 15 (dout's halo is not used)
    load_window<T, VEC, 19>(static_cast<const T *>(p.x) + b * p.x_bs + c * p.x_cs, l0, L, xw);
    load_window<T, VEC, 19>(static_cast<const T *>(p.dout) + b * p.dout_bs + c * p.dout_cs, l0, L, gw);
    int ids[19];
    if (p.seq_idx) load_ids<19>(p.seq_idx + (int64_t)b * L, l0, L, ids);
    // gradient of the pre-activation at positions l0 .. l0 + 10 (own 8 and the 3 that still see them)
    float dpre[11];
#pragma unroll
    for (int j = 0; j < 11; ++j) {
      float v = bias;
#pragma unroll
      for (int k = 0; k < MAXW; ++k) {
        float t = xw[j + k];
        if (p.seq_idx && ids[j + k] != ids[j + 3]) t = 0.f;
        v = __builtin_fmaf(w[k], t, v);
      }
      const float g = gw[j + 3];
      dpre[j] = l0 + j < L ? (p.silu ? g * dsilu(v) : g) : 0.f;
    }
    float o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float v = 0.f;
#pragma unroll
      for (int k = 0; k < MAXW; ++k) {  // x[l] enters out[l + 3 - k] through tap k
        float t = dpre[i + 3 - k];
        if (p.seq_idx && ids[i + 3 + 3 - k] != ids[i + 3]) t = 0.f;
        v = __builtin_fmaf(w[k], t, v);
      }
      o[i] = v;
#pragma unroll
      for (int k = 0; k < MAXW; ++k) {
        float t = xw[i + k];
        if (p.seq_idx && ids[i + k] != ids[i + 3]) t = 0.f;
        dw[k] = __builtin_fmaf(dpre[i], t, dw[k]);
      }
      db += dpre[i];
    }
    st8_guard<T, VEC>(static_cast<T *>(p.dx) + b * p.dx_bs + c * p.dx_cs + l0, min(8, L - l0), o);
  }
  // one atomic per wave and tap
#pragma unroll
  for (int k = 0; k < MAXW; ++k) dw[k] = wave_sum_to_last(dw[k]);
  db = wave_sum_to_last(db);
  if ((threadIdx.x & 63) == 63) {
#pragma unroll
    for (int k = 0; k < MAXW; ++k) {
      const int j = k - (MAXW - p.width);
      if (j >= 0 && dw[k] != 0.f) conv_acc_add(p, p.dweight, p.det_dweight, (int64_t)c * p.width + j, dw[k]);
    }
    if (p.dbias && db != 0.f) conv_acc_add(p, p.dbias, p.det_dbias, c, db);
  }
}

// ------------------------------------------------------------------ channel-contiguous rows
constexpr int RUN = 32;   // positions per thread
constexpr int NRUN = 4;   // runs per workgroup (256 threads = 64 channel groups x 4 runs)

template <typename T, bool VEC> DEVI void load_ch8(const T *p, int nvalid, float (&o)[8]) {
  if constexpr (VEC) ld8<T>(p, o);
  else ld8_guard<T, false>(p, nvalid, 0.f, o);
}

template <typename T, bool VEC> __global__ __launch_bounds__(256) void conv_cl_fwd_kernel(const CausalConvParams p) {
  const int L = p.seqlen, b = blockIdx.z;
  const int cg = threadIdx.x & 63, run = threadIdx.x >> 6;
  const int c0 = (blockIdx.x * 64 + cg) * 8;
  if (c0 >= p.dim) return;
  const int nch = min(8, p.dim - c0);
  const int lbeg = (blockIdx.y * NRUN + run) * RUN, lend = min(lbeg + RUN, L);
  if (lbeg >= L) return;
  float w[8][MAXW], bias[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) load_taps(p, min(c0 + e, p.dim - 1), w[e], bias[e]);
  const T *xb = static_cast<const T *>(p.x) + b * p.x_bs + c0;
  T *ob = static_cast<T *>(p.out) + b * p.out_bs + c0;
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L : nullptr;
  float xw[3][8];  // x at l - 3, l - 2, l - 1
  int idw[3] = {-0x7fffffff, -0x7fffffff, -0x7fffffff};
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    const int l = lbeg - 3 + j;
#pragma unroll
    for (int e = 0; e < 8; ++e) xw[j][e] = 0.f;
    if (l >= 0) {
      load_ch8<T, VEC>(xb + (int64_t)l * p.x_ls, nch, xw[j]);
      if (seq) idw[j] = seq[l];
    }
  }
  for (int l4 = lbeg; l4 < lend; l4 += 4) {
    float xin[4][8];
    int idn[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {  // the loads of four positions first
      const int l = min(l4 + u, L - 1);
      load_ch8<T, VEC>(xb + (int64_t)l * p.x_ls, nch, xin[u]);
      idn[u] = seq ? seq[l] : 0;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int l = l4 + u;
      if (l >= lend) break;
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float v = __builtin_fmaf(w[e][3], xin[u][e], bias[e]);
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          float t = xw[j][e];
          if (seq && idw[j] != idn[u]) t = 0.f;
          v = __builtin_fmaf(w[e][j], t, v);
        }
        o[e] = p.silu ? silu_f(v) : v;
      }
      st8_guard<T, VEC>(ob + (int64_t)l * p.out_ls, nch, o);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        xw[0][e] = xw[1][e];
        xw[1][e] = xw[2][e];
        xw[2][e] = xin[u][e];
      }
      idw[0] = idw[1];
      idw[1] = idw[2];
      idw[2] = idn[u];
    }
  }
}

template <typename T, bool VEC> __global__ __launch_bounds__(256) void conv_cl_bwd_kernel(const CausalConvParams p) {
  __shared__ float red[NRUN - 1][64][8 * (MAXW + 1)];
  const int L = p.seqlen, b = blockIdx.z;
  const int cg = threadIdx.x & 63, run = threadIdx.x >> 6;
  const int c0 = (blockIdx.x * 64 + cg) * 8;
  const int nch = max(0, min(8, p.dim - c0));
  const int lbeg = (blockIdx.y * NRUN + run) * RUN, lend = min(lbeg + RUN, L);
  float dw[8][MAXW], db[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    db[e] = 0.f;
#pragma unroll
    for (int k = 0; k < MAXW; ++k) dw[e][k] = 0.f;
  }
  if (nch > 0 && lbeg < L) {
    float w[8][MAXW], bias[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) load_taps(p, min(c0 + e, p.dim - 1), w[e], bias[e]);
    const T *xb = static_cast<const T *>(p.x) + b * p.x_bs + c0;
    const T *gb = static_cast<const T *>(p.dout) + b * p.dout_bs + c0;
    T *dxb = static_cast<T *>(p.dx) + b * p.dx_bs + c0;
    const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L : nullptr;
    // Walk down from lend + 2: the first three steps only rebuild dpre at the positions after the run.
    const int ltop = min(lend + 2, L - 1);
    float xw[4][8];   // x at l - 3 .. l
    float dp[4][8];   // dpre at l .. l + 3
    int idx[7];       // sequence ids at l - 3 .. l + 3
#pragma unroll
    for (int j = 0; j < 7; ++j) {
      const int l = ltop - 3 + j;
      idx[j] = (seq && l >= 0 && l < L) ? seq[l] : -0x7fffffff;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int l = ltop - 3 + j;
#pragma unroll
      for (int e = 0; e < 8; ++e) xw[j][e] = dp[j][e] = 0.f;
      if (l >= 0) load_ch8<T, VEC>(xb + (int64_t)l * p.x_ls, nch, xw[j]);
    }
    for (int l4 = ltop; l4 >= lbeg; l4 -= 4) {
      // the loads of four steps first (dout at l4 .. l4 - 3, x at l4 - 4 .. l4 - 7): the stores of dx in
      // between would otherwise keep the compiler from moving them up
      float g4[4][8], x4[4][8];
      int id4[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int l = l4 - u;
        load_ch8<T, VEC>(gb + (int64_t)max(l, 0) * p.dout_ls, nch, g4[u]);
        load_ch8<T, VEC>(xb + (int64_t)max(l - 4, 0) * p.x_ls, nch, x4[u]);
        id4[u] = (seq && l - 4 >= 0) ? seq[l - 4] : -0x7fffffff;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int l = l4 - u;
        if (l < lbeg) break;
        // dpre at l
        float dcur[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float v = bias[e];
#pragma unroll
          for (int k = 0; k < MAXW; ++k) {
            float t = xw[k][e];
            if (seq && idx[k] != idx[3]) t = 0.f;
            v = __builtin_fmaf(w[e][k], t, v);
          }
          dcur[e] = p.silu ? g4[u][e] * dsilu(v) : g4[u][e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          dp[3][e] = dp[2][e];
          dp[2][e] = dp[1][e];
          dp[1][e] = dp[0][e];
          dp[0][e] = dcur[e];
        }
        if (l < lend) {
          float o[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float v = 0.f;
#pragma unroll
            for (int k = 0; k < MAXW; ++k) {  // x[l] enters out[l + 3 - k] through tap k
              float t = dp[3 - k][e];
              if (seq && idx[3 + 3 - k] != idx[3]) t = 0.f;
              v = __builtin_fmaf(w[e][k], t, v);
            }
            o[e] = v;
#pragma unroll
            for (int k = 0; k < MAXW; ++k) {
              float t = xw[k][e];
              if (seq && idx[k] != idx[3]) t = 0.f;
              dw[e][k] = __builtin_fmaf(dcur[e], t, dw[e][k]);
            }
            db[e] += dcur[e];
          }
          st8_guard<T, VEC>(dxb + (int64_t)l * p.dx_ls, nch, o);
        }
        // slide both windows one position down
        const bool has = l - 4 >= 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          xw[3][e] = xw[2][e];
          xw[2][e] = xw[1][e];
          xw[1][e] = xw[0][e];
          xw[0][e] = has ? x4[u][e] : 0.f;
        }
#pragma unroll
        for (int j = 6; j > 0; --j) idx[j] = idx[j - 1];
        idx[0] = id4[u];
      }
    }
  }
  // the four runs of a channel group are summed in LDS, then one atomic per channel and tap
  if (run > 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
#pragma unroll
      for (int k = 0; k < MAXW; ++k) red[run - 1][cg][e * (MAXW + 1) + k] = dw[e][k];
      red[run - 1][cg][e * (MAXW + 1) + MAXW] = db[e];
    }
  }
  __syncthreads();
  if (run == 0 && nch > 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (e >= nch) break;
#pragma unroll
      for (int k = 0; k < MAXW; ++k) {
        float v = dw[e][k];
#pragma unroll
        for (int r = 0; r < NRUN - 1; ++r) v += red[r][cg][e * (MAXW + 1) + k];
        const int j = k - (MAXW - p.width);
        if (j >= 0 && v != 0.f) conv_acc_add(p, p.dweight, p.det_dweight, (int64_t)(c0 + e) * p.width + j, v);
      }
      float v = db[e];
#pragma unroll
      for (int r = 0; r < NRUN - 1; ++r) v += red[r][cg][e * (MAXW + 1) + MAXW];
      if (p.dbias && v != 0.f) conv_acc_add(p, p.dbias, p.det_dbias, c0 + e, v);
    }
  }
}

// The backward pass with 4 channels per thread (rows whose 4-channel pieces are aligned: the VEC case).  The
// 8-channel kernel above keeps two windows, the taps and their gradients for 8 channels in 232 registers, two waves
// per SIMD; half the channels per thread is half the registers and twice the waves.  A thread's loads of the next
// four steps are requested, and kept in their storage format, before it works on the current four: memory and the
// SiLU re-computation overlap instead of alternating.
template <typename T> struct Raw4 {
  typedef u32x2 type;
};
template <> struct Raw4<float> {
  typedef u32x4 type;
};
template <typename T> DEVI void unpack4(const typename Raw4<T>::type &r, float (&o)[4]);
template <> DEVI void unpack4<bf16_t>(const u32x2 &r, float (&o)[4]) {
  o[0] = bf16_lo(r.x); o[1] = bf16_hi(r.x); o[2] = bf16_lo(r.y); o[3] = bf16_hi(r.y);
}
template <> DEVI void unpack4<f16_t>(const u32x2 &r, float (&o)[4]) {
  o[0] = f16_lo(r.x); o[1] = f16_hi(r.x); o[2] = f16_lo(r.y); o[3] = f16_hi(r.y);
}
template <> DEVI void unpack4<float>(const u32x4 &r, float (&o)[4]) {
  const f32x4 f = __builtin_bit_cast(f32x4, r);  // (the whole vector: a bit cast of one element of it is not one)
  o[0] = f.x; o[1] = f.y; o[2] = f.z; o[3] = f.w;
}
template <typename T> DEVI typename Raw4<T>::type pack4(const float (&v)[4]);
template <> DEVI u32x2 pack4<bf16_t>(const float (&v)[4]) { return u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])}; }
template <> DEVI u32x2 pack4<f16_t>(const float (&v)[4]) { return u32x2{pack_f16(v[0], v[1]), pack_f16(v[2], v[3])}; }
template <> DEVI u32x4 pack4<float>(const float (&v)[4]) {
  const f32x4 f = {v[0], v[1], v[2], v[3]};
  return __builtin_bit_cast(u32x4, f);
}

// The forward pass in the same form: 4 channels per thread, the next four positions requested before the current
// four are worked on.
template <typename T> __global__ __launch_bounds__(256) void conv_cl_fwd4_kernel(const CausalConvParams p) {
  typedef typename Raw4<T>::type raw_t;
  constexpr int CPT = 4;
  const int L = p.seqlen, b = blockIdx.z;
  const int cg = threadIdx.x & 63, run = threadIdx.x >> 6;
  const int c0 = (blockIdx.x * 64 + cg) * CPT;
  if (c0 >= p.dim) return;
  const int lbeg = (blockIdx.y * NRUN + run) * RUN, lend = min(lbeg + RUN, L);
  if (lbeg >= L) return;
  float w[CPT][MAXW], bias[CPT];
#pragma unroll
  for (int e = 0; e < CPT; ++e) load_taps(p, c0 + e, w[e], bias[e]);
  const T *xb = static_cast<const T *>(p.x) + b * p.x_bs + c0;
  T *ob = static_cast<T *>(p.out) + b * p.out_bs + c0;
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L : nullptr;
  float xw[3][CPT];  // x at l - 3, l - 2, l - 1
  int idw[3] = {-0x7fffffff, -0x7fffffff, -0x7fffffff};
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    const int l = lbeg - 3 + j;
#pragma unroll
    for (int e = 0; e < CPT; ++e) xw[j][e] = 0.f;
    if (l >= 0) {
      unpack4<T>(*reinterpret_cast<const raw_t *>(xb + (int64_t)l * p.x_ls), xw[j]);
      if (seq) idw[j] = seq[l];
    }
  }
  raw_t xn[4];
  int idn[4];
  auto fetch = [&](int l4) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int l = min(l4 + u, L - 1);
      xn[u] = *reinterpret_cast<const raw_t *>(xb + (int64_t)l * p.x_ls);
      idn[u] = seq ? seq[l] : 0;
    }
  };
  fetch(lbeg);
  for (int l4 = lbeg; l4 < lend; l4 += 4) {
    raw_t x4[4];
    int id4[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) x4[u] = xn[u], id4[u] = idn[u];
    fetch(l4 + 4);  // (past the run on the last turn: rows that exist, never used)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int l = l4 + u;
      if (l >= lend) break;
      float xin[CPT], o[CPT];
      unpack4<T>(x4[u], xin);
#pragma unroll
      for (int e = 0; e < CPT; ++e) {
        float v = __builtin_fmaf(w[e][3], xin[e], bias[e]);
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          float t = xw[j][e];
          if (seq && idw[j] != id4[u]) t = 0.f;
          v = __builtin_fmaf(w[e][j], t, v);
        }
        o[e] = p.silu ? silu_f(v) : v;
      }
      *reinterpret_cast<raw_t *>(ob + (int64_t)l * p.out_ls) = pack4<T>(o);
#pragma unroll
      for (int e = 0; e < CPT; ++e) {
        xw[0][e] = xw[1][e];
        xw[1][e] = xw[2][e];
        xw[2][e] = xin[e];
      }
      idw[0] = idw[1];
      idw[1] = idw[2];
      idw[2] = id4[u];
    }
  }
}

// RUN: positions per thread.  A run costs a 6-position warm-up, the taps, and its share of the reduction of the
// filter gradients: long runs (128) where the grid still fills the chip, the forward kernel's 32 otherwise.
template <typename T, int RUN> __global__ __launch_bounds__(256) void conv_cl_bwd4_kernel(const CausalConvParams p) {
  typedef typename Raw4<T>::type raw_t;
  constexpr int CPT = 4;
  __shared__ float red[NRUN - 1][64][CPT * (MAXW + 1)];
  const int L = p.seqlen, b = blockIdx.z;
  const int cg = threadIdx.x & 63, run = threadIdx.x >> 6;
  const int c0 = (blockIdx.x * 64 + cg) * CPT;
  const bool live = c0 < p.dim;  // (dim is a multiple of 8 here: a thread has all of its 4 channels or none)
  const int lbeg = (blockIdx.y * NRUN + run) * RUN, lend = min(lbeg + RUN, L);
  float dw[CPT][MAXW], db[CPT];
#pragma unroll
  for (int e = 0; e < CPT; ++e) {
    db[e] = 0.f;
#pragma unroll
    for (int k = 0; k < MAXW; ++k) dw[e][k] = 0.f;
  }
  if (live && lbeg < L) {
    float w[CPT][MAXW], bias[CPT];
#pragma unroll
    for (int e = 0; e < CPT; ++e) load_taps(p, c0 + e, w[e], bias[e]);
    const T *xb = static_cast<const T *>(p.x) + b * p.x_bs + c0;
    const T *gb = static_cast<const T *>(p.dout) + b * p.dout_bs + c0;
    T *dxb = static_cast<T *>(p.dx) + b * p.dx_bs + c0;
    const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L : nullptr;
    // Walk down from lend + 2: the first three steps only rebuild dpre at the positions after the run.
    const int ltop = min(lend + 2, L - 1);
    float xw[4][CPT];  // x at l - 3 .. l
    float dp[4][CPT];  // dpre at l .. l + 3
    int idx[7];        // sequence ids at l - 3 .. l + 3
#pragma unroll
    for (int j = 0; j < 7; ++j) {
      const int l = ltop - 3 + j;
      idx[j] = (seq && l >= 0 && l < L) ? seq[l] : -0x7fffffff;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int l = ltop - 3 + j;
#pragma unroll
      for (int e = 0; e < CPT; ++e) xw[j][e] = dp[j][e] = 0.f;
      if (l >= 0) unpack4<T>(*reinterpret_cast<const raw_t *>(xb + (int64_t)l * p.x_ls), xw[j]);
    }
    // the loads of four steps (dout at l4 .. l4 - 3, x at l4 - 4 .. l4 - 7), one group ahead
    raw_t gn[4], xn[4];
    int idn[4];
    auto fetch = [&](int l4) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int l = l4 - u;
        gn[u] = *reinterpret_cast<const raw_t *>(gb + (int64_t)max(l, 0) * p.dout_ls);
        xn[u] = *reinterpret_cast<const raw_t *>(xb + (int64_t)max(l - 4, 0) * p.x_ls);
        idn[u] = (seq && l - 4 >= 0) ? seq[l - 4] : -0x7fffffff;
      }
    };
    fetch(ltop);
    for (int l4 = ltop; l4 >= lbeg; l4 -= 4) {
      raw_t g4[4], x4[4];
      int id4[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) g4[u] = gn[u], x4[u] = xn[u], id4[u] = idn[u];
      fetch(l4 - 4);  // (below the run on the last turn: rows that exist, never used)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int l = l4 - u;
        if (l < lbeg) break;
        float gu[CPT], xu[CPT];
        unpack4<T>(g4[u], gu);
        unpack4<T>(x4[u], xu);
        // dpre at l
        float dcur[CPT];
#pragma unroll
        for (int e = 0; e < CPT; ++e) {
          float v = bias[e];
#pragma unroll
          for (int k = 0; k < MAXW; ++k) {
            float t = xw[k][e];
            if (seq && idx[k] != idx[3]) t = 0.f;
            v = __builtin_fmaf(w[e][k], t, v);
          }
          dcur[e] = p.silu ? gu[e] * dsilu(v) : gu[e];
        }
#pragma unroll
        for (int e = 0; e < CPT; ++e) {
          dp[3][e] = dp[2][e];
          dp[2][e] = dp[1][e];
          dp[1][e] = dp[0][e];
          dp[0][e] = dcur[e];
        }
        if (l < lend) {
          float o[CPT];
#pragma unroll
          for (int e = 0; e < CPT; ++e) {
            float v = 0.f;
#pragma unroll
            for (int k = 0; k < MAXW; ++k) {  // x[l] enters out[l + 3 - k] through tap k
              float t = dp[3 - k][e];
              if (seq && idx[3 + 3 - k] != idx[3]) t = 0.f;
              v = __builtin_fmaf(w[e][k], t, v);
            }
            o[e] = v;
#pragma unroll
            for (int k = 0; k < MAXW; ++k) {
              float t = xw[k][e];
              if (seq && idx[k] != idx[3]) t = 0.f;
              dw[e][k] = __builtin_fmaf(dcur[e], t, dw[e][k]);
            }
            db[e] += dcur[e];
          }
          *reinterpret_cast<raw_t *>(dxb + (int64_t)l * p.dx_ls) = pack4<T>(o);
        }
        // slide both windows one position down
        const bool has = l - 4 >= 0;
#pragma unroll
        for (int e = 0; e < CPT; ++e) {
          xw[3][e] = xw[2][e];
          xw[2][e] = xw[1][e];
          xw[1][e] = xw[0][e];
          xw[0][e] = has ? xu[e] : 0.f;
        }
#pragma unroll
        for (int j = 6; j > 0; --j) idx[j] = idx[j - 1];
        idx[0] = id4[u];
      }
    }
  }
  // the four runs of a channel group are summed in LDS, then one atomic per channel and tap
  if (run > 0) {
#pragma unroll
    for (int e = 0; e < CPT; ++e) {
#pragma unroll
      for (int k = 0; k < MAXW; ++k) red[run - 1][cg][e * (MAXW + 1) + k] = dw[e][k];
      red[run - 1][cg][e * (MAXW + 1) + MAXW] = db[e];
    }
  }
  __syncthreads();
  if (run == 0 && live) {
#pragma unroll
    for (int e = 0; e < CPT; ++e) {
#pragma unroll
      for (int k = 0; k < MAXW; ++k) {
        float v = dw[e][k];
#pragma unroll
        for (int r = 0; r < NRUN - 1; ++r) v += red[r][cg][e * (MAXW + 1) + k];
        const int j = k - (MAXW - p.width);
        if (j >= 0 && v != 0.f) conv_acc_add(p, p.dweight, p.det_dweight, (int64_t)(c0 + e) * p.width + j, v);
      }
      float v = db[e];
#pragma unroll
      for (int r = 0; r < NRUN - 1; ++r) v += red[r][cg][e * (MAXW + 1) + MAXW];
      if (p.dbias && v != 0.f) conv_acc_add(p, p.dbias, p.det_dbias, c0 + e, v);
    }
  }
}

// ------------------------------------------------------------------ decode step
// One thread per (batch entry, channel): with xn = [conv_state, x] along the position axis,
//   out[t] = act(bias + sum_k w[k] xn[state_len + t - (W-1) + k]),  conv_state <- last state_len of xn
// (what the reference spells, for one new position and state_len = W, as roll + insert + dot:
// mamba_ssm/modules/mamba2.py:291-296).  The shift runs in place in ascending order, which is safe
// because every entry is written from a higher index of the same thread's own row.
// one filter tap or bias value of the dtype the caller's parameters have
DEVI float ld_param(const void *base, int dtype, int64_t i) {
  switch (dtype) {
    case MAMBA_BF16: return ld1<bf16_t>(static_cast<const bf16_t *>(base) + i);
    case MAMBA_F16: return ld1<f16_t>(static_cast<const f16_t *>(base) + i);
    default: return static_cast<const float *>(base)[i];
  }
}

template <typename T, typename S> __global__ __launch_bounds__(256) void conv_update_kernel(const CausalConvUpdateParams p) {
  const int c = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
  if (c >= p.dim) return;
  const T *x = static_cast<const T *>(p.x) + b * p.x_bs + c * p.x_cs;
  T *out = static_cast<T *>(p.out) + b * p.out_bs + c * p.out_cs;
  const int slot = p.conv_state_indices ? p.conv_state_indices[b] : b;
  if (slot < 0 || slot >= p.state_rows) {  // padding entry of the batch: no state, zero output
    for (int t = 0; t < p.seqlen; ++t) st1<T>(out + t * p.out_ls, 0.f);
    return;
  }
  S *st = static_cast<S *>(p.conv_state) + slot * p.state_bs + c * p.state_cs;
  float w[MAXW], bias;
#pragma unroll
  for (int k = 0; k < MAXW; ++k) {
    const int j = k - (MAXW - p.width);
    w[k] = j >= 0 ? ld_param(p.weight, p.weight_dtype, (int64_t)c * p.width + j) : 0.f;
  }
  bias = p.bias ? ld_param(p.bias, p.weight_dtype, c) : 0.f;
  const int SL = p.state_len;
  float win[MAXW];  // win[0..2]: the three positions before the next output, win[3]: the new one
  if (p.cache_seqlens) {
    // circular buffer: position t of the sequence lives in slot t mod SL; taps the filter does not use stay 0
    const int len = p.cache_seqlens[b];
    auto slot_of = [&](int t) { return ((t % SL) + SL) % SL; };
#pragma unroll
    for (int i = 0; i < MAXW - 1; ++i)
      win[i] = i >= MAXW - p.width ? ld1<S>(st + slot_of(len - (MAXW - 1) + i) * p.state_ls) : 0.f;
    for (int t = 0; t < p.seqlen; ++t) st1<S>(st + slot_of(len + t) * p.state_ls, ld1<T>(x + t * p.x_ls));
  } else {
#pragma unroll
    for (int i = 0; i < MAXW - 1; ++i) {
      const int j = SL - (MAXW - 1) + i;
      win[i] = j >= 0 ? ld1<S>(st + j * p.state_ls) : 0.f;
    }
    for (int j = 0; j < SL; ++j) {
      const int src = j + p.seqlen;
      const float v = src < SL ? ld1<S>(st + src * p.state_ls) : ld1<T>(x + (src - SL) * p.x_ls);
      st1<S>(st + j * p.state_ls, v);
    }
  }
  for (int t = 0; t < p.seqlen; ++t) {
    win[3] = ld1<T>(x + t * p.x_ls);
    float v = bias;
#pragma unroll
    for (int k = 0; k < MAXW; ++k) v = __builtin_fmaf(w[k], win[k], v);
    st1<T>(out + t * p.out_ls, p.silu ? silu_f(v) : v);
    win[0] = win[1];
    win[1] = win[2];
    win[2] = win[3];
  }
}

// states[s, c, j] = x[cu_seqlens[s + 1] - state_len + j, c], zero where that position lies before
// the start of sequence s: the convolution state each sequence of a packed row leaves behind.
template <typename T> __global__ __launch_bounds__(256) void conv_varlen_states_kernel(const CausalConvVarlenParams p) {
  const int c = blockIdx.x * 256 + threadIdx.x, s = blockIdx.y;
  if (c >= p.dim) return;
  const int beg = p.cu_seqlens[s], end = p.cu_seqlens[s + 1];
  const T *x = static_cast<const T *>(p.x) + c * p.x_cs;
  T *o = static_cast<T *>(p.states) + s * p.states_bs + c * p.states_cs;
  for (int j = 0; j < p.state_len; ++j) {
    const int l = end - p.state_len + j;
    st1<T>(o + j * p.states_ls, l >= beg && l >= 0 && l < p.total ? ld1<T>(x + l * p.x_ls) : 0.f);
  }
}

// ------------------------------------------------------------------ launch
int check(const CausalConvParams *p, bool bwd) {
  if (!p || !p->x || !p->weight) return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->dim <= 0 || p->seqlen <= 0) return MAMBA_E_BADARG;
  if (p->width < 2 || p->width > MAXW) return MAMBA_E_UNSUPPORTED;
  if (p->dtype != MAMBA_F32 && p->dtype != MAMBA_BF16 && p->dtype != MAMBA_F16) return MAMBA_E_BADARG;
  if (p->batch > 65535) return MAMBA_E_UNSUPPORTED;
  if (!bwd && !p->out) return MAMBA_E_BADARG;
  if (bwd && (!p->dout || !p->dx || !p->dweight)) return MAMBA_E_BADARG;
  if (bwd && p->det_scale && (!p->det_dweight || (p->dbias && !p->det_dbias))) return MAMBA_E_BADARG;
  if (p->x_ls != 1 && p->x_cs != 1) return MAMBA_E_UNSUPPORTED;
  return MAMBA_OK;
}

bool al16(const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; }

template <typename T> int launch_conv(const CausalConvParams &p, bool bwd, hipStream_t s) {
  const int64_t m = 16 / sizeof(T);
  const bool rows = p.x_ls == 1 && (bwd ? p.dout_ls == 1 && p.dx_ls == 1 : p.out_ls == 1);
  auto ok = [&](const void *q, int64_t a, int64_t b2) { return al16(q) && a % m == 0 && b2 % m == 0; };
  if (rows) {
    if (p.dim > 65535) return MAMBA_E_UNSUPPORTED;
    const bool vec = p.seqlen % 8 == 0 && ok(p.x, p.x_bs, p.x_cs) &&
                     (bwd ? ok(p.dout, p.dout_bs, p.dout_cs) && ok(p.dx, p.dx_bs, p.dx_cs) : ok(p.out, p.out_bs, p.out_cs));
    dim3 grid((p.seqlen + 2047) / 2048, p.dim, p.batch);
    if (bwd) {
      if (vec) hipLaunchKernelGGL((conv_rows_bwd_kernel<T, true>), grid, dim3(256), 0, s, p);
      else hipLaunchKernelGGL((conv_rows_bwd_kernel<T, false>), grid, dim3(256), 0, s, p);
    } else {
      if (vec) hipLaunchKernelGGL((conv_rows_fwd_kernel<T, true>), grid, dim3(256), 0, s, p);
      else hipLaunchKernelGGL((conv_rows_fwd_kernel<T, false>), grid, dim3(256), 0, s, p);
    }
  } else {
    const bool cl = p.x_cs == 1 && (bwd ? p.dout_cs == 1 && p.dx_cs == 1 : p.out_cs == 1);
    if (!cl) return MAMBA_E_UNSUPPORTED;
    const bool vec = p.dim % 8 == 0 && ok(p.x, p.x_bs, p.x_ls) &&
                     (bwd ? ok(p.dout, p.dout_bs, p.dout_ls) && ok(p.dx, p.dx_bs, p.dx_ls) : ok(p.out, p.out_bs, p.out_ls));
    const int ygrid = (p.seqlen + RUN * NRUN - 1) / (RUN * NRUN);
    if (ygrid > 65535) return MAMBA_E_UNSUPPORTED;
    dim3 grid((p.dim + 511) / 512, ygrid, p.batch);
    if (bwd) {
      if (vec) {
        constexpr int LONG = 128;
        const int xg = (p.dim + 255) / 256, ylong = (p.seqlen + LONG * NRUN - 1) / (LONG * NRUN);
        if ((int64_t)xg * ylong * p.batch >= 2 * (int64_t)cu_count())
          hipLaunchKernelGGL((conv_cl_bwd4_kernel<T, LONG>), dim3(xg, ylong, p.batch), dim3(256), 0, s, p);
        else
          hipLaunchKernelGGL((conv_cl_bwd4_kernel<T, RUN>), dim3(xg, ygrid, p.batch), dim3(256), 0, s, p);
      }
      else hipLaunchKernelGGL((conv_cl_bwd_kernel<T, false>), grid, dim3(256), 0, s, p);
    } else {
      if (vec) hipLaunchKernelGGL((conv_cl_fwd4_kernel<T>), dim3((p.dim + 255) / 256, ygrid, p.batch), dim3(256), 0, s, p);
      else hipLaunchKernelGGL((conv_cl_fwd_kernel<T, false>), grid, dim3(256), 0, s, p);
    }
  }
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

int dispatch(const CausalConvParams *p, bool bwd, mamba_stream_t stream) {
  int rc = check(p, bwd);
  if (rc != MAMBA_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (p->dtype) {
    case MAMBA_F32: return launch_conv<float>(*p, bwd, s);
    case MAMBA_BF16: return launch_conv<bf16_t>(*p, bwd, s);
    default: return launch_conv<f16_t>(*p, bwd, s);
  }
}

template <typename T> int launch_update(const CausalConvUpdateParams &p, hipStream_t s) {
  dim3 grid((p.dim + 255) / 256, p.batch);
  switch (p.state_dtype) {
    case MAMBA_F32: hipLaunchKernelGGL((conv_update_kernel<T, float>), grid, dim3(256), 0, s, p); break;
    case MAMBA_BF16: hipLaunchKernelGGL((conv_update_kernel<T, bf16_t>), grid, dim3(256), 0, s, p); break;
    case MAMBA_F16: hipLaunchKernelGGL((conv_update_kernel<T, f16_t>), grid, dim3(256), 0, s, p); break;
    default: return MAMBA_E_BADARG;
  }
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

}  // namespace

extern "C" int causal_conv1d_fwd(const CausalConvParams *p, mamba_stream_t stream) { return dispatch(p, false, stream); }
extern "C" int causal_conv1d_bwd(const CausalConvParams *p, mamba_stream_t stream) { return dispatch(p, true, stream); }

extern "C" int causal_conv1d_update(const CausalConvUpdateParams *p, mamba_stream_t stream) {
  if (!p || !p->x || !p->conv_state || !p->weight || !p->out) return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->dim <= 0 || p->seqlen <= 0 || p->state_len < 0) return MAMBA_E_BADARG;
  if (p->width < 2 || p->width > MAXW) return MAMBA_E_UNSUPPORTED;
  if (p->state_len < p->width - 1 || p->state_rows <= 0) return MAMBA_E_BADARG;
  if (!p->conv_state_indices && p->state_rows < p->batch) return MAMBA_E_BADARG;
  if (p->batch > 65535) return MAMBA_E_UNSUPPORTED;
  if (p->weight_dtype < MAMBA_F32 || p->weight_dtype > MAMBA_F16) return MAMBA_E_BADARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (p->dtype) {
    case MAMBA_F32: return launch_update<float>(*p, s);
    case MAMBA_BF16: return launch_update<bf16_t>(*p, s);
    case MAMBA_F16: return launch_update<f16_t>(*p, s);
    default: return MAMBA_E_BADARG;
  }
}

extern "C" int causal_conv1d_varlen_states(const CausalConvVarlenParams *p, mamba_stream_t stream) {
  if (!p || !p->x || !p->cu_seqlens || !p->states) return MAMBA_E_BADARG;
  if (p->nseq <= 0 || p->dim <= 0 || p->total < 0 || p->state_len <= 0) return MAMBA_E_BADARG;
  if (p->nseq > 65535) return MAMBA_E_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((p->dim + 255) / 256, p->nseq);
  switch (p->dtype) {
    case MAMBA_F32: hipLaunchKernelGGL((conv_varlen_states_kernel<float>), grid, dim3(256), 0, s, *p); break;
    case MAMBA_BF16: hipLaunchKernelGGL((conv_varlen_states_kernel<bf16_t>), grid, dim3(256), 0, s, *p); break;
    case MAMBA_F16: hipLaunchKernelGGL((conv_varlen_states_kernel<f16_t>), grid, dim3(256), 0, s, *p); break;
    default: return MAMBA_E_BADARG;
  }
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}
