// Mamba-1 selective scan with a complex state matrix A (complex state, B, C; output = 2 Re <h, C>),
// forward and backward, for gfx950.
//
// Same decomposition in time as the real kernels (a lane owns 8 consecutive positions, a wave one
// 512-step tile per pass, DPP scans of (decay, value) pairs over the 64 lanes, the state after every
// tile checkpointed for the backward pass) with complex pairs; a wave owns one channel.  B and C are
// read by every lane straight from memory (per-position operands carry (re, im) pairs interleaved
// along the sequence, so a lane's 8 positions are 16 consecutive values) and their gradients go to
// the global fp32 accumulators with atomics.  This path serves the S4D-style complex variant and is
// not tuned like the real one.
#include "common.hpp"

namespace {

constexpr int KI = 8;
constexpr int TILE = 64 * KI;
constexpr int MAXN = 256;
constexpr int NW = 4;  // waves (= channels) per workgroup

struct cx {
  float r, i;
};
DEVI cx cmul(cx a, cx b) { return {a.r * b.r - a.i * b.i, a.r * b.i + a.i * b.r}; }
DEVI cx cmadd(cx a, cx b, cx c) {  // a * b + c
  return {__builtin_fmaf(a.r, b.r, __builtin_fmaf(-a.i, b.i, c.r)), __builtin_fmaf(a.r, b.i, __builtin_fmaf(a.i, b.r, c.i))};
}
DEVI cx cconj(cx a) { return {a.r, -a.i}; }
DEVI cx cscale(float s, cx a) { return {s * a.r, s * a.i}; }
template <int CTRL, int MASK = 0xf> DEVI cx dpp_c(cx old, cx v) {
  return {dpp_f<CTRL, MASK>(old.r, v.r), dpp_f<CTRL, MASK>(old.i, v.i)};
}
DEVI cx readlane_c(cx v, int l) { return {readlane_f(v.r, l), readlane_f(v.i, l)}; }

// inclusive scans of segments h_out = a h_in + b over the wave: lane 0 first / lane 63 first
DEVI void scan_fwd_c(cx &a, cx &b) {
#define STEP(CTRL, MASK)                            \
  {                                                 \
    const cx bp = dpp_c<CTRL, MASK>({0.f, 0.f}, b); \
    const cx ap = dpp_c<CTRL, MASK>({1.f, 0.f}, a); \
    b = cmadd(a, bp, b);                            \
    a = cmul(a, ap);                                \
  }
  STEP(DPP_ROW_SHR + 1, 0xf)
  STEP(DPP_ROW_SHR + 2, 0xf)
  STEP(DPP_ROW_SHR + 4, 0xf)
  STEP(DPP_ROW_SHR + 8, 0xf)
  STEP(DPP_ROW_BCAST15, 0xa)
  STEP(DPP_ROW_BCAST31, 0xc)
#undef STEP
}
DEVI void scan_rev_c(cx &a, cx &b, int lane) {
#define STEP(N)                                          \
  {                                                      \
    const cx bp = dpp_c<DPP_ROW_SHL + N>({0.f, 0.f}, b); \
    const cx ap = dpp_c<DPP_ROW_SHL + N>({1.f, 0.f}, a); \
    b = cmadd(a, bp, b);                                 \
    a = cmul(a, ap);                                     \
  }
  STEP(1)
  STEP(2)
  STEP(4)
  STEP(8)
#undef STEP
  const cx a1 = readlane_c(a, 16), b1 = readlane_c(b, 16);
  const cx a2 = readlane_c(a, 32), b2 = readlane_c(b, 32);
  const cx a3 = readlane_c(a, 48), b3 = readlane_c(b, 48);
  const cx a23 = cmul(a2, a3), b23 = cmadd(a2, b3, b2);
  const cx a123 = cmul(a1, a23), b123 = cmadd(a1, b23, b1);
  const int row = lane >> 4;
  const cx an = row == 0 ? a123 : (row == 1 ? a23 : (row == 2 ? a3 : cx{1.f, 0.f}));
  const cx bn = row == 0 ? b123 : (row == 1 ? b23 : (row == 2 ? b3 : cx{0.f, 0.f}));
  b = cmadd(a, bn, b);
  a = cmul(a, an);
}

// exp(dl * A) for complex A = (Ar, Ai)
DEVI cx cexp_step(float dl, float Ar, float Ai) {
  const float e = fast_exp(dl * Ar);
  float s, c;
  sincosf(dl * Ai, &s, &c);  // the accurate routine: phase errors compound over the sequence
  return {e * c, e * s};
}

// A lane's 8 positions of a per-position complex operand: 16 consecutive values (re, im pairs) at
// row + 2 * tl; or the channel's matrix entry for every position.
template <typename T, bool VEC, bool CONST>
DEVI void load_cx8(cx (&v)[8], const void *base, const T *row, int d, int N, int n, int tl, int nvalid) {
  if constexpr (CONST) {
    const float *m = static_cast<const float *>(base) + ((int64_t)d * N + n) * 2;
    const cx c = {m[0], m[1]};
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = c;
  } else {
    float lo[8], hi[8];
    ld8_guard<T, VEC>(row + 2 * tl, min(2 * nvalid, 8), 0.f, lo);
    ld8_guard<T, VEC>(row + 2 * tl + 8, max(2 * nvalid - 8, 0), 0.f, hi);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = {lo[2 * i], lo[2 * i + 1]};
      v[4 + i] = {hi[2 * i], hi[2 * i + 1]};
    }
  }
}

struct Geo {
  int d, g, b, ntiles;
  bool valid;
};
DEVI Geo geometry(const MambaScanParams &p, int wave) {
  Geo q;
  q.d = blockIdx.x * NW + wave;
  q.b = blockIdx.y;
  q.valid = q.d < p.dim;
  q.g = min(q.d, p.dim - 1) / (p.dim / p.ngroups);
  q.ntiles = (p.seqlen + TILE - 1) / TILE;
  return q;
}

// One term of a sum that every channel of a group adds into: a float atomic, or (dsc != 0) a 64-bit integer atomic
// on the term scaled to a fixed point, whose result does not depend on the order of the adds.
DEVI void add_term(float *dst, int64_t *shadow, int64_t idx, float v, float dsc) {
  if (dsc != 0.f) {
    det_add(shadow, idx, v, dsc);
  } else {
    unsafeAtomicAdd(dst + idx, v);
  }
}

// ------------------------------------------------------------------ forward
template <typename T, bool VEC, int BC> __global__ __launch_bounds__(NW * 64) void cscan_fwd_kernel(const MambaScanParams p) {
  __shared__ cx hcar[NW][MAXN];  // state carried across tiles
  const int N = p.dstate, L = p.seqlen;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const Geo q = geometry(p, wave);
  if (!q.valid) return;  // no workgroup barriers below
  const int d = q.d, b = q.b;
  const T *Bg = (const T *)p.B + b * p.B_bs + q.g * p.B_gs;
  const T *Cg = (const T *)p.C + b * p.C_bs + q.g * p.C_gs;
  const float *Ad = (const float *)p.A + (int64_t)d * N * 2;
  for (int n = lane; n < N; n += 64) hcar[wave][n] = {0.f, 0.f};
  const float bias = p.delta_bias ? ((const float *)p.delta_bias)[d] : 0.f;
  for (int tile = 0; tile < q.ntiles; ++tile) {
    const int tl = tile * TILE + lane * KI;
    const int nvalid = min(max(L - tl, 0), KI);
    float u[8], dl[8], du[8], y[8];
    ld8_guard<T, VEC>((const T *)p.u + b * p.u_bs + d * p.u_ds + tl, nvalid, 0.f, u);
    ld8_guard<T, VEC>((const T *)p.delta + b * p.delta_bs + d * p.delta_ds + tl, nvalid, 0.f, dl);
#pragma unroll
    for (int i = 0; i < KI; ++i) {
      float x = dl[i] + bias;
      if (p.delta_softplus) x = softplus_f(x);
      dl[i] = (i < nvalid) ? x : 0.f;
      du[i] = dl[i] * u[i];
      y[i] = 0.f;
    }
    for (int n = 0; n < N; ++n) {
      const float Ar = Ad[2 * n], Ai = Ad[2 * n + 1];
      cx Bv[8], Cv[8], ac[8], hh[8];
      load_cx8<T, VEC, (BC & 1) != 0>(Bv, p.B, Bg + (int64_t)n * p.B_ns, d, N, n, tl, nvalid);
      load_cx8<T, VEC, (BC & 2) != 0>(Cv, p.C, Cg + (int64_t)n * p.C_ns, d, N, n, tl, nvalid);
      ac[0] = cexp_step(dl[0], Ar, Ai);
      hh[0] = cscale(du[0], Bv[0]);
#pragma unroll
      for (int i = 1; i < KI; ++i) {
        const cx a = cexp_step(dl[i], Ar, Ai);
        hh[i] = cmadd(a, hh[i - 1], cscale(du[i], Bv[i]));
        ac[i] = cmul(ac[i - 1], a);
      }
      cx sa = ac[KI - 1], sb = hh[KI - 1];
      scan_fwd_c(sa, sb);
      const cx hc = hcar[wave][n];
      const cx hend = cmadd(sa, hc, sb);
      const cx hx = dpp_c<DPP_WAVE_SHR1>(hc, hend);  // state entering this lane
      if (lane == 63) hcar[wave][n] = hend;
#pragma unroll
      for (int i = 0; i < KI; ++i) {
        const cx h = cmadd(ac[i], hx, hh[i]);
        y[i] += 2.f * (Cv[i].r * h.r - Cv[i].i * h.i);
      }
    }
    if (p.D) {
      const float Dd = ((const float *)p.D)[d];
#pragma unroll
      for (int i = 0; i < KI; ++i) y[i] = __builtin_fmaf(Dd, u[i], y[i]);
    }
    if (p.z) {
      float z[8];
      ld8_guard<T, VEC>((const T *)p.z + b * p.z_bs + d * p.z_ds + tl, nvalid, 0.f, z);
#pragma unroll
      for (int i = 0; i < KI; ++i) y[i] *= z[i] * sigmoid_f(z[i]);
    }
    st8_guard<T, VEC>((T *)p.out + b * p.out_bs + d * p.out_ds + tl, nvalid, y);
    float *ck = p.ckpt + ((((int64_t)b * p.dim + d) * q.ntiles + tile) * N) * 2;
    for (int n = lane; n < N; n += 64) {
      const cx h = hcar[wave][n];
      ck[2 * n] = h.r;
      ck[2 * n + 1] = h.i;
    }
  }
}

// ----------------------------------------------------------------- backward
template <typename T, bool VEC, int BC> __global__ __launch_bounds__(NW * 64) void cscan_bwd_kernel(const MambaScanParams p) {
  __shared__ cx gcar[NW][MAXN];   // adjoint at the first position of the following tile
  __shared__ cx anx[NW][MAXN];    // decay at the first position of the following tile
  __shared__ cx dAacc[NW][MAXN], dBcacc[NW][MAXN], dCcacc[NW][MAXN];
  const int N = p.dstate, L = p.seqlen;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const Geo q = geometry(p, wave);
  if (!q.valid) return;
  const int d = q.d, b = q.b;
  const bool has_z = p.z != nullptr;
  const T *Bg = (const T *)p.B + b * p.B_bs + q.g * p.B_gs;
  const T *Cg = (const T *)p.C + b * p.C_bs + q.g * p.C_gs;
  const float *Ad = (const float *)p.A + (int64_t)d * N * 2;
  float *dBg = p.dB32 + ((int64_t)b * p.ngroups + q.g) * N * 2 * L;  // (batch, ngroups, dstate, 2 L)
  float *dCg = p.dC32 + ((int64_t)b * p.ngroups + q.g) * N * 2 * L;
  // deterministic mode: the same sums as 64-bit integers of fixed-point terms (order-independent)
  const float dsc = p.det_scale ? p.det_scale[0] : 0.f;
  int64_t *det_dBg = p.det_dB ? p.det_dB + ((int64_t)b * p.ngroups + q.g) * N * 2 * L : nullptr;
  int64_t *det_dCg = p.det_dC ? p.det_dC + ((int64_t)b * p.ngroups + q.g) * N * 2 * L : nullptr;
  for (int n = lane; n < N; n += 64) {
    gcar[wave][n] = anx[wave][n] = dAacc[wave][n] = dBcacc[wave][n] = dCcacc[wave][n] = {0.f, 0.f};
  }
  const float bias = p.delta_bias ? ((const float *)p.delta_bias)[d] : 0.f;
  const float Dd = p.D ? ((const float *)p.D)[d] : 0.f;
  float dbsum = 0.f, dDsum = 0.f;
  for (int tile = q.ntiles - 1; tile >= 0; --tile) {
    const int tl = tile * TILE + lane * KI;
    const int nvalid = min(max(L - tl, 0), KI);
    float u[8], draw[8], dl[8], du[8], dout[8], dy[8], z[8], acc[8], dd[8], y[8];
    ld8_guard<T, VEC>((const T *)p.u + b * p.u_bs + d * p.u_ds + tl, nvalid, 0.f, u);
    ld8_guard<T, VEC>((const T *)p.delta + b * p.delta_bs + d * p.delta_ds + tl, nvalid, 0.f, draw);
    ld8_guard<T, VEC>((const T *)p.dout + b * p.dout_bs + d * p.dout_ds + tl, nvalid, 0.f, dout);
#pragma unroll
    for (int i = 0; i < KI; ++i) {
      dy[i] = dout[i];
      z[i] = 0.f;
    }
    if (has_z) {
      ld8_guard<T, VEC>((const T *)p.z + b * p.z_bs + d * p.z_ds + tl, nvalid, 0.f, z);
#pragma unroll
      for (int i = 0; i < KI; ++i) dy[i] *= z[i] * sigmoid_f(z[i]);
    }
#pragma unroll
    for (int i = 0; i < KI; ++i) {
      float x = draw[i] + bias;
      if (p.delta_softplus) x = softplus_f(x);
      dl[i] = (i < nvalid) ? x : 0.f;
      du[i] = dl[i] * u[i];
      acc[i] = dd[i] = y[i] = 0.f;
    }
    const float *ck = tile > 0 ? p.ckpt + ((((int64_t)b * p.dim + d) * q.ntiles + tile - 1) * N) * 2 : nullptr;
    for (int n = 0; n < N; ++n) {
      const float Ar = Ad[2 * n], Ai = Ad[2 * n + 1];
      const cx hc = ck ? cx{ck[2 * n], ck[2 * n + 1]} : cx{0.f, 0.f};
      cx Bv[8], Cv[8], a[8], ac[8], bb[8], h[8];
      load_cx8<T, VEC, (BC & 1) != 0>(Bv, p.B, Bg + (int64_t)n * p.B_ns, d, N, n, tl, nvalid);
      load_cx8<T, VEC, (BC & 2) != 0>(Cv, p.C, Cg + (int64_t)n * p.C_ns, d, N, n, tl, nvalid);
#pragma unroll
      for (int i = 0; i < KI; ++i) {
        a[i] = cexp_step(dl[i], Ar, Ai);
        bb[i] = cscale(du[i], Bv[i]);
      }
      h[0] = bb[0];
      ac[0] = a[0];
#pragma unroll
      for (int i = 1; i < KI; ++i) {
        h[i] = cmadd(a[i], h[i - 1], bb[i]);
        ac[i] = cmul(ac[i - 1], a[i]);
      }
      cx sa = ac[KI - 1], sb = h[KI - 1];
      scan_fwd_c(sa, sb);
      const cx hend = cmadd(sa, hc, sb);
      const cx hx = dpp_c<DPP_WAVE_SHR1>(hc, hend);
#pragma unroll
      for (int i = 0; i < KI; ++i) h[i] = cmadd(ac[i], hx, h[i]);  // true states
      if (has_z) {
#pragma unroll
        for (int i = 0; i < KI; ++i) y[i] += 2.f * (Cv[i].r * h[i].r - Cv[i].i * h[i].i);
      }
      // adjoint recurrence g[t] = 2 dy[t] conj(C[t]) + conj(a[t+1]) g[t+1]
      const cx a_next = dpp_c<DPP_WAVE_SHL1>(anx[wave][n], a[0]);
      cx gg[8], ar[8];
      gg[KI - 1] = cscale(2.f * dy[KI - 1], cconj(Cv[KI - 1]));
      ar[KI - 1] = cconj(a_next);
#pragma unroll
      for (int i = KI - 2; i >= 0; --i) {
        gg[i] = cmadd(cconj(a[i + 1]), gg[i + 1], cscale(2.f * dy[i], cconj(Cv[i])));
        ar[i] = cmul(ar[i + 1], cconj(a[i + 1]));
      }
      cx ra = ar[0], rb = gg[0];
      scan_rev_c(ra, rb, lane);
      const cx gc = gcar[wave][n];
      const cx gfirst = cmadd(ra, gc, rb);
      const cx gx = dpp_c<DPP_WAVE_SHL1>(gc, gfirst);  // adjoint at the next lane's first position
      if (lane == 0) {
        gcar[wave][n] = gfirst;
        anx[wave][n] = a[0];
      }
      cx dAp = {0.f, 0.f}, dBp = {0.f, 0.f}, dCp = {0.f, 0.f};
#pragma unroll
      for (int i = 0; i < KI; ++i) {
        const cx g = cmadd(ar[i], gx, gg[i]);
        const cx dC = cscale(2.f * dy[i], cconj(h[i]));
        const cx dB = cscale(du[i], g);
        if constexpr (BC & 2) {
          dCp.r += dC.r;
          dCp.i += dC.i;
        } else if (i < nvalid) {
          add_term(dCg, det_dCg, (int64_t)n * 2 * L + 2 * (tl + i), dC.r, dsc);
          add_term(dCg, det_dCg, (int64_t)n * 2 * L + 2 * (tl + i) + 1, dC.i, dsc);
        }
        if constexpr (BC & 1) {
          dBp.r += dB.r;
          dBp.i += dB.i;
        } else if (i < nvalid) {
          add_term(dBg, det_dBg, (int64_t)n * 2 * L + 2 * (tl + i), dB.r, dsc);
          add_term(dBg, det_dBg, (int64_t)n * 2 * L + 2 * (tl + i) + 1, dB.i, dsc);
        }
        acc[i] += Bv[i].r * g.r + Bv[i].i * g.i;                      // Re(conj(B) g)
        const cx w = cmul(cconj(cx{h[i].r - bb[i].r, h[i].i - bb[i].i}), g);  // conj(a h[t-1]) g
        dd[i] += Ar * w.r + Ai * w.i;                                  // Re(conj(A) w)
        dAp.r = __builtin_fmaf(dl[i], w.r, dAp.r);
        dAp.i = __builtin_fmaf(dl[i], w.i, dAp.i);
      }
      dAp = {wave_sum_to_last(dAp.r), wave_sum_to_last(dAp.i)};
      if (lane == 63) {
        dAacc[wave][n].r += dAp.r;
        dAacc[wave][n].i += dAp.i;
      }
      if constexpr (BC & 1) {
        dBp = {wave_sum_to_last(dBp.r), wave_sum_to_last(dBp.i)};
        if (lane == 63) {
          dBcacc[wave][n].r += dBp.r;
          dBcacc[wave][n].i += dBp.i;
        }
      }
      if constexpr (BC & 2) {
        dCp = {wave_sum_to_last(dCp.r), wave_sum_to_last(dCp.i)};
        if (lane == 63) {
          dCcacc[wave][n].r += dCp.r;
          dCcacc[wave][n].i += dCp.i;
        }
      }
    }
    float o[8];
#pragma unroll
    for (int i = 0; i < KI; ++i) o[i] = __builtin_fmaf(dl[i], acc[i], Dd * dy[i]);
    st8_guard<T, VEC>((T *)p.du + b * p.du_bs + d * p.du_ds + tl, nvalid, o);
#pragma unroll
    for (int i = 0; i < KI; ++i) {
      const float x = draw[i] + bias;
      float gd = __builtin_fmaf(u[i], acc[i], dd[i]);
      if (p.delta_softplus && x <= 20.f) gd *= sigmoid_f(x);
      gd = (i < nvalid) ? gd : 0.f;
      o[i] = gd;
      dbsum += gd;
      dDsum = __builtin_fmaf(dy[i], u[i], dDsum);
    }
    st8_guard<T, VEC>((T *)p.ddelta + b * p.ddelta_bs + d * p.ddelta_ds + tl, nvalid, o);
    if (has_z) {
      float oz[8];
#pragma unroll
      for (int i = 0; i < KI; ++i) {
        const float yf = __builtin_fmaf(Dd, u[i], y[i]);
        const float s = sigmoid_f(z[i]);
        o[i] = dout[i] * yf * s * (1.f + z[i] * (1.f - s));
        oz[i] = yf * z[i] * s;
      }
      st8_guard<T, VEC>((T *)p.dz + b * p.dz_bs + d * p.dz_ds + tl, nvalid, o);
      if (p.out_z) st8_guard<T, VEC>((T *)p.out_z + b * p.outz_bs + d * p.outz_ds + tl, nvalid, oz);
    }
  }
  dbsum = wave_sum_to_last(dbsum);
  dDsum = wave_sum_to_last(dDsum);
  if (lane == 63) {
    p.dD_part[(int64_t)b * p.dim + d] = dDsum;
    p.ddelta_bias_part[(int64_t)b * p.dim + d] = dbsum;
  }
  for (int n = lane; n < N; n += 64) {
    float *o = p.dA_part + (((int64_t)b * p.dim + d) * N + n) * 2;
    o[0] = dAacc[wave][n].r;
    o[1] = dAacc[wave][n].i;
    if constexpr (BC & 1) {
      float *ob = p.dB32 + (((int64_t)b * p.dim + d) * N + n) * 2;
      ob[0] = dBcacc[wave][n].r;
      ob[1] = dBcacc[wave][n].i;
    }
    if constexpr (BC & 2) {
      float *oc = p.dC32 + (((int64_t)b * p.dim + d) * N + n) * 2;
      oc[0] = dCcacc[wave][n].r;
      oc[1] = dCcacc[wave][n].i;
    }
  }
}

inline bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

bool vec_ok(const MambaScanParams &p, bool bwd) {
  const int es = p.dtype == MAMBA_F32 ? 4 : 2;
  const int64_t m = 16 / es;
  auto ok = [&](const void *ptr, int64_t s0, int64_t s1) { return !ptr || (aligned16(ptr) && s0 % m == 0 && s1 % m == 0); };
  if (p.seqlen % 8 != 0) return false;
  bool v = ok(p.u, p.u_bs, p.u_ds) && ok(p.delta, p.delta_bs, p.delta_ds) && ok(p.z, p.z_bs, p.z_ds);
  if (!(p.bc_const & 1)) v = v && ok(p.B, p.B_bs, p.B_gs) && p.B_ns % m == 0;
  if (!(p.bc_const & 2)) v = v && ok(p.C, p.C_bs, p.C_gs) && p.C_ns % m == 0;
  if (!bwd) return v && ok(p.out, p.out_bs, p.out_ds);
  return v && ok(p.dout, p.dout_bs, p.dout_ds) && ok(p.du, p.du_bs, p.du_ds) &&
         ok(p.ddelta, p.ddelta_bs, p.ddelta_ds) && ok(p.dz, p.dz_bs, p.dz_ds) && ok(p.out_z, p.outz_bs, p.outz_ds);
}

template <typename T, bool BWD, int BC> int launch_bc(const MambaScanParams &p, hipStream_t s) {
  dim3 grid((p.dim + NW - 1) / NW, p.batch), block(NW * 64);
  const bool vec = vec_ok(p, BWD);
  if (BWD) {
    if (vec) hipLaunchKernelGGL((cscan_bwd_kernel<T, true, BC>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((cscan_bwd_kernel<T, false, BC>), grid, block, 0, s, p);
  } else {
    if (vec) hipLaunchKernelGGL((cscan_fwd_kernel<T, true, BC>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((cscan_fwd_kernel<T, false, BC>), grid, block, 0, s, p);
  }
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

template <typename T, bool BWD> int launch_t(const MambaScanParams &p, hipStream_t s) {
  switch (p.bc_const & 3) {
    case 0: return launch_bc<T, BWD, 0>(p, s);
    case 1: return launch_bc<T, BWD, 1>(p, s);
    case 2: return launch_bc<T, BWD, 2>(p, s);
    default: return launch_bc<T, BWD, 3>(p, s);
  }
}

}  // namespace

// Called by mamba1_scan_fwd / mamba1_scan_bwd when p->a_complex is set; arguments already checked.
int mamba1_scan_complex(const MambaScanParams *p, hipStream_t s, bool bwd) {
  if (p->dstate > MAXN) return MAMBA_E_UNSUPPORTED;
  switch (p->dtype) {
    case MAMBA_F32: return bwd ? launch_t<float, true>(*p, s) : launch_t<float, false>(*p, s);
    case MAMBA_BF16: return bwd ? launch_t<bf16_t, true>(*p, s) : launch_t<bf16_t, false>(*p, s);
    default: return bwd ? launch_t<f16_t, true>(*p, s) : launch_t<f16_t, false>(*p, s);
  }
}
