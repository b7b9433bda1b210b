// Mamba-1 backward with 4 items per lane: the kernel of mamba1_scan.hip (scan_bwd_kernel) on 64-position tiles, for
// bf16 rows with per-position B / C, a real A and at most 16 states (reference
// csrc/selective_scan/selective_scan_bwd_kernel.cuh:83).  Half the per-lane working set of the 8-item kernel, so that a
// workgroup needs at most 128 registers and ~half the LDS and two workgroups (16 waves) share a compute unit: twice
// the resident waves per SIMD, paid for with twice the per-lane costs of a state per element (boundary exps, row
// scans, neighbour moves, row sums) and a checkpoint every 64 positions from the forward kernel.  Opt-in
// (MAMBA_AMD_M1_BWD=k4), for measurement against the default kernel; same results to rounding, and bit-for-bit
// repeatable like it (no atomics: dB / dC leave as per-workgroup partials that reduce_parts_kernel adds in order).
#include "mamba1_scan.hpp"

namespace {
namespace k4 {

constexpr int KI4 = 4;                     // items per lane
constexpr int TILE4 = RL * KI4;            // 64 positions per tile
constexpr int BC4_FLOATS = NB16 * TILE4;   // one staged operand: [n][segment][4]
constexpr int ACC4_PITCH = TILE4 * ROWS;   // floats per state row of a dB / dC accumulator: [lane][4]
constexpr int ACC4_FLOATS = NB16 * ACC4_PITCH;

struct Pack4 {
  u32x2 w;
  DEVI void load_global(const bf16_t *p) { w = *(const GLOBAL_AS u32x2 *)p; }
  DEVI void unpack(float (&o)[4]) const {
    o[0] = bf16_lo(w.x); o[1] = bf16_hi(w.x); o[2] = bf16_lo(w.y); o[3] = bf16_hi(w.y);
  }
};
DEVI void st4_or_spare(bf16_t *p, bool wanted, bf16_t *spare, const float (&v)[4]) {
  bf16_t *dst = wanted ? p : spare;
  *(GLOBAL_AS u32x2 *)dst = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
}

// B and C rows 0..15 of the tile starting at t0 -> LDS as fp32, [n][segment c][4]: 2 operands x 16 states x 8 pieces
// of 8 positions = 256 pieces, one per thread of the first four waves.
DEVI void stage_bc4(float *Bs, float *Cs, const bf16_t *Bg, int64_t B_ns, const bf16_t *Cg, int64_t C_ns, int N, int t0,
                    int L, int tid) {
  if (tid >= 256) return;
  const int which = tid >> 7, n = (tid >> 3) & 15, j = tid & 7;
  Pack8<bf16_t> raw;
  const int nc = min(n, N - 1), t = min(t0 + 8 * j, L - 8);
  raw.load((which ? Cg + (int64_t)nc * C_ns : Bg + (int64_t)nc * B_ns) + t);
  float v[8];
  raw.unpack(v);
  const bool ok = n < N && t0 + 8 * j < L;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = ok ? v[i] : 0.f;
  float *dst = (which ? Cs : Bs) + n * TILE4 + j * 8;
  *reinterpret_cast<f32x4 *>(dst) = f32x4{v[0], v[1], v[2], v[3]};
  *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{v[4], v[5], v[6], v[7]};
}
DEVI void ld4(const float *p, float (&o)[4]) {
  const f32x4 v = *reinterpret_cast<const f32x4 *>(p);
  o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
DEVI void st4(float *p, const float (&v)[4]) { *reinterpret_cast<f32x4 *>(p) = f32x4{v[0], v[1], v[2], v[3]}; }

// Which channels a workgroup takes.  pa == pb: workgroup cb of a group takes pa passes of 32 channels from channel
// 32 pa cb on, and blockIdx.y is the batch row.  pa != pb: the channels of a group are cut into blocks of pa + pb
// passes, each served by a long workgroup (the first pa passes) and a short one (the other pb); in launch order the
// first half of the grid holds the long ones and the second half the short ones in the same order, so that a long
// workgroup and its short partner, dispatched half a grid apart, tend to land on the same compute unit and every
// unit gets pa + pb passes.
struct Geo4 {
  int g, b, Dg, dend, d0, passes, part;
};
DEVI Geo4 geometry4(const MambaScanParams &p, int pa, int pb) {
  Geo4 q;
  q.Dg = p.dim / p.ngroups;
  if (pa == pb) {
    const int cblocks = (q.Dg + PASS_CH * pa - 1) / (PASS_CH * pa);
    q.b = blockIdx.y;
    q.g = blockIdx.x / cblocks;
    const int cb = blockIdx.x % cblocks;
    q.d0 = q.g * q.Dg + cb * pa * PASS_CH;
    q.passes = pa;
    q.part = cb;
  } else {
    const int pairs = (q.Dg + PASS_CH * (pa + pb) - 1) / (PASS_CH * (pa + pb));
    const int per_row = p.ngroups * pairs;                    // pairs of a batch row; gridDim.x = 2 per_row
    const int half = per_row * gridDim.y;                     // pairs of the launch
    const int k = blockIdx.y * gridDim.x + blockIdx.x;        // place in launch order
    const int second = k >= half ? 1 : 0;
    const int id = k - second * half;
    q.b = id / per_row;
    const int rest = id % per_row;
    q.g = rest / pairs;
    const int pr = rest % pairs;
    q.d0 = q.g * q.Dg + pr * (pa + pb) * PASS_CH + second * pa * PASS_CH;
    q.passes = second ? pb : pa;
    q.part = 2 * pr + second;
  }
  q.dend = (q.g + 1) * q.Dg;
  return q;
}

__global__ __launch_bounds__(NTHREADS, 4) void scan_bwd_k4_kernel(const MambaScanParams p, const int pa, const int pb,
                                                                  const int nparts) {
  extern __shared__ __align__(16) float smem[];
  typedef bf16_t T;
  const int N = p.dstate, L = p.seqlen;
  constexpr int NP = NB16;
  const int maxp = max(pa, pb), WCHMAX = maxp * PASS_CH;
  float *Bs = smem;
  float *Cs = Bs + BC4_FLOATS;
  float *dBs = Cs + BC4_FLOATS;       // fp32 sums over the workgroup's channels: [n][lane][4]
  float *dCs = dBs + ACC4_FLOATS;
  float *hcar = dCs + ACC4_FLOATS;    // [PASS_CH][NP] state entering the tile (from ckpt), per pass
  float *A1s = hcar + PASS_CH * NP;   // [WCH][NP] A
  float *gcar = A1s + WCHMAX * NP;    // adjoint at the first position of the following tile
  float *anx = gcar + WCHMAX * NP;    // decay at the first position of the following tile
  float *dAacc = anx + WCHMAX * NP;   // [WCH][NP]
  float *dDacc = dAacc + WCHMAX * NP; // [WCH]
  float *dbacc = dDacc + WCHMAX;      // [WCH]
  BwdRow<T> *rows = reinterpret_cast<BwdRow<T> *>(dbacc + WCHMAX);  // [WCH]

  const int tid = threadIdx.x, lane = tid & 63, c = lane & (RL - 1), rsel = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Geo4 q = geometry4(p, pa, pb);
  const int b = q.b, passes = q.passes, WCH = passes * PASS_CH;
  const int chl = wave * ROWS + rsel;
  const int d0 = q.d0;
  const int ntiles = (L + TILE4 - 1) / TILE4;
  const bool has_z = p.z != nullptr;
  T *const spare = reinterpret_cast<T *>(bwd_spare + tid * 8);

  const T *Bg = (const T *)p.B + b * p.B_bs + q.g * p.B_gs;
  const T *Cg = (const T *)p.C + b * p.C_bs + q.g * p.C_gs;
  const float *Ag = (const float *)p.A;
  const int64_t part0 = ((int64_t)b * p.ngroups + q.g) * nparts + q.part;

  for (int i = tid; i < WCH * NP; i += NTHREADS) {
    const int ch = i / NP, n = i % NP, d = d0 + ch;
    A1s[i] = (d < q.dend && n < N) ? Ag[(int64_t)d * N + n] : 0.f;
    gcar[i] = 0.f;
    anx[i] = 0.f;
    dAacc[i] = 0.f;
  }
  for (int i = tid; i < WCH; i += NTHREADS) {
    dDacc[i] = 0.f;
    dbacc[i] = 0.f;
    const int d = min(d0 + i, q.dend - 1);
    BwdRow<T> w;
    w.u = (const T *)p.u + b * p.u_bs + d * p.u_ds;
    w.delta = (const T *)p.delta + b * p.delta_bs + d * p.delta_ds;
    w.dout = (const T *)p.dout + b * p.dout_bs + d * p.dout_ds;
    w.z = has_z ? (const T *)p.z + b * p.z_bs + d * p.z_ds : w.u;
    w.du = (T *)p.du + b * p.du_bs + d * p.du_ds;
    w.ddelta = (T *)p.ddelta + b * p.ddelta_bs + d * p.ddelta_ds;
    w.dz = has_z ? (T *)p.dz + b * p.dz_bs + d * p.dz_ds : nullptr;
    w.out_z = (has_z && p.out_z) ? (T *)p.out_z + b * p.outz_bs + d * p.outz_ds : nullptr;
    w.ckpt = p.ckpt + ((int64_t)b * p.dim + d) * ntiles * N;
    w.D = p.D ? ((const float *)p.D)[d] : 0.f;
    w.bias = p.delta_bias ? ((const float *)p.delta_bias)[d] : 0.f;
    rows[i] = w;
  }
  lds_barrier();

  constexpr int NPP = NB16 / NWAVES, NPH = NB16 / NPP;
  struct Rows {
    Pack4 u, delta, dout, z;
    float ck;
  };
  auto fetch_rows = [&](Rows &k, int tile, int r) {
    const BwdRow<T> &w = rows[r * PASS_CH + chl];
    const int tl = min(tile * TILE4 + c * KI4, L - KI4);  // lanes past the end read a valid position and are masked
    k.ck = *(const GLOBAL_AS float *)(w.ckpt + (int64_t)max(tile - 1, 0) * N + min(c, N - 1));
    k.u.load_global(w.u + tl);
    k.delta.load_global(w.delta + tl);
    k.dout.load_global(w.dout + tl);
    k.z.load_global(w.z + tl);
  };
  int npass = 0;
  while (npass < passes && d0 + npass * PASS_CH < q.dend) ++npass;
  if (npass == 0) {
    // a short workgroup whose channels all lie past the group: its partial of dB / dC is zero
    for (int64_t i = (int64_t)tid * 4; i < (int64_t)N * L; i += NTHREADS * 4) {
      *reinterpret_cast<f32x4 *>(p.dB32 + part0 * N * L + i) = f32x4{0.f, 0.f, 0.f, 0.f};
      *reinterpret_cast<f32x4 *>(p.dC32 + part0 * N * L + i) = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    return;
  }
  Rows nxt;
  fetch_rows(nxt, ntiles - 1, 0);

  for (int tile = ntiles - 1; tile >= 0; --tile) {
    const int t0 = tile * TILE4, tl = t0 + c * KI4;
    for (int r = 0; r < npass; ++r) {
      const int chw = r * PASS_CH + chl;
      const bool valid = d0 + chw < q.dend;
      const bool live = valid && tl < L;  // whole lanes only: the rows are 8-position aligned
      float u[4], dl[4], du[4], dy[4], acc[4], dd[4], y[4], dsum = 0.f, dtail = 0.f;
      const float Dd = rows[chw].D, bias = rows[chw].bias;
      {
        nxt.u.unpack(u);
        nxt.delta.unpack(dl);
        nxt.dout.unpack(dy);
#pragma unroll
        for (int i = 0; i < KI4; ++i) {
          u[i] = live ? u[i] : 0.f;
          dy[i] = live ? dy[i] : 0.f;
        }
        if (has_z) {
          float z[4];
          nxt.z.unpack(z);
#pragma unroll
          for (int i = 0; i < KI4; ++i) dy[i] *= z[i] * sigmoid_f(z[i]);
        }
#pragma unroll
        for (int i = 0; i < KI4; ++i) {
          float x = dl[i] + bias;
          if (p.delta_softplus) x = softplus_f(x);
          dl[i] = live ? x : 0.f;
          du[i] = dl[i] * u[i];
          acc[i] = 0.f;
          dd[i] = 0.f;
          y[i] = 0.f;
        }
#pragma unroll
        for (int i = 1; i < KI4; ++i) dtail += dl[i];
        dsum = dtail + dl[0];
        hcar[chl * NP + c] = (c < N && tile > 0) ? nxt.ck : 0.f;
        {
          const bool more = r + 1 < npass;
          fetch_rows(nxt, more ? tile : max(tile - 1, 0), more ? r + 1 : 0);
        }
      }
      if (r == 0) {
        lds_barrier();
        stage_bc4(Bs, Cs, Bg, p.B_ns, Cg, p.C_ns, N, t0, L, tid);
        for (int i = tid * 4; i < 2 * ACC4_FLOATS; i += NTHREADS * 4)  // dBs and dCs are adjacent
          *reinterpret_cast<f32x4 *>(dBs + i) = f32x4{0.f, 0.f, 0.f, 0.f};
        lds_barrier();
      }
      {
        // the rotation of the 8 waves over the 8 state pairs, staggered by half a phase between the two waves of a
        // workgroup that share a SIMD: as in scan_bwd_kernel
        const bool early = wave < NWAVES / 2;
        const int slot_shift = early ? 0 : NPH - 1;
        const float *A1row = A1s + chw * NP;
        const float *hrow = hcar + chl * NP;
        float *grow = gcar + chw * NP;
        float *arow = anx + chw * NP;
        float *dArow = dAacc + chw * NP;
        struct Operands {
          float A1[2], hc[2], gc[2], an[2], Bv[2][4], Cv[2][4];
        };
        auto fetch_operands = [&](Operands &o, int ph) {
          const int n = ((wave + ph + slot_shift) % NPH) * NPP;
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            o.A1[s] = A1row[n + s];
            o.hc[s] = hrow[n + s];
            o.gc[s] = grow[n + s];
            o.an[s] = arow[n + s];
            ld4(Bs + (n + s) * TILE4 + c * 4, o.Bv[s]);
            ld4(Cs + (n + s) * TILE4 + c * 4, o.Cv[s]);
          }
        };
        // (the operands of a phase are fetched at its start: a prefetch one phase ahead, as in the 8-item kernel,
        // costs registers this kernel does not have, and measured slower)
        Operands ops;
        for (int ph = 0; ph < NPH; ++ph) {
          fetch_operands(ops, ph);
          const int n = ((wave + ph + slot_shift) % NPH) * NPP;
          float A1[2], gc[2], an[2];
          float Cv[2][4], a[2][4], bb[2][4], h[2][4];
          float gfirst[2], a_next_lane[2];
          {
            float hc[2], sa[2], sb[2], hend[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
              A1[s] = ops.A1[s];
              hc[s] = ops.hc[s];
              gc[s] = ops.gc[s];
              an[s] = ops.an[s];
              const float A2 = A1[s] * kLog2e;
#pragma unroll
              for (int i = 0; i < KI4; ++i) {
                Cv[s][i] = ops.Cv[s][i];
                a[s][i] = fast_exp2(dl[i] * A2);
                bb[s][i] = du[i] * ops.Bv[s][i];
              }
              sa[s] = fast_exp2(dsum * A2);
              float hl = bb[s][0];
#pragma unroll
              for (int i = 1; i < KI4; ++i) hl = __builtin_fmaf(a[s][i], hl, bb[s][i]);
              sb[s] = hl;
            }
            row_scan_fwd2(sa[0], sb[0], sa[1], sb[1]);
#pragma unroll
            for (int s = 0; s < 2; ++s) hend[s] = __builtin_fmaf(sa[s], hc[s], sb[s]);
            float ra[2], rb[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
              float hp = dpp_f<DPP_ROW_SHR + 1>(hc[s], hend[s]);
#pragma unroll
              for (int i = 0; i < KI4; ++i) {
                hp = __builtin_fmaf(a[s][i], hp, bb[s][i]);
                h[s][i] = hp;
              }
              if (has_z) {
#pragma unroll
                for (int i = 0; i < KI4; ++i) y[i] = __builtin_fmaf(h[s][i], Cv[s][i], y[i]);
              }
              a_next_lane[s] = dpp_f<DPP_ROW_SHL + 1>(an[s], a[s][0]);
#pragma unroll
              for (int i = 0; i < KI4; ++i) Cv[s][i] *= dy[i];
              float gl = Cv[s][KI4 - 1];
#pragma unroll
              for (int i = KI4 - 2; i >= 0; --i) gl = __builtin_fmaf(a[s][i + 1], gl, Cv[s][i]);
              ra[s] = fast_exp2(dtail * (A1[s] * kLog2e)) * a_next_lane[s];
              rb[s] = gl;
            }
            row_scan_rev2(ra[0], rb[0], ra[1], rb[1]);
#pragma unroll
            for (int s = 0; s < 2; ++s) gfirst[s] = __builtin_fmaf(ra[s], gc[s], rb[s]);
          }
          if (early) lds_barrier();
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const float gx = dpp_f<DPP_ROW_SHL + 1>(gc[s], gfirst[s]);
            if (c == 0) {
              grow[n + s] = gfirst[s];
              arow[n + s] = a[s][0];
            }
            float dAp = 0.f;
            float sB[4], sC[4];
            float Bq[4];
            ld4(Bs + (n + s) * TILE4 + c * 4, Bq);
            ld4(dBs + (n + s) * ACC4_PITCH + lane * 4, sB);
            ld4(dCs + (n + s) * ACC4_PITCH + lane * 4, sC);
            float gi = gx, an_i = a_next_lane[s];
#pragma unroll
            for (int i = KI4 - 1; i >= 0; --i) {
              gi = __builtin_fmaf(an_i, gi, Cv[s][i]);
              an_i = a[s][i];
              sC[i] = __builtin_fmaf(dy[i], h[s][i], sC[i]);
              sB[i] = __builtin_fmaf(gi, du[i], sB[i]);
              acc[i] = __builtin_fmaf(gi, Bq[i], acc[i]);
              const float w = gi * (h[s][i] - bb[s][i]);  // g * a * h[t-1]
              dd[i] = __builtin_fmaf(A1[s], w, dd[i]);
              dAp = __builtin_fmaf(dl[i], w, dAp);
            }
            st4(dBs + (n + s) * ACC4_PITCH + lane * 4, sB);
            st4(dCs + (n + s) * ACC4_PITCH + lane * 4, sC);
            dAp = row_sum_to_last(dAp);
            if (c == RL - 1) dArow[n + s] += dAp;
          }
          if (!early) lds_barrier();
        }
      }
      if (r == npass - 1) {
        lds_barrier();
        // one partial per workgroup: the sum over the 4 channel slots of every (state, 4 positions)
        for (int o = tid; o < 2 * NB16 * RL; o += NTHREADS) {
          const int which = o >> 8, n = (o >> 4) & 15, q4 = o & 15;
          const float *src = (which ? dCs : dBs) + n * ACC4_PITCH + q4 * 4;
          f32x4 v = *reinterpret_cast<const f32x4 *>(src);
#pragma unroll
          for (int k = 1; k < ROWS; ++k) {
            const f32x4 w = *reinterpret_cast<const f32x4 *>(src + k * RL * 4);
            v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
          }
          const int t = t0 + 4 * q4;
          if (n >= N || t >= L) continue;
          float *dst = (which ? p.dC32 : p.dB32) + (part0 * N + n) * L + t;
          *reinterpret_cast<f32x4 *>(dst) = v;
        }
      }
      {
        float o[4];
        const BwdRow<T> w = rows[chw];
        Pack4 z_k, dout_k;
        const int tlc = min(tl, L - KI4);
        z_k.load_global(w.z + tlc);
        dout_k.load_global(w.dout + tlc);
        float dbs = 0.f, dDs = 0.f;
#pragma unroll
        for (int i = 0; i < KI4; ++i) o[i] = __builtin_fmaf(dl[i], acc[i], Dd * dy[i]);
        st4_or_spare(w.du + tl, live, spare, o);
#pragma unroll
        for (int i = 0; i < KI4; ++i) {
          float gd = __builtin_fmaf(u[i], acc[i], dd[i]);
          if (p.delta_softplus) gd *= softplus_slope_f(dl[i]);
          gd = live ? gd : 0.f;
          o[i] = gd;
          dbs += gd;
          dDs = __builtin_fmaf(dy[i], u[i], dDs);
        }
        st4_or_spare(w.ddelta + tl, live, spare, o);
        float oz[4] = {0.f, 0.f, 0.f, 0.f};
        if (has_z) {
          float z[4], dout[4];
          z_k.unpack(z);
          dout_k.unpack(dout);
#pragma unroll
          for (int i = 0; i < KI4; ++i) {
            const float yf = __builtin_fmaf(Dd, u[i], y[i]);
            const float s = sigmoid_f(z[i]);
            o[i] = dout[i] * yf * s * (1.f + z[i] * (1.f - s));
            oz[i] = yf * z[i] * s;
          }
        }
        st4_or_spare(w.dz + tl, live && has_z, spare, o);
        st4_or_spare(w.out_z + tl, live && w.out_z != nullptr, spare, oz);
        dbs = row_sum_to_last(dbs);
        dDs = row_sum_to_last(dDs);
        if (c == RL - 1) {
          dbacc[chw] += dbs;
          dDacc[chw] += dDs;
        }
      }
    }
  }
  lds_barrier();
  for (int i = tid; i < WCH * N; i += NTHREADS) {
    const int ch = i / N, n = i % N, d = d0 + ch;
    if (d >= q.dend) continue;
    p.dA_part[((int64_t)b * p.dim + d) * N + n] = dAacc[ch * NP + n];
  }
  for (int ch = tid; ch < WCH; ch += NTHREADS) {
    const int d = d0 + ch;
    if (d >= q.dend) continue;
    p.dD_part[(int64_t)b * p.dim + d] = dDacc[ch];
    p.ddelta_bias_part[(int64_t)b * p.dim + d] = dbacc[ch];
  }
}

}  // namespace k4
}  // namespace

// LDS bytes of a workgroup that takes `passes` passes.
size_t mamba1_bwd_k4_lds(int passes) {
  const int wch = passes * PASS_CH, np = NB16;
  return sizeof(float) * (2 * k4::BC4_FLOATS + 2 * k4::ACC4_FLOATS + PASS_CH * np + 4 * wch * np + 2 * wch) + (size_t)wch * 80;
}

// Whether the kernel serves the problem: bf16 rows whose 16-byte pieces are aligned (the caller checks that), a real A,
// per-position B and C, at most 16 states.
bool mamba1_bwd_k4_serves(const MambaScanParams &p) {
  return p.dtype == MAMBA_BF16 && !(p.bc_const & 3) && !p.a_complex && p.dstate <= NB16 && p.seqlen % 8 == 0;
}

bool mamba1_allow_lds(const void *kernel, size_t lds);  // mamba1_scan.hip

// pa, pb: passes of the long and the short workgroups (equal: every workgroup the same); nparts: partial sums of
// dB / dC per (batch, group), as the caller sized the workspace.
int mamba1_bwd_k4_launch(const MambaScanParams &p, int pa, int pb, int nparts, hipStream_t stream) {
  const size_t lds = mamba1_bwd_k4_lds(pa > pb ? pa : pb);
  const void *kernel = reinterpret_cast<const void *>(k4::scan_bwd_k4_kernel);
  if (!mamba1_allow_lds(kernel, lds)) return MAMBA_E_LAUNCH;
  const int Dg = p.dim / p.ngroups;
  const int blocks = pa == pb ? (Dg + PASS_CH * pa - 1) / (PASS_CH * pa)
                              : 2 * ((Dg + PASS_CH * (pa + pb) - 1) / (PASS_CH * (pa + pb)));
  dim3 grid(p.ngroups * blocks, p.batch), block(NTHREADS);
  hipLaunchKernelGGL(k4::scan_bwd_k4_kernel, grid, block, lds, stream, p, pa, pb, nparts);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}
