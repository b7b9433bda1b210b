// Mamba-1 selective scan, forward and backward, for gfx950 (wave64).
//
// Work decomposition
//   * a wave owns R channels of one (batch, group); its 64 lanes hold 64
//     consecutive 8-step segments of the sequence, i.e. one 512-step tile per
//     pass.  Lane l loads its 8 items of u/delta/z with one 16-byte access.
//   * the NW waves of a workgroup walk the tiles together and share the B and
//     C rows of the tile, staged once per tile in LDS as fp32.
//   * per state n: an 8-step in-register recurrence per lane, a DPP scan of
//     the (decay, value) pairs across the 64 lanes, and a carry from the
//     previous tile kept in LDS.
//   * the state after every tile is written to `ckpt`; the backward pass walks
//     the tiles in reverse, restarts each tile from ckpt, and runs the adjoint
//     recurrence with a lane-reversed scan.  dB/dC are summed over the
//     channels of the workgroup in LDS (waves take turns on disjoint state
//     rows; LDS float atomics are far too slow for this) and added to global
//     fp32 buffers once per tile.
#include "common.hpp"

namespace {

constexpr int KI = 8;           // items per lane
constexpr int TILE = 64 * KI;   // sequence positions per tile
constexpr int NB16 = 16;        // states staged per LDS block
constexpr int BC_FLOATS = NB16 * TILE;        // one staged tensor
constexpr int MAX_DSTATE = 256;

// B or C rows n0..n0+15 of the tile starting at t0 -> LDS as fp32, laid out
// [n][half][lane][4] so that a lane reads its 8 items with two conflict-free
// 16-byte LDS loads.
// BC: bit 0 set = B is not staged (input-independent), bit 1 = C likewise.
template <typename T, bool VEC, int NTHREADS, int BC>
DEVI void stage_bc(float *Bs, float *Cs, const T *Bg, int64_t B_ns, const T *Cg, int64_t C_ns, int n0, int N, int t0,
                   int L, int tid) {
  constexpr int FIRST = (BC & 1) ? NB16 * 64 : 0, LAST = (BC & 2) ? NB16 * 64 : 2 * NB16 * 64;
  if constexpr (BC == 3) {
    return;  // nothing is staged
  } else if constexpr (VEC) {
    // all loads first, from clamped (valid) addresses, then the masked LDS stores: a load under
    // a branch, or converted right away, would make every load wait for the one before
    constexpr int UNITS = (LAST - FIRST) / NTHREADS;
    static_assert(UNITS * NTHREADS == LAST - FIRST, "whole units per thread");
    Pack8<T> raw[UNITS];
#pragma unroll
    for (int q = 0; q < UNITS; ++q) {
      const int unit = FIRST + tid + q * NTHREADS;
      const int which = unit >> 10, n = min(n0 + ((unit >> 6) & 15), N - 1), t = min(t0 + KI * (unit & 63), L - KI);
      raw[q].load((which ? Cg + (int64_t)n * C_ns : Bg + (int64_t)n * B_ns) + t);
    }
#pragma unroll
    for (int q = 0; q < UNITS; ++q) {
      const int unit = FIRST + tid + q * NTHREADS;
      const int which = unit >> 10, n = (unit >> 6) & 15, j = unit & 63;
      float v[8];
      raw[q].unpack(v);
      const bool ok = n0 + n < N && t0 + KI * j < L;
      float *dst = (which ? Cs : Bs) + n * TILE + j * 4;
      const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
      const f32x4 lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
      *reinterpret_cast<f32x4 *>(dst) = ok ? lo : zero;
      *reinterpret_cast<f32x4 *>(dst + 256) = ok ? hi : zero;
    }
  } else {
    for (int unit = FIRST + tid; unit < LAST; unit += NTHREADS) {
      const int which = unit >> 10, n = (unit >> 6) & 15, j = unit & 63;
      const int t = t0 + KI * j;
      const T *src = (which ? Cg + (int64_t)(n0 + n) * C_ns : Bg + (int64_t)(n0 + n) * B_ns) + t;
      int nvalid = (n0 + n < N) ? min(max(L - t, 0), KI) : 0;
      float v[8];
      ld8_guard<T, false>(src, nvalid, 0.f, v);
      float *dst = (which ? Cs : Bs) + n * TILE + j * 4;
      f32x4 lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
      *reinterpret_cast<f32x4 *>(dst) = lo;
      *reinterpret_cast<f32x4 *>(dst + 256) = hi;
    }
  }
}

// The 8 items of one (batch, channel) row owned by this lane, as stored: VEC reads 16 bytes from a
// clamped position (the caller masks lanes past the end), else element by element.
template <typename T, bool VEC> DEVI void load_items(Pack8<T> &k, const T *row, int tl, int L, int nvalid) {
  if constexpr (VEC) {
    k.load(row + min(tl, L - KI));
  } else {
    float v[8];
    ld8_guard<T, false>(row + tl, nvalid, 0.f, v);
    k.pack(v);
  }
}

DEVI void lds_st8(float *base, int lane, const float (&v)[8]) {
  f32x4 lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
  *reinterpret_cast<f32x4 *>(base + lane * 4) = lo;
  *reinterpret_cast<f32x4 *>(base + 256 + lane * 4) = hi;
}

DEVI void lds_ld8(const float *base, int lane, float (&o)[8]) {
  f32x4 lo = *reinterpret_cast<const f32x4 *>(base + lane * 4);
  f32x4 hi = *reinterpret_cast<const f32x4 *>(base + 256 + lane * 4);
  o[0] = lo.x; o[1] = lo.y; o[2] = lo.z; o[3] = lo.w;
  o[4] = hi.x; o[5] = hi.y; o[6] = hi.z; o[7] = hi.w;
}

// The 8 items of B (or C) for state n of channel d: from the staged tile, or, when the operand is an
// input-independent (dim, dstate) fp32 matrix, its one value for every position (0 for padded states).
template <int CONST>
DEVI void load_bc(float (&v)[8], const float *staged, const void *mat, int d, int N, int n_abs, int n_loc, int lane) {
  if constexpr (CONST != 0) {
    const float c = n_abs < N ? static_cast<const float *>(mat)[(int64_t)d * N + n_abs] : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = c;
  } else {
    lds_ld8(staged + n_loc * TILE, lane, v);
  }
}

// ------------------------------------------------------------------ forward
// BC: bit 0 = B is an input-independent (dim, dstate) fp32 matrix, bit 1 = C likewise
// (selective_scan_fwd_kernel.cuh:74 kIsVariableB / kIsVariableC false).
template <typename T, int NW, int R, bool VEC, int BC>
__global__ __launch_bounds__(NW * 64, 4) void scan_fwd_kernel(const MambaScanParams p) {
  extern __shared__ __align__(16) float smem[];
  const int N = p.dstate, L = p.seqlen;
  const int NBLK = (N + NB16 - 1) / NB16, NP = NBLK * NB16;
  float *Bs = smem;
  float *Cs = Bs + BC_FLOATS;
  float *A2s = Cs + BC_FLOATS;       // [NW*R][NP]  A * log2(e)
  float *hcar = A2s + NW * R * NP;   // [NW*R][NP]  state carried across tiles

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int Dg = p.dim / p.ngroups;
  const int cblocks = (Dg + NW * R - 1) / (NW * R);
  const int g = blockIdx.x / cblocks, cb = blockIdx.x % cblocks;
  const int b = blockIdx.y;
  const int dbase = g * Dg + cb * NW * R + wave * R;
  const int dend = (g + 1) * Dg;
  const int ntiles = (L + TILE - 1) / TILE;

  const T *Bg = (const T *)p.B + b * p.B_bs + g * p.B_gs;
  const T *Cg = (const T *)p.C + b * p.C_bs + g * p.C_gs;
  const float *Ag = (const float *)p.A;

  for (int i = lane; i < R * NP; i += 64) {
    const int r = i / NP, n = i % NP, d = dbase + r;
    A2s[wave * R * NP + i] = (d < dend && n < N) ? Ag[(int64_t)d * N + n] * kLog2e : 0.f;
    hcar[wave * R * NP + i] = 0.f;
  }

  for (int tile = 0; tile < ntiles; ++tile) {
    const int t0 = tile * TILE, tl = t0 + lane * KI;
    const int nvalid = min(max(L - tl, 0), KI);
    for (int r = 0; r < R; ++r) {
      const int d = dbase + r;
      const bool valid = d < dend;
      float u[8], dl[8], du[8], y[8], dsum = 0.f;
      Pack8<T> ku, kd, kz;  // raw rows: every load is issued before the first conversion
      kz.zero();
      // lane states of this (tile, channel), when the caller keeps them for the backward pass
      float *lanes = (p.lane_state && valid) ? p.lane_state + (((int64_t)b * p.dim + d) * ntiles + tile) * N * 64 : nullptr;
      if (valid) {
        load_items<T, VEC>(ku, (const T *)p.u + b * p.u_bs + d * p.u_ds, tl, L, nvalid);
        load_items<T, VEC>(kd, (const T *)p.delta + b * p.delta_bs + d * p.delta_ds, tl, L, nvalid);
        if (p.z) load_items<T, VEC>(kz, (const T *)p.z + b * p.z_bs + d * p.z_ds, tl, L, nvalid);
        const float bias = p.delta_bias ? ((const float *)p.delta_bias)[d] : 0.f;
        ku.unpack(u);
        kd.unpack(dl);
#pragma unroll
        for (int i = 0; i < KI; ++i) {
          float x = dl[i] + bias;
          if (p.delta_softplus) x = softplus_f(x);
          dl[i] = (i < nvalid) ? x : 0.f;
          u[i] = (i < nvalid) ? u[i] : 0.f;
          du[i] = dl[i] * u[i];
          y[i] = 0.f;
        }
#pragma unroll
        for (int i = 0; i < KI; ++i) dsum += dl[i];
      }
      for (int nb = 0; nb < NBLK; ++nb) {
        if (BC != 3 && (NBLK > 1 || r == 0)) {
          __syncthreads();
          stage_bc<T, VEC, NW * 64, BC>(Bs, Cs, Bg, p.B_ns, Cg, p.C_ns, nb * NB16, N, t0, L, tid);
          __syncthreads();
        }
        if (valid) {
          const float *A2row = A2s + (wave * R + r) * NP + nb * NB16;
          float *hrow = hcar + (wave * R + r) * NP + nb * NB16;
          const int nmax = min(NB16, N - nb * NB16);
          // two states per iteration: their wave scans are interleaved (padded rows are inert:
          // A = 0, B = C = 0)
          for (int n = 0; n < nmax; n += 2) {
            // Pass 1 runs the lane's 8 steps from a zero state to get the lane's (decay, value) pair;
            // the decay over the lane is one exp of the summed delta instead of 7 products. Pass 2
            // reruns the 8 steps from the state the wave scan gives this lane.
            float a[2][8], bb[2][8], Cv[2][8], hc[2];
            float sa[2], sb[2];
#pragma unroll
            for (int q = 0; q < 2; ++q) {
              const float A2 = A2row[n + q];
              hc[q] = hrow[n + q];
              float Bv[8];
              load_bc<BC & 1>(Bv, Bs, p.B, d, N, nb * NB16 + n + q, n + q, lane);
              load_bc<BC & 2>(Cv[q], Cs, p.C, d, N, nb * NB16 + n + q, n + q, lane);
              sa[q] = fast_exp2(dsum * A2);
#pragma unroll
              for (int i = 0; i < KI; ++i) {
                a[q][i] = fast_exp2(dl[i] * A2);
                bb[q][i] = du[i] * Bv[i];
              }
              float hl = bb[q][0];
#pragma unroll
              for (int i = 1; i < KI; ++i) hl = __builtin_fmaf(a[q][i], hl, bb[q][i]);
              sb[q] = hl;
            }
            wave_scan_fwd2(sa[0], sb[0], sa[1], sb[1]);
            const float hend[2] = {__builtin_fmaf(sa[0], hc[0], sb[0]), __builtin_fmaf(sa[1], hc[1], sb[1])};
#pragma unroll
            for (int q = 0; q < 2; ++q) {
              float h = dpp_f<DPP_WAVE_SHR1>(hc[q], hend[q]);  // state entering this lane
              if (lane == 63) hrow[n + q] = hend[q];           // state after the tile
              if (lanes && nb * NB16 + n + q < N) lanes[(nb * NB16 + n + q) * 64 + lane] = h;
#pragma unroll
              for (int i = 0; i < KI; ++i) {
                h = __builtin_fmaf(a[q][i], h, bb[q][i]);
                y[i] = __builtin_fmaf(h, Cv[q][i], y[i]);
              }
            }
          }
        }
      }
      if (valid) {
        if (p.D) {
          const float Dd = ((const float *)p.D)[d];
#pragma unroll
          for (int i = 0; i < KI; ++i) y[i] = __builtin_fmaf(Dd, u[i], y[i]);
        }
        if (p.z) {
          float z[8];
          kz.unpack(z);
#pragma unroll
          for (int i = 0; i < KI; ++i) y[i] *= z[i] * sigmoid_f(z[i]);
        }
        st8_guard<T, VEC>((T *)p.out + b * p.out_bs + d * p.out_ds + tl, nvalid, y);
        float *ck = p.ckpt + (((int64_t)b * p.dim + d) * ntiles + tile) * N;
        const float *hfin = hcar + (wave * R + r) * NP;
        for (int n = lane; n < N; n += 64) ck[n] = hfin[n];
      }
    }
  }
}

// ----------------------------------------------------------------- backward
// Row starts of one channel of the workgroup, kept in LDS: every (tile, channel) step needs nine
// addresses, and as scalars next to the loop state they did not fit the scalar registers (each step
// then re-read some 250 spilled scalars through v_readlane).
template <typename T> struct BwdRow {
  const T *u, *delta, *dout, *z;
  T *du, *ddelta, *dz, *out_z;
  const float *ckpt;  // tile 0 of this channel: the tile checkpoints, or with LS the lane states
  float D, bias;
};

// LS: the forward pass left the state entering every lane's 8 positions (lane_state); the states of a
// tile are then re-computed from those directly, without the lane-local pass and the wave scan.
template <typename T, int NW, int R, bool VEC, int BC, bool LS>
__global__ __launch_bounds__(NW * 64) void scan_bwd_kernel(const MambaScanParams p) {
  static_assert(sizeof(BwdRow<T>) == 80, "the host side sizes the LDS table with 80 bytes per channel");
  extern __shared__ __align__(16) float smem[];
  const int N = p.dstate, L = p.seqlen;
  const int NBLK = (N + NB16 - 1) / NB16, NP = NBLK * NB16;
  constexpr int WR = NW * R;
  float *Bs = smem;
  float *Cs = Bs + BC_FLOATS;
  float *dBs = Cs + BC_FLOATS;        // fp32 sums over the workgroup's channels, same layout as Bs
  float *dCs = dBs + BC_FLOATS;
  float *A1s = dCs + BC_FLOATS;       // [WR][NP] A
  float *hcar = A1s + WR * NP;        // state entering the tile (from ckpt)
  float *gcar = hcar + WR * NP;       // adjoint at the first position of the following tile
  float *anx = gcar + WR * NP;        // decay at the first position of the following tile
  float *dAacc = anx + WR * NP;       // [WR][NP]
  float *dDacc = dAacc + WR * NP;     // [WR]
  float *dbacc = dDacc + WR;          // [WR]
  float *dBcacc = dbacc + WR;         // [WR][NP] gradients of input-independent B / C
  float *dCcacc = dBcacc + WR * NP;
  BwdRow<T> *rows = reinterpret_cast<BwdRow<T> *>(dCcacc + WR * NP);  // [WR]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int Dg = p.dim / p.ngroups;
  const int cblocks = (Dg + WR - 1) / WR;
  const int g = blockIdx.x / cblocks, cb = blockIdx.x % cblocks;
  const int b = blockIdx.y;
  const int dbase = g * Dg + cb * WR + wave * R;
  const int dend = (g + 1) * Dg;
  const int ntiles = (L + TILE - 1) / TILE;
  const bool has_z = p.z != nullptr;
  if (lane < R) {  // each wave fills and reads only its own rows
    const int d = min(dbase + lane, dend - 1);
    BwdRow<T> q;
    q.u = (const T *)p.u + b * p.u_bs + d * p.u_ds;
    q.delta = (const T *)p.delta + b * p.delta_bs + d * p.delta_ds;
    q.dout = (const T *)p.dout + b * p.dout_bs + d * p.dout_ds;
    q.z = has_z ? (const T *)p.z + b * p.z_bs + d * p.z_ds : nullptr;
    q.du = (T *)p.du + b * p.du_bs + d * p.du_ds;
    q.ddelta = (T *)p.ddelta + b * p.ddelta_bs + d * p.ddelta_ds;
    q.dz = has_z ? (T *)p.dz + b * p.dz_bs + d * p.dz_ds : nullptr;
    q.out_z = (has_z && p.out_z) ? (T *)p.out_z + b * p.outz_bs + d * p.outz_ds : nullptr;
    q.ckpt = LS ? p.lane_state + ((int64_t)b * p.dim + d) * ntiles * N * 64 : p.ckpt + ((int64_t)b * p.dim + d) * ntiles * N;
    q.D = p.D ? ((const float *)p.D)[d] : 0.f;
    q.bias = p.delta_bias ? ((const float *)p.delta_bias)[d] : 0.f;
    rows[wave * R + lane] = q;
  }

  const T *Bg = (const T *)p.B + b * p.B_bs + g * p.B_gs;
  const T *Cg = (const T *)p.C + b * p.C_bs + g * p.C_gs;
  const float *Ag = (const float *)p.A;
  float *dBg = p.dB32 + ((int64_t)b * p.ngroups + g) * N * L;
  float *dCg = p.dC32 + ((int64_t)b * p.ngroups + g) * N * L;

  for (int i = lane; i < R * NP; i += 64) {
    const int r = i / NP, n = i % NP, d = dbase + r;
    const int o = wave * R * NP + i;
    A1s[o] = (d < dend && n < N) ? Ag[(int64_t)d * N + n] : 0.f;
    gcar[o] = 0.f;
    anx[o] = 0.f;
    dAacc[o] = 0.f;
    dBcacc[o] = 0.f;
    dCcacc[o] = 0.f;
  }
  if (lane < R) {
    dDacc[wave * R + lane] = 0.f;
    dbacc[wave * R + lane] = 0.f;
  }

  // The rows of the next (tile, channel) are fetched while the current one is computed.
  constexpr int NPP = NB16 / NW > 0 ? NB16 / NW : 1;  // state rows per wave and phase (see the state loop)
  constexpr int NPH = NB16 / NPP;
  constexpr int Q = NPP >= 2 ? 2 : 1;                 // states per step; two keep two scan chains in flight
  struct Rows {
    Pack8<T> u, delta, dout, z;
    float ck;     // !LS: checkpointed state n = lane entering the tile (when the padded state count fits a wave)
    float h0[Q];  // LS: lane states of the first step's states
  };
  // lane states of step (nb, ph, j) of a (tile, channel): rows past N read a clamped row and are never used
  auto lane_states = [&](const float *tile_base, int nb, int ph, int j, float (&o)[Q]) {
    const int n = nb * NB16 + ((wave + ph) % NPH) * NPP + j;
#pragma unroll
    for (int q = 0; q < Q; ++q) o[q] = tile_base[(int64_t)min(n + q, N - 1) * 64 + lane];
  };
  auto fetch_rows = [&](Rows &k, int tile, int r) {
    const int d = dbase + r, tl = tile * TILE + lane * KI;
    const int nvalid = min(max(L - tl, 0), KI);
    k.z.zero();
    k.ck = 0.f;
#pragma unroll
    for (int q = 0; q < Q; ++q) k.h0[q] = 0.f;
    if (d < dend) {
      const BwdRow<T> &q = rows[wave * R + r];
      if constexpr (LS) lane_states(q.ckpt + (int64_t)tile * N * 64, 0, 0, 0, k.h0);
      else if (NP <= 64 && tile > 0 && lane < N) k.ck = q.ckpt[(int64_t)(tile - 1) * N + lane];
      load_items<T, VEC>(k.u, q.u, tl, L, nvalid);
      load_items<T, VEC>(k.delta, q.delta, tl, L, nvalid);
      load_items<T, VEC>(k.dout, q.dout, tl, L, nvalid);
      if (has_z) load_items<T, VEC>(k.z, q.z, tl, L, nvalid);
    }
  };
  Rows nxt;
  fetch_rows(nxt, ntiles - 1, 0);

  for (int tile = ntiles - 1; tile >= 0; --tile) {
    const int t0 = tile * TILE, tl = t0 + lane * KI;
    const int nvalid = min(max(L - tl, 0), KI);
    for (int r = 0; r < R; ++r) {
      const int d = dbase + r;
      const bool valid = d < dend;
      const int row = wave * R + r;
      float u[8], dl[8], du[8], dy[8], acc[8], dd[8], y[8], dsum = 0.f, dtail = 0.f;
      // raw delta, z and dout stay in registers in their storage format for the epilogue
      const Rows cur = nxt;
      float hnext[Q];  // LS: lane states of the step about to run
#pragma unroll
      for (int q = 0; q < Q; ++q) hnext[q] = cur.h0[q];
      Pack8<T> draw_k = cur.delta, z_k = cur.z, dout_k = cur.dout;
      if (r + 1 < R) fetch_rows(nxt, tile, r + 1);
      else if (tile > 0) fetch_rows(nxt, tile - 1, 0);
      float Dd = 0.f;
      if (valid) {
        Dd = rows[row].D;
        const Pack8<T> u_k = cur.u;
        const float bias = rows[row].bias;
        u_k.unpack(u);
        draw_k.unpack(dl);
        dout_k.unpack(dy);
#pragma unroll
        for (int i = 0; i < KI; ++i) {  // lanes past the end read a clamped position: mask them
          u[i] = (i < nvalid) ? u[i] : 0.f;
          dy[i] = (i < nvalid) ? dy[i] : 0.f;
        }
        if (has_z) {
          float z[8];
          z_k.unpack(z);
#pragma unroll
          for (int i = 0; i < KI; ++i) dy[i] *= z[i] * sigmoid_f(z[i]);
        }
#pragma unroll
        for (int i = 0; i < KI; ++i) {
          float x = dl[i] + bias;
          if (p.delta_softplus) x = softplus_f(x);
          dl[i] = (i < nvalid) ? x : 0.f;
          du[i] = dl[i] * u[i];
          acc[i] = 0.f;
          dd[i] = 0.f;
          y[i] = 0.f;
        }
        dtail = 0.f;
#pragma unroll
        for (int i = 1; i < KI; ++i) dtail += dl[i];
        dsum = dtail + dl[0];
        // state entering this tile
        if constexpr (LS) {
        } else if (NP <= 64) {
          if (lane < NP) hcar[row * NP + lane] = cur.ck;
        } else {
          for (int n = lane; n < NP; n += 64) {
            float v = 0.f;
            if (tile > 0 && n < N) v = rows[row].ckpt[(int64_t)(tile - 1) * N + n];
            hcar[row * NP + n] = v;
          }
        }
      }
      for (int nb = 0; nb < NBLK; ++nb) {
        if (BC != 3 && (NBLK > 1 || r == 0)) {
          __syncthreads();
          stage_bc<T, VEC, NW * 64, BC>(Bs, Cs, Bg, p.B_ns, Cg, p.C_ns, nb * NB16, N, t0, L, tid);
          for (int i = tid * 4; i < 2 * BC_FLOATS; i += NW * 256)  // dBs and dCs are adjacent
            *reinterpret_cast<f32x4 *>(dBs + i) = f32x4{0.f, 0.f, 0.f, 0.f};
          __syncthreads();
        }
        {
          // The NW waves add their channels' dB/dC terms into the shared LDS sums without
          // atomics: in phase ph wave w owns state rows (w + ph) % NPH * NPP .. + NPP - 1,
          // so no two waves touch a row between two barriers.
          static_assert(NW <= NPH, "one row slot per wave and phase");
          const float *A1row = A1s + row * NP + nb * NB16;
          const float *hrow = hcar + row * NP + nb * NB16;
          float *grow = gcar + row * NP + nb * NB16;
          float *arow = anx + row * NP + nb * NB16;
          float *dArow = dAacc + row * NP + nb * NB16;
          const int nmax = min(NB16, N - nb * NB16);
          static_assert(NPP % Q == 0, "whole steps per phase");
          for (int ph = 0; ph < NPH; ++ph) {
            const int slot = (wave + ph) % NPH;
            for (int j = 0; j < NPP; j += Q) {
              const int n = slot * NPP + j;
              float hin[Q];
              if constexpr (LS) {
                // this step's lane states arrived during the previous step (the first step's with the rows);
                // the next step's are requested now
#pragma unroll
                for (int q = 0; q < Q; ++q) hin[q] = hnext[q];
                int j2 = j + Q, ph2 = ph, nb2 = nb;
                if (j2 >= NPP) { j2 = 0; ++ph2; }
                if (ph2 >= NPH) { ph2 = 0; ++nb2; }
                if (valid && nb2 < NBLK) lane_states(rows[row].ckpt + (int64_t)tile * N * 64, nb2, ph2, j2, hnext);
              }
              if (!valid || n >= nmax) continue;
              // Forward states: pass 1 runs the lane's 8 steps from zero for the lane's (decay, value)
              // pair, the decay being one exp of the summed delta; pass 2 reruns them from the state
              // the wave scan gives this lane. The adjoint is handled the same way in reverse.
              float A1[Q], hc[Q], gc[Q], an[Q];
              float Cv[Q][8], a[Q][8], bb[Q][8], h[Q][8];
              float sa[Q], sb[Q], hend[Q];
#pragma unroll
              for (int q = 0; q < Q; ++q) {
                A1[q] = A1row[n + q];
                hc[q] = LS ? 0.f : hrow[n + q];
                gc[q] = grow[n + q];
                an[q] = arow[n + q];
                float Bv[8];  // read again for the last loop: 16 registers fewer held through the scans
                load_bc<BC & 1>(Bv, Bs, p.B, d, N, nb * NB16 + n + q, n + q, lane);
                load_bc<BC & 2>(Cv[q], Cs, p.C, d, N, nb * NB16 + n + q, n + q, lane);
                const float A2 = A1[q] * kLog2e;
#pragma unroll
                for (int i = 0; i < KI; ++i) {
                  a[q][i] = fast_exp2(dl[i] * A2);
                  bb[q][i] = du[i] * Bv[i];
                }
                if constexpr (!LS) {
                  sa[q] = fast_exp2(dsum * A2);
                  float hl = bb[q][0];
#pragma unroll
                  for (int i = 1; i < KI; ++i) hl = __builtin_fmaf(a[q][i], hl, bb[q][i]);
                  sb[q] = hl;
                }
              }
              if constexpr (!LS) {
                if constexpr (Q == 2) wave_scan_fwd2(sa[0], sb[0], sa[1], sb[1]);
                else wave_scan_fwd(sa[0], sb[0]);
#pragma unroll
                for (int q = 0; q < Q; ++q) hend[q] = __builtin_fmaf(sa[q], hc[q], sb[q]);
              }
              float ra[Q], rb[Q], gfirst[Q], a_next_lane[Q];
#pragma unroll
              for (int q = 0; q < Q; ++q) {
                float hp;
                if constexpr (LS) hp = hin[q];
                else hp = dpp_f<DPP_WAVE_SHR1>(hc[q], hend[q]);
#pragma unroll
                for (int i = 0; i < KI; ++i) {
                  hp = __builtin_fmaf(a[q][i], hp, bb[q][i]);
                  h[q][i] = hp;  // true states
                }
                if (has_z) {
#pragma unroll
                  for (int i = 0; i < KI; ++i) y[i] = __builtin_fmaf(h[q][i], Cv[q][i], y[i]);
                }
                // adjoint recurrence g[t] = dy[t] C[t] + a[t+1] g[t+1]; Cv becomes dy * C
                a_next_lane[q] = dpp_f<DPP_WAVE_SHL1>(an[q], a[q][0]);
#pragma unroll
                for (int i = 0; i < KI; ++i) Cv[q][i] *= dy[i];
                float gl = Cv[q][KI - 1];
#pragma unroll
                for (int i = KI - 2; i >= 0; --i) gl = __builtin_fmaf(a[q][i + 1], gl, Cv[q][i]);
                ra[q] = fast_exp2(dtail * (A1[q] * kLog2e)) * a_next_lane[q];
                rb[q] = gl;
              }
              if constexpr (Q == 2) {
                row_scan_rev2(ra[0], rb[0], ra[1], rb[1]);
                wave_scan_rev_finish(ra[0], rb[0], lane);
                wave_scan_rev_finish(ra[1], rb[1], lane);
              } else {
                wave_scan_rev(ra[0], rb[0], lane);
              }
#pragma unroll
              for (int q = 0; q < Q; ++q) gfirst[q] = __builtin_fmaf(ra[q], gc[q], rb[q]);
#pragma unroll
              for (int q = 0; q < Q; ++q) {
                const float gx = dpp_f<DPP_WAVE_SHL1>(gc[q], gfirst[q]);  // adjoint at the next lane's first item
                if (lane == 0) {
                  grow[n + q] = gfirst[q];
                  arow[n + q] = a[q][0];
                }
                float dAp = 0.f, dBp = 0.f, dCp = 0.f;
                float sB[8], sC[8], Bv[8];
                load_bc<BC & 1>(Bv, Bs, p.B, d, N, nb * NB16 + n + q, n + q, lane);
                if constexpr (!(BC & 1)) lds_ld8(dBs + (n + q) * TILE, lane, sB);
                if constexpr (!(BC & 2)) lds_ld8(dCs + (n + q) * TILE, lane, sC);
                float gi = gx, an_i = a_next_lane[q];
#pragma unroll
                for (int i = KI - 1; i >= 0; --i) {
                  gi = __builtin_fmaf(an_i, gi, Cv[q][i]);
                  an_i = a[q][i];
                  if constexpr (BC & 2) dCp = __builtin_fmaf(dy[i], h[q][i], dCp);
                  else sC[i] = __builtin_fmaf(dy[i], h[q][i], sC[i]);
                  if constexpr (BC & 1) dBp = __builtin_fmaf(gi, du[i], dBp);
                  else sB[i] = __builtin_fmaf(gi, du[i], sB[i]);
                  acc[i] = __builtin_fmaf(gi, Bv[i], acc[i]);
                  const float w = gi * (h[q][i] - bb[q][i]);  // g * a * h[t-1]
                  dd[i] = __builtin_fmaf(A1[q], w, dd[i]);
                  dAp = __builtin_fmaf(dl[i], w, dAp);
                }
                if constexpr (!(BC & 1)) lds_st8(dBs + (n + q) * TILE, lane, sB);
                if constexpr (!(BC & 2)) lds_st8(dCs + (n + q) * TILE, lane, sC);
                dAp = wave_sum_to_last(dAp);
                if (lane == 63) dArow[n + q] += dAp;  // the row belongs to this wave alone
                if constexpr (BC & 1) {
                  dBp = wave_sum_to_last(dBp);
                  if (lane == 63) dBcacc[row * NP + nb * NB16 + n + q] += dBp;
                }
                if constexpr (BC & 2) {
                  dCp = wave_sum_to_last(dCp);
                  if (lane == 63) dCcacc[row * NP + nb * NB16 + n + q] += dCp;
                }
              }
            }
            __syncthreads();
          }
        }
        if (BC != 3 && (NBLK > 1 || r == R - 1)) {
          const int n0 = nb * NB16;
          constexpr int FIRST = (BC & 1) ? NB16 * TILE : 0, LAST = (BC & 2) ? NB16 * TILE : 2 * NB16 * TILE;
          for (int i = FIRST + tid; i < LAST; i += NW * 64) {
            const int which = i >> 13, n = (i >> 9) & 15, t = i & (TILE - 1);
            const float v = (which ? dCs : dBs)[n * TILE + ((t >> 2) & 1) * 256 + (t >> 3) * 4 + (t & 3)];
            if (n0 + n < N && t0 + t < L) unsafeAtomicAdd((which ? dCg : dBg) + (int64_t)(n0 + n) * L + t0 + t, v);
          }
        }
      }
      if (valid) {
        float draw[8], o[8];
        draw_k.unpack(draw);
        const BwdRow<T> q = rows[row];
        const float bias = q.bias;
        float dbs = 0.f, dDs = 0.f;
#pragma unroll
        for (int i = 0; i < KI; ++i) o[i] = __builtin_fmaf(dl[i], acc[i], Dd * dy[i]);
        st8_guard<T, VEC>(q.du + tl, nvalid, o);
#pragma unroll
        for (int i = 0; i < KI; ++i) {
          const float x = draw[i] + bias;
          float gd = __builtin_fmaf(u[i], acc[i], dd[i]);
          if (p.delta_softplus && x <= 20.f) gd *= sigmoid_f(x);
          gd = (i < nvalid) ? gd : 0.f;
          o[i] = gd;
          dbs += gd;
          dDs = __builtin_fmaf(dy[i], u[i], dDs);
        }
        st8_guard<T, VEC>(q.ddelta + tl, nvalid, o);
        if (has_z) {
          float z[8], dout[8], oz[8];
          z_k.unpack(z);
          dout_k.unpack(dout);
#pragma unroll
          for (int i = 0; i < KI; ++i) {
            const float yf = __builtin_fmaf(Dd, u[i], y[i]);
            const float s = sigmoid_f(z[i]);
            o[i] = dout[i] * yf * s * (1.f + z[i] * (1.f - s));
            oz[i] = yf * z[i] * s;
          }
          st8_guard<T, VEC>(q.dz + tl, nvalid, o);
          if (q.out_z) st8_guard<T, VEC>(q.out_z + tl, nvalid, oz);
        }
        dbs = wave_sum_to_last(dbs);
        dDs = wave_sum_to_last(dDs);
        if (lane == 63) {
          dbacc[row] += dbs;
          dDacc[row] += dDs;
        }
      }
    }
  }
  // per-(batch, channel) partial sums; the caller reduces over batch
  for (int r = 0; r < R; ++r) {
    const int d = dbase + r;
    if (d >= dend) continue;
    const int row = wave * R + r;
    for (int n = lane; n < N; n += 64) {
      p.dA_part[((int64_t)b * p.dim + d) * N + n] = dAacc[row * NP + n];
      if constexpr (BC & 1) p.dB32[((int64_t)b * p.dim + d) * N + n] = dBcacc[row * NP + n];
      if constexpr (BC & 2) p.dC32[((int64_t)b * p.dim + d) * N + n] = dCcacc[row * NP + n];
    }
    if (lane == 0) {
      p.dD_part[(int64_t)b * p.dim + d] = dDacc[row];
      p.ddelta_bias_part[(int64_t)b * p.dim + d] = dbacc[row];
    }
  }
}

// ------------------------------------------------------------------ launch
inline bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

struct Cfg {
  int nw, r;
};

inline size_t fwd_lds(int nw, int r, int np) { return sizeof(float) * (2 * BC_FLOATS + 2 * nw * r * np); }
inline size_t bwd_lds(int nw, int r, int np) {
  return sizeof(float) * (4 * BC_FLOATS + 7 * nw * r * np + 2 * nw * r) + (size_t)nw * r * 80;  // + BwdRow per channel
}

template <typename KernelT>
int launch(KernelT kernel, const MambaScanParams &p, int nw, int r, size_t lds, hipStream_t stream) {
  const int Dg = p.dim / p.ngroups;
  const int cblocks = (Dg + nw * r - 1) / (nw * r);
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)lds) != hipSuccess) {
    (void)hipGetLastError();
    return MAMBA_E_LAUNCH;
  }
  dim3 grid(p.ngroups * cblocks, p.batch), block(nw * 64);
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

int check_common(const MambaScanParams *p) {
  if (!p || !p->u || !p->delta || !p->A || !p->B || !p->C || !p->ckpt) return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->dim <= 0 || p->seqlen <= 0 || p->dstate <= 0 || p->ngroups <= 0) return MAMBA_E_BADARG;
  if (p->dim % p->ngroups != 0) return MAMBA_E_BADARG;
  if (p->batch > 65535) return MAMBA_E_UNSUPPORTED;
  if (p->dstate > MAX_DSTATE) return MAMBA_E_UNSUPPORTED;
  if (p->dtype != MAMBA_F32 && p->dtype != MAMBA_BF16 && p->dtype != MAMBA_F16) return MAMBA_E_BADARG;
  return MAMBA_OK;
}

// 16-byte accesses need every row start aligned and whole 8-item groups.
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

template <typename T, bool BWD, int BC> int dispatch_bc(const MambaScanParams &p, hipStream_t stream) {
  const int np = (p.dstate + NB16 - 1) / NB16 * NB16;
  const bool vec = vec_ok(p, BWD);
  const bool small = p.dstate <= NB16;
  if (!BWD) {
    if (small) {
      const size_t lds = fwd_lds(8, 4, np);
      return vec ? launch(scan_fwd_kernel<T, 8, 4, true, BC>, p, 8, 4, lds, stream)
                 : launch(scan_fwd_kernel<T, 8, 4, false, BC>, p, 8, 4, lds, stream);
    }
    const size_t lds = fwd_lds(8, 1, np);
    return vec ? launch(scan_fwd_kernel<T, 8, 1, true, BC>, p, 8, 1, lds, stream)
               : launch(scan_fwd_kernel<T, 8, 1, false, BC>, p, 8, 1, lds, stream);
  } else {
    if (small) {
      const size_t lds = bwd_lds(8, 4, np);
      if (p.lane_state)
        return vec ? launch(scan_bwd_kernel<T, 8, 4, true, BC, true>, p, 8, 4, lds, stream)
                   : launch(scan_bwd_kernel<T, 8, 4, false, BC, true>, p, 8, 4, lds, stream);
      return vec ? launch(scan_bwd_kernel<T, 8, 4, true, BC, false>, p, 8, 4, lds, stream)
                 : launch(scan_bwd_kernel<T, 8, 4, false, BC, false>, p, 8, 4, lds, stream);
    }
    const size_t lds = bwd_lds(4, 1, np);
    if (p.lane_state)
      return vec ? launch(scan_bwd_kernel<T, 4, 1, true, BC, true>, p, 4, 1, lds, stream)
                 : launch(scan_bwd_kernel<T, 4, 1, false, BC, true>, p, 4, 1, lds, stream);
    return vec ? launch(scan_bwd_kernel<T, 4, 1, true, BC, false>, p, 4, 1, lds, stream)
               : launch(scan_bwd_kernel<T, 4, 1, false, BC, false>, p, 4, 1, lds, stream);
  }
}

template <typename T, bool BWD> int dispatch(const MambaScanParams &p, hipStream_t stream) {
  switch (p.bc_const & 3) {
    case 0: return dispatch_bc<T, BWD, 0>(p, stream);
    case 1: return dispatch_bc<T, BWD, 1>(p, stream);
    case 2: return dispatch_bc<T, BWD, 2>(p, stream);
    default: return dispatch_bc<T, BWD, 3>(p, stream);
  }
}

}  // namespace

int mamba1_scan_complex(const MambaScanParams *p, hipStream_t s, bool bwd);  // mamba1_scan_complex.hip

extern "C" int mamba1_scan_fwd(const MambaScanParams *p, mamba_stream_t stream) {
  int rc = check_common(p);
  if (rc != MAMBA_OK) return rc;
  if (!p->out) return MAMBA_E_BADARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (p->a_complex) return mamba1_scan_complex(p, s, false);
  switch (p->dtype) {
    case MAMBA_F32: return dispatch<float, false>(*p, s);
    case MAMBA_BF16: return dispatch<bf16_t, false>(*p, s);
    default: return dispatch<f16_t, false>(*p, s);
  }
}

// ----------------------------------------------------- forward without a caller workspace
// The tile checkpoints of mamba1_scan_fwd_noalloc live in this array instead of a caller buffer.
// Host code never uses the array's name as an address: the device address is looked up once per
// device with hipGetSymbolAddress and kept in g_scratch_ptr.
constexpr int64_t SCRATCH_FLOATS = (int64_t)MAMBA_NOALLOC_SCRATCH_BYTES / 4;
constexpr int SCRATCH_MAX_DEVICES = 64;
static __device__ __align__(256) float scratch[SCRATCH_FLOATS];
static float *g_scratch_ptr[SCRATCH_MAX_DEVICES];  // per device, null until resolved

namespace {
// Device address of `scratch` on the current device (resolved on first use), or null on failure.
float *scratch_for_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SCRATCH_MAX_DEVICES) {
    (void)hipGetLastError();
    return nullptr;
  }
  float *ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (ptr) return ptr;
  if (hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
    (void)hipGetLastError();
    return nullptr;
  }
  __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
  return ptr;
}

// last_state[b, d, :] = ckpt[b, d, ntiles - 1, :]; `width` floats per (b, d) row (dstate, or 2 * dstate
// for a complex state).
__global__ __launch_bounds__(256) void gather_last_state_kernel(const float *__restrict__ ckpt, float *__restrict__ last,
                                                                int64_t rows, int ntiles, int width) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * width) return;
  const int64_t row = i / width;
  const int n = (int)(i - row * width);
  last[i] = ckpt[(row * ntiles + (ntiles - 1)) * width + n];
}
}  // namespace

extern "C" int mamba_hip_init(void) { return scratch_for_current_device() ? MAMBA_OK : MAMBA_E_LAUNCH; }

extern "C" int mamba1_scan_fwd_noalloc(const MambaScanParams *p, float *last_state, mamba_stream_t stream) {
  if (!p) return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->dim <= 0 || p->seqlen <= 0 || p->dstate <= 0) return MAMBA_E_BADARG;
  const int ntiles = (p->seqlen + TILE - 1) / TILE;
  const int width = p->dstate * (p->a_complex ? 2 : 1);
  const int64_t rows = (int64_t)p->batch * p->dim;
  if (rows * ntiles > SCRATCH_FLOATS / width) return MAMBA_E_UNSUPPORTED;  // checkpoints beyond the fixed buffer
  float *ws = scratch_for_current_device();
  if (!ws) return MAMBA_E_LAUNCH;
  MambaScanParams q = *p;
  q.ckpt = ws;
  q.lane_state = nullptr;
  const int rc = mamba1_scan_fwd(&q, stream);
  if (rc != MAMBA_OK || !last_state) return rc;
  const int64_t n = rows * width;
  if ((n + 255) / 256 > 0x7fffffff) return MAMBA_E_UNSUPPORTED;
  hipLaunchKernelGGL(gather_last_state_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), ws, last_state, rows, ntiles, width);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

extern "C" int mamba1_scan_bwd(const MambaScanParams *p, mamba_stream_t stream) {
  int rc = check_common(p);
  if (rc != MAMBA_OK) return rc;
  if (!p->dout || !p->du || !p->ddelta || !p->dB32 || !p->dC32 || !p->dA_part || !p->dD_part || !p->ddelta_bias_part)
    return MAMBA_E_BADARG;
  if (p->z && !p->dz) return MAMBA_E_BADARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (p->a_complex) return mamba1_scan_complex(p, s, true);
  switch (p->dtype) {
    case MAMBA_F32: return dispatch<float, true>(*p, s);
    case MAMBA_BF16: return dispatch<bf16_t, true>(*p, s);
    default: return dispatch<f16_t, true>(*p, s);
  }
}
