// Mamba-1 selective scan, forward and backward, for gfx950 (wave64).
//
// Work decomposition
//   * a wave owns 4 channels of one (batch, group) at a time, one per DPP row of 16 lanes; the 16
//     lanes of a row hold 16 consecutive 8-step segments of the sequence, i.e. one 128-step tile
//     per pass.  A lane loads its 8 items of u/delta/z with one 16-byte access.  Every cross-lane
//     step of the scans then stays inside a DPP row (row_shr / row_shl), which is the cheap kind.
//   * the 8 waves of a workgroup walk the tiles together and share the B and C rows of the tile,
//     staged once per tile in LDS as fp32; a backward workgroup takes several passes of 32 channels
//     over a tile.
//   * per state n: an 8-step in-register recurrence per lane, a row scan of the (decay, value)
//     pairs across the 16 lanes, and a carry from the previous tile kept in LDS.
//   * the state after every tile is written to `ckpt`; the backward pass walks the tiles in
//     reverse, restarts each tile from ckpt, and runs the adjoint recurrence with a reversed row
//     scan.  dB/dC are summed over the channels of the workgroup in LDS (waves take turns on
//     disjoint state rows; LDS float atomics are far too slow for this), written once per tile as
//     one partial per workgroup, and summed over the workgroups in a fixed order by a second
//     kernel: no float atomics anywhere, so every gradient repeats bit for bit.
#include "mamba1_scan.hpp"

#include <stdlib.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>

size_t mamba1_bwd_mx_lds(int passes, int np);                                                       // mamba1_scan_bwd_mx.hip
int mamba1_bwd_mx_launch(const MambaScanParams &p, int passes, bool vec, hipStream_t stream);  // likewise
size_t mamba1_bwd_k4_lds(int passes);                                                          // mamba1_scan_bwd_k4.hip
bool mamba1_bwd_k4_serves(const MambaScanParams &p);                                           // likewise
int mamba1_bwd_k4_launch(const MambaScanParams &p, int pa, int pb, int nparts, hipStream_t stream);  // likewise

namespace {

// ------------------------------------------------------------------ forward
// BC: bit 0 = B is an input-independent (dim, dstate) fp32 matrix, bit 1 = C likewise
// (selective_scan_fwd_kernel.cuh:74 kIsVariableB / kIsVariableC false).
// HALF: a checkpoint every 64 positions instead of every 128 (the state entering lane 8 of a row is the state after
// the tile's first 64 positions): ckpt is then (batch, dim, ceil(L / 64), N).  For the backward kernel that walks
// 64-position tiles (mamba1_scan_bwd_k4.hip).
template <typename T, bool VEC, int BC, bool HALF>
__global__ __launch_bounds__(NTHREADS, 4) void scan_fwd_kernel(const MambaScanParams p, const int passes) {
  extern __shared__ __align__(16) float smem[];
  const int N = p.dstate, L = p.seqlen;
  const int NBLK = (N + NB16 - 1) / NB16, NP = NBLK * NB16;
  float *Bs = smem;
  float *Cs = Bs + BC_FLOATS;
  float *A2s = Cs + BC_FLOATS;                 // [passes * PASS_CH][NP]  A * log2(e)
  float *hcar = A2s + passes * PASS_CH * NP;   // [passes * PASS_CH][NP]  state carried across tiles
  float *hmid = hcar + passes * PASS_CH * NP;  // [passes * PASS_CH][NP]  state after the tile's first half (HALF)

  const int tid = threadIdx.x, lane = tid & 63, c = lane & (RL - 1), rsel = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Geo q = geometry(p, passes);
  const int b = q.b;
  const int chl = wave * ROWS + rsel;  // this lane's channel within a pass
  const T *Bg = (const T *)p.B + b * p.B_bs + q.g * p.B_gs;
  const T *Cg = (const T *)p.C + b * p.C_bs + q.g * p.C_gs;
  const float *Ag = (const float *)p.A;
  const int d0 = q.g * q.Dg + q.cb * passes * PASS_CH;  // first channel of the workgroup

  for (int i = tid; i < passes * PASS_CH * NP; i += NTHREADS) {
    const int ch = i / NP, n = i % NP, d = d0 + ch;
    A2s[i] = (d < q.dend && n < N) ? Ag[(int64_t)d * N + n] * kLog2e : 0.f;
    hcar[i] = 0.f;
  }
  lds_barrier();

  for (int tile = 0; tile < q.ntiles; ++tile) {
    const int t0 = tile * TILE, tl = t0 + c * KI;
    for (int r = 0; r < passes; ++r) {
      if (d0 + r * PASS_CH >= q.dend) break;  // the whole pass lies past the group (the same in every wave)
      const int chw = r * PASS_CH + chl;
      const bool valid = d0 + chw < q.dend;
      const int d = min(d0 + chw, q.dend - 1);
      const int nvalid = valid ? min(max(L - tl, 0), KI) : 0;
      float u[8], dl[8], du[8], y[8], dsum = 0.f;
      Pack8<T> ku, kd, kz;  // raw rows: every load is issued before the first conversion
      kz.zero();
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
      for (int nb = 0; nb < NBLK; ++nb) {
        if (BC != 3 && (NBLK > 1 || r == 0)) {
          lds_barrier();
          stage_bc<T, VEC, BC>(Bs, Cs, Bg, p.B_ns, Cg, p.C_ns, nb * NB16, N, t0, L, tid);
          lds_barrier();
        }
        const float *A2row = A2s + chw * NP + nb * NB16;
        float *hrow = hcar + chw * NP + nb * NB16;
        float *mrow = hmid + chw * NP + nb * NB16;
        const int nmax = min(NB16, N - nb * NB16);
        // two states per iteration: their row scans are interleaved (padded rows are inert:
        // A = 0, B = C = 0)
        for (int n = 0; n < nmax; n += 2) {
          // Pass 1 runs the lane's 8 steps from a zero state to get the lane's (decay, value) pair;
          // the decay over the lane is one exp of the summed delta instead of 7 products. Pass 2
          // reruns the 8 steps from the state the row scan gives this lane.
          float a[2][8], bb[2][8], Cv[2][8], hc[2];
          float sa[2], sb[2];
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const float A2 = A2row[n + s];
            hc[s] = hrow[n + s];
            float Bv[8];
            load_bc<BC & 1>(Bv, Bs, p.B, d, N, nb * NB16 + n + s, n + s, c);
            load_bc<BC & 2>(Cv[s], Cs, p.C, d, N, nb * NB16 + n + s, n + s, c);
            sa[s] = fast_exp2(dsum * A2);
#pragma unroll
            for (int i = 0; i < KI; ++i) {
              a[s][i] = fast_exp2(dl[i] * A2);
              bb[s][i] = du[i] * Bv[i];
            }
            float hl = bb[s][0];
#pragma unroll
            for (int i = 1; i < KI; ++i) hl = __builtin_fmaf(a[s][i], hl, bb[s][i]);
            sb[s] = hl;
          }
          row_scan_fwd2(sa[0], sb[0], sa[1], sb[1]);
          const float hend[2] = {__builtin_fmaf(sa[0], hc[0], sb[0]), __builtin_fmaf(sa[1], hc[1], sb[1])};
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            float h = dpp_f<DPP_ROW_SHR + 1>(hc[s], hend[s]);  // state entering this lane
            if (c == RL - 1) hrow[n + s] = hend[s];            // state after the tile
            if constexpr (HALF) {
              if (c == RL / 2) mrow[n + s] = h;                // state after the tile's first half
            }
#pragma unroll
            for (int i = 0; i < KI; ++i) {
              h = __builtin_fmaf(a[s][i], h, bb[s][i]);
              y[i] = __builtin_fmaf(h, Cv[s][i], y[i]);
            }
          }
        }
      }
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
      if (valid) {  // a row's own lanes wrote its slots of hcar: no other wave touches them
        const float *hfin = hcar + chw * NP;
        if constexpr (HALF) {
          const int nhalf = (L + TILE / 2 - 1) / (TILE / 2);
          float *ck = p.ckpt + (((int64_t)b * p.dim + d) * nhalf + 2 * tile) * N;
          const float *hm = hmid + chw * NP;
          for (int n = c; n < N; n += RL) ck[n] = hm[n];
          if (2 * tile + 1 < nhalf)
            for (int n = c; n < N; n += RL) ck[N + n] = hfin[n];
        } else {
          float *ck = p.ckpt + (((int64_t)b * p.dim + d) * q.ntiles + tile) * N;
          for (int n = c; n < N; n += RL) ck[n] = hfin[n];
        }
      }
    }
  }
}

// ----------------------------------------------------------------- backward

// `passes` passes of PASS_CH channels per tile; the dB / dC sums of all of them leave once per tile as
// partial number (workgroup's place in its group), or after every pass and block when the states come
// in blocks of 16 (the host side then asks for one pass).
// CKH: the checkpoints come every 64 positions (see scan_fwd_kernel): the state entering tile t is slot 2 t - 1.
template <typename T, bool VEC, int BC, bool CKH>
__global__ __launch_bounds__(NTHREADS) void scan_bwd_kernel(const MambaScanParams p, const int passes) {
  constexpr bool ck_half = CKH;
  extern __shared__ __align__(16) float smem[];
  const int N = p.dstate, L = p.seqlen;
  const int NBLK = (N + NB16 - 1) / NB16, NP = NBLK * NB16;
  const int WCH = passes * PASS_CH;
  float *Bs = smem;
  float *Cs = Bs + BC_FLOATS;
  float *dBs = Cs + BC_FLOATS;        // fp32 sums over the workgroup's channels: [n][half][lane][4]
  float *dCs = dBs + ACC_FLOATS;
  float *hcar = dCs + ACC_FLOATS;     // [PASS_CH][NP] state entering the tile (from ckpt), per pass
  float *A1s = hcar + PASS_CH * NP;   // [WCH][NP] A
  float *gcar = A1s + WCH * NP;       // adjoint at the first position of the following tile
  float *anx = gcar + WCH * NP;       // decay at the first position of the following tile
  float *dAacc = anx + WCH * NP;      // [WCH][NP]
  float *dDacc = dAacc + WCH * NP;    // [WCH]
  float *dbacc = dDacc + WCH;         // [WCH]
  BwdRow<T> *rows = reinterpret_cast<BwdRow<T> *>(dbacc + WCH);  // [WCH]
  float *dBcacc = reinterpret_cast<float *>(rows + WCH);  // [WCH][NP] gradients of input-independent B / C (BC != 0)
  float *dCcacc = dBcacc + WCH * NP;
  static_assert(sizeof(BwdRow<T>) == 80, "the host side sizes the LDS table with 80 bytes per channel");

  const int tid = threadIdx.x, lane = tid & 63, c = lane & (RL - 1), rsel = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Geo q = geometry(p, passes);
  const int b = q.b;
  const int chl = wave * ROWS + rsel;
  const int d0 = q.g * q.Dg + q.cb * WCH;
  const int ntiles = q.ntiles;
  const bool has_z = p.z != nullptr;
  T *const spare = reinterpret_cast<T *>(bwd_spare + tid * 8);  // where this thread's unwanted row stores go

  const T *Bg = (const T *)p.B + b * p.B_bs + q.g * p.B_gs;
  const T *Cg = (const T *)p.C + b * p.C_bs + q.g * p.C_gs;
  const float *Ag = (const float *)p.A;
  // partials of this workgroup: (batch, ngroups, nparts, dstate, seqlen), nparts = cblocks (x passes when NBLK > 1)
  const int per_wg = NBLK > 1 ? passes : 1;
  const int64_t part0 = ((int64_t)b * p.ngroups + q.g) * (q.cblocks * per_wg) + (int64_t)q.cb * per_wg;

  for (int i = tid; i < WCH * NP; i += NTHREADS) {
    const int ch = i / NP, n = i % NP, d = d0 + ch;
    A1s[i] = (d < q.dend && n < N) ? Ag[(int64_t)d * N + n] : 0.f;
    gcar[i] = 0.f;
    anx[i] = 0.f;
    dAacc[i] = 0.f;
    if constexpr (BC != 0) {
      dBcacc[i] = 0.f;
      dCcacc[i] = 0.f;
    }
  }
  for (int i = tid; i < WCH; i += NTHREADS) {
    dDacc[i] = 0.f;
    dbacc[i] = 0.f;
    const int d = min(d0 + i, q.dend - 1);  // channels past the group stand on its last one; their lanes are masked
    BwdRow<T> w;
    w.u = (const T *)p.u + b * p.u_bs + d * p.u_ds;
    w.delta = (const T *)p.delta + b * p.delta_bs + d * p.delta_ds;
    w.dout = (const T *)p.dout + b * p.dout_bs + d * p.dout_ds;
    w.z = has_z ? (const T *)p.z + b * p.z_bs + d * p.z_ds : w.u;  // without z the u row stands in, read and unused
    w.du = (T *)p.du + b * p.du_bs + d * p.du_ds;
    w.ddelta = (T *)p.ddelta + b * p.ddelta_bs + d * p.ddelta_ds;
    w.dz = has_z ? (T *)p.dz + b * p.dz_bs + d * p.dz_ds : nullptr;
    w.out_z = (has_z && p.out_z) ? (T *)p.out_z + b * p.outz_bs + d * p.outz_ds : nullptr;
    w.ckpt = p.ckpt + ((int64_t)b * p.dim + d) * (ck_half ? (L + TILE / 2 - 1) / (TILE / 2) : ntiles) * N;
    w.D = p.D ? ((const float *)p.D)[d] : 0.f;
    w.bias = p.delta_bias ? ((const float *)p.delta_bias)[d] : 0.f;
    rows[i] = w;
  }
  lds_barrier();

  constexpr int NPP = NB16 / NWAVES;  // state rows per wave and phase (see the state loop)
  constexpr int NPH = NB16 / NPP;
  static_assert(NPP == 2 && NPH == NWAVES, "two states per step, one row slot per wave and phase");
  // The rows of the next (tile, pass) are fetched while the current one is computed.
  struct Rows {
    Pack8<T> u, delta, dout, z;
    float ck;  // checkpointed state n = c entering the tile (when the padded state count is 16)
  };
  auto fetch_rows = [&](Rows &k, int tile, int r) {
    const BwdRow<T> &w = rows[r * PASS_CH + chl];
    const int tl = tile * TILE + c * KI;
    const int nvalid = min(max(L - tl, 0), KI);
    // No branch around any of these loads (the checkpoint of tile 0 stands in where there is none to read, the u
    // row where there is no z): with the same memory operations on every path through a step the compiler counts
    // those in flight exactly, and a wait for these rows leaves the younger stores of the step before draining.
    k.ck = *(const GLOBAL_AS float *)(w.ckpt + (int64_t)max(ck_half ? 2 * tile - 1 : tile - 1, 0) * N + min(c, N - 1));
    load_items<T, VEC>(k.u, w.u, tl, L, nvalid);
    load_items<T, VEC>(k.delta, w.delta, tl, L, nvalid);
    load_items<T, VEC>(k.dout, w.dout, tl, L, nvalid);
    load_items<T, VEC>(k.z, w.z, tl, L, nvalid);
  };
  int npass = 0;  // passes that hold at least one channel of the group (the same in every wave)
  while (npass < passes && d0 + npass * PASS_CH < q.dend) ++npass;
  Rows nxt;
  fetch_rows(nxt, ntiles - 1, 0);

  for (int tile = ntiles - 1; tile >= 0; --tile) {
    const int t0 = tile * TILE, tl = t0 + c * KI;
    for (int r = 0; r < npass; ++r) {
      const int chw = r * PASS_CH + chl;
      const bool valid = d0 + chw < q.dend;
      const int d = min(d0 + chw, q.dend - 1);
      const int nvalid = valid ? min(max(L - tl, 0), KI) : 0;
      float u[8], dl[8], du[8], dy[8], acc[8], dd[8], y[8], dsum = 0.f, dtail = 0.f;
      const float Dd = rows[chw].D, bias = rows[chw].bias;
      {
        // The rows requested during the previous step are unpacked where they were loaded, and only then are the
        // next step's rows requested into the same registers: nothing of them has to be copied (a copy held
        // across the loop's back edge went through scratch memory).  The epilogue reads z and dout again.
        nxt.u.unpack(u);
        nxt.delta.unpack(dl);
        nxt.dout.unpack(dy);
#pragma unroll
        for (int i = 0; i < KI; ++i) {  // lanes past the end read a clamped position: mask them
          u[i] = (i < nvalid) ? u[i] : 0.f;
          dy[i] = (i < nvalid) ? dy[i] : 0.f;
        }
        if (has_z) {
          float z[8];
          nxt.z.unpack(z);
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
#pragma unroll
        for (int i = 1; i < KI; ++i) dtail += dl[i];
        dsum = dtail + dl[0];
        // state entering this tile (a row's own lanes write and read its slots)
        if (NBLK == 1) {
          hcar[chl * NP + c] = (c < N && tile > 0) ? nxt.ck : 0.f;
        } else {
          for (int n = c; n < NP; n += RL) {
            float v = 0.f;
            if (tile > 0 && n < N)
              v = *(const GLOBAL_AS float *)(rows[chw].ckpt + (int64_t)(ck_half ? 2 * tile - 1 : tile - 1) * N + n);
            hcar[chl * NP + n] = v;
          }
        }
        {  // the very last step fetches tile 0 once more rather than branch around the loads
          const bool more = r + 1 < npass;
          fetch_rows(nxt, more ? tile : max(tile - 1, 0), more ? r + 1 : 0);
        }
      }
      for (int nb = 0; nb < NBLK; ++nb) {
        if (BC != 3 && (NBLK > 1 || r == 0)) {
          lds_barrier();
          stage_bc<T, VEC, BC>(Bs, Cs, Bg, p.B_ns, Cg, p.C_ns, nb * NB16, N, t0, L, tid);
          for (int i = tid * 4; i < 2 * ACC_FLOATS; i += NTHREADS * 4)  // dBs and dCs are adjacent
            *reinterpret_cast<f32x4 *>(dBs + i) = f32x4{0.f, 0.f, 0.f, 0.f};
          lds_barrier();
        }
        {
          // The 8 waves add their channels' dB/dC terms into the shared LDS sums without atomics: between
          // two workgroup barriers every wave adds into another pair of state rows, and the 4 channels of a
          // wave have their own slots of a row.  A phase has two halves, the states and adjoints of the pair
          // (vector ALU work) and the sums (LDS traffic).  Waves 4-7 meet the barrier at the end of a phase;
          // waves 0-3 meet the same barrier between their two halves, so they run half a phase behind and
          // the two waves of a SIMD are never in the same half: one computes while the other waits for LDS.
          // Between barriers j and j + 1 waves 0-3 add the sums of phase j into rows (w + j) % 8 * 2, + 1 and
          // waves 4-7 those of phase j + 1 into rows (w + j) % 8 * 2, + 1 (their rows run one phase behind):
          // eight different pairs.
          const bool early = wave < NWAVES / 2;
          const int slot_shift = early ? 0 : NPH - 1;
          const float *A1row = A1s + chw * NP + nb * NB16;
          const float *hrow = hcar + chl * NP + nb * NB16;
          float *grow = gcar + chw * NP + nb * NB16;
          float *arow = anx + chw * NP + nb * NB16;
          float *dArow = dAacc + chw * NP + nb * NB16;
          // the LDS operands of a phase's two states: A, the carries, the B and C rows
          struct Operands {
            float A1[2], hc[2], gc[2], an[2], Bv[2][8], Cv[2][8];
          };
          auto fetch_operands = [&](Operands &o, int ph) {
            const int n = ((wave + ph + slot_shift) % NPH) * NPP;
#pragma unroll
            for (int s = 0; s < 2; ++s) {
              o.A1[s] = A1row[n + s];
              o.hc[s] = hrow[n + s];
              o.gc[s] = grow[n + s];
              o.an[s] = arow[n + s];
              load_bc<BC & 1>(o.Bv[s], Bs, p.B, d, N, nb * NB16 + n + s, n + s, c);
              load_bc<BC & 2>(o.Cv[s], Cs, p.C, d, N, nb * NB16 + n + s, n + s, c);
            }
          };
          Operands ops;
          fetch_operands(ops, 0);
          for (int ph = 0; ph < NPH; ++ph) {
            const int n = ((wave + ph + slot_shift) % NPH) * NPP;
            constexpr bool active = true;  // padded states run on zeros (A = B = C = 0)
            float A1[2], gc[2], an[2];
            float Cv[2][8], a[2][8], bb[2][8], h[2][8];
            float gfirst[2], a_next_lane[2];
            if (active) {
              // Forward states: pass 1 runs the lane's 8 steps from zero for the lane's (decay, value)
              // pair, the decay being one exp of the summed delta; pass 2 reruns them from the state
              // the row scan gives this lane. The adjoint is handled the same way in reverse.
              float hc[2], sa[2], sb[2], hend[2];
#pragma unroll
              for (int s = 0; s < 2; ++s) {
                A1[s] = ops.A1[s];
                hc[s] = ops.hc[s];
                gc[s] = ops.gc[s];
                an[s] = ops.an[s];
                const float A2 = A1[s] * kLog2e;
#pragma unroll
                for (int i = 0; i < KI; ++i) {
                  Cv[s][i] = ops.Cv[s][i];
                  a[s][i] = fast_exp2(dl[i] * A2);
                  bb[s][i] = du[i] * ops.Bv[s][i];
                }
                sa[s] = fast_exp2(dsum * A2);
                float hl = bb[s][0];
#pragma unroll
                for (int i = 1; i < KI; ++i) hl = __builtin_fmaf(a[s][i], hl, bb[s][i]);
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
                for (int i = 0; i < KI; ++i) {
                  hp = __builtin_fmaf(a[s][i], hp, bb[s][i]);
                  h[s][i] = hp;  // true states
                }
                if (has_z) {
#pragma unroll
                  for (int i = 0; i < KI; ++i) y[i] = __builtin_fmaf(h[s][i], Cv[s][i], y[i]);
                }
                // adjoint recurrence g[t] = dy[t] C[t] + a[t+1] g[t+1]; Cv becomes dy * C
                a_next_lane[s] = dpp_f<DPP_ROW_SHL + 1>(an[s], a[s][0]);
#pragma unroll
                for (int i = 0; i < KI; ++i) Cv[s][i] *= dy[i];
                float gl = Cv[s][KI - 1];
#pragma unroll
                for (int i = KI - 2; i >= 0; --i) gl = __builtin_fmaf(a[s][i + 1], gl, Cv[s][i]);
                ra[s] = fast_exp2(dtail * (A1[s] * kLog2e)) * a_next_lane[s];
                rb[s] = gl;
              }
              row_scan_rev2(ra[0], rb[0], ra[1], rb[1]);
#pragma unroll
              for (int s = 0; s < 2; ++s) gfirst[s] = __builtin_fmaf(ra[s], gc[s], rb[s]);
            }
            if (early) lds_barrier();  // the early waves meet the others here, between the two halves
            if (active) {
#pragma unroll
              for (int s = 0; s < 2; ++s) {
                const float gx = dpp_f<DPP_ROW_SHL + 1>(gc[s], gfirst[s]);  // adjoint at the next lane's first item
                if (c == 0) {
                  grow[n + s] = gfirst[s];
                  arow[n + s] = a[s][0];
                }
                float dAp = 0.f, dBp = 0.f, dCp = 0.f;
                float sB[8], sC[8], Bv[8];
                load_bc<BC & 1>(Bv, Bs, p.B, d, N, nb * NB16 + n + s, n + s, c);
                if constexpr (!(BC & 1)) lds_ld8<4 * 64>(dBs + (n + s) * ACC_PITCH, lane, sB);
                if constexpr (!(BC & 2)) lds_ld8<4 * 64>(dCs + (n + s) * ACC_PITCH, lane, sC);
                float gi = gx, an_i = a_next_lane[s];
#pragma unroll
                for (int i = KI - 1; i >= 0; --i) {
                  gi = __builtin_fmaf(an_i, gi, Cv[s][i]);
                  an_i = a[s][i];
                  if constexpr (BC & 2) dCp = __builtin_fmaf(dy[i], h[s][i], dCp);
                  else sC[i] = __builtin_fmaf(dy[i], h[s][i], sC[i]);
                  if constexpr (BC & 1) dBp = __builtin_fmaf(gi, du[i], dBp);
                  else sB[i] = __builtin_fmaf(gi, du[i], sB[i]);
                  acc[i] = __builtin_fmaf(gi, Bv[i], acc[i]);
                  const float w = gi * (h[s][i] - bb[s][i]);  // g * a * h[t-1]
                  dd[i] = __builtin_fmaf(A1[s], w, dd[i]);
                  dAp = __builtin_fmaf(dl[i], w, dAp);
                }
                if constexpr (!(BC & 1)) lds_st8<4 * 64>(dBs + (n + s) * ACC_PITCH, lane, sB);
                if constexpr (!(BC & 2)) lds_st8<4 * 64>(dCs + (n + s) * ACC_PITCH, lane, sC);
                dAp = row_sum_to_last(dAp);
                if (c == RL - 1) dArow[n + s] += dAp;  // the slot belongs to this row alone
                if constexpr (BC & 1) {
                  dBp = row_sum_to_last(dBp);
                  if (c == RL - 1) dBcacc[chw * NP + nb * NB16 + n + s] += dBp;
                }
                if constexpr (BC & 2) {
                  dCp = row_sum_to_last(dCp);
                  if (c == RL - 1) dCcacc[chw * NP + nb * NB16 + n + s] += dCp;
                }
              }
            }
            if (ph + 1 < NPH) fetch_operands(ops, ph + 1);
            if (!early) lds_barrier();
          }
        }
        if (BC != 3 && (NBLK > 1 || r == npass - 1)) {
          lds_barrier();  // waves 0-3 add their last sums after the last barrier of the phases
          // One partial per workgroup: the sum over the 4 channel slots of every (state, position), written
          // with plain stores (positions past the end and padded states are skipped).
          const int n0 = nb * NB16;
          const int64_t part = part0 + (NBLK > 1 ? r : 0);
          constexpr int FIRST = (BC & 1) ? NB16 * TILE / 4 : 0, LAST = (BC & 2) ? NB16 * TILE / 4 : 2 * NB16 * TILE / 4;
          for (int o = FIRST + tid; o < LAST; o += NTHREADS) {
            const int which = o >> 9, n = (o >> 5) & 15, q4 = o & 31;  // positions 4 q4 .. 4 q4 + 3 of state n
            const float *src = (which ? dCs : dBs) + n * ACC_PITCH + (q4 & 1) * 256 + (q4 >> 1) * 4;
            f32x4 v = *reinterpret_cast<const f32x4 *>(src);
#pragma unroll
            for (int k = 1; k < ROWS; ++k) {
              const f32x4 w = *reinterpret_cast<const f32x4 *>(src + k * RL * 4);
              v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
            }
            const int t = t0 + 4 * q4;
            if (n0 + n >= N || t >= L) continue;
            float *dst = (which ? p.dC32 : p.dB32) + (part * N + n0 + n) * L + t;
            if (VEC) {
              *reinterpret_cast<f32x4 *>(dst) = v;
            } else {
              dst[0] = v.x;
              if (t + 1 < L) dst[1] = v.y;
              if (t + 2 < L) dst[2] = v.z;
              if (t + 3 < L) dst[3] = v.w;
            }
          }
        }
      }
      {
        float o[8];
        const BwdRow<T> w = rows[chw];
        Pack8<T> z_k, dout_k;  // read again here rather than held through the state loop: they come from the caches
        load_items<T, VEC>(z_k, w.z, tl, L, nvalid);
        load_items<T, VEC>(dout_k, w.dout, tl, L, nvalid);
        float dbs = 0.f, dDs = 0.f;
#pragma unroll
        for (int i = 0; i < KI; ++i) o[i] = __builtin_fmaf(dl[i], acc[i], Dd * dy[i]);
        st8_or_spare_global<T, VEC>(w.du + tl, nvalid, true, spare, o);
#pragma unroll
        for (int i = 0; i < KI; ++i) {
          float gd = __builtin_fmaf(u[i], acc[i], dd[i]);
          if (p.delta_softplus) gd *= softplus_slope_f(dl[i]);
          gd = (i < nvalid) ? gd : 0.f;
          o[i] = gd;
          dbs += gd;
          dDs = __builtin_fmaf(dy[i], u[i], dDs);
        }
        st8_or_spare_global<T, VEC>(w.ddelta + tl, nvalid, true, spare, o);
        float oz[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (has_z) {
          float z[8], dout[8];
          z_k.unpack(z);
          dout_k.unpack(dout);
#pragma unroll
          for (int i = 0; i < KI; ++i) {
            const float yf = __builtin_fmaf(Dd, u[i], y[i]);
            const float s = sigmoid_f(z[i]);
            o[i] = dout[i] * yf * s * (1.f + z[i] * (1.f - s));
            oz[i] = yf * z[i] * s;
          }
        }
        st8_or_spare_global<T, VEC>(w.dz + tl, nvalid, has_z, spare, o);
        st8_or_spare_global<T, VEC>(w.out_z + tl, nvalid, w.out_z != nullptr, spare, oz);
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
  // per-(batch, channel) partial sums; the caller reduces over batch
  for (int i = tid; i < WCH * N; i += NTHREADS) {
    const int ch = i / N, n = i % N, d = d0 + ch;
    if (d >= q.dend) continue;
    p.dA_part[((int64_t)b * p.dim + d) * N + n] = dAacc[ch * NP + n];
    if constexpr (BC & 1) p.dB32[((int64_t)b * p.dim + d) * N + n] = dBcacc[ch * NP + n];
    if constexpr (BC & 2) p.dC32[((int64_t)b * p.dim + d) * N + n] = dCcacc[ch * NP + n];
  }
  for (int ch = tid; ch < WCH; ch += NTHREADS) {
    const int d = d0 + ch;
    if (d >= q.dend) continue;
    p.dD_part[(int64_t)b * p.dim + d] = dDacc[ch];
    p.ddelta_bias_part[(int64_t)b * p.dim + d] = dbacc[ch];
  }
}

// out[row, e] = sum over parts of part[row, part, e], in the order of the parts, converted to T; one
// thread per 4 consecutive elements e of the row's `row_len`.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void reduce_parts_kernel(const float *__restrict__ parts, T *__restrict__ out,
                                                           int64_t rows, int nparts, int64_t row_len) {
  const int64_t quad = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t per_row = (row_len + 3) / 4;
  if (quad >= rows * per_row) return;
  const int64_t row = quad / per_row, e = (quad - row * per_row) * 4;
  const float *src = parts + row * nparts * row_len + e;
  T *dst = out + row * row_len + e;
  if (VEC) {
    f32x4 v = *reinterpret_cast<const f32x4 *>(src);
    for (int k = 1; k < nparts; ++k) {
      const f32x4 w = *reinterpret_cast<const f32x4 *>(src + (int64_t)k * row_len);
      v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
    }
    if constexpr (DT<T>::id == MAMBA_F32) {
      *reinterpret_cast<f32x4 *>(dst) = v;
    } else if constexpr (DT<T>::id == MAMBA_BF16) {
      *reinterpret_cast<u32x2 *>(dst) = u32x2{pack_bf16(v.x, v.y), pack_bf16(v.z, v.w)};
    } else {
      *reinterpret_cast<u32x2 *>(dst) = u32x2{pack_f16(v.x, v.y), pack_f16(v.z, v.w)};
    }
  } else {
    for (int i = 0; i < 4 && e + i < row_len; ++i) {
      float v = src[i];
      for (int k = 1; k < nparts; ++k) v += src[(int64_t)k * row_len + i];
      st1<T>(dst + i, v);
    }
  }
}

// ------------------------------------------------------------------ launch
inline bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

inline size_t fwd_lds(int passes, int np, bool half) {
  return sizeof(float) * (2 * BC_FLOATS + (half ? 3 : 2) * passes * PASS_CH * np);
}
inline size_t bwd_lds(int passes, int np, int bc) {
  const int wch = passes * PASS_CH;
  return sizeof(float) * (2 * BC_FLOATS + 2 * ACC_FLOATS + PASS_CH * np + (bc ? 6 : 4) * wch * np + 2 * wch) +
         (size_t)wch * 80;  // + BwdRow per channel
}
constexpr size_t LDS_LIMIT = 160 * 1024;

int compute_units() {
  static int cus = 0;
  if (cus > 0) return cus;
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return 256;  // not cached: asked again on the next call
  }
  cus = n;
  return n;
}

// Which backward kernel serves a problem.  The kernel with fp32 sums of dB / dC in LDS (below) serves every problem by
// default.  MAMBA_AMD_M1_BWD=mx in the environment (read once) sends bf16 rows with per-position B and C to the kernel
// whose dB / dC sums are formed by the matrix cores (mamba1_scan_bwd_mx.hip): measured 8 % slower at batch 8 x 5120
// channels x 4096 positions x 16 states, kept for comparisons.
// MAMBA_AMD_M1_BWD=k4 (read once): checkpoints every 64 positions from the forward kernel, and the backward kernel
// that walks 64-position tiles with 4 items per lane (mamba1_scan_bwd_k4.hip) where it serves the problem; the default
// backward kernel reads the denser checkpoints everywhere else.
bool k4_mode() {
  static const int want = [] {
    const char *e = getenv("MAMBA_AMD_M1_BWD");
    return (e && e[0] == 'k') ? 1 : 0;
  }();
  return want != 0;
}
int ckpt_tile(bool a_complex) { return a_complex ? TILE_COMPLEX : (k4_mode() ? TILE / 2 : TILE); }

bool use_mx(const MambaScanParams &p) {
  static const int want_mx = [] {
    const char *e = getenv("MAMBA_AMD_M1_BWD");
    return (e && e[0] == 'm') ? 1 : 0;
  }();
  return want_mx && p.dtype == MAMBA_BF16 && !(p.bc_const & 3) && !p.a_complex;
}

// Passes of PASS_CH channels a backward workgroup takes per tile.  More passes mean fewer, larger
// partials of dB / dC; the count is chosen so that the workgroups still fill whole rounds over the
// compute units (one workgroup per unit): the smallest rounds * passes wins, ties go to more passes.
int bwd_passes(const MambaScanParams &p) {
  const int np = (p.dstate + NB16 - 1) / NB16 * NB16;
  if (np > NB16) return 1;  // states in blocks: the sums leave after every block
  const int Dg = p.dim / p.ngroups, cus = compute_units();
  int best = 1;
  int64_t best_cost = -1;
  for (int r = 1; r <= MAX_PASSES; ++r) {
    if ((use_mx(p) ? mamba1_bwd_mx_lds(r, np) : bwd_lds(r, np, p.bc_const & 3)) > LDS_LIMIT) break;
    if (r > 1 && (r - 1) * PASS_CH >= Dg) break;
    const int64_t wgs = (int64_t)p.batch * p.ngroups * ((Dg + PASS_CH * r - 1) / (PASS_CH * r));
    const int64_t cost = (wgs + cus - 1) / cus * r;
    if (best_cost < 0 || cost <= best_cost) {
      best_cost = cost;
      best = r;
    }
  }
  return best;
}

// The 4-items-per-lane backward kernel (k4 mode): two workgroups share a compute unit, so its workgroups may take
// pa and pb passes alternately (the long and the short one of a unit); pa == pb: all the same.  Chosen like
// bwd_passes: rounds of workgroups over the units' two places, times the mean passes of a round.
struct K4Plan {
  int pa, pb, nparts;
};
K4Plan k4_plan(const MambaScanParams &p) {
  const int Dg = p.dim / p.ngroups, cus = compute_units();
  static const int cand[6][2] = {{1, 1}, {2, 1}, {2, 2}, {3, 1}, {3, 2}, {3, 3}};
  K4Plan best{1, 1, 1};
  double best_cost = -1;
  for (const auto &c : cand) {
    const int pa = c[0], pb = c[1];
    if (mamba1_bwd_k4_lds(pa) > LDS_LIMIT / 2) continue;
    if (pa > 1 && (pa - 1) * PASS_CH >= Dg) continue;
    const int per = pa == pb ? (Dg + PASS_CH * pa - 1) / (PASS_CH * pa) : 2 * ((Dg + PASS_CH * (pa + pb) - 1) / (PASS_CH * (pa + pb)));
    const int64_t wgs = (int64_t)p.batch * p.ngroups * per;
    const double cost = (double)((wgs + 2 * cus - 1) / (2 * cus)) * 0.5 * (pa + pb);
    if (best_cost < 0 || cost <= best_cost) best_cost = cost, best = K4Plan{pa, pb, per};
  }
  return best;
}
bool use_k4(const MambaScanParams &p) { return k4_mode() && mamba1_bwd_k4_serves(p); }

int bwd_nparts(const MambaScanParams &p) {
  if (use_k4(p)) return k4_plan(p).nparts;
  const int Dg = p.dim / p.ngroups, r = bwd_passes(p);
  return (Dg + PASS_CH * r - 1) / (PASS_CH * r) * (p.dstate > NB16 ? r : 1);
}

// Raises a kernel's dynamic LDS limit to `lds` bytes on the current device, once: the largest size granted so far is
// remembered per (device, kernel), so that repeated launches (and launches under stream capture) make no runtime call.
}  // namespace

bool mamba1_allow_lds(const void *kernel, size_t lds) {
  static std::mutex mu;
  static std::map<std::pair<int, const void *>, size_t> granted;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  std::lock_guard<std::mutex> lock(mu);
  size_t &have = granted[{dev, kernel}];
  if (lds <= have) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  have = lds;
  return true;
}

namespace {

template <typename KernelT>
int launch(KernelT kernel, const MambaScanParams &p, int passes, size_t lds, hipStream_t stream) {
  const int Dg = p.dim / p.ngroups;
  const int cblocks = (Dg + PASS_CH * passes - 1) / (PASS_CH * passes);
  if (lds > LDS_LIMIT) return MAMBA_E_UNSUPPORTED;
  if (!mamba1_allow_lds(reinterpret_cast<const void *>(kernel), lds)) return MAMBA_E_LAUNCH;
  dim3 grid(p.ngroups * cblocks, p.batch), block(NTHREADS);
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, p, passes);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

int check_common(const MambaScanParams *p) {
  if (!p || !p->u || !p->delta || !p->A || !p->B || !p->C || !p->ckpt) return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->dim <= 0 || p->seqlen <= 0 || p->dstate <= 0 || p->ngroups <= 0) return MAMBA_E_BADARG;
  if (p->dim % p->ngroups != 0) return MAMBA_E_BADARG;
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
  if (!(p.bc_const & 1)) v = v && aligned16(p.dB32);
  if (!(p.bc_const & 2)) v = v && aligned16(p.dC32);
  return v && ok(p.dout, p.dout_bs, p.dout_ds) && ok(p.du, p.du_bs, p.du_ds) &&
         ok(p.ddelta, p.ddelta_bs, p.ddelta_ds) && ok(p.dz, p.dz_bs, p.dz_ds) && ok(p.out_z, p.outz_bs, p.outz_ds);
}

template <typename T>
int reduce_parts(const float *parts, void *out, int64_t rows, int nparts, int64_t row_len, hipStream_t stream) {
  const int64_t quads = rows * ((row_len + 3) / 4);
  if ((quads + 255) / 256 > 0x7fffffff) return MAMBA_E_UNSUPPORTED;
  const dim3 grid((unsigned)((quads + 255) / 256)), block(256);
  T *o = static_cast<T *>(out);
  if (row_len % 4 == 0 && aligned16(parts) && aligned16(out))
    hipLaunchKernelGGL((reduce_parts_kernel<T, true>), grid, block, 0, stream, parts, o, rows, nparts, row_len);
  else
    hipLaunchKernelGGL((reduce_parts_kernel<T, false>), grid, block, 0, stream, parts, o, rows, nparts, row_len);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

// dB / dC of per-position operands: the partials summed in a fixed order into the outputs
template <typename T> int reduce_dBC(const MambaScanParams &p, int nparts, hipStream_t stream) {
  const int64_t rows = (int64_t)p.batch * p.ngroups;
  const int64_t row_len = (int64_t)p.dstate * p.seqlen * (p.a_complex ? 2 : 1);
  int rc = MAMBA_OK;
  if (!(p.bc_const & 1)) rc = reduce_parts<T>(p.dB32, p.dB, rows, nparts, row_len, stream);
  if (rc == MAMBA_OK && !(p.bc_const & 2)) rc = reduce_parts<T>(p.dC32, p.dC, rows, nparts, row_len, stream);
  return rc;
}

// `plan`: the whole problem, of which p may be a slice of batch rows; it decides the passes per workgroup and with
// them the number of dB / dC partials, which must be the same for every slice.
template <typename T, bool BWD, int BC> int dispatch_bc(const MambaScanParams &p, const MambaScanParams &plan, hipStream_t stream) {
  const int np = (p.dstate + NB16 - 1) / NB16 * NB16;
  const bool vec = vec_ok(p, BWD);
  if (!BWD) {
    // MAMBA_AMD_FWD_MIN_LDS (bytes): a measurement hook.  A workgroup that asks for more LDS shares its CU with fewer
    // others (160 KB per CU), which is how the kernel's speed against resident waves per SIMD is measured.
    static const size_t min_lds = getenv("MAMBA_AMD_FWD_MIN_LDS") ? (size_t)atol(getenv("MAMBA_AMD_FWD_MIN_LDS")) : 0;
    const bool half = k4_mode();
    const size_t lds = fwd_lds(1, np, half) > min_lds ? fwd_lds(1, np, half) : min_lds;
    if (half)
      return vec ? launch(scan_fwd_kernel<T, true, BC, true>, p, 1, lds, stream)
                 : launch(scan_fwd_kernel<T, false, BC, true>, p, 1, lds, stream);
    return vec ? launch(scan_fwd_kernel<T, true, BC, false>, p, 1, lds, stream)
               : launch(scan_fwd_kernel<T, false, BC, false>, p, 1, lds, stream);
  }
  if (use_k4(plan)) {
    const K4Plan k = k4_plan(plan);
    if (vec) {
      if constexpr (std::is_same_v<T, bf16_t> && BC == 0) {
        const int rc = mamba1_bwd_k4_launch(p, k.pa, k.pb, k.nparts, stream);
        return rc != MAMBA_OK ? rc : reduce_dBC<T>(p, k.nparts, stream);
      }
    }
    // rows the 4-item kernel does not take (unaligned views): the default kernel with as many passes as a long and a
    // short workgroup together, whose partials are fewer than the workspace was sized for: the others are cleared
    const int64_t bytes = (int64_t)p.batch * p.ngroups * k.nparts * p.dstate * p.seqlen * 4;
    int rc = mamba_hip_zero(p.dB32, bytes, stream);
    if (rc == MAMBA_OK) rc = mamba_hip_zero(p.dC32, bytes, stream);
    if (rc != MAMBA_OK) return rc;
    const int passes = k.pa == k.pb ? k.pa : k.pa + k.pb;
    rc = launch(scan_bwd_kernel<T, false, BC, true>, p, passes, bwd_lds(passes, np, BC), stream);
    return rc != MAMBA_OK ? rc : reduce_dBC<T>(p, k.nparts, stream);
  }
  const int passes = bwd_passes(plan);
  if (use_mx(p)) {
    const int rc = mamba1_bwd_mx_launch(p, passes, vec, stream);
    return rc != MAMBA_OK ? rc : reduce_dBC<T>(p, bwd_nparts(plan), stream);
  }
  const size_t lds = bwd_lds(passes, np, BC);
  int rc;
  if (k4_mode())
    rc = vec ? launch(scan_bwd_kernel<T, true, BC, true>, p, passes, lds, stream)
             : launch(scan_bwd_kernel<T, false, BC, true>, p, passes, lds, stream);
  else
    rc = vec ? launch(scan_bwd_kernel<T, true, BC, false>, p, passes, lds, stream)
             : launch(scan_bwd_kernel<T, false, BC, false>, p, passes, lds, stream);
  return rc != MAMBA_OK ? rc : reduce_dBC<T>(p, bwd_nparts(plan), stream);
}

template <typename T, bool BWD> int dispatch(const MambaScanParams &p, const MambaScanParams &plan, hipStream_t stream) {
  switch (p.bc_const & 3) {
    case 0: return dispatch_bc<T, BWD, 0>(p, plan, stream);
    case 1: return dispatch_bc<T, BWD, 1>(p, plan, stream);
    case 2: return dispatch_bc<T, BWD, 2>(p, plan, stream);
    default: return dispatch_bc<T, BWD, 3>(p, plan, stream);
  }
}

// The grid's batch coordinate is 16 bits wide: a larger batch is served in slices of rows (rows are independent; every
// per-row pointer is advanced, the per-(batch, channel) partial sums included).
constexpr int MAX_GRID_BATCH = 65535;

MambaScanParams batch_slice(const MambaScanParams &p, int64_t b0, int nb, int nparts) {
  MambaScanParams q = p;
  q.batch = nb;
  const int64_t es = p.dtype == MAMBA_F32 ? 4 : 2, cx = p.a_complex ? 2 : 1;
  const int tile = ckpt_tile(p.a_complex);
  const int64_t ntiles = (p.seqlen + tile - 1) / tile, N = p.dstate, L = p.seqlen, G = p.ngroups, D = p.dim;
  auto adv = [&](auto *&ptr, int64_t elems, int64_t size) {
    if (ptr) ptr = reinterpret_cast<std::remove_reference_t<decltype(ptr)>>(
                 reinterpret_cast<uintptr_t>(ptr) + (uintptr_t)(b0 * elems * size));
  };
  adv(q.u, p.u_bs, es), adv(q.delta, p.delta_bs, es), adv(q.z, p.z_bs, es), adv(q.out, p.out_bs, es);
  if (!(p.bc_const & 1)) adv(q.B, p.B_bs, es);
  if (!(p.bc_const & 2)) adv(q.C, p.C_bs, es);
  adv(q.ckpt, D * ntiles * N * cx, 4);
  adv(q.dout, p.dout_bs, es), adv(q.du, p.du_bs, es), adv(q.ddelta, p.ddelta_bs, es), adv(q.dz, p.dz_bs, es);
  adv(q.out_z, p.outz_bs, es);
  adv(q.dB32, (p.bc_const & 1) ? D * N * cx : G * nparts * N * L * cx, 4);
  adv(q.dC32, (p.bc_const & 2) ? D * N * cx : G * nparts * N * L * cx, 4);
  adv(q.dA_part, D * N * cx, 4), adv(q.dD_part, D, 4), adv(q.ddelta_bias_part, D, 4);
  adv(q.dB, G * N * L * cx, es), adv(q.dC, G * N * L * cx, es);
  adv(q.det_dB, G * N * L * cx, 8), adv(q.det_dC, G * N * L * cx, 8);
  return q;
}

}  // namespace

int mamba1_scan_complex(const MambaScanParams *p, hipStream_t s, bool bwd);  // mamba1_scan_complex.hip

int mamba1_scan_tile(bool a_complex) { return ckpt_tile(a_complex); }  // positions per checkpoint tile

namespace {
int scan_fwd_one(const MambaScanParams &p, hipStream_t s) {
  if (p.a_complex) return mamba1_scan_complex(&p, s, false);
  switch (p.dtype) {
    case MAMBA_F32: return dispatch<float, false>(p, p, s);
    case MAMBA_BF16: return dispatch<bf16_t, false>(p, p, s);
    default: return dispatch<f16_t, false>(p, p, s);
  }
}

int scan_bwd_one(const MambaScanParams &p, const MambaScanParams &plan, mamba_stream_t stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (p.a_complex) {
    // the complex kernels add their dB / dC terms into one fp32 copy with atomics: clear it, run, convert
    const int64_t bytes = (int64_t)p.batch * p.ngroups * p.dstate * 2 * p.seqlen * 4;
    int rc = MAMBA_OK;
    if (!(p.bc_const & 1)) rc = mamba_hip_zero(p.dB32, bytes, stream);
    if (rc == MAMBA_OK && !(p.bc_const & 2)) rc = mamba_hip_zero(p.dC32, bytes, stream);
    if (p.det_scale && ((!(p.bc_const & 1) && !p.det_dB) || (!(p.bc_const & 2) && !p.det_dC))) return MAMBA_E_BADARG;
    if (rc == MAMBA_OK) rc = mamba1_scan_complex(&p, s, true);
    if (rc == MAMBA_OK && p.det_scale) {  // the integer sums -> the fp32 sums the conversion below reads
      if (!(p.bc_const & 1)) rc = ssd_det_convert(p.det_dB, p.dB32, bytes / 4, p.det_scale, stream);
      if (rc == MAMBA_OK && !(p.bc_const & 2)) rc = ssd_det_convert(p.det_dC, p.dC32, bytes / 4, p.det_scale, stream);
    }
    if (rc != MAMBA_OK) return rc;
    switch (p.dtype) {
      case MAMBA_F32: return reduce_dBC<float>(p, 1, s);
      case MAMBA_BF16: return reduce_dBC<bf16_t>(p, 1, s);
      default: return reduce_dBC<f16_t>(p, 1, s);
    }
  }
  switch (p.dtype) {
    case MAMBA_F32: return dispatch<float, true>(p, plan, s);
    case MAMBA_BF16: return dispatch<bf16_t, true>(p, plan, s);
    default: return dispatch<f16_t, true>(p, plan, s);
  }
}
}  // namespace

extern "C" int mamba1_scan_fwd(const MambaScanParams *p, mamba_stream_t stream) {
  int rc = check_common(p);
  if (rc != MAMBA_OK) return rc;
  if (!p->out) return MAMBA_E_BADARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  for (int64_t b0 = 0; b0 < p->batch; b0 += MAX_GRID_BATCH) {
    const int nb = (int)std::min<int64_t>(MAX_GRID_BATCH, p->batch - b0);
    rc = p->batch <= MAX_GRID_BATCH ? scan_fwd_one(*p, s) : scan_fwd_one(batch_slice(*p, b0, nb, 1), s);
    if (rc != MAMBA_OK) return rc;
  }
  return MAMBA_OK;
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
  const int tile = ckpt_tile(p->a_complex);
  const int ntiles = (p->seqlen + tile - 1) / tile;
  const int width = p->dstate * (p->a_complex ? 2 : 1);
  const int64_t rows = (int64_t)p->batch * p->dim;
  if (rows * ntiles > SCRATCH_FLOATS / width) return MAMBA_E_UNSUPPORTED;  // checkpoints beyond the fixed buffer
  float *ws = scratch_for_current_device();
  if (!ws) return MAMBA_E_LAUNCH;
  MambaScanParams q = *p;
  q.ckpt = ws;
  const int rc = mamba1_scan_fwd(&q, stream);
  if (rc != MAMBA_OK || !last_state) return rc;
  const int64_t n = rows * width;
  if ((n + 255) / 256 > 0x7fffffff) return MAMBA_E_UNSUPPORTED;
  hipLaunchKernelGGL(gather_last_state_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), ws, last_state, rows, ntiles, width);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

extern "C" int mamba1_scan_bwd_nparts(const MambaScanParams *p) {
  if (!p || p->batch <= 0 || p->dim <= 0 || p->seqlen <= 0 || p->dstate <= 0 || p->ngroups <= 0 ||
      p->dim % p->ngroups != 0)
    return MAMBA_E_BADARG;
  if (p->dstate > MAX_DSTATE) return MAMBA_E_UNSUPPORTED;
  return p->a_complex ? 1 : bwd_nparts(*p);
}

extern "C" int mamba1_scan_bwd(const MambaScanParams *p, mamba_stream_t stream) {
  int rc = check_common(p);
  if (rc != MAMBA_OK) return rc;
  if (!p->dout || !p->du || !p->ddelta || !p->dB32 || !p->dC32 || !p->dA_part || !p->dD_part || !p->ddelta_bias_part)
    return MAMBA_E_BADARG;
  if ((!(p->bc_const & 1) && !p->dB) || (!(p->bc_const & 2) && !p->dC)) return MAMBA_E_BADARG;
  if (p->z && !p->dz) return MAMBA_E_BADARG;
  const int nparts = p->a_complex ? 1 : bwd_nparts(*p);
  for (int64_t b0 = 0; b0 < p->batch; b0 += MAX_GRID_BATCH) {
    const int nb = (int)std::min<int64_t>(MAX_GRID_BATCH, p->batch - b0);
    rc = p->batch <= MAX_GRID_BATCH ? scan_bwd_one(*p, *p, stream) : scan_bwd_one(batch_slice(*p, b0, nb, nparts), *p, stream);
    if (rc != MAMBA_OK) return rc;
  }
  return MAMBA_OK;
}
