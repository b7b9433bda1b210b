// Mamba-1 selective scan, backward, for 16-bit inputs with per-position B and C: the variant whose dB / dC
// sums over channels are formed by the matrix cores.
//
// Same decomposition as scan_bwd_kernel (mamba1_scan.hip): a wave owns 4 channels, one per DPP row of 16
// lanes, a lane 8 consecutive positions of a 128-position tile; tiles in reverse order, states recomputed
// from the checkpoints, adjoint recurrence with a reversed row scan.  What differs is where the sums of
// dB[n, t] = sum over channels of g * delta * u and dC[n, t] = sum over channels of dy * h are kept:
//   * a lane's 8 products of one state are rounded to bf16 and handed to v_mfma_f32_16x16x32_bf16 as the
//     32 x 16 operand P[k = 8 row + item][column = the lane's place in its row]; the other operand is a 0/1
//     selector S[i][8 row + item] = (i == item) (dB) or (i == item + 8) (dC), so the product adds
//     D[i][column] += sum over the 4 rows (channels) of item i (dB) / item i - 8 (dC);
//   * one 16 x 16 fp32 accumulator tile per state (4 registers per lane) stays with the wave over every pass
//     of a tile, so the state loop has no shared sums, no LDS read-add-write and no barrier;
//   * once per tile the 8 waves' tiles are added through LDS in wave order and written as the workgroup's
//     partial of dB32 / dC32, which reduce_parts_kernel adds over the workgroups in index order.
// The terms are rounded to bf16 once (relative error 2^-9 per term, random in sign) before an fp32 sum whose
// result is itself stored as bf16: this is why the variant serves bf16 inputs only; fp32 and fp16 inputs keep
// the kernel with fp32 sums in LDS.  The order of every sum is fixed, so results repeat bit for bit.
#include "mamba1_scan.hpp"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

constexpr int RED_STATES = 4;                              // states per round of the cross-wave sum
constexpr int RED_FLOATS = NWAVES * RED_STATES * 64 * 4;   // its scratch: [wave][state][lane] 16-byte tile parts

// The two selector operands.  Lane with row index i (= its place c in its DPP row) supplies S[i][8 r + e],
// e = 0..7, for its own r; the selector does not depend on r.
struct Selectors {
  bf16x8_t s[2];
  DEVI void init(int i) {
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    s16x8 v0, v1;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v0[e] = (i == e) ? (short)0x3f80 : (short)0;
      v1[e] = (i == e + 8) ? (short)0x3f80 : (short)0;
    }
    s[0] = __builtin_bit_cast(bf16x8_t, v0);
    s[1] = __builtin_bit_cast(bf16x8_t, v1);
  }
  // rows 8 W .. 8 W + 7 of the tile, column c += the sum over the 4 DPP rows of v[0..7]
  template <int W> DEVI void add(f32x4 &tile, const float (&v)[8]) const {
    const u32x4 w = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
    tile = __builtin_amdgcn_mfma_f32_16x16x32_bf16(s[W], __builtin_bit_cast(bf16x8_t, w), tile, 0, 0, 0);
  }
};

// HAS_Z: a gate z is given (a compile-time switch: as a run-time flag inside the unrolled state loop the compiler
// moved all sixteen states' y sums behind the loop and kept their operands in scratch memory until then).
DEVI void pin8(float (&v)[8]) {
  asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
}

template <typename T, bool VEC, bool HAS_Z>
__global__ __launch_bounds__(NTHREADS) void scan_bwd_mx_kernel(const MambaScanParams p, const int passes) {
  static_assert(sizeof(T) == 2, "16-bit rows: the parked copies take one 16-byte slot per lane");
  extern __shared__ __align__(16) float smem[];
  const int N = p.dstate, L = p.seqlen;
  const int NBLK = (N + NB16 - 1) / NB16, NP = NBLK * NB16;
  const int WCH = passes * PASS_CH;
  // The arrays the state loop reads lie in the first 64 KB, where an access reaches them with an immediate offset.
  float *Bs = smem;
  float *Cs = Bs + BC_FLOATS;
  f32x4 *st4 = reinterpret_cast<f32x4 *>(Cs + BC_FLOATS);  // [WCH][NP] per channel and state: A, the adjoint and the decay
                                                           // at the first position of the following tile, the dA sum
  float *hcar = reinterpret_cast<float *>(st4 + WCH * NP);  // [PASS_CH][NP] state entering the tile
  float *dDacc = hcar + PASS_CH * NP;  // [WCH]
  float *dbacc = dDacc + WCH;          // [WCH]
  BwdRow<T> *rows = reinterpret_cast<BwdRow<T> *>(dbacc + WCH);  // [WCH]
  u32x4 *park = reinterpret_cast<u32x4 *>(rows + WCH);  // [3][NTHREADS] u, z, dout of the step as stored
  float *red = reinterpret_cast<float *>(park + 3 * NTHREADS);  // scratch of the cross-wave sum of the dB / dC tiles
  static_assert(sizeof(BwdRow<T>) == 80, "the host side sizes the LDS table with 80 bytes per channel");

  const int tid = threadIdx.x, lane = tid & 63, c = lane & (RL - 1), rsel = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Geo q = geometry(p, passes);
  const int b = q.b;
  const int chl = wave * ROWS + rsel;
  const int d0 = q.g * q.Dg + q.cb * WCH;
  const int ntiles = q.ntiles;
  constexpr bool has_z = HAS_Z;
  T *const spare = reinterpret_cast<T *>(bwd_spare + tid * 8);  // where this thread's unwanted row stores go

  const T *Bg = (const T *)p.B + b * p.B_bs + q.g * p.B_gs;
  const T *Cg = (const T *)p.C + b * p.C_bs + q.g * p.C_gs;
  const float *Ag = (const float *)p.A;
  // partials of this workgroup: (batch, ngroups, nparts, dstate, seqlen), nparts = cblocks (x passes when NBLK > 1)
  const int per_wg = NBLK > 1 ? passes : 1;
  const int64_t part0 = ((int64_t)b * p.ngroups + q.g) * (q.cblocks * per_wg) + (int64_t)q.cb * per_wg;

  for (int i = tid; i < WCH * NP; i += NTHREADS) {
    const int ch = i / NP, n = i % NP, d = d0 + ch;
    st4[i] = f32x4{(d < q.dend && n < N) ? Ag[(int64_t)d * N + n] : 0.f, 0.f, 0.f, 0.f};
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
    w.ckpt = p.ckpt + ((int64_t)b * p.dim + d) * ntiles * N;
    w.D = p.D ? ((const float *)p.D)[d] : 0.f;
    w.bias = p.delta_bias ? ((const float *)p.delta_bias)[d] : 0.f;
    rows[i] = w;
  }
  lds_barrier();

  Selectors sel;
  sel.init(c);
  f32x4 tiles[NB16];  // tile n: rows 0-7 = dB of items 0-7, rows 8-15 = dC of items 0-7, column = place in the row
#pragma unroll
  for (int n = 0; n < NB16; ++n) tiles[n] = f32x4{0.f, 0.f, 0.f, 0.f};

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
    // row where there is no z): the compiler then counts the memory operations in flight exactly.
    k.ck = *(const GLOBAL_AS float *)(w.ckpt + (int64_t)max(tile - 1, 0) * N + min(c, N - 1));
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
      (void)d;
      const int nvalid = valid ? min(max(L - tl, 0), KI) : 0;
      float dl[8], du[8], dy[8], acc[8], dd[8], y[8], dsum = 0.f, dtail = 0.f;
      const float bias = rows[chw].bias;
      {
        // The rows requested during the previous step are unpacked where they were loaded; u, z and dout are
        // parked in LDS as stored for the epilogue; then the next step's rows are requested into the same registers.
        float u[8];
        nxt.u.unpack(u);
        nxt.delta.unpack(dl);
        nxt.dout.unpack(dy);
        park[tid] = nxt.u.w;
        park[NTHREADS + tid] = nxt.z.w;
        park[2 * NTHREADS + tid] = nxt.dout.w;
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
            if (tile > 0 && n < N) v = *(const GLOBAL_AS float *)(rows[chw].ckpt + (int64_t)(tile - 1) * N + n);
            hcar[chl * NP + n] = v;
          }
        }
        {  // the very last step fetches tile 0 once more rather than branch around the loads
          const bool more = r + 1 < npass;
          fetch_rows(nxt, more ? tile : max(tile - 1, 0), more ? r + 1 : 0);
        }
      }
      for (int nb = 0; nb < NBLK; ++nb) {
        if (NBLK > 1 || r == 0) {
          lds_barrier();  // every wave has left the previous tile's (block's) B and C rows
          stage_bc<T, VEC, 0>(Bs, Cs, Bg, p.B_ns, Cg, p.C_ns, nb * NB16, N, t0, L, tid);
          lds_barrier();
        }
        f32x4 *srow = st4 + chw * NP + nb * NB16;
        const float *hrow = hcar + chl * NP + nb * NB16;
        // The LDS operands of a state: its record, the state entering the tile, its B and C rows.  Those of the
        // next state are requested before the current state is computed.
        struct Operands {
          f32x4 st;
          float hc, Bv[8], Cv[8];
        };
        auto fetch_operands = [&](Operands &o, int n) {
          o.st = srow[n];
          o.hc = hrow[n];
          lds_ld8<4 * RL>(Bs + n * TILE, c, o.Bv);
          lds_ld8<4 * RL>(Cs + n * TILE, c, o.Cv);
        };
        Operands ops;
        fetch_operands(ops, 0);
        // One state at a time (padded states run on zeros: A = B = C = 0).  The loop is unrolled because each
        // state's accumulator tile is a register of its own.
#pragma unroll
        for (int n = 0; n < NB16; ++n) {
          __builtin_amdgcn_sched_barrier(0);  // one scheduling region per state: nothing of the next one is hoisted
          // Forward states: pass 1 runs the lane's 8 steps from zero for the lane's (decay, value) pair, the
          // decay being one exp of the summed delta; pass 2 reruns them from the state the row scan gives this
          // lane.  The adjoint is handled the same way in reverse.
          const float A1 = ops.st.x, gc = ops.st.y, an = ops.st.z, dA_old = ops.st.w, hc = ops.hc;
          float Bv[8], Cv[8], a[8], h[8];
          const float A2 = A1 * kLog2e;
#pragma unroll
          for (int i = 0; i < KI; ++i) {
            Bv[i] = ops.Bv[i];
            Cv[i] = ops.Cv[i];
            a[i] = fast_exp2(dl[i] * A2);
            h[i] = du[i] * Bv[i];  // the input term; pass 2 turns it into the state
          }
          if (n + 1 < NB16) fetch_operands(ops, n + 1);
          float sa = fast_exp2(dsum * A2), sb = h[0];
#pragma unroll
          for (int i = 1; i < KI; ++i) sb = __builtin_fmaf(a[i], sb, h[i]);
          row_scan_fwd1(sa, sb);
          const float hend = __builtin_fmaf(sa, hc, sb);
          const float hin = dpp_f<DPP_ROW_SHR + 1>(hc, hend);  // state entering this lane
          {
            float hp = hin;
#pragma unroll
            for (int i = 0; i < KI; ++i) {
              hp = __builtin_fmaf(a[i], hp, h[i]);
              h[i] = hp;  // true states
            }
          }
          {
            float pC[8];
#pragma unroll
            for (int i = 0; i < KI; ++i) pC[i] = dy[i] * h[i];
            sel.add<1>(tiles[n], pC);
          }
          if (has_z) {
#pragma unroll
            for (int i = 0; i < KI; ++i) y[i] = __builtin_fmaf(h[i], Cv[i], y[i]);
          }
          // adjoint recurrence g[t] = dy[t] C[t] + a[t+1] g[t+1]; Cv becomes dy * C
          const float a_next_lane = dpp_f<DPP_ROW_SHL + 1>(an, a[0]);
#pragma unroll
          for (int i = 0; i < KI; ++i) Cv[i] *= dy[i];
          float rb = Cv[KI - 1];
#pragma unroll
          for (int i = KI - 2; i >= 0; --i) rb = __builtin_fmaf(a[i + 1], rb, Cv[i]);
          float ra = fast_exp2(dtail * A2) * a_next_lane;
          row_scan_rev1(ra, rb);
          const float gfirst = __builtin_fmaf(ra, gc, rb);
          const float gx = dpp_f<DPP_ROW_SHL + 1>(gc, gfirst);  // adjoint at the next lane's first item
          float dAp = 0.f;
          float pB[8];
          float gi = gx, an_i = a_next_lane;
#pragma unroll
          for (int i = KI - 1; i >= 0; --i) {
            gi = __builtin_fmaf(an_i, gi, Cv[i]);
            an_i = a[i];
            pB[i] = gi * du[i];
            acc[i] = __builtin_fmaf(gi, Bv[i], acc[i]);
            const float w = (gi * a[i]) * (i > 0 ? h[i - 1] : hin);  // g * a * h[t-1]
            dd[i] = __builtin_fmaf(A1, w, dd[i]);
            dAp = __builtin_fmaf(dl[i], w, dAp);
          }
          sel.add<0>(tiles[n], pB);
          dAp = row_sum_to_last(dAp);
          // the record's carries belong to the row's first lane, its dA sum to the row's last lane
          float *rec = reinterpret_cast<float *>(srow + n);
          if (c == 0) *reinterpret_cast<f32x2 *>(rec + 1) = f32x2{gfirst, a[0]};
          if (c == RL - 1) rec[3] = dA_old + dAp;
          // The running sums are pinned here: left alone, the compiler moves a state's additions to the sums' first
          // reader behind the loop and keeps the operands of all sixteen states in scratch memory until then.
          pin8(acc);
          pin8(dd);
          if (has_z) pin8(y);
        }
        if (NBLK > 1 || r == npass - 1) {
          // One partial per workgroup: the tiles of the 8 waves added through LDS in wave order and written with
          // plain stores (positions past the end and padded states are skipped).  Lane l of tile n holds rows
          // 4 (l / 16) .. + 3 of column l % 16: dB (l < 32) or dC of positions 8 (l % 16) + 4 (l / 16 % 2) .. + 3.
          const int n0 = nb * NB16;
          const int64_t part = part0 + (NBLK > 1 ? r : 0);
          f32x4 *red4 = reinterpret_cast<f32x4 *>(red);
#pragma unroll
          for (int chunk = 0; chunk < NB16 / RED_STATES; ++chunk) {
            lds_barrier();  // the scratch is free
#pragma unroll
            for (int k = 0; k < RED_STATES; ++k) {
              red4[(wave * RED_STATES + k) * 64 + lane] = tiles[chunk * RED_STATES + k];
              tiles[chunk * RED_STATES + k] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            lds_barrier();
            if (wave < RED_STATES) {  // wave w adds state chunk * RED_STATES + w
              f32x4 v = red4[wave * 64 + lane];
#pragma unroll
              for (int k = 1; k < NWAVES; ++k) {
                const f32x4 w = red4[(k * RED_STATES + wave) * 64 + lane];
                v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
              }
              const int n = chunk * RED_STATES + wave, which = lane >> 5;
              const int t = t0 + KI * c + 4 * ((lane >> 4) & 1);
              if (n0 + n < N && t < L) {
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
        }
      }
      {
        float o[8], u[8];
        const BwdRow<T> w = rows[chw];
        const float Dd = w.D;
        Pack8<T> u_k, z_k, dout_k;  // the step's rows as stored, parked in LDS by this lane
        u_k.w = park[tid];
        z_k.w = park[NTHREADS + tid];
        dout_k.w = park[2 * NTHREADS + tid];
        u_k.unpack(u);
        float dbs = 0.f, dDs = 0.f;
#pragma unroll
        for (int i = 0; i < KI; ++i) {
          u[i] = (i < nvalid) ? u[i] : 0.f;
          o[i] = __builtin_fmaf(dl[i], acc[i], Dd * dy[i]);
        }
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
    p.dA_part[((int64_t)b * p.dim + d) * N + n] = st4[ch * NP + n].w;
  }
  for (int ch = tid; ch < WCH; ch += NTHREADS) {
    const int d = d0 + ch;
    if (d >= q.dend) continue;
    p.dD_part[(int64_t)b * p.dim + d] = dDacc[ch];
    p.ddelta_bias_part[(int64_t)b * p.dim + d] = dbacc[ch];
  }
}

}  // namespace

bool mamba1_allow_lds(const void *kernel, size_t lds);  // mamba1_scan.hip

// LDS bytes of the kernel above for `passes` passes of PASS_CH channels and `np` padded states.
size_t mamba1_bwd_mx_lds(int passes, int np) {
  const int wch = passes * PASS_CH;
  return sizeof(float) * (2 * BC_FLOATS + RED_FLOATS + PASS_CH * np + 4 * wch * np + 2 * wch) +
         (size_t)3 * NTHREADS * 16 + (size_t)wch * 80;  // + parked rows + BwdRow per channel
}

// Launches the kernel (bf16 rows, per-position B and C).  `vec`: every row is 16-byte aligned and whole groups of 8.
int mamba1_bwd_mx_launch(const MambaScanParams &p, int passes, bool vec, hipStream_t stream) {
  const int np = (p.dstate + NB16 - 1) / NB16 * NB16;
  const size_t lds = mamba1_bwd_mx_lds(passes, np);
  if (lds > 160 * 1024 || p.dtype != MAMBA_BF16 || (p.bc_const & 3)) return MAMBA_E_UNSUPPORTED;
  const int Dg = p.dim / p.ngroups;
  const int cblocks = (Dg + PASS_CH * passes - 1) / (PASS_CH * passes);
  auto kernel = p.z ? (vec ? scan_bwd_mx_kernel<bf16_t, true, true> : scan_bwd_mx_kernel<bf16_t, false, true>)
                    : (vec ? scan_bwd_mx_kernel<bf16_t, true, false> : scan_bwd_mx_kernel<bf16_t, false, false>);
  if (!mamba1_allow_lds(reinterpret_cast<const void *>(kernel), lds)) return MAMBA_E_LAUNCH;
  dim3 grid(p.ngroups * cblocks, p.batch), block(NTHREADS);
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, p, passes);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}
