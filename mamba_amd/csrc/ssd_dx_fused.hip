// SSD backward, dx (and the ddt / chunk-state ddA terms that come with it), fused with the C B^T contraction, for
// bf16 on gfx950.  The mirror image of the fused forward scan (ssd_scan_fused.hip; reference
// mamba_ssm/ops/triton/ssd_combined.py:94 _chunk_scan_chunk_state_bwd_dx, which reads a stored CB):
//     acc[p, s]  = w_s sum_n dS[p, n] B[s, n]                                  (carried-state part, MFMA)
//                + sum_{l >= s, same sequence} g[l, p] exp(a_l - a_s) sum_n C[l, n] B[s, n]
//     dx[s, p]   = dt_s acc[p, s] + D_p g[s, p]
//     ddt_out[s] += <x_s, acc_s>;  ddA_cumsum[s] -= dt_s <x_s, state part>, the same sum added at the chunk's end.
// One workgroup of one wave per 16 positions; wave w owns the positions s of tile w and keeps their B rows in
// registers as the B operand of both contractions.  S'[l, s] = C_l . B_s leaves the first MFMA with 4 consecutive l
// per lane for one s, which is the B-operand layout of the second one (k = l), so the masked product never leaves
// registers and CB is not read.  The chunk's C rows (the same for every head of the group) sit in LDS for the
// workgroup's whole list of heads, a head's g rows and state gradient for that head; between the barrier that
// publishes them and the one before the epilogue the waves run free.  Below the diagonal tile the decay is factored
// as exp(a_l - a_t) exp(a_t - a_s) with a_t the first a of the l tile (both exponents <= 0): one multiply per element
// and one exponential per lane and tile; the diagonal tile uses the exact form.
#include "ssd_common.hpp"

namespace {

DEVI f32x4 mfma_bf16(bf16x8_t a, bf16x8_t b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
DEVI bf16x8_t ld_frag(const uint16_t *p) { return *reinterpret_cast<const bf16x8_t *>(p); }

template <int PT, int NK, int QT, bool DET>
__global__ __launch_bounds__(64 * QT) void bwd_dx_fused_kernel(const SsdParams p, const int hb, const int sum_dD) {
  constexpr int P = 16 * PT, N = 32 * NK, Q = 16 * QT, NSB = Q / 32, NT = 64 * QT;
  constexpr int BP = N + 8;   // LDS pitch of a C row / dS row (bf16): 16-byte aligned, bank-spread
  constexpr int XP = P + 16;  // LDS pitch of a g row (one position, P values + pad), as it lies in memory
  constexpr int YP = P + 4;   // fp32 pitch of the epilogue's per-wave transpose patch (rows 4 banks apart)
  __shared__ __align__(16) uint16_t Cs[Q * BP];  // the chunk's C rows
  struct Head {
    uint16_t Gs[Q * XP];  // the head's g rows
    uint16_t Ss[P * BP];  // the gradient of the state the chunk hands on, rows p
  };
  union __align__(16) Shared {
    Head hd;                     // state product and causal loop
    float ypatch[QT * 16 * YP];  // epilogue (g and the state gradient are dead by then)
  };
  __shared__ Shared shm;
  auto &Gs = shm.hd.Gs;
  auto &Ss = shm.hd.Ss;
  __shared__ __align__(16) float a2_s[Q], el_s[Q], dt_s[Q], w_s[Q];
  __shared__ int seq_s[Q];
  __shared__ __align__(16) float d_s[P];
  __shared__ float dd_s[QT];  // sum_dD: each wave's <g, x> of the head over its 16 positions

  int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int j = lane & 15, g = lane >> 4;
  const int H = p.nheads, G = p.ngroups, L = p.seqlen;
  // the heads of a workgroup are `per` apart: workgroups in flight together touch neighbouring heads
  const int hpg = H / G, per = hpg / hb;
  const int grp = blockIdx.x / per, h_first = grp * hpg + blockIdx.x % per;
  const int c = blockIdx.y, b = blockIdx.z;
  const int lt = wave, first = lt >> 1;  // this wave's s tile; the l block that holds its diagonal
  const int t0 = c * Q;
  const int qlim = min(Q, L - t0);
  const bf16_t *Bg = static_cast<const bf16_t *>(p.B) + b * p.B_bs + grp * p.B_gs;
  const bf16_t *Cg = static_cast<const bf16_t *>(p.C) + b * p.C_bs + grp * p.C_gs;
  const bool has_seq = p.seq_idx != nullptr;
  const float *Dp = static_cast<const float *>(p.D);
  const View4 gv = g_view(p);
  const float dsc = det_scale_of(p);

  // ---- global -> registers -> LDS in 16-byte pieces, every piece of a tensor dealt to a thread, no branch around a
  // load (rows past the end of the sequence re-read its last row and are zeroed at the commit)
  constexpr int CCH = Q * N / 8 / NT, GCH = Q * P / 8 / NT;
  static_assert(CCH * NT * 8 == Q * N && GCH * NT * 8 == Q * P, "whole pieces per thread");
  constexpr int HCH = (P * N / 8 + NT - 1) / NT;
  static_assert(NT >= Q && NT >= P, "one position / one channel per thread");
  const int s_own = lt * 16 + j;           // the position this lane's column stands for
  const int s_row = min(s_own, qlim - 1);  // its row in memory (positions past the end are never stored)
  u32x4 gregs[GCH], hraw[HCH];
  u32x2 xl[PT];  // x of this lane's column s in the accumulator layout: rows p = 16 pt + 4 g .. + 3
  float sc_a = 0.f, sc_at = 0.f, sc_alast = 0.f, sc_dt = 0.f, sc_d = 0.f;
  bool in_last = false;  // position tid belongs to the last sequence of the chunk
  auto load_head = [&](int h) {
    const bf16_t *gg = static_cast<const bf16_t *>(gv.ptr) + b * gv.bs + h * gv.hs;
#pragma unroll
    for (int q = 0; q < GCH; ++q) {
      const int id = tid + q * NT, r = id / (P / 8), c8 = id % (P / 8);
      gregs[q] = *(const GLOBAL_AS u32x4 *)(gg + (int64_t)(t0 + min(r, qlim - 1)) * gv.ls + c8 * 8);
    }
    const bf16_t *dS = static_cast<const bf16_t *>(p.dstates_lp) + (((int64_t)b * p.nchunks + c) * H + h) * P * N;
#pragma unroll
    for (int q = 0; q < HCH; ++q)
      hraw[q] = *(const GLOBAL_AS u32x4 *)(dS + (int64_t)min(tid + q * NT, P * N / 8 - 1) * 8);
    const float *dA = p.dA_cumsum + (((int64_t)b * H + h) * p.nchunks + c) * Q;
    const float *dt = p.dt_out + (((int64_t)b * H + h) * p.nchunks + c) * Q;
    const int pos = min(tid, Q - 1);
    sc_a = *(const GLOBAL_AS float *)(dA + pos);
    sc_at = *(const GLOBAL_AS float *)(dA + (pos & ~15));
    sc_alast = *(const GLOBAL_AS float *)(dA + Q - 1);
    sc_dt = *(const GLOBAL_AS float *)(dt + pos);
    const float *dsrc = Dp ? Dp + (p.D_has_hdim ? h * P + min(tid, P - 1) : h) : dA;  // any valid address without D
    sc_d = *(const GLOBAL_AS float *)dsrc;
    const bf16_t *xcol = static_cast<const bf16_t *>(p.x) + b * p.x_bs + h * p.x_hs + (int64_t)(t0 + s_row) * p.x_ls + 4 * g;
#pragma unroll
    for (int pt = 0; pt < PT; ++pt) xl[pt] = *(const GLOBAL_AS u32x2 *)(xcol + pt * 16);
  };
  auto commit_head = [&]() {
#pragma unroll
    for (int q = 0; q < GCH; ++q) {
      const int id = tid + q * NT, r = id / (P / 8), c8 = id % (P / 8);
      const bool live = r < qlim;
      const u32x4 v = {live ? gregs[q].x : 0u, live ? gregs[q].y : 0u, live ? gregs[q].z : 0u, live ? gregs[q].w : 0u};
      *reinterpret_cast<u32x4 *>(&Gs[r * XP + c8 * 8]) = v;
    }
#pragma unroll
    for (int q = 0; q < HCH; ++q) {
      const int id = tid + q * NT, pp = id / (N / 8), c8 = id % (N / 8);
      if (id < P * N / 8) *reinterpret_cast<u32x4 *>(&Ss[pp * BP + c8 * 8]) = hraw[q];
    }
    if (tid < Q) {
      a2_s[tid] = sc_a * kLog2e;
      el_s[tid] = fast_exp(fminf(sc_a - sc_at, 0.f));
      dt_s[tid] = sc_dt;
      w_s[tid] = in_last ? fast_exp(fminf(sc_alast - sc_a, 0.f)) : 0.f;
    }
    if (tid < P) d_s[tid] = Dp ? sc_d : 0.f;
  };
  // G^T fragment of p tile pt for l block sb: lane (j, g) gets row p = 16 pt + j and the k slots of lane group g,
  // which are positions 4 g .. 4 g + 3 of the block's first 16-tile, then of its second: the layout in which the
  // first MFMA leaves the masked product.  Each half is one transposing load of a 4 x 16 patch.
  auto g_frag = [&](int sb, int pt) {
    typedef __attribute__((address_space(3))) i16x4_t *lds_ptr;
    typedef short i16x8_t __attribute__((ext_vector_type(8)));
    const uint16_t *src = &Gs[(sb * 32 + 4 * g + (j >> 2)) * XP + pt * 16 + 4 * (j & 3)];
    const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)src);
    const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(src + 16 * XP));
    return __builtin_bit_cast(bf16x8_t, (i16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // ---- prologue: every global load is issued before anything waits
  load_head(h_first);
  bf16x8_t Bf[NK];  // B rows of this wave's s tile: B operand of both contractions (col s = j, k = n)
#pragma unroll
  for (int kk = 0; kk < NK; ++kk)
    Bf[kk] = __builtin_bit_cast(bf16x8_t, *(const GLOBAL_AS u32x4 *)(Bg + (int64_t)(t0 + s_row) * p.B_ls + kk * 32 + g * 8));
  {
    u32x4 craw[CCH];
#pragma unroll
    for (int q = 0; q < CCH; ++q) {
      const int id = tid + q * NT, r = id / (N / 8), c8 = id % (N / 8);
      craw[q] = *(const GLOBAL_AS u32x4 *)(Cg + (int64_t)(t0 + min(r, qlim - 1)) * p.C_ls + c8 * 8);
    }
    if (tid < Q) {
      bool ok = tid < qlim;
      int id = 0;
      if (has_seq) {
        const int32_t *seq = p.seq_idx + (int64_t)b * L + t0;
        id = tid < qlim ? seq[tid] : -2;
        const int lastid = seq[qlim - 1];
        ok = ok && lastid >= 0 && id == lastid;
      }
      seq_s[tid] = id;
      in_last = ok;
    }
#pragma unroll
    for (int q = 0; q < CCH; ++q) {
      const int id = tid + q * NT, r = id / (N / 8), c8 = id % (N / 8);
      const bool live = r < qlim;
      const u32x4 v = {live ? craw[q].x : 0u, live ? craw[q].y : 0u, live ? craw[q].z : 0u, live ? craw[q].w : 0u};
      *reinterpret_cast<u32x4 *>(&Cs[r * BP + c8 * 8]) = v;
    }
  }

  constexpr int EQ = 16 * P / 8 / 64;  // 16-byte pieces per lane of one 16 x P tile
  static_assert(EQ * 64 * 8 == 16 * P, "whole pieces per lane");
  float *Ys = shm.ypatch + wave * 16 * YP;

#pragma unroll 1
  for (int hh = 0; hh < hb; ++hh) {
    const int h = h_first + hh * per;
    // the thread's indices pass through an empty asm once per head, so that the addresses derived from them are
    // computed where they are used instead of being carried (or spilled) across the loop over the heads
    asm volatile("" : "+v"(tid), "+v"(lane), "+v"(j), "+v"(g));
    commit_head();
    lds_barrier();

    f32x4 acc[PT];
    // ---- carried-state part: acc[p, s] = w_s sum_n dS[p, n] B[s, n]
    {
      const float w = w_s[s_own];
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) {
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) v = mfma_bf16(ld_frag(&Ss[(pt * 16 + j) * BP + kk * 32 + g * 8]), Bf[kk], v);
        acc[pt] = v * w;
      }
    }
    // <x_s, a_s>: over this lane's rows, then over the four lane groups of the column
    auto x_dot = [&](const f32x4 (&a)[PT]) {
      float q = 0.f;
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) {
        q = __builtin_fmaf(bf16_lo(xl[pt].x), a[pt][0], q);
        q = __builtin_fmaf(bf16_hi(xl[pt].x), a[pt][1], q);
        q = __builtin_fmaf(bf16_lo(xl[pt].y), a[pt][2], q);
        q = __builtin_fmaf(bf16_hi(xl[pt].y), a[pt][3], q);
      }
      q += __shfl_xor(q, 16, 64);
      q += __shfl_xor(q, 32, 64);
      return q;
    };
    const float q1 = x_dot(acc);

    u32x4 ge[EQ];

    // ---- inside the chunk: the l blocks from the one that holds the wave's diagonal on
    const float as2 = a2_s[s_own];
    const int sid = seq_s[s_own];
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
      if (sb < first) continue;
      float m[8];
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const int ltp = 2 * sb + h2;  // l tile
        if (ltp < lt) {
#pragma unroll
          for (int r = 0; r < 4; ++r) m[h2 * 4 + r] = 0.f;
          continue;
        }
        f32x4 S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) S = mfma_bf16(ld_frag(&Cs[(ltp * 16 + j) * BP + kk * 32 + g * 8]), Bf[kk], S);
        const int l0 = ltp * 16 + 4 * g;
        if (ltp > lt) {
          const float cs = fast_exp2(fminf(a2_s[ltp * 16] - as2, 0.f));
          const f32x4 el = *reinterpret_cast<const f32x4 *>(&el_s[l0]);
#pragma unroll
          for (int r = 0; r < 4; ++r) m[h2 * 4 + r] = S[r] * el[r] * cs;
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            m[h2 * 4 + r] = l0 + r >= s_own ? S[r] * fast_exp2(fminf(a2_s[l0 + r] - as2, 0.f)) : 0.f;
        }
        if (has_seq) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (seq_s[l0 + r] != sid) m[h2 * 4 + r] = 0.f;
        }
      }
      const u32x4 mp = {pack_bf16(m[0], m[1]), pack_bf16(m[2], m[3]), pack_bf16(m[4], m[5]), pack_bf16(m[6], m[7])};
      const bf16x8_t Mf = __builtin_bit_cast(bf16x8_t, mp);
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) acc[pt] = mfma_bf16(g_frag(sb, pt), Mf, acc[pt]);
    }

    // ---- ddt and the chunk-state terms of ddA, from the accumulator layout
    const int64_t row_off = (((int64_t)b * H + h) * p.nchunks + c) * Q;
    {
      const float dts = dt_s[s_own];
      const bool live = g == 0 && s_own < qlim;
      const float q2 = x_dot(acc);
      if (live) {
        acc_add<DET ? 1 : 0>(p.ddt_out, p.det_ddt_out, row_off + s_own, q2, dsc);
        acc_add<DET ? 1 : 0>(p.ddA_cumsum, p.det_ddA_cumsum, row_off + s_own, -dts * q1, dsc);
      }
      const float e = wave_sum_to_last(live ? dts * q1 : 0.f);  // ... and + at the chunk end: one add per wave
      if (lane == 63) acc_add<DET ? 1 : 0>(p.ddA_cumsum, p.det_ddA_cumsum, row_off + Q - 1, e, dsc);
    }

    // ---- dD[h] += sum_{s, p} g[s, p] x[s, p] (a D per head and no gate: g is dout): x in this lane's registers,
    // g of the same column and rows from the head's rows in LDS (zero past the end of the sequence)
    if (sum_dD) {
      float dd = 0.f;
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) {
        const u32x2 gw = *reinterpret_cast<const u32x2 *>(&Gs[s_own * XP + pt * 16 + 4 * g]);
        dd = __builtin_fmaf(bf16_lo(xl[pt].x), bf16_lo(gw.x), dd);
        dd = __builtin_fmaf(bf16_hi(xl[pt].x), bf16_hi(gw.x), dd);
        dd = __builtin_fmaf(bf16_lo(xl[pt].y), bf16_lo(gw.y), dd);
        dd = __builtin_fmaf(bf16_hi(xl[pt].y), bf16_hi(gw.y), dd);
      }
      dd = wave_sum_to_last(dd);
      if (lane == 63) dd_s[wave] = dd;
    }

    // ---- each wave requests the next head's operands as it leaves the loop; the epilogue's patches lie over g and
    // the state gradient, so it starts once every wave has left
    if (hh + 1 < hb) load_head(h + per);
    // the epilogue's g rows (for D) come from the head's rows in LDS, before the patches overlay them
#pragma unroll
    for (int q = 0; q < EQ; ++q) {
      const int id = lane + q * 64, rr = id / (P / 8), c8 = id % (P / 8);
      ge[q] = *reinterpret_cast<const u32x4 *>(&Gs[(lt * 16 + rr) * XP + c8 * 8]);
    }
    lds_barrier();
    if (sum_dD && tid == 0) {  // every wave's part is in (added in a fixed order); the next head's follow two barriers on
      float dd = 0.f;
#pragma unroll
      for (int w = 0; w < QT; ++w) dd += dd_s[w];
      acc_add<DET ? 1 : 0>(p.dD, p.det_dD, h, dd, dsc);
    }
    {
      bf16_t *dxg = static_cast<bf16_t *>(p.dx) + b * p.dx_bs + h * p.dx_hs + (int64_t)(t0 + lt * 16) * p.dx_ls;
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) *reinterpret_cast<f32x4 *>(&Ys[j * YP + pt * 16 + 4 * g]) = acc[pt];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int q = 0; q < EQ; ++q) {  // 16 rows x P/8 pieces of 8 columns
        const int id = lane + q * 64, rr = id / (P / 8), c8 = id % (P / 8);
        if (lt * 16 + rr >= qlim) continue;
        const f32x4 y0 = *reinterpret_cast<const f32x4 *>(&Ys[rr * YP + c8 * 8]);
        const f32x4 y1 = *reinterpret_cast<const f32x4 *>(&Ys[rr * YP + c8 * 8 + 4]);
        const float dts = dt_s[lt * 16 + rr];
        float v[8] = {y0.x, y0.y, y0.z, y0.w, y1.x, y1.y, y1.z, y1.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= dts;
        if (Dp) {
          const u32x4 gw = ge[q];
          const float gf[8] = {bf16_lo(gw.x), bf16_hi(gw.x), bf16_lo(gw.y), bf16_hi(gw.y),
                               bf16_lo(gw.z), bf16_hi(gw.z), bf16_lo(gw.w), bf16_hi(gw.w)};
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = __builtin_fmaf(d_s[c8 * 8 + e], gf[e], v[e]);
        }
        st8<bf16_t>(dxg + (int64_t)rr * p.dx_ls + c8 * 8, v);
      }
    }
    lds_barrier();  // the next head's operands overwrite the patches
  }
}

template <int PT, int NK, bool DET> int launch_q(const SsdParams &p, hipStream_t s, int dd) {
  const int hb = heads_per_workgroup(p);
  dim3 grid(p.nheads / hb, p.nchunks, p.batch);
  switch (p.chunk_size) {
    case 256: hipLaunchKernelGGL((bwd_dx_fused_kernel<PT, NK, 16, DET>), grid, dim3(1024), 0, s, p, hb, dd); break;
    case 128: hipLaunchKernelGGL((bwd_dx_fused_kernel<PT, NK, 8, DET>), grid, dim3(512), 0, s, p, hb, dd); break;
    case 64: hipLaunchKernelGGL((bwd_dx_fused_kernel<PT, NK, 4, DET>), grid, dim3(256), 0, s, p, hb, dd); break;
    default: return MAMBA_E_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}
template <int PT, bool DET> int launch_n(const SsdParams &p, hipStream_t s, int dd) {
  switch (p.dstate) {
    case 64: return launch_q<PT, 2, DET>(p, s, dd);
    case 128: return launch_q<PT, 4, DET>(p, s, dd);
    default: return MAMBA_E_UNSUPPORTED;
  }
}
template <bool DET> int launch_p(const SsdParams &p, hipStream_t s, int dd) {
  return p.headdim == 64 ? launch_n<4, DET>(p, s, dd) : launch_n<2, DET>(p, s, dd);
}

bool supported(const SsdParams *p) {
  if (p->dtype != MAMBA_BF16 || !p->dstates_lp) return false;
  if (p->headdim != 32 && p->headdim != 64) return false;
  if (p->dstate != 64 && p->dstate != 128) return false;
  if (p->chunk_size != 64 && p->chunk_size != 128 && p->chunk_size != 256) return false;
  // 16-byte pieces of rows everywhere
  const void *gptr = p->z ? static_cast<const void *>(p->gbuf) : p->dout;
  if (!gptr) return false;
  if (!aligned(p->x, 16) || !aligned(p->B, 16) || !aligned(p->C, 16) || !aligned(p->dx, 16) || !aligned(gptr, 16) ||
      !aligned(p->dstates_lp, 16))
    return false;
  if (p->x_bs % 8 || p->x_ls % 8 || p->x_hs % 8 || p->B_bs % 8 || p->B_ls % 8 || p->B_gs % 8 || p->C_bs % 8 ||
      p->C_ls % 8 || p->C_gs % 8 || p->dx_bs % 8 || p->dx_ls % 8 || p->dx_hs % 8)
    return false;
  if (!p->z && (p->dout_bs % 8 || p->dout_ls % 8 || p->dout_hs % 8)) return false;
  if (p->batch > 65535 || p->nchunks > 65535) return false;
  return true;
}

}  // namespace

bool ssd_bwd_dx_fused_supported(const SsdParams *p) { return supported(p); }

// With sum_dD the launch also adds the heads' <g, x> to dD (one D per head): the whole of dD where no gate stands
// between dout and g.
int ssd_bwd_dx_fused_launch(const SsdParams *p, hipStream_t stream, bool sum_dD) {
  if (!supported(p)) return MAMBA_E_UNSUPPORTED;
  if (sum_dD && (!p->dD || p->D_has_hdim || (p->det_scale && !p->det_dD))) return MAMBA_E_BADARG;
  return p->det_scale ? launch_p<true>(*p, stream, sum_dD) : launch_p<false>(*p, stream, sum_dD);
}
