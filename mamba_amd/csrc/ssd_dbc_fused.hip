// SSD backward, the chunk-state parts of dB and dC (and the ddA_cumsum rows that come with dC), for bf16 on gfx950
// (reference mamba_ssm/ops/triton/ssd_chunk_state.py:902 _chunk_state_bwd_db and ssd_chunk_scan.py:1451
// _chunk_scan_bwd_dC; the same sums as bwd_dB_state_wide_kernel / bwd_dC_state_wide_kernel in ssd_bwd.hip):
//     dB[s, n] += sum_{h in group} w_h[s] sum_p x[s, h, p] dS[h, p, n],   w_h[s] = dt_s exp(a_last - a_s), s in the
//                                                                          chunk's last sequence, else 0
//     dC[l, n] += sum_{h in group} v_h[l] sum_p g[l, h, p] H[h, p, n],    v_h[l] = exp(a_l), l in the sequence the
//                                                                          chunk was entered in, else 0
//     ddA_cumsum[h, l] += sum_n (v_h[l] sum_p g[l, h, p] H[h, p, n]) C[l, n]
// with dS the gradient of the state a chunk hands on and H the state it was entered with.  One launch does both: half
// of its workgroups take dC, half dB.  One workgroup of one wave
// per 16 positions works through a list of heads of one (batch, chunk, group): a head's rows (x or g, as they lie in
// memory) and its P x N matrix are staged in LDS, two heads deep, so that a single barrier per head separates the
// waves' products from the next commit and the loads of the head after next are in flight meanwhile.  Wave w owns
// positions 16 w .. 16 w + 15 and keeps their sum over the heads in registers (fp32, N / 16 tiles); the per-position
// weight is applied to the fp32 product of each head, not to the bf16 operand.  The matrix is the B operand with
// k = p: its fragments come from transposing LDS reads.
#include "ssd_common.hpp"

namespace {

DEVI f32x4 mfma_bf16(bf16x8_t a, bf16x8_t b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

constexpr int MAXHB = 40;  // heads per workgroup at most (dbc_heads_per_workgroup never picks more)

// LDS of one staged head: rows of x / g (pitch P + 8: 16-byte aligned pieces), the matrix (pitch N + 16: the
// transposing reads of a half-wave cover all 64 banks once), the weight per position.
template <int PT, int NK, int QT> struct DbcBuf {
  uint16_t Rs[16 * QT * (16 * PT + 8)];
  uint16_t Ms[16 * PT * (32 * NK + 16)];
  float w[16 * QT];
};

// One of the two products for the workgroup's list of heads (list number `lb` of those of the launch).
template <int PT, int NK, int QT, bool IS_C, bool DET>
DEVI void dbc_body(const SsdParams &p, const int hb, const int lb, DbcBuf<PT, NK, QT> *buf, float (*dda_s)[16 * QT]) {
  constexpr int P = 16 * PT, N = 32 * NK, Q = 16 * QT, NT = 64 * QT, NTL = N / 16, KK = P / 32;
  constexpr int XP = P + 8, BP = N + 16;
  using Buf = DbcBuf<PT, NK, QT>;

  int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int j = lane & 15, g = lane >> 4;
  const int H = p.nheads, G = p.ngroups, L = p.seqlen;
  // the heads of a workgroup are `per` apart: workgroups in flight together touch neighbouring heads
  const int hpg = H / G, per = hpg / hb;
  const int grp = lb / per, h_first = grp * hpg + lb % per;
  const int c = blockIdx.y, b = blockIdx.z;
  const int t0 = c * Q;
  const int qlim = min(Q, L - t0);
  const float dsc = det_scale_of(p);
  const View4 gv = g_view(p);
  const bf16_t *rows_base = IS_C ? static_cast<const bf16_t *>(gv.ptr) + b * gv.bs : static_cast<const bf16_t *>(p.x) + b * p.x_bs;
  const int64_t r_ls = IS_C ? gv.ls : p.x_ls, r_hs = IS_C ? gv.hs : p.x_hs;
  const bf16_t *mats = static_cast<const bf16_t *>(IS_C ? p.states_lp : p.dstates_lp) + ((int64_t)b * p.nchunks + c) * H * P * N;

  // position tid takes part: inside the sequence, and in the sequence the carried state belongs to
  bool row_ok = false;
  if (tid < Q) {
    row_ok = tid < qlim;
    if (p.seq_idx && row_ok) {
      const int32_t *seq = p.seq_idx + (int64_t)b * L + t0;
      if (IS_C) {
        row_ok = seq[tid] == (c > 0 ? seq[-1] : 0);
      } else {
        const int last = seq[qlim - 1];
        row_ok = last >= 0 && seq[tid] == last;
      }
    }
  }

  // ---- global -> registers -> LDS in 16-byte pieces, no branch around a load (rows past the end of the sequence
  // re-read its last row; their weight is zero)
  constexpr int GCH = Q * P / 8 / NT;
  static_assert(GCH * NT * 8 == Q * P, "whole pieces per thread");
  constexpr int HCH = (P * N / 8 + NT - 1) / NT;
  static_assert(NT >= Q, "one position per thread");
  u32x4 rregs[GCH], mregs[HCH];
  float sc_a = 0.f, sc_alast = 0.f, sc_dt = 0.f;
  auto load_head = [&](int h) {
    const bf16_t *rr = rows_base + h * r_hs;
#pragma unroll
    for (int q = 0; q < GCH; ++q) {
      const int id = tid + q * NT, r = id / (P / 8), c8 = id % (P / 8);
      rregs[q] = *(const GLOBAL_AS u32x4 *)(rr + (int64_t)(t0 + min(r, qlim - 1)) * r_ls + c8 * 8);
    }
    const bf16_t *mm = mats + (int64_t)h * P * N;
#pragma unroll
    for (int q = 0; q < HCH; ++q) mregs[q] = *(const GLOBAL_AS u32x4 *)(mm + (int64_t)min(tid + q * NT, P * N / 8 - 1) * 8);
    const float *dA = p.dA_cumsum + (((int64_t)b * H + h) * p.nchunks + c) * Q;
    const int pos = min(tid, Q - 1);
    sc_a = *(const GLOBAL_AS float *)(dA + pos);
    if (!IS_C) {
      sc_alast = *(const GLOBAL_AS float *)(dA + Q - 1);
      sc_dt = *(const GLOBAL_AS float *)(p.dt_out + (((int64_t)b * H + h) * p.nchunks + c) * Q + pos);
    }
  };
  auto commit_head = [&](Buf &B) {
#pragma unroll
    for (int q = 0; q < GCH; ++q) {
      const int id = tid + q * NT, r = id / (P / 8), c8 = id % (P / 8);
      *reinterpret_cast<u32x4 *>(&B.Rs[r * XP + c8 * 8]) = rregs[q];
    }
#pragma unroll
    for (int q = 0; q < HCH; ++q) {
      const int id = tid + q * NT, pp = id / (N / 8), c8 = id % (N / 8);
      if (id < P * N / 8) *reinterpret_cast<u32x4 *>(&B.Ms[pp * BP + c8 * 8]) = mregs[q];
    }
    if (tid < Q) {
      const float wv = IS_C ? fast_exp(sc_a) : fast_exp(fminf(sc_alast - sc_a, 0.f)) * sc_dt;
      B.w[tid] = row_ok ? wv : 0.f;
    }
  };

  load_head(h_first);

  // C at this lane's accumulator positions (rows 16 wave + 4 g + r, columns 16 nt + j): the wave's 16 rows go to
  // LDS as they lie in memory (the staging buffers are still empty) and a transposing read hands lane (j, g) column
  // 16 nt + j of rows 4 g .. 4 g + 3, which is that layout; cr(nt, r) is then one half of a register.
  u32x2 crp[IS_C ? NTL : 1];
  if (IS_C) {
    constexpr int CPP = 64 + 16;  // pitch of the patch (bf16): 16 rows x 64 columns at a time
    static_assert(sizeof(Buf) * 2 >= (size_t)(Q / 16) * 16 * CPP * 2, "the waves' patches fit in the staging buffers");
    uint16_t *Cw = reinterpret_cast<uint16_t *>(&buf[0]) + wave * 16 * CPP;
    const bf16_t *Cg = static_cast<const bf16_t *>(p.C) + b * p.C_bs + grp * p.C_gs;
#pragma unroll
    for (int half = 0; half < N / 64; ++half) {
#pragma unroll
      for (int q = 0; q < 2; ++q) {  // 16 rows x 8 pieces of 8 columns
        const int id = lane + q * 64, rr = id >> 3, c8 = id & 7;
        const u32x4 v = *(const GLOBAL_AS u32x4 *)(Cg + (int64_t)(t0 + min(wave * 16 + rr, qlim - 1)) * p.C_ls + half * 64 + c8 * 8);
        *reinterpret_cast<u32x4 *>(&Cw[rr * CPP + c8 * 8]) = v;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        typedef __attribute__((address_space(3))) i16x4_t *lds_ptr;
        const i16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)&Cw[(4 * g + (j >> 2)) * CPP + t * 16 + 4 * (j & 3)]);
        crp[half * 4 + t] = __builtin_bit_cast(u32x2, v);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    lds_barrier();  // every wave has its C values before the first head is committed over the patches
  }
  auto cr = [&](int nt, int r) {
    const uint32_t w = (r & 2) ? crp[nt].y : crp[nt].x;
    return (r & 1) ? bf16_hi(w) : bf16_lo(w);
  };

  f32x4 sum[NTL];
#pragma unroll
  for (int nt = 0; nt < NTL; ++nt) sum[nt] = f32x4{0.f, 0.f, 0.f, 0.f};

  commit_head(buf[0]);
  load_head(h_first + min(1, hb - 1) * per);
  lds_barrier();

#pragma unroll 1
  for (int hh = 0; hh < hb; ++hh) {
    // the thread's indices pass through an empty asm once per head, so that the addresses derived from them are
    // computed where they are used instead of being carried (or spilled) across the loop over the heads
    asm volatile("" : "+v"(tid), "+v"(lane), "+v"(j), "+v"(g));
    Buf &B = buf[hh & 1];
    f32x4 acc[NTL];
#pragma unroll
    for (int nt = 0; nt < NTL; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      // k slots of lane group g: p = 32 kk + 4 g .. + 3, then 16 further on (both operands alike)
      const uint16_t *ar = &B.Rs[(wave * 16 + j) * XP + kk * 32 + 4 * g];
      const u32x2 a_lo = *reinterpret_cast<const u32x2 *>(ar), a_hi = *reinterpret_cast<const u32x2 *>(ar + 16);
      const bf16x8_t af = __builtin_bit_cast(bf16x8_t, u32x4{a_lo.x, a_lo.y, a_hi.x, a_hi.y});
#pragma unroll
      for (int nt = 0; nt < NTL; ++nt) {
        typedef __attribute__((address_space(3))) i16x4_t *lds_ptr;
        typedef short i16x8_t __attribute__((ext_vector_type(8)));
        const uint16_t *src = &B.Ms[(kk * 32 + 4 * g + (j >> 2)) * BP + nt * 16 + 4 * (j & 3)];
        const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)src);
        const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(src + 16 * BP));
        const bf16x8_t bfr = __builtin_bit_cast(bf16x8_t, (i16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        acc[nt] = mfma_bf16(af, bfr, acc[nt]);
      }
    }
    const f32x4 wv = *reinterpret_cast<const f32x4 *>(&B.w[wave * 16 + 4 * g]);
    if (IS_C) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float rs = 0.f;
#pragma unroll
        for (int nt = 0; nt < NTL; ++nt) rs = __builtin_fmaf(acc[nt][r], cr(nt, r), rs);
        rs *= wv[r];
        rs += dpp_f<DPP_ROW_SHR + 1>(0.f, rs);
        rs += dpp_f<DPP_ROW_SHR + 2>(0.f, rs);
        rs += dpp_f<DPP_ROW_SHR + 4>(0.f, rs);
        rs += dpp_f<DPP_ROW_SHR + 8>(0.f, rs);
        if (j == 15) dda_s[hh][wave * 16 + 4 * g + r] = rs;
      }
    }
#pragma unroll
    for (int nt = 0; nt < NTL; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) sum[nt][r] = __builtin_fmaf(acc[nt][r], wv[r], sum[nt][r]);

    // the next head's operands go to the other buffer (last read one head ago, before the barrier that ended that
    // head); the loads of the head after it follow, then the one barrier of this head
    commit_head(buf[(hh + 1) & 1]);
    load_head(h_first + min(hh + 2, hb - 1) * per);
    lds_barrier();
  }

  // ---- the sums over this workgroup's heads join those of the others
  float *dst = IS_C ? p.dC32 : p.dB32;
  int64_t *shadow = IS_C ? p.det_dC : p.det_dB;
  // (the same adds as whole 128-byte lines of a row, through a patch per wave, measured no faster: 20 of a launch's
  // ~85 us go into these atomics, and it is their number that costs).  A workgroup that holds all heads of its group
  // is the only one to touch its rows of dB / dC, and the first of the backward pass to do so: it stores them, so
  // the caller need not clear them (ssd_bwd_overwrites reports this case).
  const bool alone = per == 1 && !DET;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int l = wave * 16 + 4 * g + r;
    if (l >= qlim) continue;
    const int64_t row = (((int64_t)b * L + t0 + l) * G + grp) * N + j;
    if (alone) {
#pragma unroll
      for (int nt = 0; nt < NTL; ++nt) dst[row + nt * 16] = sum[nt][r];
    } else {
#pragma unroll
      for (int nt = 0; nt < NTL; ++nt) acc_add<DET ? 1 : 0>(dst, shadow, row + nt * 16, sum[nt][r], dsc);
    }
  }
  if (IS_C) {
    for (int idx = tid; idx < hb * Q; idx += NT) {
      const int hh = idx / Q, l = idx % Q;
      const float d = dda_s[hh][l];
      if (l < qlim && d != 0.f)
        acc_add<DET ? 1 : 0>(p.ddA_cumsum, p.det_ddA_cumsum, chunk_off(p, b, h_first + hh * per, c) + l, d, dsc);
    }
  }
}

// Both products in one launch: the first half of the workgroups along x takes dC, the second dB, each for one list
// of heads.  With lists twice as long as a launch per product would use to fill the chip there are half as many
// lists to add up with atomics, the two prologues run side by side, and the whole chip is busy to the end.
template <int PT, int NK, int QT, bool DET>
__global__ __launch_bounds__(64 * QT) void bwd_dbc_fused_kernel(const SsdParams p, const int hb) {
  __shared__ __align__(16) DbcBuf<PT, NK, QT> buf[2];
  __shared__ float dda_s[MAXHB][16 * QT];  // the heads' ddA_cumsum rows of the dC product, flushed at the end
  const int nlists = gridDim.x / 2;
  if ((int)blockIdx.x < nlists) dbc_body<PT, NK, QT, true, DET>(p, hb, blockIdx.x, buf, dda_s);
  else dbc_body<PT, NK, QT, false, DET>(p, hb, blockIdx.x - nlists, buf, dda_s);
}

// Heads per workgroup for that launch: a divisor of the heads per group, MAXHB at most, by the same estimate as
// heads_per_workgroup with the fixed cost these kernels measure (prologue and final adds: about 8 heads' worth).
inline int dbc_heads_per_workgroup(const SsdParams &p) {
  const int hpg = p.nheads / p.ngroups, cus = cu_count();
  const int64_t tiles = (int64_t)p.nchunks * p.batch;
  int best = 1;
  double best_cost = 1e30;
  for (int hb = 1; hb <= MAXHB && hb <= hpg; ++hb) {
    if (hpg % hb) continue;
    const int64_t wgs = 2 * tiles * (p.nheads / hb);
    const double cost = (double)((wgs + cus - 1) / cus) * (8.0 + hb);
    if (cost < best_cost - 1e-9) best = hb, best_cost = cost;
  }
  return best;
}

template <int PT, int NK, bool DET> int launch_q(const SsdParams &p, hipStream_t s) {
  const int hb = dbc_heads_per_workgroup(p);
  dim3 grid(2 * (p.nheads / hb), p.nchunks, p.batch);
  switch (p.chunk_size) {
    case 256: hipLaunchKernelGGL((bwd_dbc_fused_kernel<PT, NK, 16, DET>), grid, dim3(1024), 0, s, p, hb); break;
    case 128: hipLaunchKernelGGL((bwd_dbc_fused_kernel<PT, NK, 8, DET>), grid, dim3(512), 0, s, p, hb); break;
    case 64: hipLaunchKernelGGL((bwd_dbc_fused_kernel<PT, NK, 4, DET>), grid, dim3(256), 0, s, p, hb); break;
    default: return MAMBA_E_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}
template <bool DET> int launch_pn(const SsdParams &p, hipStream_t s) {
  if (p.headdim == 64) return p.dstate == 128 ? launch_q<4, 4, DET>(p, s) : launch_q<4, 2, DET>(p, s);
  return p.dstate == 128 ? launch_q<2, 4, DET>(p, s) : launch_q<2, 2, DET>(p, s);
}

bool supported(const SsdParams *p) {
  if (p->dtype != MAMBA_BF16 || !p->dstates_lp || !p->states_lp) return false;
  if (p->headdim != 32 && p->headdim != 64) return false;
  if (p->dstate != 64 && p->dstate != 128) return false;
  if (p->chunk_size != 64 && p->chunk_size != 128 && p->chunk_size != 256) return false;
  // 16-byte pieces of the x and g rows
  const void *gptr = p->z ? static_cast<const void *>(p->gbuf) : p->dout;
  if (!gptr || !p->dB32 || !p->dC32 || !p->ddA_cumsum) return false;
  if (!aligned(p->x, 16) || !aligned(gptr, 16) || !aligned(p->dstates_lp, 16) || !aligned(p->states_lp, 16)) return false;
  if (p->x_bs % 8 || p->x_ls % 8 || p->x_hs % 8) return false;
  if (!p->z && (p->dout_bs % 8 || p->dout_ls % 8 || p->dout_hs % 8)) return false;
  if (p->batch > 65535 || p->nchunks > 65535) return false;
  return true;
}

}  // namespace

// True when ssd_bwd_dbc_fused_launch runs for this problem with one workgroup per (chunk, group): that workgroup
// stores its rows of dB32 / dC32.
bool ssd_bwd_dbc_fused_owns(const SsdParams *p) {
  if (p->det_scale || !supported(p)) return false;
  const int hb = dbc_heads_per_workgroup(*p);
  return hb == p->nheads / p->ngroups && 2 * (p->nheads / hb) <= 65535;
}

int ssd_bwd_dbc_fused_launch(const SsdParams *p, hipStream_t stream) {
  if (!supported(p)) return MAMBA_E_UNSUPPORTED;
  if (2 * (p->nheads / dbc_heads_per_workgroup(*p)) > 65535) return MAMBA_E_UNSUPPORTED;
  return p->det_scale ? launch_pn<true>(*p, stream) : launch_pn<false>(*p, stream);
}
