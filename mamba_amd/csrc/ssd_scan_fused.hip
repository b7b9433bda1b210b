// SSD chunk_scan forward, fused with the C B^T contraction, for bf16 on gfx950.
//
// One workgroup (one wave per 16 positions of the chunk) computes the whole (chunk_size x headdim) output
// tile of one (batch, chunk, head), and then that of the next head of its list: a workgroup works through
// several heads of one group, whose C rows are the same and stay in registers, and fetches a head's first
// blocks, carried state and scalars before the previous head's epilogue.  A tile is organised like a causal
// attention forward pass whose softmax is replaced by the decay mask:
//     S^T[s, l] = sum_n B[s, n] C[l, n]                       (MFMA; C rows live in registers)
//     M^T[s, l] = S^T[s, l] * dt_s * exp(a_l - a_s)   (s <= l, same sequence)
//     y^T[p, l] += sum_s X^T[p, s] M^T[s, l]                 (MFMA)
// plus the carried state  y^T[p, l] += exp(a_l) sum_n H[p, n] C[l, n].
// Working on the transposes makes the accumulator layout of the first MFMA (4 consecutive s per
// lane for one l) equal to the B-operand layout of the second one, so M never leaves registers
// and CB never goes to memory.  X is staged as it lies in memory (rows of positions) and the second
// MFMA's X^T fragments, with the k order that M^T has, come out of it through the transposing LDS load.
// For positions more than one 16-tile apart the decay is
// factored as exp(a_l - a_end) * exp(a_end - a_s) with a_end the last a of the s tile (both
// exponents <= 0), so the inner loop has one multiply per element instead of an exponential;
// diagonal tiles use the exact form.
#include "ssd_common.hpp"

namespace {

DEVI f32x4 mfma_bf16(bf16x8_t a, bf16x8_t b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
DEVI bf16x8_t ld_frag(const uint16_t *p) { return *reinterpret_cast<const bf16x8_t *>(p); }

// One workgroup of QT waves; wave w owns the 16 positions l of tile w.  The chunk's B rows (the same for every head
// of the group) are put into LDS once, a head's X rows, carried state and scalars once per head, all requested
// before the previous head's epilogue; between the barrier that publishes them and the one before the epilogue the
// waves run free: no staging and no barrier inside the causal loop, so that waves at different places in it keep
// the LDS, matrix and vector pipes busy at the same time (in step, every wave read its fragments, then multiplied,
// then masked, and each pipe idled two thirds of the time).
template <int PT, int NK, int QT>
__global__ __launch_bounds__(64 * QT) void chunk_scan_fwd_fused_kernel(const SsdParams p, const int hb) {
  constexpr int P = 16 * PT, N = 32 * NK, Q = 16 * QT, NSB = Q / 32, NT = 64 * QT;
  constexpr int BP = N + 8;   // LDS pitch of a B row / H row (bf16): 16-byte aligned, bank-spread
  constexpr int XP = P + 16;  // LDS pitch of an X row (one position, P values + pad), as it lies in memory
  constexpr int YP = P + 4;   // fp32 pitch of the epilogue's per-wave transpose patch (rows 4 banks apart)
  __shared__ __align__(16) uint16_t Bs[Q * BP];  // the chunk's B rows
  struct Head {
    uint16_t Xs[Q * XP];  // the head's X rows
    uint16_t Hs[P * BP];  // its carried state, rows p
  };
  union __align__(16) Shared {
    Head hd;                    // state product and causal loop
    float ypatch[QT * 16 * YP]; // epilogue (X and the state are dead by then)
  };
  __shared__ Shared shm;
  auto &Xs = shm.hd.Xs;
  auto &Hs = shm.hd.Hs;
  __shared__ float a2_s[Q], dt_s[Q], cs_s[Q], rs_s[Q];
  __shared__ int seq_s[Q];
  __shared__ __align__(16) float d_s[P];

  int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int j = lane & 15, g = lane >> 4;
  const int H = p.nheads, G = p.ngroups, L = p.seqlen;
  // A workgroup works through hb heads of one group, one after the other; its heads are `per` apart, so that
  // workgroups in flight together, which sit at about the same place in their lists, touch neighbouring heads.
  const int hpg = H / G, per = hpg / hb;
  const int grp = blockIdx.x / per, h_first = grp * hpg + blockIdx.x % per;
  const int c = blockIdx.y, b = blockIdx.z;
  const int lt = wave, last = lt >> 1;  // this wave's l tile; the s block that holds its diagonal
  const int t0 = c * Q;
  const int qlim = min(Q, L - t0);
  const bf16_t *Bg = static_cast<const bf16_t *>(p.B) + b * p.B_bs + grp * p.B_gs;
  const bf16_t *Cg = static_cast<const bf16_t *>(p.C) + b * p.C_bs + grp * p.C_gs;
  const bool has_seq = p.seq_idx != nullptr;
  const bool has_z = p.z != nullptr;
  const float *Dp = static_cast<const float *>(p.D);

  // ---- global -> registers -> LDS in 16-byte pieces, every piece of a tensor dealt to a thread: no thread is idle
  // and no branch surrounds a load (rows past the end of the sequence re-read its last row and are zeroed at the
  // commit), so the compiler's count of the loads in flight is exact.
  constexpr int BCH = Q * N / 8 / NT, XCH = Q * P / 8 / NT;
  static_assert(BCH * NT * 8 == Q * N && XCH * NT * 8 == Q * P, "whole pieces per thread");
  constexpr int HCH = (P * N / 8 + NT - 1) / NT;
  static_assert(NT >= Q && NT >= P, "one position / one channel per thread");
  u32x4 xregs[XCH], hraw[HCH];
  float sc_a = 0.f, sc_aend = 0.f, sc_dt = 0.f, sc_d = 0.f;
  bool carried_ok = false;
  // Everything a head needs from memory: its X rows, the carried state, the per-position scalars, D.  For the
  // first head this is requested together with the B and C rows; for every later head as soon as a wave has left
  // the previous head's causal loop, and it arrives behind the epilogue.
  auto load_head = [&](int h) {
    const bf16_t *xg = static_cast<const bf16_t *>(p.x) + b * p.x_bs + h * p.x_hs;
#pragma unroll
    for (int q = 0; q < XCH; ++q) {
      const int id = tid + q * NT, r = id / (P / 8), c8 = id % (P / 8);
      xregs[q] = *(const GLOBAL_AS u32x4 *)(xg + (int64_t)(t0 + min(r, qlim - 1)) * p.x_ls + c8 * 8);
    }
    const bf16_t *Hc = static_cast<const bf16_t *>(p.states_lp) + (((int64_t)b * p.nchunks + c) * H + h) * P * N;
#pragma unroll
    for (int q = 0; q < HCH; ++q)
      hraw[q] = *(const GLOBAL_AS u32x4 *)(Hc + (int64_t)min(tid + q * NT, P * N / 8 - 1) * 8);
    const float *dA = p.dA_cumsum + (((int64_t)b * H + h) * p.nchunks + c) * Q;
    const float *dt = p.dt_out + (((int64_t)b * H + h) * p.nchunks + c) * Q;
    const int pos = min(tid, Q - 1);
    sc_a = *(const GLOBAL_AS float *)(dA + pos);
    sc_aend = *(const GLOBAL_AS float *)(dA + (pos | 15));
    sc_dt = *(const GLOBAL_AS float *)(dt + pos);
    // D of channel min(tid, P - 1) of this head (0 without D); any valid address stands in when there is no D
    const float *dsrc = Dp ? Dp + (p.D_has_hdim ? h * P + min(tid, P - 1) : h) : dA;
    sc_d = *(const GLOBAL_AS float *)dsrc;
  };
  auto commit_head = [&]() {
#pragma unroll
    for (int q = 0; q < XCH; ++q) {
      const int id = tid + q * NT, r = id / (P / 8), c8 = id % (P / 8);
      const bool live = r < qlim;
      const u32x4 v = {live ? xregs[q].x : 0u, live ? xregs[q].y : 0u, live ? xregs[q].z : 0u, live ? xregs[q].w : 0u};
      *reinterpret_cast<u32x4 *>(&Xs[r * XP + c8 * 8]) = v;
    }
#pragma unroll
    for (int q = 0; q < HCH; ++q) {
      const int id = tid + q * NT, pp = id / (N / 8), c8 = id % (N / 8);
      if (id < P * N / 8) *reinterpret_cast<u32x4 *>(&Hs[pp * BP + c8 * 8]) = hraw[q];
    }
    if (tid < Q) {
      a2_s[tid] = sc_a * kLog2e;
      dt_s[tid] = sc_dt;
      cs_s[tid] = sc_dt * fast_exp(sc_aend - sc_a);
      rs_s[tid] = carried_ok ? fast_exp(sc_a) : 0.f;
    }
    if (tid < P) d_s[tid] = Dp ? sc_d : 0.f;
  };
  // X^T fragment of p tile pt for block sb: lane (j, g) gets row p = 16 pt + j and the k slots of lane group g,
  // which are positions 4 g .. 4 g + 3 of the block's first 16-tile, then of its second: the layout in which the
  // first MFMA leaves M^T.  Each half is one transposing load of a 4 x 16 patch.
  auto x_frag = [&](int sb, int pt) {
    typedef __attribute__((address_space(3))) i16x4_t *lds_ptr;
    typedef short i16x8_t __attribute__((ext_vector_type(8)));
    const uint16_t *src = &Xs[(sb * 32 + 4 * g + (j >> 2)) * XP + pt * 16 + 4 * (j & 3)];
    const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)src);
    const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(src + 16 * XP));
    return __builtin_bit_cast(bf16x8_t, (i16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // ---- prologue: every global load is issued before anything waits
  load_head(h_first);
  bf16x8_t Cf[NK];  // C rows of this wave's l tile: B operand of both contractions (col l = j, k = n)
  {
    const int l = min(lt * 16 + j, qlim - 1);  // rows past the end are never stored
#pragma unroll
    for (int kk = 0; kk < NK; ++kk)
      Cf[kk] = __builtin_bit_cast(bf16x8_t, *(const GLOBAL_AS u32x4 *)(Cg + (int64_t)(t0 + l) * p.C_ls + kk * 32 + g * 8));
  }
  {
    u32x4 braw[BCH];
#pragma unroll
    for (int q = 0; q < BCH; ++q) {
      const int id = tid + q * NT, r = id / (N / 8), c8 = id % (N / 8);
      braw[q] = *(const GLOBAL_AS u32x4 *)(Bg + (int64_t)(t0 + min(r, qlim - 1)) * p.B_ls + c8 * 8);
    }
    // sequence ids of the chunk's positions (the same for every head), and whether the state entering the chunk
    // belongs to the position's sequence
    if (tid < Q) {
      bool ok = tid < qlim;
      int id = 0;
      if (has_seq) {
        const int32_t *seq = p.seq_idx + (int64_t)b * L + t0;
        id = tid < qlim ? seq[tid] : -2;
        ok = ok && id == (c > 0 ? seq[-1] : 0);
      }
      seq_s[tid] = id;
      carried_ok = ok;
    }
#pragma unroll
    for (int q = 0; q < BCH; ++q) {
      const int id = tid + q * NT, r = id / (N / 8), c8 = id % (N / 8);
      const bool live = r < qlim;
      const u32x4 v = {live ? braw[q].x : 0u, live ? braw[q].y : 0u, live ? braw[q].z : 0u, live ? braw[q].w : 0u};
      *reinterpret_cast<u32x4 *>(&Bs[r * BP + c8 * 8]) = v;
    }
  }

  constexpr int EQ = 16 * P / 8 / 64;  // 16-byte pieces per lane of one 16 x P tile
  static_assert(EQ * 64 * 8 == 16 * P, "whole pieces per lane");
  float *Ys = shm.ypatch + wave * 16 * YP;

#pragma unroll 1
  for (int hh = 0; hh < hb; ++hh) {
    const int h = h_first + hh * per;
    // The thread's indices pass through an empty asm once per head: to the compiler they are new values, so the
    // addresses derived from them are computed where they are used, as in a kernel without this loop, instead of
    // being kept in registers (or spilled) across it.
    asm volatile("" : "+v"(tid), "+v"(lane), "+v"(j), "+v"(g));
    commit_head();
    lds_barrier();

    f32x4 acc[PT];
    // ---- carried state: y^T[p, l] = rs_l * sum_n H[p, n] C[l, n]
    {
      const float rs = rs_s[lt * 16 + j];
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) {
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) v = mfma_bf16(ld_frag(&Hs[(pt * 16 + j) * BP + kk * 32 + g * 8]), Cf[kk], v);
        acc[pt] = v * rs;
      }
    }
    // The epilogue's z rows are requested two blocks before the wave's last one.  No branch around these loads
    // either (rows past the end re-read the last row and are not stored; without z the x row stands in).  Its x rows
    // (for D) are taken from the head's X rows in LDS when the wave leaves the loop, before the patches overlay them.
    const bf16_t *xt = static_cast<const bf16_t *>(p.x) + b * p.x_bs + h * p.x_hs + (int64_t)t0 * p.x_ls;
    const bf16_t *zt = has_z ? static_cast<const bf16_t *>(p.z) + b * p.z_bs + h * p.z_hs + (int64_t)t0 * p.z_ls : xt;
    const int64_t zls = has_z ? p.z_ls : p.x_ls;
    u32x4 xe[EQ], ze[EQ];
    auto epilogue_prefetch = [&]() {
#pragma unroll
      for (int q = 0; q < EQ; ++q) {
        const int id = lane + q * 64, rr = id / (P / 8), c8 = id % (P / 8);
        const int64_t row = min(lt * 16 + rr, qlim - 1);
        ze[q] = *(const GLOBAL_AS u32x4 *)(zt + row * zls + c8 * 8);
      }
    };

    // ---- inside the chunk: the wave's blocks, up to the one that holds its diagonal
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
      if (sb > last) break;
      if (sb == max(last - 2, 0)) epilogue_prefetch();
      const int l = lt * 16 + j;
      const float al2 = a2_s[l];
      const int lid = seq_s[l];
      float m[8];
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const int st = 2 * sb + h2;
        if (st > lt) {
#pragma unroll
          for (int r = 0; r < 4; ++r) m[h2 * 4 + r] = 0.f;
          continue;
        }
        f32x4 S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) S = mfma_bf16(ld_frag(&Bs[(st * 16 + j) * BP + kk * 32 + g * 8]), Cf[kk], S);
        const int s0 = st * 16 + 4 * g;
        if (st < lt) {
          const float rl = fast_exp2(al2 - a2_s[st * 16 + 15]);
          const f32x4 cs = *reinterpret_cast<const f32x4 *>(&cs_s[s0]);
#pragma unroll
          for (int r = 0; r < 4; ++r) m[h2 * 4 + r] = S[r] * cs[r] * rl;
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int s = s0 + r;
            m[h2 * 4 + r] = s <= l ? S[r] * dt_s[s] * fast_exp2(fminf(al2 - a2_s[s], 0.f)) : 0.f;
          }
        }
        if (has_seq) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (seq_s[s0 + r] != lid) m[h2 * 4 + r] = 0.f;
        }
      }
      const u32x4 mp = {pack_bf16(m[0], m[1]), pack_bf16(m[2], m[3]), pack_bf16(m[4], m[5]), pack_bf16(m[6], m[7])};
      const bf16x8_t Mf = __builtin_bit_cast(bf16x8_t, mp);
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) acc[pt] = mfma_bf16(x_frag(sb, pt), Mf, acc[pt]);
    }

    // ---- the next head's operands are requested by each wave as it leaves the loop; the epilogue's patches lie
    // over X and the state, so it starts once every wave has left
    if (hh + 1 < hb) load_head(h + per);
#pragma unroll
    for (int q = 0; q < EQ; ++q) {
      const int id = lane + q * 64, rr = id / (P / 8), c8 = id % (P / 8);
      xe[q] = *reinterpret_cast<const u32x4 *>(&Xs[(lt * 16 + rr) * XP + c8 * 8]);
    }
    lds_barrier();
    // epilogue: + D x, pre-gate copy, gate.  Each wave transposes its 16 rows through a private LDS patch so that
    // out / out_x stores are 16-byte pieces of contiguous rows (the accumulator layout itself would scatter 8-byte
    // pieces over 16 rows).
    {
      const int64_t otile = b * p.out_bs + h * p.out_hs + (int64_t)(t0 + lt * 16) * p.out_ls;
      bf16_t *og = static_cast<bf16_t *>(p.out) + otile;
      // without a pre-gate buffer (a forward pass nobody differentiates) the pre-gate store lands on the out row
      // and the gated one after it replaces it in the cache: no branch around a store
      bf16_t *oxg = has_z && p.out_x ? static_cast<bf16_t *>(p.out_x) + otile : og;
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
        float v[8] = {y0.x, y0.y, y0.z, y0.w, y1.x, y1.y, y1.z, y1.w};
        if (Dp) {
          const u32x4 xw = xe[q];
          const float xf[8] = {bf16_lo(xw.x), bf16_hi(xw.x), bf16_lo(xw.y), bf16_hi(xw.y),
                               bf16_lo(xw.z), bf16_hi(xw.z), bf16_lo(xw.w), bf16_hi(xw.w)};
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = __builtin_fmaf(d_s[c8 * 8 + e], xf[e], v[e]);
        }
        const int64_t oi = (int64_t)rr * p.out_ls + c8 * 8;
        if (has_z) {
          st8<bf16_t>(oxg + oi, v);
          const u32x4 zw = ze[q];
          const float zf[8] = {bf16_lo(zw.x), bf16_hi(zw.x), bf16_lo(zw.y), bf16_hi(zw.y),
                               bf16_lo(zw.z), bf16_hi(zw.z), bf16_lo(zw.w), bf16_hi(zw.w)};
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] *= zf[e] * sigmoid_f(zf[e]);
        }
        st8<bf16_t>(og + oi, v);
      }
    }
    lds_barrier();  // the next head's operands overwrite the patches
  }
}

template <int PT, int NK> int launch_q(const SsdParams &p, hipStream_t s) {
  if (ssd_scan_paired_serves(p) && !ssd_single_tile_only()) return ssd_scan_paired_launch(p, s);
  const int hb = heads_per_workgroup(p);
  dim3 grid(p.nheads / hb, p.nchunks, p.batch);
  switch (p.chunk_size) {
    case 256: hipLaunchKernelGGL((chunk_scan_fwd_fused_kernel<PT, NK, 16>), grid, dim3(1024), 0, s, p, hb); break;
    case 128: hipLaunchKernelGGL((chunk_scan_fwd_fused_kernel<PT, NK, 8>), grid, dim3(512), 0, s, p, hb); break;
    case 64: hipLaunchKernelGGL((chunk_scan_fwd_fused_kernel<PT, NK, 4>), grid, dim3(256), 0, s, p, hb); break;
    default: return MAMBA_E_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

template <int PT> int launch_n(const SsdParams &p, hipStream_t s) {
  switch (p.dstate) {
    case 64: return launch_q<PT, 2>(p, s);
    case 128: return launch_q<PT, 4>(p, s);
    default: return MAMBA_E_UNSUPPORTED;
  }
}

}  // namespace

// 1 if ssd_chunk_scan_fwd_fused has a kernel for this problem, else 0.
extern "C" int ssd_chunk_scan_fwd_fused_supported(const SsdParams *p) {
  if (!p || p->dtype != MAMBA_BF16) return 0;
  if (p->headdim != 32 && p->headdim != 64) return 0;
  if (p->dstate != 64 && p->dstate != 128) return 0;
  if (p->chunk_size != 64 && p->chunk_size != 128 && p->chunk_size != 256) return 0;
  // 16-byte pieces of rows everywhere
  if (!aligned(p->x, 16) || !aligned(p->B, 16) || !aligned(p->C, 16) || !aligned(p->out, 16)) return 0;
  if (p->x_bs % 8 || p->x_ls % 8 || p->x_hs % 8 || p->B_bs % 8 || p->B_ls % 8 || p->B_gs % 8 || p->C_bs % 8 ||
      p->C_ls % 8 || p->C_gs % 8)
    return 0;
  if (p->out_bs % 8 || p->out_ls % 8 || p->out_hs % 8) return 0;
  if (p->z && (!aligned(p->z, 16) || !aligned(p->out_x, 16) || p->z_bs % 8 || p->z_ls % 8 || p->z_hs % 8)) return 0;  // (a null out_x is aligned)
  if (p->states_lp && !aligned(p->states_lp, 16)) return 0;
  if (p->batch > 65535 || p->nheads > 65535) return 0;
  return 1;
}

static int ssd_chunk_scan_fwd_fused_one(const SsdParams *p, mamba_stream_t stream) {
  if (!p || !p->x || !p->B || !p->C || !p->states_lp || !p->out || !p->dt_out || !p->dA_cumsum) return MAMBA_E_BADARG;
  if (!ssd_chunk_scan_fwd_fused_supported(p)) return MAMBA_E_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return p->headdim == 64 ? launch_n<4>(*p, s) : launch_n<2>(*p, s);
}

// Public entry points: the whole problem in one go when one launch can index it, else in slices of batch rows.
extern "C" int ssd_chunk_scan_fwd_fused(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_chunk_scan_fwd_fused_one); }
