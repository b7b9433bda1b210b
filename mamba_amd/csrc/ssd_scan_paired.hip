// SSD chunk_scan forward fused with the C B^T contraction (bf16, gfx950): the form in which every wave owns TWO
// 16-position tiles of the chunk, a short one and a long one.
//
// The mathematics and the register hand-over between the two MFMAs are those of chunk_scan_fwd_fused_kernel
// (ssd_scan_fused.hip):
//     S^T[s, l] = sum_n B[s, n] C[l, n]           M^T[s, l] = S^T[s, l] dt_s exp(a_l - a_s)  (s <= l, same sequence)
//     y^T[p, l] += sum_s X^T[p, s] M^T[s, l]      y^T[p, l] += exp(a_l) sum_n H[p, n] C[l, n]
// What differs is the division of the causal triangle.  With one tile per wave, the wave of tile t walks
// t / 2 + 1 blocks of 32 positions: the last wave 8 of them at chunk size 256, the first one 1, and a workgroup
// (the only one its CU has room for) lasts as long as its last wave.  Here wave w owns tiles w and QT - 1 - w,
// which is 9 blocks for every wave at chunk size 256: no wave waits for another one, and both tiles of a wave
// take the B rows and the X^T columns of a block from the same fragment registers (28 % fewer fragment reads from
// LDS), as two independent MFMA chains in one instruction stream.  Half as many waves share the CU's registers, so
// a block's body is straight-line code with the next block's fragments requested under it.
// Reference: mamba_ssm/ops/triton/ssd_chunk_scan.py:49 (_chunk_scan_fwd_kernel), :1259 (_chunk_scan_fwd).
#include <type_traits>

#include "ssd_common.hpp"

namespace {

DEVI f32x4 mfma_bf16(bf16x8_t a, bf16x8_t b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
DEVI bf16x8_t ld_frag(const uint16_t *p) { return *reinterpret_cast<const bf16x8_t *>(p); }
typedef int i32x4 __attribute__((ext_vector_type(4)));

template <int V> using Int = std::integral_constant<int, V>;

template <int PT, int NK, int QT, bool SEQ, bool GATED>
__global__ __launch_bounds__(32 * QT) void chunk_scan_fwd_paired_kernel(const SsdParams p, const int hb) {
  constexpr int P = 16 * PT, N = 32 * NK, Q = 16 * QT, NW = QT / 2, NT = 64 * NW;
  constexpr int BP = N + 8;   // LDS pitch of a B row / H row (bf16): 16-byte aligned, bank-spread
  constexpr int XP = P + 16;  // LDS pitch of an X row (one position, P values + pad), as it lies in memory
  constexpr int YP = P + 4;   // fp32 pitch of the epilogue's per-tile transpose patch (rows 4 banks apart)
  static_assert(QT >= 4 && QT % 2 == 0, "a short and a long tile per wave, on different blocks");
  __shared__ __align__(16) uint16_t Bs[Q * BP];  // the chunk's B rows
  struct Head {
    uint16_t Xs[Q * XP];  // the head's X rows
    uint16_t Hs[P * BP];  // its carried state, rows p
  };
  union __align__(16) Shared {
    Head hd;                     // state product and causal loop
    float ypatch[QT * 16 * YP];  // epilogue (X and the state are dead by then)
  };
  __shared__ Shared shm;
  auto &Xs = shm.hd.Xs;
  auto &Hs = shm.hd.Hs;
  __shared__ __align__(16) float a2_s[Q], dt_s[Q], cs_s[Q], rs_s[Q];
  __shared__ __align__(16) int seq_s[Q];
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
  // this wave's two l tiles and the s blocks that hold their diagonals (last_a < last_b for every wave)
  const int ta = wave, tb = QT - 1 - wave;
  const int last_a = ta >> 1, last_b = tb >> 1;
  const int t0 = c * Q;
  const int qlim = min(Q, L - t0);
  const bf16_t *Bg = static_cast<const bf16_t *>(p.B) + b * p.B_bs + grp * p.B_gs;
  const bf16_t *Cg = static_cast<const bf16_t *>(p.C) + b * p.C_bs + grp * p.C_gs;
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
  // A thread's byte offsets into a head's tensors are the same for every head: they are computed once, and a
  // head's loads are a uniform base (scalar registers) plus a 32-bit offset each, with no address arithmetic in
  // the vector pipe.
  typedef const GLOBAL_AS char *gptr;
  uint32_t xoff[XCH], hoff[HCH];
#pragma unroll
  for (int q = 0; q < XCH; ++q) {
    const int id = tid + q * NT, r = id / (P / 8), c8 = id % (P / 8);
    xoff[q] = (uint32_t)(min(r, qlim - 1) * (int)p.x_ls + c8 * 8) * 2u;
  }
#pragma unroll
  for (int q = 0; q < HCH; ++q) hoff[q] = (uint32_t)min(tid + q * NT, P * N / 8 - 1) * 16u;
  const uint32_t pos_off = (uint32_t)min(tid, Q - 1) * 4u, end_off = (uint32_t)(min(tid, Q - 1) | 15) * 4u;
  const uint32_t d_off = Dp && p.D_has_hdim ? (uint32_t)min(tid, P - 1) * 4u : 0u;
  auto load_head = [&](int h) {
    const gptr xg = (gptr)(static_cast<const bf16_t *>(p.x) + b * p.x_bs + h * p.x_hs + (int64_t)t0 * p.x_ls);
#pragma unroll
    for (int q = 0; q < XCH; ++q) xregs[q] = *(const GLOBAL_AS u32x4 *)(xg + xoff[q]);
    const gptr Hc = (gptr)(static_cast<const bf16_t *>(p.states_lp) + (((int64_t)b * p.nchunks + c) * H + h) * P * N);
#pragma unroll
    for (int q = 0; q < HCH; ++q) hraw[q] = *(const GLOBAL_AS u32x4 *)(Hc + hoff[q]);
    const gptr dA = (gptr)(p.dA_cumsum + (((int64_t)b * H + h) * p.nchunks + c) * Q);
    const gptr dt = (gptr)(p.dt_out + (((int64_t)b * H + h) * p.nchunks + c) * Q);
    sc_a = *(const GLOBAL_AS float *)(dA + pos_off);
    sc_aend = *(const GLOBAL_AS float *)(dA + end_off);
    sc_dt = *(const GLOBAL_AS float *)(dt + pos_off);
    // D of channel min(tid, P - 1) of this head (0 without D); any valid address stands in when there is no D
    const gptr dsrc = Dp ? (gptr)(Dp + (p.D_has_hdim ? h * P : h)) : dA;
    sc_d = *(const GLOBAL_AS float *)(dsrc + d_off);
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
  // The B rows of block sb as the first MFMA's A operand: row s = 16 (2 sb + half) + j, k slots n = 32 kk + 8 g ..
  auto load_b = [&](int sb, bf16x8_t (&bf)[2][NK]) {
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
      for (int kk = 0; kk < NK; ++kk) bf[h2][kk] = ld_frag(&Bs[((2 * sb + h2) * 16 + j) * BP + kk * 32 + g * 8]);
  };

  // ---- prologue: every global load is issued before anything waits
  load_head(h_first);
  bf16x8_t Cfa[NK], Cfb[NK];  // C rows of the two l tiles: B operand of both contractions (col l = j, k = n)
  {
    const int la = min(ta * 16 + j, qlim - 1), lb = min(tb * 16 + j, qlim - 1);  // rows past the end are never stored
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) {
      Cfa[kk] = __builtin_bit_cast(bf16x8_t, *(const GLOBAL_AS u32x4 *)(Cg + (int64_t)(t0 + la) * p.C_ls + kk * 32 + g * 8));
      Cfb[kk] = __builtin_bit_cast(bf16x8_t, *(const GLOBAL_AS u32x4 *)(Cg + (int64_t)(t0 + lb) * p.C_ls + kk * 32 + g * 8));
    }
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
      if (SEQ) {
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
  // the epilogue's pieces: 16 rows x P/8 pieces of 8 columns per tile; byte offsets from the chunk's first row
  uint32_t zoff[2][EQ], ooff[2][EQ];
  bool olive[2][EQ];
#pragma unroll
  for (int e = 0; e < 2; ++e)
#pragma unroll
    for (int q = 0; q < EQ; ++q) {
      const int id = lane + q * 64, row = (e ? tb : ta) * 16 + id / (P / 8), c8 = id % (P / 8);
      zoff[e][q] = GATED ? (uint32_t)(min(row, qlim - 1) * (int)p.z_ls + c8 * 8) * 2u : 0u;
      ooff[e][q] = (uint32_t)(row * (int)p.out_ls + c8 * 8) * 2u;
      olive[e][q] = row < qlim;
    }
  commit_head();
  lds_barrier();

  // A head's pass: the products on what lies in LDS; the request for the next head's operands; the epilogue; the
  // next head's operands into LDS.  Every load and every store sits in straight-line code between the point where
  // it is issued and the point that waits for it (the last head requests its own operands once more instead of
  // branching around the request; stores of rows past the end of the sequence are masked, not branched around), so
  // each wait names exactly the accesses it needs: the epilogue does not wait for the next head's operands, and the
  // commit of those does not wait for the epilogue's stores.
#pragma unroll 1
  for (int hh = 0; hh < hb; ++hh) {
    const int h = h_first + hh * per;
    // The thread's indices pass through an empty asm once per head: to the compiler they are new values, so the
    // addresses derived from them are computed where they are used instead of being kept in registers across the loop.
    asm volatile("" : "+v"(tid), "+v"(lane), "+v"(j), "+v"(g));

    // The epilogue's z rows of both tiles are requested here and arrive under the loop (rows past the end re-read
    // the last row and are not stored).
    u32x4 xe[2][EQ], ze[2][EQ];
    if (GATED) {
      const gptr zt = (gptr)(static_cast<const bf16_t *>(p.z) + b * p.z_bs + h * p.z_hs + (int64_t)t0 * p.z_ls);
#pragma unroll
      for (int e = 0; e < 2; ++e)
#pragma unroll
        for (int q = 0; q < EQ; ++q) ze[e][q] = *(const GLOBAL_AS u32x4 *)(zt + zoff[e][q]);
    }

    const int l_a = ta * 16 + j, l_b = tb * 16 + j;
    const float al2a = a2_s[l_a], al2b = a2_s[l_b];
    const int lida = seq_s[l_a], lidb = seq_s[l_b];

    f32x4 acca[PT], accb[PT];
    // ---- carried state: y^T[p, l] = rs_l * sum_n H[p, n] C[l, n]; a state fragment serves both tiles
    {
      const float rsa = rs_s[l_a], rsb = rs_s[l_b];
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) {
        f32x4 va = {0.f, 0.f, 0.f, 0.f}, vb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) {
          const bf16x8_t hf = ld_frag(&Hs[(pt * 16 + j) * BP + kk * 32 + g * 8]);
          va = mfma_bf16(hf, Cfa[kk], va);
          vb = mfma_bf16(hf, Cfb[kk], vb);
        }
        acca[pt] = va * rsa;
        accb[pt] = vb * rsb;
      }
    }

    // ---- masks.  Below a tile's diagonal the decay is exp(a_l - a_end) * (dt_s exp(a_end - a_s)) with a_end the last
    // a of the 16 positions s (both exponents <= 0): one exponential per lane and 16 positions.
    auto mask_full = [&](const f32x4 &S, const f32x4 &cs, const i32x4 &sq, float aend2, float al2, int lid, float *m) {
      const float rl = fast_exp2(al2 - aend2);
#pragma unroll
      for (int r = 0; r < 4; ++r) m[r] = S[r] * cs[r] * rl;
      if (SEQ) {
#pragma unroll
        for (int r = 0; r < 4; ++r) m[r] = sq[r] != lid ? 0.f : m[r];
      }
    };
    // the 16 positions that hold the tile's diagonal: the exact decay, s <= l
    auto mask_diag = [&](const f32x4 &S, const i32x4 &sq, int st, int l, float al2, int lid, float *m) {
      const int s0 = st * 16 + 4 * g;
      const f32x4 dts = *reinterpret_cast<const f32x4 *>(&dt_s[s0]);
      const f32x4 as2 = *reinterpret_cast<const f32x4 *>(&a2_s[s0]);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float v = S[r] * dts[r] * fast_exp2(fminf(al2 - as2[r], 0.f));
        m[r] = s0 + r <= l ? v : 0.f;
      }
      if (SEQ) {
#pragma unroll
        for (int r = 0; r < 4; ++r) m[r] = sq[r] != lid ? 0.f : m[r];
      }
    };

    bf16x8_t bf[2][NK];
    load_b(0, bf);
    // One block of 32 positions s for the long tile and, while the short tile still has blocks, for it too.
    //   KA: 0 = the short tile is done, 1 = the block lies below its diagonal, 2 = the block holds its diagonal
    //   DB: the block holds the long tile's diagonal (the wave's last block)
    auto step = [&](const int sb, auto ka_tag, auto db_tag) {
      constexpr int KA = decltype(ka_tag)::value;
      constexpr bool DB = decltype(db_tag)::value != 0;
      f32x4 Sa[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, Sb[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
      // the first 16 positions' chains before the second 16's: their masks are vector work under the second's MFMAs
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) {
          Sb[h2] = mfma_bf16(bf[h2][kk], Cfb[kk], Sb[h2]);
          if (KA) Sa[h2] = mfma_bf16(bf[h2][kk], Cfa[kk], Sa[h2]);
        }
      bf16x8_t xf[PT];
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) xf[pt] = x_frag(sb, pt);
      // the per-position factors of the block, shared by both tiles
      f32x4 cs[2];
      i32x4 sq[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
      float aend2[2];
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const int st = 2 * sb + h2;
        cs[h2] = *reinterpret_cast<const f32x4 *>(&cs_s[st * 16 + 4 * g]);
        aend2[h2] = a2_s[st * 16 + 15];
        if (SEQ) sq[h2] = *reinterpret_cast<const i32x4 *>(&seq_s[st * 16 + 4 * g]);
      }
      if (!DB) load_b(sb + 1, bf);  // the next block's B fragments arrive under the masks (sb < last_b here)
      float ma[8], mb[8];
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const int st = 2 * sb + h2;
        if (!DB) {
          mask_full(Sb[h2], cs[h2], sq[h2], aend2[h2], al2b, lidb, mb + 4 * h2);
        } else if (st < tb) {
          mask_full(Sb[h2], cs[h2], sq[h2], aend2[h2], al2b, lidb, mb + 4 * h2);
        } else if (st == tb) {
          mask_diag(Sb[h2], sq[h2], st, l_b, al2b, lidb, mb + 4 * h2);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r) mb[4 * h2 + r] = 0.f;
        }
        if (KA == 1) {
          mask_full(Sa[h2], cs[h2], sq[h2], aend2[h2], al2a, lida, ma + 4 * h2);
        } else if (KA == 2) {
          if (st < ta) {
            mask_full(Sa[h2], cs[h2], sq[h2], aend2[h2], al2a, lida, ma + 4 * h2);
          } else if (st == ta) {
            mask_diag(Sa[h2], sq[h2], st, l_a, al2a, lida, ma + 4 * h2);
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) ma[4 * h2 + r] = 0.f;
          }
        }
      }
      const u32x4 mpb = {pack_bf16(mb[0], mb[1]), pack_bf16(mb[2], mb[3]), pack_bf16(mb[4], mb[5]), pack_bf16(mb[6], mb[7])};
      const bf16x8_t Mfb = __builtin_bit_cast(bf16x8_t, mpb);
      if (KA) {
        const u32x4 mpa = {pack_bf16(ma[0], ma[1]), pack_bf16(ma[2], ma[3]), pack_bf16(ma[4], ma[5]), pack_bf16(ma[6], ma[7])};
        const bf16x8_t Mfa = __builtin_bit_cast(bf16x8_t, mpa);
#pragma unroll
        for (int pt = 0; pt < PT; ++pt) {
          accb[pt] = mfma_bf16(xf[pt], Mfb, accb[pt]);
          acca[pt] = mfma_bf16(xf[pt], Mfa, acca[pt]);
        }
      } else {
#pragma unroll
        for (int pt = 0; pt < PT; ++pt) accb[pt] = mfma_bf16(xf[pt], Mfb, accb[pt]);
      }
      // Order within the block below both diagonals: the chains of the first 16 positions; then those of the second
      // 16, each MFMA followed by three vector instructions of the first 16's masks (an MFMA holds the matrix pipe
      // for four issue slots).
      if (KA == 1 && !DB) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * NK, 0);
#pragma unroll
        for (int i = 0; i < 2 * NK; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
        }
      }
    };

    // ---- inside the chunk: blocks 0 .. last_a for both tiles, last_a + 1 .. last_b for the long one
    {
      int sb = 0;
#pragma unroll 1
      for (; sb < last_a; ++sb) step(sb, Int<1>{}, Int<0>{});
      step(sb, Int<2>{}, Int<0>{});
      ++sb;
#pragma unroll 1
      for (; sb < last_b; ++sb) step(sb, Int<0>{}, Int<0>{});
      step(sb, Int<0>{}, Int<1>{});
    }

    // ---- the next head's operands are requested by each wave as it leaves the loop; the epilogue's patches lie
    // over X and the state, so it starts once every wave has left.  Its x rows (for D) are taken from the head's X
    // rows in LDS before that.
    load_head(h_first + min(hh + 1, hb - 1) * per);
#pragma unroll
    for (int e = 0; e < 2; ++e)
#pragma unroll
      for (int q = 0; q < EQ; ++q) {
        const int id = lane + q * 64, rr = id / (P / 8), c8 = id % (P / 8);
        xe[e][q] = *reinterpret_cast<const u32x4 *>(&Xs[((e ? tb : ta) * 16 + rr) * XP + c8 * 8]);
      }
    lds_barrier();
    // epilogue: + D x, pre-gate copy, gate.  A tile's 16 rows are transposed through an LDS patch of its own so that
    // out / out_x stores are 16-byte pieces of contiguous rows (the accumulator layout itself would scatter 8-byte
    // pieces over 16 rows).
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int lt = e ? tb : ta;
      float *Ys = shm.ypatch + lt * 16 * YP;
      typedef GLOBAL_AS char *gwptr;
      auto store8 = [](gwptr dst, const float (&v)[8]) {
        const u32x4 pk = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
        *(GLOBAL_AS u32x4 *)dst = pk;
      };
      const int64_t otile = b * p.out_bs + h * p.out_hs + (int64_t)t0 * p.out_ls;
      const gwptr og = (gwptr)(static_cast<bf16_t *>(p.out) + otile);
      // without a pre-gate buffer (a forward pass nobody differentiates) the pre-gate store lands on the out row
      // and the gated one after it replaces it in the cache
      const gwptr oxg = p.out_x ? (gwptr)(static_cast<bf16_t *>(p.out_x) + otile) : og;
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) *reinterpret_cast<f32x4 *>(&Ys[j * YP + pt * 16 + 4 * g]) = e ? accb[pt] : acca[pt];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int q = 0; q < EQ; ++q) {  // 16 rows x P/8 pieces of 8 columns
        const int id = lane + q * 64, rr = id / (P / 8), c8 = id % (P / 8);
        const bool live = olive[e][q];
        const f32x4 y0 = *reinterpret_cast<const f32x4 *>(&Ys[rr * YP + c8 * 8]);
        const f32x4 y1 = *reinterpret_cast<const f32x4 *>(&Ys[rr * YP + c8 * 8 + 4]);
        float v[8] = {y0.x, y0.y, y0.z, y0.w, y1.x, y1.y, y1.z, y1.w};
        if (Dp) {
          const u32x4 xw = xe[e][q];
          const float xf[8] = {bf16_lo(xw.x), bf16_hi(xw.x), bf16_lo(xw.y), bf16_hi(xw.y),
                               bf16_lo(xw.z), bf16_hi(xw.z), bf16_lo(xw.w), bf16_hi(xw.w)};
#pragma unroll
          for (int k = 0; k < 8; ++k) v[k] = __builtin_fmaf(d_s[c8 * 8 + k], xf[k], v[k]);
        }
        const uint32_t oi = ooff[e][q];
        if (GATED) {
          if (live) store8(oxg + oi, v);
          const u32x4 zw = ze[e][q];
          const float zf[8] = {bf16_lo(zw.x), bf16_hi(zw.x), bf16_lo(zw.y), bf16_hi(zw.y),
                               bf16_lo(zw.z), bf16_hi(zw.z), bf16_lo(zw.w), bf16_hi(zw.w)};
#pragma unroll
          for (int k = 0; k < 8; ++k) v[k] *= zf[k] * sigmoid_f(zf[k]);
        }
        if (live) store8(og + oi, v);
      }
    }
    lds_barrier();  // the next head's operands overwrite the patches
    commit_head();
    lds_barrier();
  }
}

template <int PT, int NK, int QT> int launch_seq(const SsdParams &p, hipStream_t s) {
  const int hb = heads_per_workgroup(p);
  dim3 grid(p.nheads / hb, p.nchunks, p.batch);
  const dim3 block(32 * QT);
  if (p.seq_idx && p.z)
    hipLaunchKernelGGL((chunk_scan_fwd_paired_kernel<PT, NK, QT, true, true>), grid, block, 0, s, p, hb);
  else if (p.seq_idx)
    hipLaunchKernelGGL((chunk_scan_fwd_paired_kernel<PT, NK, QT, true, false>), grid, block, 0, s, p, hb);
  else if (p.z)
    hipLaunchKernelGGL((chunk_scan_fwd_paired_kernel<PT, NK, QT, false, true>), grid, block, 0, s, p, hb);
  else
    hipLaunchKernelGGL((chunk_scan_fwd_paired_kernel<PT, NK, QT, false, false>), grid, block, 0, s, p, hb);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

template <int PT> int launch_n(const SsdParams &p, hipStream_t s) {
  switch (p.dstate) {
    case 64: return launch_seq<PT, 2, 16>(p, s);
    case 128: return launch_seq<PT, 4, 16>(p, s);
    default: return MAMBA_E_UNSUPPORTED;
  }
}

}  // namespace

// Whether the two-tiles-per-wave kernel serves a problem that ssd_chunk_scan_fwd_fused_supported accepts: chunk size
// 256, where the one-tile form leaves the last wave eight blocks and the first one a single block.
// (Its per-thread offsets are 32-bit byte offsets from a chunk's first row: rows up to 8 MB apart.)
bool ssd_scan_paired_serves(const SsdParams &p) {
  const int64_t lim = 1 << 22;
  return p.chunk_size == 256 && p.x_ls < lim && p.out_ls < lim && (!p.z || p.z_ls < lim);
}

int ssd_scan_paired_launch(const SsdParams &p, hipStream_t s) {
  return p.headdim == 64 ? launch_n<4>(p, s) : launch_n<2>(p, s);
}
