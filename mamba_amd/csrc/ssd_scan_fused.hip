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

// l tile k (0 .. LT-1) of wave w, QT tiles in all, NWV waves
template <int QT, int NWV> DEVI int l_tile(int w, int k) {
  constexpr int LT = QT / NWV;
  if (LT == 1) return w;
  constexpr int HALF = LT / 2;
  return k < HALF ? HALF * w + k : QT - 1 - (HALF * w + (k - HALF));
}

// NWV waves share the l tiles of one (batch, chunk, head); they are spread over SPLIT workgroups
// of NWV / SPLIT waves each (the pairing of tile i with tile QT-1-i keeps the workgroups balanced
// as well).  Smaller workgroups let several of them, at different stages, share a CU.
template <int PT, int NK, int QT, int NWV, int SPLIT>
__global__ __launch_bounds__(64 * NWV / SPLIT) void chunk_scan_fwd_fused_kernel(const SsdParams p, const int hb) {
  constexpr int P = 16 * PT, N = 32 * NK, Q = 16 * QT, LT = QT / NWV, NSB = Q / 32, NWG = NWV / SPLIT, NT = 64 * NWG;
  static_assert(LT >= 1 && LT * NWV == QT, "l tiles divide evenly over the waves");
  static_assert(NWG * SPLIT == NWV, "waves divide evenly over the workgroups");
  constexpr int BP = N + 8;  // LDS pitch of a B row / H row (bf16): 16-byte aligned, bank-spread
  constexpr int XP = P + 16; // LDS pitch of an X row (one position, P values + pad), as it lies in memory
  constexpr int YP = P + 4;  // fp32 pitch of the epilogue's per-wave transpose patch (rows 4 banks apart)
  struct Stage {
    uint16_t Bs[2][32 * BP];
    uint16_t Xs[2][32 * XP];
    uint16_t Hs[P * BP];
  };
  union __align__(16) Shared {
    Stage st;                       // main loop
    float ypatch[NWG * 16 * YP];    // epilogue (the staging buffers are dead by then)
  };
  __shared__ Shared shm;
  auto &Bs = shm.st.Bs;
  auto &Xs = shm.st.Xs;
  auto &Hs = shm.st.Hs;
  __shared__ float a2_s[Q], dt_s[Q], cs_s[Q], rs_s[Q];
  __shared__ int seq_s[Q];
  __shared__ __align__(16) float d_s[P];

  int tid = threadIdx.x, lane = tid & 63;
  const int lwave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave inside this workgroup
  int j = lane & 15, g = lane >> 4;
  const int H = p.nheads, G = p.ngroups, L = p.seqlen;
  // heads vary fastest over the grid: workgroups in flight together then read and write whole
  // (position, all heads) rows of x, z and out between them
  // A workgroup works through hb heads of one group, one after the other (their C rows are the same and stay in
  // registers); its heads are `per` apart, so that workgroups in flight together, which sit at about the same place
  // in their lists, touch neighbouring heads.
  const int hpg = H / G, per = hpg / hb;
  const int grp = blockIdx.x / per, h_first = grp * hpg + blockIdx.x % per;
  const int c = blockIdx.y / SPLIT, part = blockIdx.y % SPLIT, b = blockIdx.z;
  const int wave = part * NWG + lwave;  // wave among the NWV that share the chunk
  // s blocks this workgroup needs: up to its last l tile
  int last_tile = 0;
#pragma unroll
  for (int k = 0; k < LT; ++k)
    last_tile = max(last_tile, max(l_tile<QT, NWV>(part * NWG, k), l_tile<QT, NWV>(part * NWG + NWG - 1, k)));
  const int nsb = SPLIT == 1 ? NSB : min(NSB, (last_tile * 16 + 15) / 32 + 1);
  const int t0 = c * Q;
  const int qlim = min(Q, L - t0);
  const bf16_t *xg = static_cast<const bf16_t *>(p.x) + b * p.x_bs + h_first * p.x_hs;  // of the head being staged
  const bf16_t *Bg = static_cast<const bf16_t *>(p.B) + b * p.B_bs + grp * p.B_gs;
  const bf16_t *Cg = static_cast<const bf16_t *>(p.C) + b * p.C_bs + grp * p.C_gs;
  const bool has_seq = p.seq_idx != nullptr;

  // ---- staging (global -> registers -> LDS), one s block of 32 positions: the 16-byte pieces of its B rows and of
  // its X rows (X as it lies in memory: the second MFMA reads its X^T fragments with the transposing LDS load) are
  // one list of tasks, dealt to the threads.  Every thread issues the same number of loads whatever its task (an
  // idle thread or a row past the end re-reads a valid piece that is dropped or zeroed at the commit): with no
  // branch around a global load the compiler counts the loads in flight exactly, and the wait before a commit
  // lets the loads of the blocks behind it stay in flight.
  constexpr int TB = 32 * N / 8, TX = 32 * P / 8, TPT = (TB + TX + NT - 1) / NT;
  u32x4 sregs[2][TPT];  // two blocks in flight: global loads run two blocks ahead
  uint16_t *const stage0 = &shm.st.Bs[0][0];
  static_assert(offsetof(Stage, Xs) == sizeof(uint16_t) * 2 * 32 * BP, "X tiles follow the B tiles");
  const int64_t B_ls = p.B_ls, x_ls = p.x_ls;  // in registers: a select between them must not become a load
  auto load_block = [&](int sb, u32x4 (&reg)[TPT]) {
#pragma unroll
    for (int q = 0; q < TPT; ++q) {
      const int t = tid + q * NT;
      const bool is_b = t < TB;
      const int u = is_b ? t : min(t - TB, TX - 1);
      const int r = is_b ? u / (N / 8) : u / (P / 8), c8 = is_b ? u % (N / 8) : u % (P / 8);
      const int64_t row = t0 + min(sb * 32 + r, qlim - 1);
      const bf16_t *base = is_b ? Bg : xg;
      reg[q] = *(const GLOBAL_AS u32x4 *)(base + row * (is_b ? B_ls : x_ls) + c8 * 8);
    }
  };
  auto store_block = [&](int sb, int buf, const u32x4 (&reg)[TPT]) {
#pragma unroll
    for (int q = 0; q < TPT; ++q) {
      const int t = tid + q * NT;
      const bool is_b = t < TB;
      const int u = t - (is_b ? 0 : TB);
      const int r = is_b ? u / (N / 8) : u / (P / 8), c8 = is_b ? u % (N / 8) : u % (P / 8);
      const bool live = sb * 32 + r < qlim;
      const u32x4 v = {live ? reg[q].x : 0u, live ? reg[q].y : 0u, live ? reg[q].z : 0u, live ? reg[q].w : 0u};
      const int off = is_b ? buf * 32 * BP + r * BP + c8 * 8 : 2 * 32 * BP + buf * 32 * XP + r * XP + c8 * 8;
      if (t < TB + TX) *reinterpret_cast<u32x4 *>(stage0 + off) = v;
    }
  };
  // X^T fragment of p tile pt: lane (j, g) gets row p = 16 pt + j and the k slots of lane group g, which are
  // positions 4 g .. 4 g + 3 of the block's first 16-tile, then of its second: the layout in which the first
  // MFMA leaves M^T.  Each half is one transposing load of a 4 x 16 patch.
  auto x_frag = [&](int buf, int pt) {
    typedef __attribute__((address_space(3))) i16x4_t *lds_ptr;
    typedef short i16x8_t __attribute__((ext_vector_type(8)));
    const uint16_t *src = &Xs[buf][(4 * g + (j >> 2)) * XP + pt * 16 + 4 * (j & 3)];
    const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)src);
    const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(src + 16 * XP));
    return __builtin_bit_cast(bf16x8_t, (i16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // carried state (bf16 in memory), rows p, k = n
  constexpr int HCH = (P * N / 8 + NT - 1) / NT;
  u32x4 hraw[HCH];
  // Everything a head needs from memory before its first block: the first two s blocks, the carried state and the
  // per-position scalars.  For the first head this is issued together with the C rows, so that the workgroup pays one
  // memory latency; for every later head it is issued before the previous head's epilogue and arrives behind it.
  static_assert(NT >= Q && NT >= P, "one position / one channel per thread");
  const float *Dp = static_cast<const float *>(p.D);
  float sc_a = 0.f, sc_aend = 0.f, sc_dt = 0.f;
  bool carried_ok = false;
  float sc_d = 0.f;
  auto load_head = [&](int h) {
    xg = static_cast<const bf16_t *>(p.x) + b * p.x_bs + h * p.x_hs;
    load_block(0, sregs[0]);
    if (nsb > 1) load_block(1, sregs[1]);
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
  load_head(h_first);
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
  // C rows of this wave's l tiles: B operand of both contractions (col l = j, k = n)
  bf16x8_t Cf[LT][NK];
#pragma unroll
  for (int k = 0; k < LT; ++k) {
    const int l = l_tile<QT, NWV>(wave, k) * 16 + j;
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) {
      u32x4 v = {0, 0, 0, 0};
      if (l < qlim) v = *reinterpret_cast<const u32x4 *>(Cg + (int64_t)(t0 + l) * p.C_ls + kk * 32 + g * 8);
      Cf[k][kk] = __builtin_bit_cast(bf16x8_t, v);
    }
  }
#pragma unroll 1
  for (int hh = 0; hh < hb; ++hh) {
  const int h = h_first + hh * per;
  // The thread's indices pass through an empty asm once per head: to the compiler they are new values, so the
  // addresses derived from them are computed where they are used, as in a kernel without this loop, instead of
  // being kept in registers (or spilled) across it.
  asm volatile("" : "+v"(tid), "+v"(lane), "+v"(j), "+v"(g));
  // ---- per-position scalars of this (batch, head, chunk): thread s holds position s
  if (tid < Q) {
    a2_s[tid] = sc_a * kLog2e;
    dt_s[tid] = sc_dt;
    cs_s[tid] = sc_dt * fast_exp(sc_aend - sc_a);
    rs_s[tid] = carried_ok ? fast_exp(sc_a) : 0.f;
  }
  if (tid < P) d_s[tid] = Dp ? sc_d : 0.f;

#pragma unroll
  for (int q = 0; q < HCH; ++q) {
    const int id = tid + q * NT, pp = id / (N / 8), c8 = id % (N / 8);
    if (id < P * N / 8) *reinterpret_cast<u32x4 *>(&Hs[pp * BP + c8 * 8]) = hraw[q];
  }
  store_block(0, 0, sregs[0]);
  lds_barrier();

  f32x4 acc[LT][PT];
  // ---- carried state: y^T[p, l] = rs_l * sum_n H[p, n] C[l, n]
#pragma unroll
  for (int k = 0; k < LT; ++k) {
#pragma unroll
    for (int pt = 0; pt < PT; ++pt) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NK; ++kk) v = mfma_bf16(ld_frag(&Hs[(pt * 16 + j) * BP + kk * 32 + g * 8]), Cf[k][kk], v);
      acc[k][pt] = v * rs_s[l_tile<QT, NWV>(wave, k) * 16 + j];
    }
  }

  // The epilogue's x (for D) and z rows are fetched a few blocks before the main loop ends, so
  // that their latency is covered by the remaining blocks.
  constexpr int EQ = (16 * P / 8 + 63) / 64;  // 16-byte chunks per lane of one 16 x P tile
  const bf16_t *xe_g = static_cast<const bf16_t *>(p.x) + b * p.x_bs + h * p.x_hs;
  const bf16_t *zg = p.z ? static_cast<const bf16_t *>(p.z) + b * p.z_bs + h * p.z_hs : nullptr;
  u32x4 xe[LT][EQ], ze[LT][EQ];
  auto epilogue_prefetch = [&]() {
#pragma unroll
    for (int k = 0; k < LT; ++k)
#pragma unroll
      for (int q = 0; q < EQ; ++q) {
        const int id = lane + q * 64, rr = id / (P / 8), c8 = id % (P / 8);
        const int l = l_tile<QT, NWV>(wave, k) * 16 + rr;
        // no branch around these loads either (rows past the end re-read the last row and are not stored;
        // without z the x row stands in and is not used)
        static_assert(EQ * 64 == 16 * P / 8, "whole 16-byte pieces per lane");
        const int64_t row = t0 + min(l, qlim - 1);
        xe[k][q] = *(const GLOBAL_AS u32x4 *)(xe_g + row * p.x_ls + c8 * 8);
        ze[k][q] = *(const GLOBAL_AS u32x4 *)(zg ? zg + row * p.z_ls + c8 * 8 : xe_g + row * p.x_ls + c8 * 8);
      }
  };

  // ---- inside the chunk
#pragma unroll
  for (int sb = 0; sb < NSB; ++sb) {
    const int buf = sb & 1;
    if (SPLIT > 1 && sb >= nsb) break;
    if (sb == max(nsb - 3, 0)) epilogue_prefetch();
    if (sb + 2 < nsb) load_block(sb + 2, sregs[sb & 1]);
#pragma unroll
    for (int k = 0; k < LT; ++k) {
      const int lt = l_tile<QT, NWV>(wave, k);
      if (lt * 16 + 15 < sb * 32) continue;  // every position of the block is after the tile
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
        for (int kk = 0; kk < NK; ++kk)
          S = mfma_bf16(ld_frag(&Bs[buf][(h2 * 16 + j) * BP + kk * 32 + g * 8]), Cf[k][kk], S);
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
      for (int pt = 0; pt < PT; ++pt)
        acc[k][pt] = mfma_bf16(x_frag(buf, pt), Mf, acc[k][pt]);
    }
    if (sb + 1 < nsb) store_block(sb + 1, buf ^ 1, sregs[(sb + 1) & 1]);
    lds_barrier();
  }

  // ---- epilogue: + D x, pre-gate copy, gate.  Each wave transposes its 16-row tiles through a
  // private LDS patch so that x / z loads and out / out_x stores are 16-byte pieces of
  // contiguous rows (the accumulator layout itself would scatter 8-byte pieces over 16 rows).
  if (hh + 1 < hb) load_head(h + per);
  float *Ys = shm.ypatch + lwave * 16 * YP;
  bf16_t *og = static_cast<bf16_t *>(p.out) + b * p.out_bs + h * p.out_hs;
  bf16_t *oxg = p.z ? static_cast<bf16_t *>(p.out_x) + b * p.out_bs + h * p.out_hs : nullptr;
#pragma unroll
  for (int k = 0; k < LT; ++k) {
    const int ltile = l_tile<QT, NWV>(wave, k);
#pragma unroll
    for (int pt = 0; pt < PT; ++pt) *reinterpret_cast<f32x4 *>(&Ys[j * YP + pt * 16 + 4 * g]) = acc[k][pt];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // 16 rows x P/8 chunks of 8 columns
#pragma unroll
    for (int q = 0; q < EQ; ++q) {
      const int id = lane + q * 64, rr = id / (P / 8), c8 = id % (P / 8);
      const int l = ltile * 16 + rr;
      if (id >= 16 * P / 8 || l >= qlim) continue;
      const f32x4 y0 = *reinterpret_cast<const f32x4 *>(&Ys[rr * YP + c8 * 8]);
      const f32x4 y1 = *reinterpret_cast<const f32x4 *>(&Ys[rr * YP + c8 * 8 + 4]);
      float v[8] = {y0.x, y0.y, y0.z, y0.w, y1.x, y1.y, y1.z, y1.w};
      if (Dp) {
        const u32x4 xw = xe[k][q];
        const float xf[8] = {bf16_lo(xw.x), bf16_hi(xw.x), bf16_lo(xw.y), bf16_hi(xw.y),
                             bf16_lo(xw.z), bf16_hi(xw.z), bf16_lo(xw.w), bf16_hi(xw.w)};
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = __builtin_fmaf(d_s[c8 * 8 + e], xf[e], v[e]);
      }
      const int64_t oi = (int64_t)(t0 + l) * p.out_ls + c8 * 8;
      if (zg) {
        st8<bf16_t>(oxg + oi, v);
        const u32x4 zw = ze[k][q];
        const float zf[8] = {bf16_lo(zw.x), bf16_hi(zw.x), bf16_lo(zw.y), bf16_hi(zw.y),
                             bf16_lo(zw.z), bf16_hi(zw.z), bf16_lo(zw.w), bf16_hi(zw.w)};
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= zf[e] * sigmoid_f(zf[e]);
      }
      st8<bf16_t>(og + oi, v);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  lds_barrier();  // the next head's staging overwrites the patches
  }
}

bool aligned(const void *ptr, int a) { return (reinterpret_cast<uintptr_t>(ptr) % a) == 0; }

int cu_count() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    cached[dev] = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256;
  }
  return cached[dev];
}

// Heads per workgroup: a divisor of the heads per group, 20 at most.  One workgroup fills a CU, so the launch runs in
// ceil(workgroups / CUs) rounds, each as long as what a workgroup pays once (launch, arguments, C rows, the first
// head's exposed memory latency: measured at about 0.15 of a head's work) plus its heads; the divisor with the
// shortest estimate wins.
int heads_per_workgroup(const SsdParams &p) {
  const int hpg = p.nheads / p.ngroups, cus = cu_count();
  const int64_t tiles = (int64_t)p.nchunks * p.batch;
  int best = 1;
  double best_cost = 1e30;
  for (int hb = 1; hb <= 20 && hb <= hpg; ++hb) {
    if (hpg % hb) continue;
    const int64_t wgs = tiles * (p.nheads / hb);
    const double cost = (double)((wgs + cus - 1) / cus) * (0.15 + hb);
    if (cost < best_cost - 1e-9) best = hb, best_cost = cost;
  }
  return best;
}

template <int PT, int NK> int launch_q(const SsdParams &p, hipStream_t s) {
  const int hb = heads_per_workgroup(p);
  dim3 grid(p.nheads / hb, p.nchunks, p.batch);
  switch (p.chunk_size) {
    case 256: hipLaunchKernelGGL((chunk_scan_fwd_fused_kernel<PT, NK, 16, 16, 1>), grid, dim3(1024), 0, s, p, hb); break;
    case 128: hipLaunchKernelGGL((chunk_scan_fwd_fused_kernel<PT, NK, 8, 8, 1>), grid, dim3(512), 0, s, p, hb); break;
    case 64: hipLaunchKernelGGL((chunk_scan_fwd_fused_kernel<PT, NK, 4, 4, 1>), grid, dim3(256), 0, s, p, hb); break;
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
  if (p->z && (!aligned(p->z, 16) || !aligned(p->out_x, 16) || p->z_bs % 8 || p->z_ls % 8 || p->z_hs % 8)) return 0;
  if (p->states_lp && !aligned(p->states_lp, 16)) return 0;
  if (p->batch > 65535 || p->nheads > 65535) return 0;
  return 1;
}

extern "C" int ssd_chunk_scan_fwd_fused(const SsdParams *p, mamba_stream_t stream) {
  if (!p || !p->x || !p->B || !p->C || !p->states_lp || !p->out || !p->dt_out || !p->dA_cumsum || (p->z && !p->out_x))
    return MAMBA_E_BADARG;
  if (!ssd_chunk_scan_fwd_fused_supported(p)) return MAMBA_E_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return p->headdim == 64 ? launch_n<4>(*p, s) : launch_n<2>(*p, s);
}
