// Shared pieces of the SSD kernels: the bf16 MFMA block-GEMM core on LDS tiles
// and the tile staging helpers.
//
// Block GEMM: a 256-thread workgroup (4 waves, 2 x 2) computes a 64 x 64 tile
// D[m][n] = sum_k A[m][k] * B[n][k] in steps of 32 along k.  Both operand tiles
// sit in LDS "k-contiguous" ([row][k], padded), which is exactly the register
// layout v_mfma_f32_16x16x32_bf16 wants for A and for B: lane l supplies row
// (l % 16) and the 8 k-values 8 * (l / 16) .. + 7 with one 16-byte LDS load.
// fp32 / fp16 inputs keep their precision by splitting every operand into a
// bf16 high part and a bf16 remainder and issuing three MFMAs
// (hi*hi + hi*lo + lo*hi); bf16 inputs need one.
#pragma once
#include "common.hpp"
#include <algorithm>
#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

constexpr int GB = 64;         // block tile edge (M and N)
constexpr int GK = 32;         // k step (one MFMA k-slice per barrier pair; 64 measured slower)
constexpr int GLD = GK + 8;    // LDS row pitch in bf16 (80 bytes: conflict-free 16-byte reads)
constexpr int GTILE = GB * GLD;

DEVI uint16_t bf16_bits(float x) { return (uint16_t)f32_to_bf16_bits(x); }
DEVI float bf16_val(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

template <typename T> DEVI float ldg(const void *base, int64_t idx) { return ld1<T>(static_cast<const T *>(base) + idx); }
template <typename T> DEVI void stg(void *base, int64_t idx, float v) { st1<T>(static_cast<T *>(base) + idx, v); }

DEVI float ld_dyn(const void *base, int64_t idx, int dtype) {
  switch (dtype) {
    case MAMBA_F32: return static_cast<const float *>(base)[idx];
    case MAMBA_BF16: return ld1<bf16_t>(static_cast<const bf16_t *>(base) + idx);
    default: return ld1<f16_t>(static_cast<const f16_t *>(base) + idx);
  }
}
DEVI void st_dyn(void *base, int64_t idx, int dtype, float v) {
  switch (dtype) {
    case MAMBA_F32: static_cast<float *>(base)[idx] = v; break;
    case MAMBA_BF16: st1<bf16_t>(static_cast<bf16_t *>(base) + idx, v); break;
    default: st1<f16_t>(static_cast<f16_t *>(base) + idx, v); break;
  }
}

// LDS of one block GEMM: A and B tiles, high and low parts.
struct GemmLds {
  uint16_t ah[GTILE], al[GTILE], bh[GTILE], bl[GTILE];
};

// Offset of element (row, k) inside a staged 64 x GK tile.  The 8-element k groups of a row
// are XOR-swizzled with (row / 8): 16-byte fragment reads stay conflict-free and the transposing
// stores of row-contiguous sources (8 lanes writing rows 8 apart) no longer pile on one bank.
DEVI int tile_off(int r, int k) { return r * GLD + ((((k >> 3) ^ (r >> 3)) & (GK / 8 - 1)) << 3) + (k & 7); }

// Packs 8 floats to bf16 (plus the bf16 remainders when SPLIT) and stores them with 16-byte LDS
// writes; `ok` false stores zeros instead (the mask is applied to the packed words).
template <bool SPLIT> DEVI void put8(uint16_t *hi, uint16_t *lo, int off, const float (&v)[8], bool ok = true) {
  uint32_t h[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) h[e] = pack_bf16(v[2 * e], v[2 * e + 1]);
  if (SPLIT) {
    uint32_t l[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      l[e] = pack_bf16(v[2 * e] - bf16_lo(h[e]), v[2 * e + 1] - bf16_hi(h[e]));
      l[e] = ok ? l[e] : 0u;
    }
    *reinterpret_cast<u32x4 *>(lo + off) = u32x4{l[0], l[1], l[2], l[3]};
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) h[e] = ok ? h[e] : 0u;
  *reinterpret_cast<u32x4 *>(hi + off) = u32x4{h[0], h[1], h[2], h[3]};
}

// A register slot that already holds 8 bf16 values goes to LDS as it is.
template <bool SPLIT, typename S> constexpr bool kRawCopy = !SPLIT && DT<S>::id == MAMBA_BF16;
template <typename S> DEVI void put_raw(uint16_t *hi, int off, const Pack8<S> &q, bool ok) {
  if constexpr (DT<S>::id == MAMBA_BF16) {
    *reinterpret_cast<u32x4 *>(hi + off) = u32x4{ok ? q.w.x : 0u, ok ? q.w.y : 0u, ok ? q.w.z : 0u, ok ? q.w.w : 0u};
  }
}

// ---- staging split into a fetch (global -> registers) and a commit (registers -> LDS) half, so
// that the loads of the next k step are in flight while the current one is multiplied.
// FAST is the path on which every thread's task is a whole, 16-byte aligned group of 8 elements:
// its loads are issued unguarded from clamped (always valid) addresses and masked at commit, which
// keeps branches away from the loads.  The guarded path (ragged or unaligned operands) takes any
// shape.  Both stagers take one task per thread with the 32-wide k step.
static_assert(GK == 32, "one staging task per thread");

// k-contiguous source: element (r, k) at base[r * rstride + k]; thread t takes row t / 4, 8 k values.
template <bool SPLIT, typename S> struct KcStager {
  static constexpr bool transposed = false;
  uint16_t *hi, *lo;
  const S *base;
  int64_t rstride;
  int rows_valid, k_valid;
  const float *kscale, *rscale;  // optional multipliers, by absolute k / by tile row
  bool vec;                      // rows are 16-byte aligned
  int t;
  Pack8<S> q;
  DEVI KcStager(uint16_t *hi_, uint16_t *lo_, const S *base_, int64_t rstride_, int rows_valid_, int k_valid_,
                const float *kscale_, const float *rscale_, bool vec_, int t_)
      : hi(hi_), lo(lo_), base(base_), rstride(rstride_), rows_valid(rows_valid_), k_valid(k_valid_), kscale(kscale_),
        rscale(rscale_), vec(vec_), t(t_) {}
  DEVI bool fast() const { return vec && k_valid >= 8 && k_valid % 8 == 0 && rows_valid >= 1; }
  template <bool FAST> DEVI void fetch(int k0) {
    const int r = t >> 2, k = k0 + (t & 3) * 8;
    if constexpr (FAST) {
      q.load(base + (int64_t)min(r, rows_valid - 1) * rstride + min(k, k_valid - 8));
    } else {
      q.zero();
      if (r < rows_valid && k < k_valid) {
        const S *src = base + (int64_t)r * rstride + k;
        if (vec && k + 8 <= k_valid) {
          q.load(src);
        } else {
          float v[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = k + e < k_valid ? ld1<S>(src + e) : 0.f;
          q.pack(v);
        }
      }
    }
  }
  template <bool FAST> DEVI void commit(int k0) {
    const int r = t >> 2, k8 = (t & 3) * 8;
    const bool ok = !FAST || (r < rows_valid && k0 + k8 < k_valid);
    if constexpr (kRawCopy<SPLIT, S>) {
      if (!kscale && !rscale) {
        put_raw<S>(hi, tile_off(r, k8), q, ok);
        return;
      }
    }
    float v[8];
    q.unpack(v);
    if (kscale) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] *= kscale[k0 + k8 + e];
    }
    if (rscale) {
      const float rs = rscale[r];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] *= rs;
    }
    put8<SPLIT>(hi, lo, tile_off(r, k8), v, ok);
  }
};

// Row-contiguous source kept as it lies: element (r, k) at base[k * kstride + r] goes to LDS as
// [k][r] (pitch TLD), and the MFMA fragments are read with the transposing LDS load.  Thread t takes
// k = t / 8 and 8 consecutive rows: one 16-byte load, one 16-byte LDS store, no per-element shuffling.
constexpr int TLD = GB + 16;  // [k][r] pitch in bf16 (160 bytes: the 4 rows of a transposing read hit disjoint banks)
static_assert(GK * TLD <= GTILE, "the [k][r] tile fits the operand's LDS array");
DEVI int tr_off(int k, int r) { return k * TLD + r; }

template <bool SPLIT, typename S> struct TrStager {
  static constexpr bool transposed = true;
  uint16_t *hi, *lo;
  const S *base;
  int64_t kstride;
  int rows_valid, k_valid;
  const float *kscale, *rscale;
  bool vec;
  int t;
  Pack8<S> q;
  DEVI TrStager(uint16_t *hi_, uint16_t *lo_, const S *base_, int64_t kstride_, int rows_valid_, int k_valid_,
                const float *kscale_, const float *rscale_, bool vec_, int t_)
      : hi(hi_), lo(lo_), base(base_), kstride(kstride_), rows_valid(rows_valid_), k_valid(k_valid_), kscale(kscale_),
        rscale(rscale_), vec(vec_), t(t_) {}
  DEVI bool fast() const { return vec && rows_valid >= 8 && rows_valid % 8 == 0 && k_valid >= 1; }
  template <bool FAST> DEVI void fetch(int k0) {
    const int k = k0 + (t >> 3), r8 = (t & 7) * 8;
    if constexpr (FAST) {
      q.load(base + (int64_t)min(k, k_valid - 1) * kstride + min(r8, rows_valid - 8));
    } else {
      q.zero();
      if (k < k_valid && r8 < rows_valid) {
        const S *src = base + (int64_t)k * kstride + r8;
        if (vec && r8 + 8 <= rows_valid) {
          q.load(src);
        } else {
          float v[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = r8 + e < rows_valid ? ld1<S>(src + e) : 0.f;
          q.pack(v);
        }
      }
    }
  }
  template <bool FAST> DEVI bool task_ok(int k0) const {
    return !FAST || (k0 + (t >> 3) < k_valid && (t & 7) * 8 < rows_valid);
  }
  // commit with a multiplier per element, f(tile row, absolute k), instead of the scale vectors
  template <bool FAST, typename F> DEVI void commit_each(int k0, F f) {
    const int kk = t >> 3, r8 = (t & 7) * 8;
    float v[8];
    q.unpack(v);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= f(r8 + e, k0 + kk);
    put8<SPLIT>(hi, lo, tr_off(kk, r8), v, task_ok<FAST>(k0));
  }
  template <bool FAST> DEVI void commit(int k0) {
    const int kk = t >> 3, r8 = (t & 7) * 8;
    const bool ok = task_ok<FAST>(k0);
    if constexpr (kRawCopy<SPLIT, S>) {
      if (!kscale && !rscale) {
        put_raw<S>(hi, tr_off(kk, r8), q, ok);
        return;
      }
    }
    float v[8];
    q.unpack(v);
    if (kscale) {
      const float ks = kscale[k0 + kk];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] *= ks;
    }
    if (rscale) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] *= rscale[r8 + e];
    }
    put8<SPLIT>(hi, lo, tr_off(kk, r8), v, ok);
  }
};

template <typename S> DEVI bool rows_aligned16(const S *base, int64_t stride) {
  constexpr int m = 16 / sizeof(S);
  return (reinterpret_cast<uintptr_t>(base) & 15) == 0 && stride % m == 0;
}

// Fills a 64 x 32 tile from a functor f(row, k) -> float.  K_FAST: consecutive
// threads walk k (use when the source is contiguous along k), else along rows.
template <bool SPLIT, bool K_FAST, typename F> DEVI void stage_tile(uint16_t *hi, uint16_t *lo, F f, int tid) {
#pragma unroll 2
  for (int idx = tid; idx < GB * GK; idx += 256) {
    int r, k;
    if (K_FAST) {
      k = idx % GK;
      r = idx / GK;
    } else {
      r = idx % GB;
      k = idx / GB;
    }
    const float v = f(r, k);
    const uint16_t h = bf16_bits(v);
    hi[tile_off(r, k)] = h;
    if (SPLIT) lo[tile_off(r, k)] = bf16_bits(v - bf16_val(h));
  }
}

struct GemmAcc {
  f32x4 v[2][2];
  DEVI void zero() {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) v[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
};

// MFMA fragment of a staged tile: rows row0 .. row0 + 15, lane (i, g) gets row row0 + i, k = 8 g .. 8 g + 7.
// From a [row][k] tile that is one 16-byte load.  From a [k][row] tile (TR) it is two transposing
// loads: in each, the 16 lanes of a k group read the 4 x 16 block of rows k .. k + 3 (lane i: row
// k + i / 4, 4 columns from 4 (i % 4)) and the hardware hands lane i column i of the 4 rows.
typedef short i16x4_t __attribute__((ext_vector_type(4)));
template <bool TR> DEVI bf16x8_t load_frag(const uint16_t *tile, int row0, int i, int g) {
  if constexpr (!TR) {
    return *reinterpret_cast<const bf16x8_t *>(&tile[tile_off(row0 + i, g * 8)]);
  } else {
    typedef __attribute__((address_space(3))) i16x4_t *lds_ptr;
    const uint16_t *src = tile + tr_off(g * 8 + (i >> 2), row0 + 4 * (i & 3));
    const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)src);
    const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(src + 4 * TLD));
    typedef short i16x8_t __attribute__((ext_vector_type(8)));
    const i16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, both);
  }
}

// One 32-deep step.  Wave (wm, wn) of the 2 x 2 grid owns rows 32*wm.. and columns 32*wn...
template <bool SPLIT, bool ATR = false, bool BTR = false>
DEVI void mma_step(GemmAcc &acc, const GemmLds &s, int wm, int wn, int lane) {
  static_assert(GK == 32, "one MFMA k-slice per step");
  const int i = lane & 15, g = lane >> 4;
  bf16x8_t a[2], b[2], al[2], bl[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    a[t] = load_frag<ATR>(s.ah, wm * 32 + t * 16, i, g);
    b[t] = load_frag<BTR>(s.bh, wn * 32 + t * 16, i, g);
    if (SPLIT) {
      al[t] = load_frag<ATR>(s.al, wm * 32 + t * 16, i, g);
      bl[t] = load_frag<BTR>(s.bl, wn * 32 + t * 16, i, g);
    }
  }
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
      acc.v[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[tm], b[tn], acc.v[tm][tn], 0, 0, 0);
      if (SPLIT) {
        acc.v[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[tm], bl[tn], acc.v[tm][tn], 0, 0, 0);
        acc.v[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[tm], b[tn], acc.v[tm][tn], 0, 0, 0);
      }
    }
}

// ---- wide variant: a 64 x 128 tile per workgroup, 32 x 64 per wave, both operands row-contiguous
// ([k][row] in LDS).  Per MFMA it moves three quarters of the LDS and global bytes of the 64 x 64 core.
constexpr int WB = 128;          // columns of the wide tile
constexpr int WLD = WB + 16;     // [k][row] pitch of the wide operand (288 bytes)
template <bool SPLIT> struct GemmLdsWide {
  uint16_t ah[GTILE], al[SPLIT ? GTILE : 8], bh[GK * WLD], bl[SPLIT ? GK * WLD : 8];
};
struct GemmAccWide {
  f32x4 v[2][4];
  DEVI void zero() {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) v[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
};
template <int PITCH> DEVI bf16x8_t load_frag_tr(const uint16_t *tile, int row0, int i, int g) {
  typedef __attribute__((address_space(3))) i16x4_t *lds_ptr;
  typedef short i16x8_t __attribute__((ext_vector_type(8)));
  const uint16_t *src = tile + (g * 8 + (i >> 2)) * PITCH + row0 + 4 * (i & 3);
  const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)src);
  const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(src + 4 * PITCH));
  return __builtin_bit_cast(bf16x8_t, (i16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}
// Stages ROWS rows x 32 k of a row-contiguous operand (element (r, k) at base[k * kstride + r]) as
// [k][r]: thread t takes k = t / 8 and, per 64 rows, 8 consecutive rows from 8 (t % 8).  The operand
// must be 16-byte aligned with rows_valid a multiple of 8 and k_valid a multiple of 32 (the caller
// checks); rows past rows_valid re-read the last rows and are zeroed.
template <bool SPLIT, typename S, int ROWS> struct WideTrStager {
  static constexpr int NT = ROWS / 64, PITCH = ROWS + 16;
  uint16_t *hi, *lo;
  const S *base;
  int64_t kstride;
  int rows_valid;
  const float *kscale;
  int t;
  Pack8<S> q[NT];
  WideTrStager() = default;  // for arrays of stagers, each assigned from a constructed one
  DEVI WideTrStager(uint16_t *hi_, uint16_t *lo_, const S *base_, int64_t kstride_, int rows_valid_, const float *kscale_, int t_)
      : hi(hi_), lo(lo_), base(base_), kstride(kstride_), rows_valid(rows_valid_), kscale(kscale_), t(t_) {}
  static constexpr bool transposed = true;
  DEVI bool fast() const { return true; }
  template <bool FAST = true> DEVI void fetch(int k0) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
      q[j].load(base + (int64_t)(k0 + (t >> 3)) * kstride + min((t & 7) * 8 + 64 * j, rows_valid - 8));
  }
  template <bool FAST = true> DEVI void commit(int k0) {
    const int kk = t >> 3;
    const float ks = kscale ? kscale[k0 + kk] : 1.f;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int r8 = (t & 7) * 8 + 64 * j, off = kk * PITCH + r8;
      if (r8 >= rows_valid) {
        const float zero[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        put8<SPLIT>(hi, lo, off, zero);
      } else if (kRawCopy<SPLIT, S> && !kscale) {
        put_raw<S>(hi, off, q[j], true);
      } else {
        float v[8];
        q[j].unpack(v);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= ks;
        put8<SPLIT>(hi, lo, off, v);
      }
    }
  }
};
// acc[m][n] += sum_k A[m][k] B[n][k] over k in [0, k_end), k_end a multiple of 32.  The A stager is
// a 64-row stager of either layout on its fast path, the B stager a 128-row WideTrStager (possibly
// inside a SegStager).
template <bool SPLIT, bool RING, typename SA, typename SB, typename AFTER>
DEVI void block_gemm_wide(GemmAccWide &acc, GemmLdsWide<SPLIT> &s, int k_end, SA &sa, SB &sb, int tid, AFTER after_step) {
  constexpr bool ATR = SA::transposed;
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int i = lane & 15, g = lane >> 4;
  // One k step: commit the step's operands (fetched earlier into fa / fb) to LDS, request those of step k_next
  // into the same registers, multiply.  The barriers wait for LDS only, so the loads requested here, and those
  // the other pair of stagers has in flight, stay in flight across them.
  auto step = [&](int k0, SA &fa, SB &fb, int k_next) {
    lds_barrier();
    fa.template commit<true>(k0);
    fb.template commit<true>(k0);
    lds_barrier();
    fa.template fetch<true>(k_next);
    fb.template fetch<true>(k_next);
    bf16x8_t a[2], b[4], al[2], bl[4];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      a[t] = load_frag<ATR>(s.ah, wm * 32 + t * 16, i, g);
      if (SPLIT) al[t] = load_frag<ATR>(s.al, wm * 32 + t * 16, i, g);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      b[t] = load_frag_tr<WLD>(s.bh, wn * 64 + t * 16, i, g);
      if (SPLIT) bl[t] = load_frag_tr<WLD>(s.bl, wn * 64 + t * 16, i, g);
    }
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int tn = 0; tn < 4; ++tn) {
        acc.v[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[tm], b[tn], acc.v[tm][tn], 0, 0, 0);
        if (SPLIT) {
          acc.v[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[tm], bl[tn], acc.v[tm][tn], 0, 0, 0);
          acc.v[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[tm], b[tn], acc.v[tm][tn], 0, 0, 0);
        }
      }
    after_step(k0);
  };
  if (RING && !SPLIT && (k_end / GK) % 2 == 0) {
    // Two pairs of stagers take the even and the odd steps: the operands of two steps are in flight, and a
    // step's loads have two steps of work to arrive behind.  (Measured: the head loop of the state-path dB
    // product gains 7 %, chunk_state loses as much to the registers, bwd_dstates is unchanged.)
    SA sa2 = sa;
    SB sb2 = sb;
    sa.template fetch<true>(0);
    sb.template fetch<true>(0);
    sa2.template fetch<true>(GK);
    sb2.template fetch<true>(GK);
    for (int k0 = 0; k0 < k_end; k0 += 2 * GK) {
      step(k0, sa, sb, min(k0 + 2 * GK, k_end - GK));
      step(k0 + GK, sa2, sb2, min(k0 + 3 * GK, k_end - GK));
    }
  } else {
    sa.template fetch<true>(0);
    sb.template fetch<true>(0);
    for (int k0 = 0; k0 < k_end; k0 += GK) step(k0, sa, sb, min(k0 + GK, k_end - GK));
  }
}
template <bool SPLIT, bool RING = false, typename SA, typename SB>
DEVI void block_gemm_wide(GemmAccWide &acc, GemmLdsWide<SPLIT> &s, int k_end, SA &sa, SB &sb, int tid) {
  block_gemm_wide<SPLIT, RING>(acc, s, k_end, sa, sb, tid, [](int) {});
}
// One k step of that product by itself, for callers that keep more than two pairs of stagers in flight: commits
// the operands fa / fb hold (requested earlier for step k0), requests those of step k_next into the same registers,
// multiplies.
template <typename SA, typename SB>
DEVI void wide_step(GemmAccWide &acc, GemmLdsWide<false> &s, int k0, SA &fa, SB &fb, int k_next, int tid) {
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int i = lane & 15, g = lane >> 4;
  lds_barrier();
  fa.template commit<true>(k0);
  fb.template commit<true>(k0);
  lds_barrier();
  fa.template fetch<true>(k_next);
  fb.template fetch<true>(k_next);
  bf16x8_t a[2], b[4];
#pragma unroll
  for (int t = 0; t < 2; ++t) a[t] = load_frag<SA::transposed>(s.ah, wm * 32 + t * 16, i, g);
#pragma unroll
  for (int t = 0; t < 4; ++t) b[t] = load_frag_tr<WLD>(s.bh, wn * 64 + t * 16, i, g);
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int tn = 0; tn < 4; ++tn)
      acc.v[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[tm], b[tn], acc.v[tm][tn], 0, 0, 0);
}

// dtype in which the states carried between chunks, and their gradients, pass between kernels: bf16 next to bf16
// operands (the matrix products only take that part of them), fp32 otherwise.
template <typename T> using carried_t = std::conditional_t<std::is_same_v<T, bf16_t>, bf16_t, float>;
template <typename T> DEVI carried_t<T> *carried_states(const SsdParams &p) {
  if constexpr (std::is_same_v<T, bf16_t>) return static_cast<bf16_t *>(p.states_lp);
  else return p.states;
}
template <typename T> DEVI carried_t<T> *carried_dstates(const SsdParams &p) {
  if constexpr (std::is_same_v<T, bf16_t>) return static_cast<bf16_t *>(p.dstates_lp);
  else return p.dstates;
}
DEVI void st_carried(float *p, float v) { *p = v; }
DEVI void st_carried(bf16_t *p, float v) { st1<bf16_t>(p, v); }

// Stores the wide tile as rows of dst (the tile's origin, row pitch ld; fp32 or bf16; dst 16-byte aligned, ld a
// multiple of 8), rows >= rows_valid skipped, in whole 128-byte pieces of rows: each wave turns its 32 x 64 part
// around through a patch of its own in the operand tiles' LDS, 16 rows by 128 bytes at a time, so that a lane
// stores 16 contiguous bytes and eight lanes a whole line (single elements straight from the accumulator layout
// are 32-byte runs in bf16: the state-gradient product measured 83 us with those, 71 us with these).  All 256 threads must call (one barrier: the last
// step's operand reads end before the patches overwrite them).
template <bool SPLIT, typename D, bool GUARD = true>
DEVI void store_wide_rows(const GemmAccWide &acc, GemmLdsWide<SPLIT> &s, D *dst, int64_t ld, int rows_valid, int tid) {
  constexpr int CP = 128 / sizeof(D);      // columns per pass
  constexpr int PP = CP + 16 / sizeof(D);  // patch pitch in elements (144 bytes)
  constexpr int E16 = 16 / sizeof(D);      // elements per 16-byte piece
  static_assert(sizeof(GemmLdsWide<SPLIT>) >= 4 * 16 * 144, "the four waves' patches fit in the operand tiles");
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1, i = lane & 15, g = lane >> 4;
  D *patch = reinterpret_cast<D *>(&s) + wave * 16 * PP;
  lds_barrier();
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int pass = 0; pass < 64 / CP; ++pass) {
#pragma unroll
      for (int t = 0; t < CP / 16; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) st_carried(patch + (g * 4 + r) * PP + t * 16 + i, acc.v[tm][pass * (CP / 16) + t][r]);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int row = q * 8 + (lane >> 3), piece = lane & 7;
        const u32x4 v = *reinterpret_cast<const u32x4 *>(patch + row * PP + piece * E16);
        const int m = wm * 32 + tm * 16 + row;
        // (GUARD false: all 64 rows exist, and no branch stands between the caller's loads in flight and its waits)
        if (!GUARD || m < rows_valid) *(GLOBAL_AS u32x4 *)(dst + (int64_t)m * ld + wn * 64 + pass * CP + piece * E16) = v;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}
// Host side: a (batch, position, head/group, row) operand can feed WideTrStager.
inline bool wide_operand_ok(const void *ptr, int dtype, int64_t s0, int64_t s1, int64_t s2) {
  const int64_t m = dtype == MAMBA_F32 ? 4 : 8;
  return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && s0 % m == 0 && s1 % m == 0 && s2 % m == 0;
}
// Host side: every chunk is a whole number of k steps.
inline bool whole_k_steps(const SsdParams *p) {
  const int last = p->seqlen - (p->nchunks - 1) * p->chunk_size;
  return p->chunk_size % GK == 0 && last % GK == 0;
}

// D[m][n] += sum_{k in [k_begin, k_end)} fa(m, k) * fb(n, k) for the block's 64 x 64 tile.
// fa / fb return 0 outside their valid ranges.  All 256 threads must call.
template <bool SPLIT, bool A_KFAST, bool B_KFAST, typename FA, typename FB>
DEVI void block_gemm(GemmAcc &acc, GemmLds &s, int k_begin, int k_end, FA fa, FB fb, int tid) {
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  for (int k0 = k_begin; k0 < k_end; k0 += GK) {
    __syncthreads();
    stage_tile<SPLIT, A_KFAST>(s.ah, s.al, [&](int r, int k) { return fa(r, k0 + k); }, tid);
    stage_tile<SPLIT, B_KFAST>(s.bh, s.bl, [&](int r, int k) { return fb(r, k0 + k); }, tid);
    __syncthreads();
    mma_step<SPLIT>(acc, s, wm, wn, lane);
  }
}

// Software-pipelined form: sa / sb are stager objects with fetch<FAST>(k0) (global -> registers)
// and commit<FAST>(k0) (registers -> LDS tile).  The fetch of step k0 + 32 is issued before the MFMAs
// of step k0, so its latency hides behind them and behind the next barrier.  On the FAST path the
// fetch past the last step re-reads the last step instead (never committed), which keeps the loop
// free of branches around loads.
template <bool SPLIT, bool FAST, typename SA, typename SB, typename AFTER>
DEVI void block_gemm_run(GemmAcc &acc, GemmLds &s, int k_begin, int k_end, SA &sa, SB &sb, int tid, AFTER &after_step) {
  constexpr bool ATR = SA::transposed, BTR = SB::transposed;
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int k_last = k_begin + (k_end - k_begin - 1) / GK * GK;
  sa.template fetch<FAST>(k_begin);
  sb.template fetch<FAST>(k_begin);
  for (int k0 = k_begin; k0 <= k_last; k0 += GK) {
    __syncthreads();
    sa.template commit<FAST>(k0);
    sb.template commit<FAST>(k0);
    __syncthreads();
    if (FAST || k0 + GK <= k_last) {
      sa.template fetch<FAST>(min(k0 + GK, k_last));
      sb.template fetch<FAST>(min(k0 + GK, k_last));
    }
    mma_step<SPLIT, ATR, BTR>(acc, s, wm, wn, lane);
    after_step(k0);  // e.g. to consume and clear the accumulator at segment ends
  }
}
// The fast path with two pairs of stagers, for an even number of steps: the pairs take the even and the odd steps,
// so the operands of two steps are in flight and a step's loads have two steps of work to arrive behind.  The
// barriers wait for LDS only (a barrier that also waited for the loads would put them back in step).
template <bool SPLIT, typename SA, typename SB, typename AFTER>
DEVI void block_gemm_run_ring(GemmAcc &acc, GemmLds &s, int k_begin, int k_last, SA &sa, SB &sb, int tid, AFTER &after_step) {
  constexpr bool ATR = SA::transposed, BTR = SB::transposed;
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  std::remove_reference_t<SA> sa2 = sa;
  std::remove_reference_t<SB> sb2 = sb;
  auto step = [&](int k0, auto &fa, auto &fb) {
    lds_barrier();
    fa.template commit<true>(k0);
    fb.template commit<true>(k0);
    lds_barrier();
    fa.template fetch<true>(min(k0 + 2 * GK, k_last));
    fb.template fetch<true>(min(k0 + 2 * GK, k_last));
    mma_step<SPLIT, ATR, BTR>(acc, s, wm, wn, lane);
    after_step(k0);
  };
  sa.template fetch<true>(k_begin);
  sb.template fetch<true>(k_begin);
  sa2.template fetch<true>(k_begin + GK);
  sb2.template fetch<true>(k_begin + GK);
  for (int k0 = k_begin; k0 <= k_last; k0 += 2 * GK) {
    step(k0, sa, sb);
    step(k0 + GK, sa2, sb2);
  }
}
template <bool SPLIT, bool RING, typename SA, typename SB, typename AFTER>
DEVI void block_gemm_pipe(GemmAcc &acc, GemmLds &s, int k_begin, int k_end, SA &&sa, SB &&sb, int tid, AFTER after_step) {
  if (k_begin >= k_end) return;
  if (sa.fast() && sb.fast()) {
    const int k_last = k_begin + (k_end - k_begin - 1) / GK * GK;
    if (RING && ((k_last - k_begin) / GK) % 2 == 1) block_gemm_run_ring<SPLIT>(acc, s, k_begin, k_last, sa, sb, tid, after_step);
    else block_gemm_run<SPLIT, true>(acc, s, k_begin, k_end, sa, sb, tid, after_step);
  } else {
    block_gemm_run<SPLIT, false>(acc, s, k_begin, k_end, sa, sb, tid, after_step);
  }
}
template <bool SPLIT, typename SA, typename SB, typename AFTER>
DEVI void block_gemm_pipe(GemmAcc &acc, GemmLds &s, int k_begin, int k_end, SA &&sa, SB &&sb, int tid, AFTER after_step) {
  block_gemm_pipe<SPLIT, false>(acc, s, k_begin, k_end, sa, sb, tid, after_step);
}
template <bool SPLIT, typename SA, typename SB>
DEVI void block_gemm_pipe(GemmAcc &acc, GemmLds &s, int k_begin, int k_end, SA &&sa, SB &&sb, int tid) {
  block_gemm_pipe<SPLIT, false>(acc, s, k_begin, k_end, sa, sb, tid, [](int) {});
}
template <bool SPLIT, bool RING, typename SA, typename SB>
DEVI void block_gemm_pipe(GemmAcc &acc, GemmLds &s, int k_begin, int k_end, SA &&sa, SB &&sb, int tid) {
  block_gemm_pipe<SPLIT, RING>(acc, s, k_begin, k_end, sa, sb, tid, [](int) {});
}

// A k axis made of equal segments (one per head, say), each `seg_k` long (a multiple of the k step):
// before the first fetch of segment i, point(inner, i) re-targets the wrapped stager; inside a
// segment the wrapped stager sees k relative to the segment start.  The pipeline then runs through
// all segments without draining.  The constructor points at segment 0, whose alignment stands for
// all segments when the fast path is chosen.
template <typename Inner, typename PT> struct SegStager {
  static constexpr bool transposed = Inner::transposed;
  Inner inner;
  PT point;
  int seg_k, cur_seg;  // cur_seg: the segment the wrapped stager points at (the one of this object's last fetch)
  DEVI SegStager(Inner inner_, PT point_, int seg_k_) : inner(inner_), point(point_), seg_k(seg_k_), cur_seg(0) { point(inner, 0); }
  DEVI bool fast() const { return inner.fast(); }
  template <bool FAST> DEVI void fetch(int k0) {
    const int seg = k0 / seg_k, kk = k0 - seg * seg_k;
    if (seg != cur_seg) {
      point(inner, seg);
      cur_seg = seg;
    }
    inner.template fetch<FAST>(kk);
  }
  template <bool FAST> DEVI void commit(int k0) { inner.template commit<FAST>(k0 % seg_k); }
};
template <typename Inner, typename PT> DEVI SegStager<Inner, PT> seg_stager(Inner inner, PT point, int seg_k) {
  return SegStager<Inner, PT>(inner, point, seg_k);
}

// Stager for a causal operand on top of a row-contiguous stager: k steps below `diag_end` take an
// exact per-element multiplier f(tile row, k) (mask and decay), the others the stager's rank-1
// scale vectors.  Either way the loads go through the same fetch.
template <bool SPLIT, typename F, typename Inner> struct DiagStager {
  static constexpr bool transposed = Inner::transposed;
  F f;
  int diag_end;
  Inner inner;
  DEVI DiagStager(F f_, int diag_end_, Inner inner_) : f(f_), diag_end(diag_end_), inner(inner_) {}
  DEVI bool fast() const { return inner.fast(); }
  template <bool FAST> DEVI void fetch(int k0) { inner.template fetch<FAST>(k0); }
  template <bool FAST> DEVI void commit(int k0) {
    if (k0 < diag_end) inner.template commit_each<FAST>(k0, f);
    else inner.template commit<FAST>(k0);
  }
};
template <bool SPLIT, typename F, typename Inner> DEVI DiagStager<SPLIT, F, Inner> diag_stager(F f, int diag_end, Inner inner) {
  return DiagStager<SPLIT, F, Inner>(f, diag_end, inner);
}

// Visits the block tile's accumulator: value = f(m, n, value) with m, n in [0, 64).
template <typename F> DEVI void acc_foreach(GemmAcc &acc, int tid, F f) {
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int i = lane & 15, g = lane >> 4;
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        acc.v[tm][tn][r] = f(wm * 32 + tm * 16 + g * 4 + r, wn * 32 + tn * 16 + i, acc.v[tm][tn][r]);
}

// Re-lays the block tile from the MFMA accumulator layout to rows: thread t receives row t / 4,
// columns 16 * (t % 4) .. + 15.  Goes through LDS in the storage of the GEMM tiles (free once the
// leading barrier is passed).  All 256 threads call.
DEVI void acc_to_rows(const GemmAcc &acc, GemmLds &s, int tid, float (&o)[16]) {
  constexpr int PLD = GB + 4;
  static_assert(sizeof(GemmLds) >= GB * PLD * sizeof(float), "row patch must fit in the GEMM tiles");
  float *patch = reinterpret_cast<float *>(&s);
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int i = lane & 15, g = lane >> 4;
  __syncthreads();
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        patch[(wm * 32 + tm * 16 + g * 4 + r) * PLD + wn * 32 + tn * 16 + i] = acc.v[tm][tn][r];
  __syncthreads();
  const float *src = patch + (tid >> 2) * PLD + (tid & 3) * 16;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const f32x4 v = *reinterpret_cast<const f32x4 *>(src + 4 * q);
    o[4 * q] = v.x; o[4 * q + 1] = v.y; o[4 * q + 2] = v.z; o[4 * q + 3] = v.w;
  }
}

DEVI int cdiv(int a, int b) { return (a + b - 1) / b; }

// Logical block coordinates.  The hardware deals consecutive workgroup ids to the 8 XCDs in turn,
// and every XCD has its own L2; this remap gives each XCD one contiguous range of logical ids, so
// that neighbours along x (tiles that share operands) run at about the same time behind one L2.
struct Block3 {
  int x, y, z;
};
DEVI int xcd_linear_block() {
  const int nx = gridDim.x, ny = gridDim.y, total = nx * ny * gridDim.z;
  const int pid = blockIdx.x + nx * (blockIdx.y + ny * blockIdx.z);
  const int per = total / 8;
  return pid < per * 8 ? (pid % 8) * per + pid / 8 : pid;
}
DEVI Block3 xcd_block() {
  const int nx = gridDim.x, ny = gridDim.y;
  const int lid = xcd_linear_block();
  return {lid % nx, (lid / nx) % ny, lid / (nx * ny)};
}
// For a grid of (tiles, chunks, batch * heads) whose workgroups of one (batch, chunk) share that chunk's B / C rows of
// their group: {tile, chunk, batch * H + head} with the heads next to each other in the logical order, then the
// chunks, then the batch rows.  With the chunks next to each other instead (xcd_block) a group's rows of a chunk come
// round again only after every other chunk of the sequence, and on a long sequence (128 chunks) they have left the L2
// by then: the product kernels of the packed benchmark read them once per head from memory.
DEVI Block3 xcd_block_heads(int H) {
  const int nx = gridDim.x, ny = gridDim.y;
  const int lid = xcd_linear_block();
  const int rest = lid / nx, h = rest % H, c = (rest / H) % ny, b = rest / (H * ny);
  return {lid % nx, c, b * H + h};
}

// ---- pieces shared by the backward kernels
struct View4 {  // (b, L, H, P) tensor, P stride 1
  const void *ptr;
  int64_t bs, ls, hs;
};
DEVI View4 g_view(const SsdParams &p) {
  if (p.z) return {p.gbuf, (int64_t)p.seqlen * p.nheads * p.headdim, (int64_t)p.nheads * p.headdim, p.headdim};
  return {p.dout, p.dout_bs, p.dout_ls, p.dout_hs};
}


DEVI float *chunk_row(float *base, const SsdParams &p, int b, int h, int c) {
  return base + (((int64_t)b * p.nheads + h) * p.nchunks + c) * p.chunk_size;
}
DEVI int64_t chunk_off(const SsdParams &p, int b, int h, int c) {
  return (((int64_t)b * p.nheads + h) * p.nchunks + c) * p.chunk_size;
}

// Sums that several workgroups add into one address.  Default: float atomics (the order of the adds, hence the
// last bits of the sum, changes from run to run).  Deterministic mode (p.det_scale set): the term is scaled by a
// power of two common to the whole call, rounded to an integer and added with a 64-bit integer atomic into the
// shadow of the buffer; integer addition is associative, so the sum is the same in every order, and
// det_convert_kernel turns the shadow into the float buffer before its first reader runs.
DEVI float det_scale_of(const SsdParams &p) { return p.det_scale ? p.det_scale[0] : 0.f; }
// MODE: -1 decides at run time from dsc (the small kernels), 0 / 1 are compiled for one form (the kernels whose inner
// loops hold these adds: carrying both forms costs them registers and ~10 % of their time).
template <int MODE = -1> DEVI void acc_add(float *dst, int64_t *shadow, int64_t idx, float v, float dsc) {
  if (MODE == 1 || (MODE < 0 && dsc != 0.f)) {
    det_add(shadow, idx, v, dsc);
  } else {
    unsafeAtomicAdd(dst + idx, v);
  }
}

// The fused dx kernel (ssd_dx_fused.hip): launches it and returns MAMBA_OK, or returns MAMBA_E_UNSUPPORTED when it has
// no kernel for the problem (the caller then runs the tiled bwd_dx_kernel).
__attribute__((visibility("hidden"))) int ssd_bwd_dx_fused_launch(const SsdParams *p, hipStream_t stream, bool sum_dD);
__attribute__((visibility("hidden"))) bool ssd_bwd_dx_fused_supported(const SsdParams *p);
// The fused chunk-state dB / dC kernels (ssd_dbc_fused.hip), under the same convention (the caller then runs the
// tiled bwd_d*_state kernels).
__attribute__((visibility("hidden"))) int ssd_bwd_dbc_fused_launch(const SsdParams *p, hipStream_t stream);
__attribute__((visibility("hidden"))) bool ssd_bwd_dbc_fused_owns(const SsdParams *p);

// ---- host side of the kernels that work through the heads of a group in one workgroup
inline bool aligned(const void *ptr, int a) { return (reinterpret_cast<uintptr_t>(ptr) % a) == 0; }

// Heads per workgroup: a divisor of the heads per group, 20 at most.  One workgroup fills a CU, so the launch runs in
// ceil(workgroups / CUs) rounds, each as long as what a workgroup pays once (launch, arguments, C rows, the first
// head's exposed memory latency: measured at about 0.15 of a head's work) plus its heads; the divisor with the
// shortest estimate wins.
inline int heads_per_workgroup(const SsdParams &p) {
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

// The fused chunk scan with two tiles per wave (ssd_scan_paired.hip), for problems that
// ssd_chunk_scan_fwd_fused_supported accepts.
__attribute__((visibility("hidden"))) bool ssd_scan_paired_serves(const SsdParams &p);
__attribute__((visibility("hidden"))) int ssd_scan_paired_launch(const SsdParams &p, hipStream_t s);
// MAMBA_AMD_SSD_SCAN=single keeps the one-tile-per-wave kernel for every chunk size (for measurements).
inline bool ssd_single_tile_only() {
  static const bool v = [] {
    const char *e = getenv("MAMBA_AMD_SSD_SCAN");
    return e && e[0] == 's';
  }();
  return v;
}

// ------------------------------------------------------------------ batch slices
// The kernels index (batch, head) pairs with one 16-bit grid coordinate.  A larger problem is served by the entry
// points in slices of whole batch rows (rows are independent; the sums shared by all rows -- dA, dD, ddt_bias and
// their integer shadows -- are added into by every slice): the same parameters with every per-row pointer advanced.
constexpr int64_t SSD_MAX_GRID_ROWS = 65535;

inline SsdParams ssd_batch_slice(const SsdParams &p, int64_t b0, int nb) {
  SsdParams q = p;
  q.batch = nb;
  const int64_t es = p.dtype == MAMBA_F32 ? 4 : 2, ds = p.dt_dtype == MAMBA_F32 ? 4 : 2;
  const int64_t H = p.nheads, P = p.headdim, N = p.dstate, G = p.ngroups, L = p.seqlen, Q = p.chunk_size, c = p.nchunks;
  auto adv = [&](auto *&ptr, int64_t elems, int64_t size) {
    if (ptr) ptr = reinterpret_cast<std::remove_reference_t<decltype(ptr)>>(
                 reinterpret_cast<uintptr_t>(ptr) + (uintptr_t)(b0 * elems * size));
  };
  adv(q.x, p.x_bs, es), adv(q.z, p.z_bs, es), adv(q.out, p.out_bs, es), adv(q.out_x, p.out_bs, es);
  adv(q.B, p.B_bs, es), adv(q.C, p.C_bs, es), adv(q.dt, p.dt_bs, ds);
  adv(q.initial_states, H * P * N, 4), adv(q.seq_idx, L, 4);
  adv(q.dt_out, H * c * Q, 4), adv(q.dA_cumsum, H * c * Q, 4);
  adv(q.states, c * H * P * N, 4), adv(q.states_lp, c * H * P * N, 2), adv(q.final_states, H * P * N, 4);
  adv(q.CB, c * G * Q * Q, 4);
  adv(q.dout, p.dout_bs, es), adv(q.dfinal_states, H * P * N, 4), adv(q.dx, p.dx_bs, es), adv(q.dz, L * H * P, es);
  adv(q.ddt, L * H, ds), adv(q.dB, L * G * N, es), adv(q.dC, L * G * N, es), adv(q.dinitial_states, H * P * N, 4);
  adv(q.dstates, c * H * P * N, 4), adv(q.dstates_lp, c * H * P * N, 2);
  adv(q.ddA_cumsum, H * c * Q, 4), adv(q.ddt_out, H * c * Q, 4), adv(q.dCB, c * G * Q * Q, 4);
  adv(q.dB32, L * G * N, 4), adv(q.dC32, L * G * N, 4), adv(q.gbuf, L * H * P, es);
  adv(q.det_ddA_cumsum, H * c * Q, 8), adv(q.det_ddt_out, H * c * Q, 8), adv(q.det_dCB, c * G * Q * Q, 8);
  adv(q.det_dB, L * G * N, 8), adv(q.det_dC, L * G * N, 8);
  return q;
}

// Runs `one` on the whole problem when one launch can index it, else on slices of whole batch rows.
template <typename F> inline int ssd_sliced(const SsdParams *p, mamba_stream_t stream, F one) {
  if (!p || p->batch <= 0 || p->nheads <= 0 || p->nheads > SSD_MAX_GRID_ROWS ||
      (int64_t)p->batch * p->nheads <= SSD_MAX_GRID_ROWS)
    return one(p, stream);
  const int rows = (int)(SSD_MAX_GRID_ROWS / p->nheads);
  for (int64_t b0 = 0; b0 < p->batch; b0 += rows) {
    const SsdParams q = ssd_batch_slice(*p, b0, (int)std::min<int64_t>(rows, p->batch - b0));
    const int rc = one(&q, stream);
    if (rc) return rc;
  }
  return MAMBA_OK;
}
