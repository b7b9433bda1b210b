// Device-side helpers shared by the gfx950 kernels: dtype load/store, fast
// transcendental wrappers, DPP wave64 primitives.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mamba_hip.h"

#define DEVI __device__ __forceinline__

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

struct bf16_t { uint16_t v; };
struct f16_t { uint16_t v; };

// ---------------------------------------------------------------- conversions
DEVI float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
DEVI float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
DEVI uint32_t f32_to_bf16_bits(float x) {
  __bf16 b = (__bf16)x;  // round-to-nearest-even; v_cvt_pk_bf16_f32 on gfx950
  return (uint32_t)__builtin_bit_cast(uint16_t, b);
}
DEVI uint32_t pack_bf16(float lo, float hi) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  bf2 r;
  r.x = (__bf16)lo;
  r.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, r);
}
DEVI float f16_lo(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu)); }
DEVI float f16_hi(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)); }
DEVI uint32_t pack_f16(float lo, float hi) {
  uint32_t a = __builtin_bit_cast(uint16_t, (_Float16)lo);
  uint32_t b = __builtin_bit_cast(uint16_t, (_Float16)hi);
  return a | (b << 16);
}

template <typename T> struct DT;
template <> struct DT<float> { static constexpr int id = MAMBA_F32; };
template <> struct DT<bf16_t> { static constexpr int id = MAMBA_BF16; };
template <> struct DT<f16_t> { static constexpr int id = MAMBA_F16; };

template <typename T> DEVI float ld1(const T *p);
template <> DEVI float ld1<float>(const float *p) { return *p; }
template <> DEVI float ld1<bf16_t>(const bf16_t *p) { return __builtin_bit_cast(float, (uint32_t)p->v << 16); }
template <> DEVI float ld1<f16_t>(const f16_t *p) { return (float)__builtin_bit_cast(_Float16, p->v); }

template <typename T> DEVI void st1(T *p, float x);
template <> DEVI void st1<float>(float *p, float x) { *p = x; }
template <> DEVI void st1<bf16_t>(bf16_t *p, float x) { p->v = (uint16_t)f32_to_bf16_bits(x); }
template <> DEVI void st1<f16_t>(f16_t *p, float x) { p->v = __builtin_bit_cast(uint16_t, (_Float16)x); }

// 8 consecutive elements; p must be 16-byte aligned.
template <typename T> DEVI void ld8(const T *p, float (&o)[8]);
template <> DEVI void ld8<float>(const float *p, float (&o)[8]) {
  f32x4 a = *reinterpret_cast<const f32x4 *>(p);
  f32x4 b = *reinterpret_cast<const f32x4 *>(p + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
  o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
template <> DEVI void ld8<bf16_t>(const bf16_t *p, float (&o)[8]) {
  u32x4 a = *reinterpret_cast<const u32x4 *>(p);
  o[0] = bf16_lo(a.x); o[1] = bf16_hi(a.x); o[2] = bf16_lo(a.y); o[3] = bf16_hi(a.y);
  o[4] = bf16_lo(a.z); o[5] = bf16_hi(a.z); o[6] = bf16_lo(a.w); o[7] = bf16_hi(a.w);
}
template <> DEVI void ld8<f16_t>(const f16_t *p, float (&o)[8]) {
  u32x4 a = *reinterpret_cast<const u32x4 *>(p);
  o[0] = f16_lo(a.x); o[1] = f16_hi(a.x); o[2] = f16_lo(a.y); o[3] = f16_hi(a.y);
  o[4] = f16_lo(a.z); o[5] = f16_hi(a.z); o[6] = f16_lo(a.w); o[7] = f16_hi(a.w);
}
template <typename T> DEVI void st8(T *p, const float (&v)[8]);
template <> DEVI void st8<float>(float *p, const float (&v)[8]) {
  f32x4 a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
  *reinterpret_cast<f32x4 *>(p) = a;
  *reinterpret_cast<f32x4 *>(p + 4) = b;
}
template <> DEVI void st8<bf16_t>(bf16_t *p, const float (&v)[8]) {
  u32x4 a = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
  *reinterpret_cast<u32x4 *>(p) = a;
}
template <> DEVI void st8<f16_t>(f16_t *p, const float (&v)[8]) {
  u32x4 a = {pack_f16(v[0], v[1]), pack_f16(v[2], v[3]), pack_f16(v[4], v[5]), pack_f16(v[6], v[7])};
  *reinterpret_cast<u32x4 *>(p) = a;
}

// 8 values kept in registers in the storage format of T (exact round trip for values that were
// loaded from T): 4 registers for 16-bit types, 8 for fp32.
// Accesses that name the global address space.  A pointer that a kernel reads back from LDS or from
// memory has lost its address space, and plain accesses through it become flat instructions, which
// count in the LDS counter as well as in the memory counter: every wait for an LDS read then also waits
// for the flat accesses in flight.
#define GLOBAL_AS __attribute__((address_space(1)))

template <typename T> struct Pack8 {
  u32x4 w;
  DEVI void load(const T *p) { w = *reinterpret_cast<const u32x4 *>(p); }  // 16-byte aligned
  DEVI void load_global(const T *p) { w = *(const GLOBAL_AS u32x4 *)p; }
  DEVI void store_global(T *p) const { *(GLOBAL_AS u32x4 *)p = w; }
  DEVI void zero() { w = u32x4{0, 0, 0, 0}; }
  DEVI void pack(const float (&v)[8]) {
    if constexpr (DT<T>::id == MAMBA_BF16) {
      w = u32x4{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
    } else {
      w = u32x4{pack_f16(v[0], v[1]), pack_f16(v[2], v[3]), pack_f16(v[4], v[5]), pack_f16(v[6], v[7])};
    }
  }
  DEVI void unpack(float (&o)[8]) const {
    if constexpr (DT<T>::id == MAMBA_BF16) {
      o[0] = bf16_lo(w.x); o[1] = bf16_hi(w.x); o[2] = bf16_lo(w.y); o[3] = bf16_hi(w.y);
      o[4] = bf16_lo(w.z); o[5] = bf16_hi(w.z); o[6] = bf16_lo(w.w); o[7] = bf16_hi(w.w);
    } else {
      o[0] = f16_lo(w.x); o[1] = f16_hi(w.x); o[2] = f16_lo(w.y); o[3] = f16_hi(w.y);
      o[4] = f16_lo(w.z); o[5] = f16_hi(w.z); o[6] = f16_lo(w.w); o[7] = f16_hi(w.w);
    }
  }
};
template <> struct Pack8<float> {
  float v[8];
  DEVI void load(const float *p) {
    const f32x4 a = *reinterpret_cast<const f32x4 *>(p), b = *reinterpret_cast<const f32x4 *>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  DEVI void load_global(const float *p) {
    const f32x4 a = *(const GLOBAL_AS f32x4 *)p, b = *(const GLOBAL_AS f32x4 *)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  DEVI void store_global(float *p) const {
    *(GLOBAL_AS f32x4 *)p = f32x4{v[0], v[1], v[2], v[3]};
    *(GLOBAL_AS f32x4 *)(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
  }
  DEVI void zero() {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 0.f;
  }
  DEVI void pack(const float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = x[i];
  }
  DEVI void unpack(float (&o)[8]) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = v[i];
  }
};

// 8 elements starting at p[0], of which only the first `nvalid` (0..8) exist;
// the rest read as `fill`.  VEC: all-or-nothing 16-byte path.
template <typename T, bool VEC> DEVI void ld8_guard(const T *p, int nvalid, float fill, float (&o)[8]) {
  if (VEC) {
    if (nvalid >= 8) {
      ld8<T>(p, o);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = fill;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (i < nvalid) ? ld1<T>(p + i) : fill;
  }
}
template <typename T, bool VEC> DEVI void st8_guard(T *p, int nvalid, const float (&v)[8]) {
  if (VEC) {
    if (nvalid >= 8) st8<T>(p, v);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < nvalid) st1<T>(p + i, v[i]);
  }
}

// The same through the global address space: 8 values stored as T with 16-byte accesses (all or nothing), or
// element by element through the generic path.
template <typename T, bool VEC> DEVI void st8_guard_global(T *p, int nvalid, const float (&v)[8]) {
  if constexpr (VEC) {
    if (nvalid < 8) return;
    if constexpr (DT<T>::id == MAMBA_F32) {
      *(GLOBAL_AS f32x4 *)p = f32x4{v[0], v[1], v[2], v[3]};
      *(GLOBAL_AS f32x4 *)(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
    } else {
      Pack8<T> k;
      k.pack(v);
      *(GLOBAL_AS u32x4 *)p = k.w;
    }
  } else {
    st8_guard<T, false>(p, nvalid, v);
  }
}

// The same with no branch around the store on the 16-byte path: a lane with nothing to store (too few valid values, or
// a destination that is not wanted) writes to `spare`, 32 bytes of its own that nobody reads.  A branch around a
// store makes the compiler's count of the memory operations in flight inexact after it, and the next wait for an
// older load then waits for the stores as well.
template <typename T, bool VEC>
DEVI void st8_or_spare_global(T *p, int nvalid, bool wanted, T *spare, const float (&v)[8]) {
  if constexpr (VEC) {
    T *dst = (wanted && nvalid >= 8) ? p : spare;
    if constexpr (DT<T>::id == MAMBA_F32) {
      *(GLOBAL_AS f32x4 *)dst = f32x4{v[0], v[1], v[2], v[3]};
      *(GLOBAL_AS f32x4 *)(dst + 4) = f32x4{v[4], v[5], v[6], v[7]};
    } else {
      Pack8<T> k;
      k.pack(v);
      *(GLOBAL_AS u32x4 *)dst = k.w;
    }
  } else {
    if (wanted) st8_guard<T, false>(p, nvalid, v);
  }
}

// ------------------------------------------------------------------- math
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

DEVI float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }          // v_exp_f32
DEVI float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }
DEVI float fast_log(float x) { return __builtin_amdgcn_logf(x) * kLn2; }     // v_log_f32
DEVI float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// softplus with the reference's threshold: x <= 20 ? log1p(exp(x)) : x.
// log1p(e) for small e is evaluated by its series so that tiny step sizes keep
// full relative precision.
DEVI float softplus_f(float x) {
  float e = fast_exp(fminf(x, 20.f));
  float big = fast_log(1.f + e);
  float small = e * (1.f - e * (0.5f - e * (0.33333333f - 0.25f * e)));
  float r = (e < 0.03f) ? small : big;
  return x <= 20.f ? r : x;
}
DEVI float sigmoid_f(float x) { return fast_rcp(1.f + fast_exp(-x)); }
// d softplus(x) / dx = sigmoid(x), from y = softplus(x) alone: 1 - exp(-y) (= 1 / (1 + exp(-x)); above the softplus
// threshold, where y = x, it differs from the slope 1 by less than exp(-20)).  For small y the difference is taken
// from the series so that tiny steps keep their relative precision.
DEVI float softplus_slope_f(float y) {
  const float big = 1.f - fast_exp(-y);
  const float small = y * (1.f - y * (0.5f - y * (0.16666667f - 0.041666668f * y)));
  return y < 0.03f ? small : big;
}

// Workgroup barrier for code that hands data from wave to wave through LDS only.  __syncthreads() is a fence
// as well: it waits for every outstanding global access of the wave, stores included, so a barrier that follows a
// burst of row stores sits through their whole write latency.  This one waits for the wave's LDS accesses alone;
// global stores keep draining behind it.  (Nothing read through it may come from global memory written by another
// wave of the workgroup.)
DEVI void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ------------------------------------------------------------------- fixed-point sums
// One term of a sum kept as a 64-bit integer of fixed-point terms (the deterministic mode): v * scale rounded to an
// integer and added with an integer atomic, whose result does not depend on the order of the adds.  A finite term is
// clamped to +-2^59; a term that is not finite (NaN, Inf) replaces the sum by 2^62, which later adds cannot bring back
// below 2^61 in magnitude: det_value() turns every sum of magnitude >= 2^61 -- poisoned, or overflowed -- into NaN, so
// that non-finite gradients stay visible as they do with float atomics.
DEVI void det_add(int64_t *shadow, int64_t idx, float v, float scale) {
  unsigned long long *dst = reinterpret_cast<unsigned long long *>(shadow + idx);
  const float q = v * scale;
  if (__builtin_fabsf(q) <= 3.4e38f) {  // finite
    const float c = fminf(fmaxf(q, -5.7e17f), 5.7e17f);
    __hip_atomic_fetch_add(dst, static_cast<unsigned long long>(static_cast<long long>(__builtin_rintf(c))), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
  } else {
    __hip_atomic_exchange(dst, 1ull << 62, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}
DEVI float det_value(int64_t sum, float inv_scale) {
  const int64_t mag = sum < 0 ? -sum : sum;
  if (mag >= (int64_t(1) << 61) || sum == INT64_MIN) return __builtin_nanf("");
  return (float)((double)sum * (double)inv_scale);
}

// ------------------------------------------------------------------- DPP
// dpp_ctrl encodings of the GFX9 family.
enum : int {
  DPP_ROW_SHL = 0x100,
  DPP_ROW_SHR = 0x110,
  DPP_WAVE_SHL1 = 0x130,
  DPP_WAVE_SHR1 = 0x138,
  DPP_ROW_BCAST15 = 0x142,
  DPP_ROW_BCAST31 = 0x143
};

// Lanes whose DPP source does not exist (or whose row is masked off) get `old`.
template <int CTRL, int ROW_MASK = 0xf> DEVI float dpp_f(float old, float src) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, src), CTRL, ROW_MASK,
                                         0xf, false));
}
DEVI float readlane_f(float x, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

// Inclusive scan over the 64 lanes (lane 0 first) of first-order recurrence
// segments (a, b) meaning h_out = a * h_in + b.
DEVI void wave_scan_fwd(float &a, float &b) {
#define MAMBA_STEP(CTRL, MASK)                   \
  {                                              \
    float bp = dpp_f<CTRL, MASK>(0.f, b);        \
    float ap = dpp_f<CTRL, MASK>(1.f, a);        \
    b = __builtin_fmaf(a, bp, b);                \
    a = a * ap;                                  \
  }
  MAMBA_STEP(DPP_ROW_SHR + 1, 0xf)
  MAMBA_STEP(DPP_ROW_SHR + 2, 0xf)
  MAMBA_STEP(DPP_ROW_SHR + 4, 0xf)
  MAMBA_STEP(DPP_ROW_SHR + 8, 0xf)
  MAMBA_STEP(DPP_ROW_BCAST15, 0xa)
  MAMBA_STEP(DPP_ROW_BCAST31, 0xc)
#undef MAMBA_STEP
}

// Inclusive scan in the other direction (lane 63 first): on return lane l
// holds the composition of lanes l..63, again as h_out = a * h_in + b where
// h_in enters after lane 63.
DEVI void wave_scan_rev(float &a, float &b, int lane) {
#define MAMBA_STEP(N)                                      \
  {                                                        \
    float bp = dpp_f<DPP_ROW_SHL + N>(0.f, b);             \
    float ap = dpp_f<DPP_ROW_SHL + N>(1.f, a);             \
    b = __builtin_fmaf(a, bp, b);                          \
    a = a * ap;                                            \
  }
  MAMBA_STEP(1)
  MAMBA_STEP(2)
  MAMBA_STEP(4)
  MAMBA_STEP(8)
#undef MAMBA_STEP
  // rows 1..3 as whole segments, taken from their first lanes
  float a1 = readlane_f(a, 16), b1 = readlane_f(b, 16);
  float a2 = readlane_f(a, 32), b2 = readlane_f(b, 32);
  float a3 = readlane_f(a, 48), b3 = readlane_f(b, 48);
  // segment that follows each row: row2 <- row3, row1 <- row2.row3, row0 <- row1.row2.row3
  float a23 = a2 * a3, b23 = __builtin_fmaf(a2, b3, b2);
  float a123 = a1 * a23, b123 = __builtin_fmaf(a1, b23, b1);
  int row = lane >> 4;
  float an = row == 0 ? a123 : (row == 1 ? a23 : (row == 2 ? a3 : 1.f));
  float bn = row == 0 ? b123 : (row == 1 ? b23 : (row == 2 ? b3 : 0.f));
  b = __builtin_fmaf(a, bn, b);
  a = a * an;
}

// The same two scans for two independent recurrences at once, with the DPP operand folded
// into the multiply / multiply-add (v_fmac_f32_dpp, v_mul_f32_dpp).  Lanes without a DPP source
// are left unwritten, which is the identity of the scan.  Interleaving the two chains keeps the
// two wait states the hardware wants between a VALU write and a DPP read of the same register.
#define MAMBA_DPP2(CTRL)                                                       \
  "v_fmac_f32_dpp %1, %1, %0 " CTRL " bank_mask:0xf\n\t"                      \
  "v_fmac_f32_dpp %3, %3, %2 " CTRL " bank_mask:0xf\n\t"                      \
  "v_mul_f32_dpp %0, %0, %0 " CTRL " bank_mask:0xf\n\t"                       \
  "v_mul_f32_dpp %2, %2, %2 " CTRL " bank_mask:0xf\n\t"

DEVI void wave_scan_fwd2(float &a0, float &b0, float &a1, float &b1) {
  asm volatile("s_nop 1\n\t"
               MAMBA_DPP2("row_shr:1 row_mask:0xf")
               MAMBA_DPP2("row_shr:2 row_mask:0xf")
               MAMBA_DPP2("row_shr:4 row_mask:0xf")
               MAMBA_DPP2("row_shr:8 row_mask:0xf")
               MAMBA_DPP2("row_bcast:15 row_mask:0xa")
               MAMBA_DPP2("row_bcast:31 row_mask:0xc")
               "s_nop 1\n\t"
               : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1));
}

// rows only (16 lanes each), towards lane 15 of the row: an inclusive scan per row
DEVI void row_scan_fwd2(float &a0, float &b0, float &a1, float &b1) {
  asm volatile("s_nop 1\n\t"
               MAMBA_DPP2("row_shr:1 row_mask:0xf")
               MAMBA_DPP2("row_shr:2 row_mask:0xf")
               MAMBA_DPP2("row_shr:4 row_mask:0xf")
               MAMBA_DPP2("row_shr:8 row_mask:0xf")
               "s_nop 1\n\t"
               : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1));
}

// rows only (16 lanes each), towards lane 0 of the row
DEVI void row_scan_rev2(float &a0, float &b0, float &a1, float &b1) {
  asm volatile("s_nop 1\n\t"
               MAMBA_DPP2("row_shl:1 row_mask:0xf")
               MAMBA_DPP2("row_shl:2 row_mask:0xf")
               MAMBA_DPP2("row_shl:4 row_mask:0xf")
               MAMBA_DPP2("row_shl:8 row_mask:0xf")
               "s_nop 1\n\t"
               : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1));
}
#undef MAMBA_DPP2

// The same row scans for one recurrence: a step reads through DPP what the step before wrote, which needs two
// wait states between the write and the read (the other instruction of the step plus s_nop 0).
#define MAMBA_DPP1(CTRL)                                                       \
  "v_fmac_f32_dpp %1, %1, %0 " CTRL " bank_mask:0xf\n\t"                      \
  "v_mul_f32_dpp %0, %0, %0 " CTRL " bank_mask:0xf\n\t"                       \
  "s_nop 0\n\t"
DEVI void row_scan_fwd1(float &a, float &b) {
  asm volatile("s_nop 1\n\t"
               MAMBA_DPP1("row_shr:1 row_mask:0xf")
               MAMBA_DPP1("row_shr:2 row_mask:0xf")
               MAMBA_DPP1("row_shr:4 row_mask:0xf")
               MAMBA_DPP1("row_shr:8 row_mask:0xf")
               "s_nop 0\n\t"
               : "+v"(a), "+v"(b));
}
DEVI void row_scan_rev1(float &a, float &b) {
  asm volatile("s_nop 1\n\t"
               MAMBA_DPP1("row_shl:1 row_mask:0xf")
               MAMBA_DPP1("row_shl:2 row_mask:0xf")
               MAMBA_DPP1("row_shl:4 row_mask:0xf")
               MAMBA_DPP1("row_shl:8 row_mask:0xf")
               "s_nop 0\n\t"
               : "+v"(a), "+v"(b));
}
#undef MAMBA_DPP1

// Completes a lane-reversed scan whose rows have been scanned by row_scan_rev2: appends to every
// row the composition of the rows after it.
DEVI void wave_scan_rev_finish(float &a, float &b, int lane) {
  float a1 = readlane_f(a, 16), b1 = readlane_f(b, 16);
  float a2 = readlane_f(a, 32), b2 = readlane_f(b, 32);
  float a3 = readlane_f(a, 48), b3 = readlane_f(b, 48);
  float a23 = a2 * a3, b23 = __builtin_fmaf(a2, b3, b2);
  float a123 = a1 * a23, b123 = __builtin_fmaf(a1, b23, b1);
  int row = lane >> 4;
  float an = row == 0 ? a123 : (row == 1 ? a23 : (row == 2 ? a3 : 1.f));
  float bn = row == 0 ? b123 : (row == 1 ? b23 : (row == 2 ? b3 : 0.f));
  b = __builtin_fmaf(a, bn, b);
  a = a * an;
}

// Sum over the 64 lanes by DPP adds; only lane 63 holds the full sum on return.
DEVI float wave_sum_to_last(float x) {
  x += dpp_f<DPP_ROW_SHR + 1>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 2>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 4>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 8>(0.f, x);
  x += dpp_f<DPP_ROW_BCAST15, 0xa>(0.f, x);
  x += dpp_f<DPP_ROW_BCAST31, 0xc>(0.f, x);
  return x;
}

// Sum over each row of 16 lanes; only the last lane of a row holds its sum on return.
DEVI float row_sum_to_last(float x) {
  x += dpp_f<DPP_ROW_SHR + 1>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 2>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 4>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 8>(0.f, x);
  return x;
}

DEVI float wave_sum(float x) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
  return x;
}

// Compute units of the current device (256 when the query fails).
inline int cu_count() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    cached[dev] = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256;
  }
  return cached[dev];
}
