// Pieces shared by the norm kernels (gated group norm, residual-add norm): sums over a team of
// threads, one row of channels held in registers in its packed form, the reduction of the per-part
// partial sums of dweight / dbias.
#pragma once
#include "common.hpp"

#include <type_traits>

namespace {

// Sums over the TEAM threads that share a (row, group): lanes of one wave by xor shuffles, waves of
// a workgroup through LDS.
template <int TEAM> struct TeamSum {
  static constexpr int NW = TEAM / 64;
  float *red;  // LDS: 2 slots x NW x 2 floats
  int slot = 0;
  DEVI explicit TeamSum(float *lds) : red(lds) {}
  DEVI void sum2(float &a, float &b) {
#pragma unroll
    for (int off = (TEAM < 64 ? TEAM : 64) / 2; off >= 1; off >>= 1) {
      a += __shfl_xor(a, off, 64);
      b += __shfl_xor(b, off, 64);
    }
    if constexpr (NW > 1) {
      const int wave = threadIdx.x >> 6;
      float *s = red + slot * NW * 2;
      if ((threadIdx.x & 63) == 0) {
        s[wave * 2] = a;
        s[wave * 2 + 1] = b;
      }
      __syncthreads();
      a = 0.f;
      b = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        a += s[w * 2];
        b += s[w * 2 + 1];
      }
      slot ^= 1;  // the next sum uses the other slot, so one barrier per sum is enough
    }
  }
};

// K steps of 8 channels of one row, as loaded (16 bytes per step when VEC): the next row is fetched
// into this form while the current one is worked on, at half the registers of its fp32 values.
struct F8 {
  float f[8];
};
template <typename T, bool VEC, int K, int TEAM> struct RowBuf {
  using Slot = std::conditional_t<VEC, Pack8<T>, F8>;
  Slot s[K];
  DEVI void fetch(const T *row, int col, int gs) {
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int c = col + k * TEAM * 8;
      const int nv = min(max(gs - c, 0), 8);
      if constexpr (VEC) {
        if (nv == 8) s[k].load(row + c);
        else s[k].zero();
      } else {
        ld8_guard<T, false>(row + c, nv, 0.f, s[k].f);
      }
    }
  }
  DEVI void get(float (&v)[K][8]) const {
#pragma unroll
    for (int k = 0; k < K; ++k) {
      if constexpr (VEC) s[k].unpack(v[k]);
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[k][e] = s[k].f[e];
      }
    }
  }
};

template <typename T, bool VEC, int K, int TEAM>
DEVI void load_row(const T *row, int col, int gs, float (&v)[K][8]) {
  RowBuf<T, VEC, K, TEAM> b;
  b.fetch(row, col, gs);
  b.get(v);
}
template <typename T, bool VEC, int K, int TEAM>
DEVI void store_row(T *row, int col, int gs, const float (&v)[K][8]) {
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int c = col + k * TEAM * 8;
    const int nv = min(max(gs - c, 0), 8);
    if (nv > 0) st8_guard<T, VEC>(row + c, nv, v[k]);
  }
}

// dweight[c] = sum over parts of dw_part[part][c] (and the same for dbias): 64 channels x 16 slices
// of the parts per workgroup.
__global__ __launch_bounds__(1024) void norm_reduce_kernel(const float *dw_part, const float *db_part, float *dw,
                                                           float *db, int nparts, int dim) {
  __shared__ float s[2][16][64];
  const int cl = threadIdx.x & 63, sl = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + cl;
  float a = 0.f, b = 0.f;
  if (c < dim)
    for (int q = sl; q < nparts; q += 16) {
      a += dw_part[(int64_t)q * dim + c];
      if (db_part) b += db_part[(int64_t)q * dim + c];
    }
  s[0][sl][cl] = a;
  s[1][sl][cl] = b;
  __syncthreads();
  if (sl == 0 && c < dim) {
    a = 0.f;
    b = 0.f;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      a += s[0][q][cl];
      b += s[1][q][cl];
    }
    dw[c] = a;
    if (db) db[c] = b;
  }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace
