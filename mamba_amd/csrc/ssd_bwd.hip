// Mamba-2 SSD backward for gfx950.  Dense contractions run on the bf16 MFMA
// block-GEMM core of ssd_common.hpp.
//
// Gradient of the decay exponents: every kernel adds its share of dL/da_l (a_l =
// running sum of dt * A inside the chunk) into ddA_cumsum; the last kernel turns
// that into dL/d(dt_l A) with a reverse running sum.  The shares are
//   inside the chunk, w[l, s] = (g_l . x_s) dt_s CB[l, s] exp(a_l - a_s):  + row sums at l,
//     - column sums at s, both taken from the same fp32 w so that pairs cancel in the
//     reverse running sum (the shortcut <g_l, y_l> from the stored output does not: its
//     rounding error is summed coherently over the chunk);
//   carried state:  + sum_n dC_state[l, n] C[l, n] at l;
//   chunk state:    - dt_s <x_s, state part of the dx accumulator> at s, + the same at the
//     chunk end;  state passing:  + scale <G, H> at the chunk end;
// with g = dout * silu(z).
#include "ssd_common.hpp"

namespace {

// The heads of a group are spread over this many workgroups (each sums ~8 heads in registers and
// adds its partial result atomically).
__host__ __device__ inline int head_splits(int heads_per_group) { return (heads_per_group + 7) / 8; }
// The dCB kernel's lists are twice as long (~16 heads).
__host__ __device__ inline int dcb_head_splits(int heads_per_group) { return (heads_per_group + 15) / 16; }

__global__ __launch_bounds__(256) void det_convert_kernel(const int64_t *__restrict__ src, float *__restrict__ dst, int64_t n,
                                                          const float *__restrict__ scale) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = det_value(src[i], scale[1]);
}

// Sums acc[m][n] * fx(m, n) over n for every row m of the block tile into rows[64] (LDS, zeroed
// here).  All 256 threads call; rows[] is valid after the trailing barrier.
template <typename F> DEVI void row_dot(GemmAcc &acc, float *rows, int tid, F fx) {
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int i = lane & 15, g = lane >> 4;
  __syncthreads();
  if (tid < GB) rows[tid] = 0.f;
  __syncthreads();
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = wm * 32 + tm * 16 + g * 4 + r;
      float s = 0.f;
#pragma unroll
      for (int tn = 0; tn < 2; ++tn) s += acc.v[tm][tn][r] * fx(m, wn * 32 + tn * 16 + i);
      s += dpp_f<DPP_ROW_SHR + 1>(0.f, s);
      s += dpp_f<DPP_ROW_SHR + 2>(0.f, s);
      s += dpp_f<DPP_ROW_SHR + 4>(0.f, s);
      s += dpp_f<DPP_ROW_SHR + 8>(0.f, s);
      if (i == 15) __hip_atomic_fetch_add(&rows[m], s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  __syncthreads();
}

// Row sums and column sums of the block tile held in acc, into rows[64] / cols[64] (LDS).
DEVI void row_col_sums(GemmAcc &acc, float *rows, float *cols, int tid) {
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int i = lane & 15, g = lane >> 4;
  __syncthreads();
  if (tid < GB) {
    rows[tid] = 0.f;
    cols[tid] = 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float s = acc.v[tm][0][r] + acc.v[tm][1][r];
      s += dpp_f<DPP_ROW_SHR + 1>(0.f, s);
      s += dpp_f<DPP_ROW_SHR + 2>(0.f, s);
      s += dpp_f<DPP_ROW_SHR + 4>(0.f, s);
      s += dpp_f<DPP_ROW_SHR + 8>(0.f, s);
      if (i == 15)
        __hip_atomic_fetch_add(&rows[wm * 32 + tm * 16 + g * 4 + r], s, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
    }
#pragma unroll
  for (int tn = 0; tn < 2; ++tn) {
    float s = 0.f;
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int r = 0; r < 4; ++r) s += acc.v[tm][tn][r];
    s += __shfl_xor(s, 16, 64);
    s += __shfl_xor(s, 32, 64);
    if (g == 0)
      __hip_atomic_fetch_add(&cols[wn * 32 + tn * 16 + i], s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  __syncthreads();
}

// ------------------------------------------------------------------- dz
// Per position: dz, g = dout silu(z), dD += g x.  A lane owns 8 consecutive p of one position
// (16-byte accesses when the rows allow it); a workgroup covers 64 positions of one (batch, head).
template <typename T> __global__ __launch_bounds__(256) void bwd_dz_kernel(const SsdParams p) {
  const int tid = threadIdx.x;
  const int L = p.seqlen, H = p.nheads, P = p.headdim;
  // (positions run fastest over the grid; with heads fastest -- whole rows in flight together -- it measured 14 % slower)
  const int h = blockIdx.y, b = blockIdx.z;
  const int pchunks = (P + 7) / 8;                 // 8-wide column groups per row
  const float *Dp = static_cast<const float *>(p.D);
  const void *yptr = p.z ? p.out_x : p.out;
  const bool vec = P % 8 == 0 && rows_aligned16(static_cast<const T *>(p.dout) + b * p.dout_bs + h * p.dout_hs, p.dout_ls) &&
                   rows_aligned16(static_cast<const T *>(p.x) + b * p.x_bs + h * p.x_hs, p.x_ls) &&
                   (!p.z || (rows_aligned16(static_cast<const T *>(p.z) + b * p.z_bs + h * p.z_hs, p.z_ls) &&
                             rows_aligned16(static_cast<const T *>(yptr) + b * p.out_bs + h * p.out_hs, p.out_ls)));
  // every thread keeps one column group (tid % pchunks is fixed when 256 % pchunks == 0; otherwise
  // the partial dD sums are flushed per task)
  const bool fixed_cols = 256 % pchunks == 0;
  float dDacc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int ntask = 64 * pchunks;
  for (int task = tid; task < ntask; task += 256) {
    const int t = blockIdx.x * 64 + task / pchunks, c8 = (task % pchunks) * 8;
    if (t >= L) break;
    const int nv = min(8, P - c8);
    float dout[8], x[8], g[8];
    const T *dop = static_cast<const T *>(p.dout) + b * p.dout_bs + (int64_t)t * p.dout_ls + h * p.dout_hs + c8;
    const T *xp = static_cast<const T *>(p.x) + b * p.x_bs + (int64_t)t * p.x_ls + h * p.x_hs + c8;
    if (vec) {
      ld8<T>(dop, dout);
      ld8<T>(xp, x);
    } else {
      ld8_guard<T, false>(dop, nv, 0.f, dout);
      ld8_guard<T, false>(xp, nv, 0.f, x);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] = dout[e];
    if (p.z) {
      float y[8], z[8], dz[8];
      const T *yp = static_cast<const T *>(yptr) + b * p.out_bs + (int64_t)t * p.out_ls + h * p.out_hs + c8;
      const T *zp = static_cast<const T *>(p.z) + b * p.z_bs + (int64_t)t * p.z_ls + h * p.z_hs + c8;
      if (vec) {
        ld8<T>(yp, y);
        ld8<T>(zp, z);
      } else {
        ld8_guard<T, false>(yp, nv, 0.f, y);
        ld8_guard<T, false>(zp, nv, 0.f, z);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float sg = sigmoid_f(z[e]);
        g[e] = dout[e] * z[e] * sg;
        dz[e] = dout[e] * y[e] * sg * (1.f + z[e] * (1.f - sg));
      }
      const int64_t oi = (((int64_t)b * L + t) * H + h) * P + c8;
      if (vec) {
        st8<T>(static_cast<T *>(p.dz) + oi, dz);
        st8<T>(static_cast<T *>(p.gbuf) + oi, g);
      } else {
        st8_guard<T, false>(static_cast<T *>(p.dz) + oi, nv, dz);
        st8_guard<T, false>(static_cast<T *>(p.gbuf) + oi, nv, g);
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) dDacc[e] = __builtin_fmaf(g[e], x[e], dDacc[e]);
    if (Dp && !fixed_cols) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (e < nv) acc_add(p.dD, p.det_dD, p.D_has_hdim ? h * P + c8 + e : h, dDacc[e], det_scale_of(p));
        dDacc[e] = 0.f;
      }
    }
  }
  if (Dp && fixed_cols) {
    __shared__ float red[256 * 9];                 // row stride 9: conflict-free column reads
#pragma unroll
    for (int e = 0; e < 8; ++e) red[tid * 9 + e] = dDacc[e];
    __syncthreads();
    if (p.D_has_hdim) {
      // column c of the head: threads with tid % pchunks == c / 8 hold its partial sums
      if (tid < P) {
        float sacc = 0.f;
        for (int r = tid / 8; r < 256; r += pchunks) sacc += red[r * 9 + (tid & 7)];
        acc_add(p.dD, p.det_dD, h * P + tid, sacc, det_scale_of(p));
      }
    } else if (tid < 64) {
      float sacc = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int e = 0; e < 8; ++e) sacc += red[(tid * 4 + r) * 9 + e];
      sacc = wave_sum(sacc);
      if (tid == 0) acc_add(p.dD, p.det_dD, h, sacc, det_scale_of(p));
    }
  }
}

// -------------------------------------------------------------- dstates
// dstates[b, c, h, p, n] = sum_l g[l, p] exp(a_l) [seq_l == seq before the chunk] C[l, n]
template <typename T, bool SPLIT> __global__ __launch_bounds__(256) void bwd_dstates_kernel(const SsdParams p) {
  __shared__ GemmLds lds;
  __shared__ float rs[256];
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads;
  const int ntn = cdiv(N, GB);
  const Block3 blk = xcd_block_heads(H);  // the tiles of one (chunk, head) share its x / g rows: same L2
  const int pt = blk.x / ntn, nt = blk.x % ntn;
  const int c = blk.y, b = blk.z / H, h = blk.z % H;
  const int g = h / (H / p.ngroups);
  const int t0 = c * Q, qlim = min(Q, L - t0);
  const float *dA = chunk_row(p.dA_cumsum, p, b, h, c);
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  for (int l = tid; l < Q; l += 256) {
    float v = 0.f;
    if (l < qlim) {
      bool ok = true;
      if (seq) ok = seq[l] == (c > 0 ? seq[-1] : 0);
      if (ok) v = fast_exp(dA[l]);
    }
    rs[l] = v;
  }
  const View4 gv = g_view(p);
  const int64_t gb = b * gv.bs + h * gv.hs, Cb = b * p.C_bs + g * p.C_gs;
  GemmAcc acc;
  acc.zero();
  // A = g^T (rows p, k = position), B = (C rs)^T (rows n, k = position)
  const T *ga = static_cast<const T *>(gv.ptr) + gb + (int64_t)t0 * gv.ls + pt * GB;
  const T *Ca = static_cast<const T *>(p.C) + Cb + (int64_t)t0 * p.C_ls + nt * GB;
  const bool va = rows_aligned16(ga, gv.ls), vb = rows_aligned16(Ca, p.C_ls);
  block_gemm_pipe<SPLIT>(
      acc, lds, 0, qlim,
      TrStager<SPLIT, T>(lds.ah, lds.al, ga, gv.ls, P - pt * GB, qlim, nullptr, nullptr, va, tid),
      TrStager<SPLIT, T>(lds.bh, lds.bl, Ca, p.C_ls, N - nt * GB, qlim, rs, nullptr, vb, tid),
      tid);
  carried_t<T> *ds = carried_dstates<T>(p) + (((int64_t)b * p.nchunks + c) * H + h) * P * N;
  acc_foreach(acc, tid, [&](int m, int n, float v) {
    const int pp = pt * GB + m, nn = nt * GB + n;
    if (pp < P && nn < N) st_carried(ds + (int64_t)pp * N + nn, v);
    return v;
  });
}

// The same product with a 64 x 128 tile per workgroup (whole 128-state blocks, aligned operands,
// chunks that are whole k steps).
template <typename T, bool SPLIT> __global__ __launch_bounds__(256) void bwd_dstates_wide_kernel(const SsdParams p) {
  __shared__ GemmLdsWide<SPLIT> lds;
  __shared__ float rs[256];
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads;
  const int ntn = N / WB;
  const Block3 blk = xcd_block_heads(H);
  const int pt = blk.x / ntn, nt = blk.x % ntn;
  const int c = blk.y, b = blk.z / H, h = blk.z % H;
  const int g = h / (H / p.ngroups);
  const int t0 = c * Q, qlim = min(Q, L - t0);
  const float *dA = chunk_row(p.dA_cumsum, p, b, h, c);
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  for (int l = tid; l < Q; l += 256) {
    float v = 0.f;
    if (l < qlim) {
      bool ok = true;
      if (seq) ok = seq[l] == (c > 0 ? seq[-1] : 0);
      if (ok) v = fast_exp(dA[l]);
    }
    rs[l] = v;
  }
  const View4 gv = g_view(p);
  const T *ga = static_cast<const T *>(gv.ptr) + b * gv.bs + h * gv.hs + (int64_t)t0 * gv.ls + pt * GB;
  const T *Ca = static_cast<const T *>(p.C) + b * p.C_bs + g * p.C_gs + (int64_t)t0 * p.C_ls + nt * WB;
  GemmAccWide acc;
  acc.zero();
  WideTrStager<SPLIT, T, 64> sa(lds.ah, lds.al, ga, gv.ls, P - pt * GB, nullptr, tid);
  WideTrStager<SPLIT, T, WB> sb(lds.bh, lds.bl, Ca, p.C_ls, WB, rs, tid);
  block_gemm_wide<SPLIT>(acc, lds, qlim, sa, sb, tid);  // the first barrier inside publishes rs
  carried_t<T> *ds = carried_dstates<T>(p) + (((int64_t)b * p.nchunks + c) * H + h) * P * N;
  store_wide_rows(acc, lds, ds + (int64_t)pt * GB * N + nt * WB, N, P - pt * GB, tid);
}

// dz, g = dout silu(z), dD and the state-gradient product of a (batch, chunk, head) in one pass (bf16 operands,
// 128 states, a gate): the stager of the product's A operand makes g from dout and z on its way to LDS, stores it
// and dz, and sums g x for dD; the product takes the stored (rounded) g, as the separate kernel does.  A thread's
// task per k step is one 16-byte piece of a position's row, the task of bwd_dz_kernel.
template <typename T> struct DzStager {
  static constexpr bool transposed = true;
  static constexpr int PITCH = WideTrStager<false, T, 64>::PITCH;
  uint16_t *hi;
  const T *dout, *z, *y, *x;  // at (batch, first position of the chunk, head, first p of the tile)
  T *dz, *g;
  int64_t dout_ls, z_ls, y_ls, x_ls, o_ls;
  int rows_valid, t;
  Pack8<T> qd, qz, qy, qx;
  float dD[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  DEVI bool fast() const { return true; }
  template <bool FAST = true> DEVI void fetch(int k0) {
    const int l = k0 + (t >> 3), r8 = min((t & 7) * 8, rows_valid - 8);
    qd.load(dout + (int64_t)l * dout_ls + r8);
    qz.load(z + (int64_t)l * z_ls + r8);
    qy.load(y + (int64_t)l * y_ls + r8);
    qx.load(x + (int64_t)l * x_ls + r8);
  }
  template <bool FAST = true> DEVI void commit(int k0) {
    const int kk = t >> 3, r8 = (t & 7) * 8, off = kk * PITCH + r8;
    Pack8<T> gq;
    gq.zero();
    if (r8 < rows_valid) {
      float d[8], zz[8], yy[8], xx[8], gv[8], dzv[8];
      qd.unpack(d);
      qz.unpack(zz);
      qy.unpack(yy);
      qx.unpack(xx);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float sg = sigmoid_f(zz[e]);
        gv[e] = d[e] * zz[e] * sg;
        dzv[e] = d[e] * yy[e] * sg * (1.f + zz[e] * (1.f - sg));
        dD[e] = __builtin_fmaf(gv[e], xx[e], dD[e]);
      }
      gq.pack(gv);
      Pack8<T> dq;
      dq.pack(dzv);
      const int64_t o = (int64_t)(k0 + kk) * o_ls + r8;
      *reinterpret_cast<u32x4 *>(dz + o) = dq.w;
      *reinterpret_cast<u32x4 *>(g + o) = gq.w;
    }
    *reinterpret_cast<u32x4 *>(hi + off) = gq.w;  // bf16 as it is: the MFMA operand
  }
};


template <typename T> __global__ __launch_bounds__(256) void bwd_dz_dstates_kernel(const SsdParams p) {
  __shared__ GemmLdsWide<false> lds;
  __shared__ float rs[256];
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads;
  const Block3 blk = xcd_block_heads(H);
  const int pt = blk.x;  // one 128-state tile: a p tile's rows are read by one workgroup only
  const int c = blk.y, b = blk.z / H, h = blk.z % H;
  const int g = h / (H / p.ngroups);
  const int t0 = c * Q, qlim = min(Q, L - t0);
  const float *dA = chunk_row(p.dA_cumsum, p, b, h, c);
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  for (int l = tid; l < Q; l += 256) {
    float v = 0.f;
    if (l < qlim) {
      bool ok = true;
      if (seq) ok = seq[l] == (c > 0 ? seq[-1] : 0);
      if (ok) v = fast_exp(dA[l]);
    }
    rs[l] = v;
  }
  DzStager<T> sa;
  sa.hi = lds.ah;
  sa.dout = static_cast<const T *>(p.dout) + b * p.dout_bs + h * p.dout_hs + (int64_t)t0 * p.dout_ls + pt * GB;
  sa.z = static_cast<const T *>(p.z) + b * p.z_bs + h * p.z_hs + (int64_t)t0 * p.z_ls + pt * GB;
  sa.y = static_cast<const T *>(p.out_x) + b * p.out_bs + h * p.out_hs + (int64_t)t0 * p.out_ls + pt * GB;
  sa.x = static_cast<const T *>(p.x) + b * p.x_bs + h * p.x_hs + (int64_t)t0 * p.x_ls + pt * GB;
  const int64_t o0 = (((int64_t)b * L + t0) * H + h) * P + pt * GB;
  sa.dz = static_cast<T *>(p.dz) + o0;
  sa.g = static_cast<T *>(p.gbuf) + o0;
  sa.dout_ls = p.dout_ls, sa.z_ls = p.z_ls, sa.y_ls = p.out_ls, sa.x_ls = p.x_ls, sa.o_ls = (int64_t)H * P;
  sa.rows_valid = P - pt * GB;
  sa.t = tid;
  const T *Ca = static_cast<const T *>(p.C) + b * p.C_bs + g * p.C_gs + (int64_t)t0 * p.C_ls;
  GemmAccWide acc;
  acc.zero();
  WideTrStager<false, T, WB> sb(lds.bh, lds.bl, Ca, p.C_ls, WB, rs, tid);
  block_gemm_wide<false>(acc, lds, qlim, sa, sb, tid);  // the first barrier inside publishes rs
  if (p.D) {
    // a thread's 8 columns are the same in every step: column group tid % 8, summed over the 32 threads that share it
    float *red = reinterpret_cast<float *>(&lds);  // row stride 9: conflict-free column reads
    static_assert(sizeof(lds) >= 256 * 9 * sizeof(float), "the partial sums fit in the operand tiles");
    lds_barrier();  // the last step's operand reads end before the sums overwrite them
#pragma unroll
    for (int e = 0; e < 8; ++e) red[tid * 9 + e] = sa.dD[e];
    lds_barrier();
    if (p.D_has_hdim) {
      if (tid < GB && pt * GB + tid < P) {
        float sacc = 0.f;
        for (int r = tid / 8; r < 256; r += 8) sacc += red[r * 9 + (tid & 7)];
        acc_add(p.dD, p.det_dD, h * P + pt * GB + tid, sacc, det_scale_of(p));
      }
    } else if (tid < 64) {
      float sacc = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int e = 0; e < 8; ++e) sacc += red[(tid * 4 + r) * 9 + e];
      sacc = wave_sum(sacc);
      if (tid == 0) acc_add(p.dD, p.det_dD, h, sacc, det_scale_of(p));
    }
  }
  carried_t<T> *ds = carried_dstates<T>(p) + (((int64_t)b * p.nchunks + c) * H + h) * P * N;
  store_wide_rows(acc, lds, ds + (int64_t)pt * GB * N, N, P - pt * GB, tid);
}

// ---------------------------------------------------- state_passing bwd
// Reverse recurrence over chunks.  On entry dstates[c] is the direct gradient of the state
// entering chunk c; on exit it is the gradient of chunk c's local state.
// A thread owns W consecutive elements; the direct gradients and states of the next SPB_PF chunks
// are always in flight (the serial recurrence only needs them one chunk at a time, and the
// compiler cannot hoist the loads over the in-place stores by itself).  TABLE: the per-chunk decay factors come from
// an LDS table filled before the loop, as in the forward kernel (no scalar loads, and their waits, inside the loop),
// and the ddA_cumsum terms of the chunks are kept in LDS until the loop is over.
constexpr int SPB_PF = 4;
constexpr size_t SPB_TABLE_BYTES = 40960;

template <int W> struct VecG;
template <> struct VecG<1> {
  float v[1];
  DEVI void load(const float *p) { v[0] = *p; }
  DEVI void store(float *p) const { *p = v[0]; }
  DEVI void load(const bf16_t *p) { v[0] = ld1<bf16_t>(p); }
  DEVI void store(bf16_t *p) const { st1<bf16_t>(p, v[0]); }
};
template <> struct VecG<4> {
  float v[4];
  DEVI void load(const float *p) {
    const f32x4 t = *reinterpret_cast<const f32x4 *>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  DEVI void store(float *p) const { *reinterpret_cast<f32x4 *>(p) = f32x4{v[0], v[1], v[2], v[3]}; }
  DEVI void load(const bf16_t *p) {
    const u32x2 t = *reinterpret_cast<const u32x2 *>(p);
    v[0] = bf16_lo(t.x); v[1] = bf16_hi(t.x); v[2] = bf16_lo(t.y); v[3] = bf16_hi(t.y);
  }
  DEVI void store(bf16_t *p) const { *reinterpret_cast<u32x2 *>(p) = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])}; }
};
// W elements as they lie in memory: what the prefetch holds.  They are converted when the chunk is processed; a
// conversion placed at the load makes the wave wait for the load it has just issued, i.e. no prefetch at all.
template <int W, typename CT> struct RawG;
template <> struct RawG<1, float> {
  float r;
  DEVI void load(const float *p) { r = *p; }
  DEVI void unpack(float (&v)[1]) const { v[0] = r; }
};
template <> struct RawG<4, float> {
  f32x4 r;
  DEVI void load(const float *p) { r = *reinterpret_cast<const f32x4 *>(p); }
  DEVI void unpack(float (&v)[4]) const { v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w; }
};
template <> struct RawG<1, bf16_t> {
  uint16_t r;
  DEVI void load(const bf16_t *p) { r = *reinterpret_cast<const uint16_t *>(p); }
  DEVI void unpack(float (&v)[1]) const { v[0] = __builtin_bit_cast(float, (uint32_t)r << 16); }
};
template <> struct RawG<4, bf16_t> {
  u32x2 r;
  DEVI void load(const bf16_t *p) { r = *reinterpret_cast<const u32x2 *>(p); }
  DEVI void unpack(float (&v)[4]) const { v[0] = bf16_lo(r.x); v[1] = bf16_hi(r.x); v[2] = bf16_lo(r.y); v[3] = bf16_hi(r.y); }
};

// CT: dtype of the carried states and of dstates (float, or bf16_t next to bf16 operands)
template <int W, typename CT, bool TABLE, bool FULL = false> __global__ __launch_bounds__(256) void state_passing_bwd_kernel(const SsdParams p) {
  extern __shared__ float spb_decay[];
  CT *const dst_p = std::is_same_v<CT, float> ? reinterpret_cast<CT *>(p.dstates) : static_cast<CT *>(p.dstates_lp);
  const CT *const st_p = std::is_same_v<CT, float> ? reinterpret_cast<const CT *>(p.states) : static_cast<const CT *>(p.states_lp);
  const int PN = p.headdim * p.dstate, H = p.nheads, nc = p.nchunks, Q = p.chunk_size, L = p.seqlen;
  const int e = (blockIdx.x * 256 + threadIdx.x) * W;
  const int lane = threadIdx.x & 63;
  const int h = blockIdx.y, b = blockIdx.z;
  // FULL: the state is a whole number of workgroups (no idle thread, and so no branch around the stores of the
  // loop: with one the compiler counts the memory operations in flight for the worst path and waits for all)
  const bool live = FULL || e < PN;
  const int ec = live ? e : 0;  // clamped: idle threads read valid memory and add nothing
  VecG<W> G;
#pragma unroll
  for (int i = 0; i < W; ++i) G.v[i] = 0.f;
  if (live && p.dfinal_states) G.load(p.dfinal_states + ((int64_t)b * H + h) * PN + e);
  const float *dA = p.dA_cumsum + ((int64_t)b * H + h) * nc * Q;
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L : nullptr;
  auto offset = [&](int c) { return (((int64_t)b * nc + c) * H + h) * PN + ec; };
  auto decay_of = [&](int c) {
    float scale = fast_exp(dA[c * Q + Q - 1]);
    if (seq) {
      const int end_c = seq[min((c + 1) * Q, L) - 1];
      const int end_prev = c > 0 ? seq[c * Q - 1] : 0;
      if (end_c != end_prev) scale = 0.f;
    }
    return scale;
  };
  if constexpr (TABLE) {
    for (int c = threadIdx.x; c < nc; c += 256) spb_decay[c] = decay_of(c);
    lds_barrier();
  }
  auto decay = [&](int c) { return TABLE ? spb_decay[c] : decay_of(c); };
  float *const parts = spb_decay + nc;  // [nc][4 waves] (TABLE)
  RawG<W, CT> direct[SPB_PF], state[SPB_PF];
  float scale[SPB_PF];
#pragma unroll
  for (int j = 0; j < SPB_PF; ++j) {
    const int c = max(nc - 1 - j, 0);
    direct[j].load(dst_p + offset(c));
    state[j].load(st_p + offset(c));
    scale[j] = decay(c);
  }
  // one chunk, its operands in slot j of the prefetch; `more`: request chunk c - SPB_PF into the slot
  auto step = [&](int c, int j, bool more) {
    if (live) G.store(dst_p + offset(c));
    float dir[W], st[W];
    direct[j].unpack(dir);
    state[j].unpack(st);
    const float sc = scale[j];
    if (more) {  // past the first chunk the loads repeat chunk 0 and nobody uses them: no branch, so no register
                 // copies (which would wait for the loads in flight) where the paths meet
      const int cn = max(c - SPB_PF, 0);
      direct[j].load(dst_p + offset(cn));
      state[j].load(st_p + offset(cn));
      scale[j] = decay(cn);
    }
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < W; ++i) {
      part = __builtin_fmaf(G.v[i], st[i], part);
      G.v[i] = __builtin_fmaf(sc, G.v[i], dir[i]);
    }
    part = live ? part * sc : 0.f;
    part = wave_sum_to_last(part);
    if constexpr (TABLE) {
      if (lane == 63) parts[c * 4 + (threadIdx.x >> 6)] = part;  // the wave's own slot
    } else {
      if (lane == 63 && part != 0.f)
        acc_add(p.ddA_cumsum, p.det_ddA_cumsum, (((int64_t)b * H + h) * nc + c) * Q + Q - 1, part, det_scale_of(p));
    }
  };
  // whole groups of SPB_PF chunks without a branch inside, then the chunks left over from what the slots hold
  int c0 = nc - 1;
  for (; c0 >= SPB_PF - 1; c0 -= SPB_PF) {
#pragma unroll
    for (int j = 0; j < SPB_PF; ++j) step(c0 - j, j, true);
  }
#pragma unroll
  for (int j = 0; j < SPB_PF - 1; ++j)
    if (c0 - j >= 0) step(c0 - j, j, false);
  if constexpr (TABLE) {
    // one add per chunk and workgroup, after the loop: an atomic inside it is counted with the loads, and the wait
    // for a chunk's loads then sat through the round trips of the adds before them
    lds_barrier();
    for (int c = threadIdx.x; c < nc; c += 256) {
      const float part = (parts[c * 4] + parts[c * 4 + 1]) + (parts[c * 4 + 2] + parts[c * 4 + 3]);
      if (part != 0.f)
        acc_add(p.ddA_cumsum, p.det_ddA_cumsum, (((int64_t)b * H + h) * nc + c) * Q + Q - 1, part, det_scale_of(p));
    }
  }
  if (live && p.dinitial_states) G.store(p.dinitial_states + ((int64_t)b * H + h) * PN + e);
}

// ------------------------------------------------------------------- dx
// acc[s, p] = exp(a_last - a_s) [s in the chunk's last sequence] sum_n B[s, n] dS[p, n]
//           + sum_{l >= s} CB[l, s] exp(a_l - a_s) g[l, p]
// dx = dt_s acc + D g;  ddt_out[s] += <x_s, acc_s>;  chunk-state terms of ddA_cumsum.
template <typename T, bool SPLIT, bool DET> __global__ __launch_bounds__(256) void bwd_dx_kernel(const SsdParams p) {
  __shared__ GemmLds lds;
  __shared__ float a_s[256], dt_s[256], kdec[256], rdec[GB], wrow[GB];
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads, G = p.ngroups;
  const int ntp = cdiv(P, GB);
  // Logical order: s tile fastest (the tiles of a (chunk, head) share dS and g), then head (the heads
  // of a chunk share CB and B), then chunk, then batch, behind one L2 at a time.
  int lid = xcd_linear_block();
  const int nst = gridDim.x / ntp;
  const int st = lid % nst, pt = (lid / nst) % ntp;
  lid /= gridDim.x;
  const int h = lid % H, c = (lid / H) % p.nchunks, b = lid / (H * p.nchunks);
  const int g = h / (H / G);
  const int t0 = c * Q, qlim = min(Q, L - t0);
  const float *dA = chunk_row(p.dA_cumsum, p, b, h, c);
  const float *dt = chunk_row(p.dt_out, p, b, h, c);
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  const float a_last = dA[Q - 1];
  // Below the diagonal block exp(a_l - a_s) = exp(a_l - a_ref) exp(a_ref - a_s) with a_ref taken
  // at the tile's last row: both factors are <= 1, so the rank-1 form cannot overflow.
  const float a_ref = dA[min((st + 1) * GB, qlim) - 1];
  for (int s = tid; s < Q; s += 256) {
    const float a = dA[s];
    a_s[s] = a;
    dt_s[s] = dt[s];
    kdec[s] = fast_exp(fminf(a - a_ref, 0.f));
  }
  if (tid < GB) {
    const int s = st * GB + tid;
    rdec[tid] = s < qlim ? fast_exp(fminf(a_ref - dA[s], 0.f)) : 0.f;
    float v = 0.f;
    if (s < qlim) {
      bool ok = true;
      if (seq) {
        const int last = seq[qlim - 1];
        ok = last >= 0 && seq[s] == last;
      }
      if (ok) v = fast_exp(fminf(a_last - dA[s], 0.f));
    }
    wrow[tid] = v;
  }
  const View4 gv = g_view(p);
  const int64_t gb = b * gv.bs + h * gv.hs, xb = b * p.x_bs + h * p.x_hs, Bb = b * p.B_bs + g * p.B_gs;
  const carried_t<T> *dS = carried_dstates<T>(p) + (((int64_t)b * p.nchunks + c) * H + h) * P * N;
  const float *CB = p.CB + (((int64_t)b * p.nchunks + c) * G + g) * Q * Q;
  GemmAcc acc1, acc2;  // carried-state part, in-chunk part
  acc1.zero();
  acc2.zero();
  {
    // A = B rows (s, k = n), B = dS rows (p, k = n): both k-contiguous
    const T *Ba = static_cast<const T *>(p.B) + Bb + (int64_t)(t0 + st * GB) * p.B_ls;
    const carried_t<T> *dSa = dS + (int64_t)pt * GB * N;
    const bool va = rows_aligned16(Ba, p.B_ls), vb = rows_aligned16(dSa, N);
    block_gemm_pipe<SPLIT, !SPLIT>(
        acc1, lds, 0, N,
        KcStager<SPLIT, T>(lds.ah, lds.al, Ba, p.B_ls, qlim - st * GB, N, nullptr, nullptr, va, tid),
        KcStager<SPLIT, carried_t<T>>(lds.bh, lds.bl, dSa, N, P - pt * GB, N, nullptr, nullptr, vb, tid),
        tid);
  }
  {
    // exact decay and causal mask for the diagonal 64 x 64 block: multiplier of CB[l = k, s]
    auto fa = [&](int r, int k) {
      const int s = st * GB + r;
      return (s < qlim && k < qlim && k >= s) ? fast_exp(fminf(a_s[min(k, Q - 1)] - a_s[min(s, Q - 1)], 0.f)) : 0.f;
    };
    const T *ga = static_cast<const T *>(gv.ptr) + gb + (int64_t)t0 * gv.ls + pt * GB;
    const bool vb = rows_aligned16(ga, gv.ls);
    const float *CBa = CB + st * GB;  // A rows s are contiguous in the source, k = l strides by Q
    const bool va = rows_aligned16(CBa, Q);
    block_gemm_pipe<SPLIT, !SPLIT>(
        acc2, lds, st * GB, qlim,
        // diagonal block: causal mask and the exact decay; below it CB^T with the rank-1 decays
        diag_stager<SPLIT>(fa, (st + 1) * GB,
                           TrStager<SPLIT, float>(lds.ah, lds.al, CBa, Q, qlim - st * GB, qlim, kdec, rdec, va, tid)),
        TrStager<SPLIT, T>(lds.bh, lds.bl, ga, gv.ls, P - pt * GB, qlim, nullptr, nullptr, vb, tid),
        tid);
  }
  // The epilogue's x and g rows (thread t: position s = tile row t / 4, 16 consecutive p) are
  // fetched before the accumulators are re-laid, so that they arrive during that exchange (any
  // earlier and the extra live registers cost a wave of occupancy).
  const int s = st * GB + (tid >> 2), p0 = pt * GB + (tid & 3) * 16;
  const bool row_ok = s < qlim;
  const T *xr = static_cast<const T *>(p.x) + xb + (int64_t)(t0 + s) * p.x_ls + p0;
  const T *gr = static_cast<const T *>(gv.ptr) + gb + (int64_t)(t0 + s) * gv.ls + p0;
  const bool vec = P % 8 == 0 && rows_aligned16(static_cast<const T *>(p.x) + xb, p.x_ls) &&
                   rows_aligned16(static_cast<const T *>(gv.ptr) + gb, gv.ls) &&
                   rows_aligned16(static_cast<T *>(p.dx) + b * p.dx_bs + h * p.dx_hs, p.dx_ls);
  const float *Dp = static_cast<const float *>(p.D);
  Pack8<T> xk[2], gk[2];
  if (vec) {
    const int sc = min(s, qlim - 1) - s;  // row clamp, as an offset from s
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int pc = min(p0 + 8 * j, P - 8) - p0;  // column clamp; clamped pieces are masked below
      xk[j].load(xr + (int64_t)sc * p.x_ls + pc);
      gk[j].load(gr + (int64_t)sc * gv.ls + pc);
    }
  }
  // Epilogue with rows in threads: thread t owns position s = tile row t / 4 and 16 consecutive p.
  float v1[16], v2[16];
  acc_to_rows(acc1, lds, tid, v1);
  acc_to_rows(acc2, lds, tid, v2);
  {
    const float w = wrow[tid >> 2];
#pragma unroll
    for (int e = 0; e < 16; ++e) v1[e] *= w;
  }
  T *dxr = static_cast<T *>(p.dx) + b * p.dx_bs + (int64_t)(t0 + s) * p.dx_ls + h * p.dx_hs + p0;
  float q1 = 0.f, q2 = 0.f;
  const float dts = dt_s[min(s, Q - 1)];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int nv = row_ok ? max(0, min(8, P - p0 - 8 * j)) : 0;
    float xv[8], gvv[8], o[8];
    if (vec) {
      xk[j].unpack(xv);
      gk[j].unpack(gvv);
      if (nv < 8) {
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[e] = gvv[e] = 0.f;
      }
    } else {
      ld8_guard<T, false>(xr + 8 * j, nv, 0.f, xv);
      ld8_guard<T, false>(gr + 8 * j, Dp ? nv : 0, 0.f, gvv);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float a1 = v1[8 * j + e], a = a1 + v2[8 * j + e];
      q1 = __builtin_fmaf(xv[e], a1, q1);
      q2 = __builtin_fmaf(xv[e], a, q2);
      float d = 0.f;
      if (Dp) d = p.D_has_hdim ? Dp[h * P + min(p0 + 8 * j + e, P - 1)] : Dp[h];
      o[e] = __builtin_fmaf(d, gvv[e], a * dts);
    }
    if (vec) st8_guard<T, true>(dxr + 8 * j, nv, o);
    else st8_guard<T, false>(dxr + 8 * j, nv, o);
  }
  // <x_s, acc_s> over the row's four threads
  q1 += __shfl_xor(q1, 1, 64);
  q1 += __shfl_xor(q1, 2, 64);
  q2 += __shfl_xor(q2, 1, 64);
  q2 += __shfl_xor(q2, 2, 64);
  const bool lead = (tid & 3) == 0 && row_ok;
  const int64_t row_off = chunk_off(p, b, h, c);
  const float dsc = det_scale_of(p);
  if (lead) {
    acc_add<DET ? 1 : 0>(p.ddt_out, p.det_ddt_out, row_off + s, q2, dsc);
    acc_add<DET ? 1 : 0>(p.ddA_cumsum, p.det_ddA_cumsum, row_off + s, -dts * q1, dsc);  // chunk-state terms: -dt_s <x_s, acc1_s> at s ...
  }
  // ... and + at the chunk end: one address for the whole tile, so one atomic per wave
  const float endsum = wave_sum_to_last(lead ? dts * q1 : 0.f);
  if ((tid & 63) == 63) acc_add<DET ? 1 : 0>(p.ddA_cumsum, p.det_ddA_cumsum, row_off + Q - 1, endsum, dsc);
}

// ---------------------------------------------- state-path parts of dB, dC
// dB32[s, n] = sum_{h in group} exp(a_last - a_s) dt_s [s in last sequence] sum_p x[s, p] dS[p, n]
// dC32[l, n] = sum_{h in group} exp(a_l) [seq_l == seq before the chunk]    sum_p g[l, p] Hc[p, n]
// One workgroup per (batch, chunk, group, 64 x 64 tile) loops over the heads of the group and keeps
// both sums in registers (no atomics); the per-head row factor is folded into the A operand.
// The carried-state share of ddA_cumsum, sum_n dC_h[l, n] C[l, n], is taken per head on the way.
// PARTS: bit 0 = the dB product, bit 1 = the dC product.
template <typename T, bool SPLIT, bool DET, int PARTS> DEVI void dBC_state_body(const SsdParams &p) {
  constexpr int MAXH = 8;  // heads per workgroup (head_splits keeps it at or below 8)
  __shared__ GemmLds lds;
  __shared__ float wB[MAXH][GB], wC[MAXH][GB];  // per-head row factors
  // the heads' ddA_cumsum shares per half of the tile's columns, added to global memory once at the end
  __shared__ float dda_s[(PARTS & 2) ? 2 : 1][(PARTS & 2) ? MAXH : 1][GB];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int i = lane & 15, gq = lane >> 4;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads, G = p.ngroups;
  const int ntn = cdiv(N, GB);
  const Block3 blk = xcd_block();
  const int nst = gridDim.x / ntn;
  const int st = blk.x % nst, nt = blk.x / nst;  // the s tiles of a chunk share the state tiles
  const int hpg = H / G, nsplit = head_splits(hpg);
  const int c = blk.y, bg = blk.z / nsplit, hs = blk.z % nsplit, b = bg / G, g = bg % G;
  const int nh = hs < hpg ? (hpg - hs + nsplit - 1) / nsplit : 0;  // heads hs, hs + nsplit, ...
  const int t0 = c * Q, qlim = min(Q, L - t0);
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  const View4 gv = g_view(p);
  // row factors of every head of this workgroup (published by the first barrier of the GEMM)
  for (int idx = tid; idx < nh * GB; idx += 256) {
    const int hl = idx / GB, r = idx % GB, s = st * GB + r, h = g * hpg + hs + hl * nsplit;
    float vb = 0.f, vc = 0.f;
    if (s < qlim) {
      const float *dA = chunk_row(p.dA_cumsum, p, b, h, c);
      bool okb = true, okc = true;
      if (seq) {
        const int last = seq[qlim - 1];
        okb = last >= 0 && seq[s] == last;
        okc = seq[s] == (c > 0 ? seq[-1] : 0);
      }
      if (okb) vb = fast_exp(fminf(dA[Q - 1] - dA[s], 0.f)) * chunk_row(p.dt_out, p, b, h, c)[s];
      if (okc) vc = fast_exp(dA[s]);
    }
    wB[hl][r] = vb;
    wC[hl][r] = vc;
  }
  // The k axis of both products concatenates the heads (k = (head, p)), so each runs as one
  // pipelined GEMM: A = (w x) or (w g) rows (position, k = p), k-contiguous; B = state rows n,
  // k = p: row-contiguous fp32.
  const int seg_k = cdiv(P, GK) * GK;
  auto state_off = [&](int hl) {
    return (((int64_t)b * p.nchunks + c) * H + g * hpg + hs + hl * nsplit) * P * N + nt * GB;
  };
  if constexpr ((PARTS & 1) != 0) {  // dB32 += (wB x)^T-rows times dS
    GemmAcc accB;
    accB.zero();
    block_gemm_pipe<SPLIT>(
        accB, lds, 0, nh * seg_k,
        seg_stager(KcStager<SPLIT, T>(lds.ah, lds.al, nullptr, p.x_ls, qlim - st * GB, P, nullptr, nullptr, false, tid),
                   [&](KcStager<SPLIT, T> &q, int hl) {
                     q.base = static_cast<const T *>(p.x) + b * p.x_bs + (g * hpg + hs + hl * nsplit) * p.x_hs +
                              (int64_t)(t0 + st * GB) * p.x_ls;
                     q.vec = rows_aligned16(q.base, p.x_ls);
                     q.rscale = wB[hl];
                   },
                   seg_k),
        seg_stager(TrStager<SPLIT, carried_t<T>>(lds.bh, lds.bl, nullptr, N, N - nt * GB, P, nullptr, nullptr, false, tid),
                   [&](TrStager<SPLIT, carried_t<T>> &q, int hl) {
                     q.base = carried_dstates<T>(p) + state_off(hl);
                     q.vec = rows_aligned16(q.base, N);
                   },
                   seg_k),
        tid);
    acc_foreach(accB, tid, [&](int m, int n, float v) {
      const int s = st * GB + m, nn = nt * GB + n;
      if (s < qlim && nn < N) acc_add<DET ? 1 : 0>(p.dB32, p.det_dB, (((int64_t)b * L + t0 + s) * G + g) * N + nn, v, det_scale_of(p));
      return v;
    });
  }
  if constexpr ((PARTS & 2) != 0) {  // dC32 += (wC g) rows times H, and per head the carried-state share of ddA_cumsum
    const int64_t Cb = b * p.C_bs + g * p.C_gs;
    // C at this lane's 16 accumulator positions (shared by the heads of the group)
    float cr[2][2][4];
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int tn = 0; tn < 2; ++tn)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int l = st * GB + wm * 32 + tm * 16 + gq * 4 + r, nn = nt * GB + wn * 32 + tn * 16 + i;
          cr[tm][tn][r] = (l < qlim && nn < N) ? ldg<T>(p.C, Cb + (int64_t)(t0 + l) * p.C_ls + nn) : 0.f;
        }
    GemmAcc accC, accH;
    accC.zero();
    accH.zero();
    block_gemm_pipe<SPLIT>(
        accH, lds, 0, nh * seg_k,
        seg_stager(KcStager<SPLIT, T>(lds.ah, lds.al, nullptr, gv.ls, qlim - st * GB, P, nullptr, nullptr, false, tid),
                   [&](KcStager<SPLIT, T> &q, int hl) {
                     q.base = static_cast<const T *>(gv.ptr) + b * gv.bs + (g * hpg + hs + hl * nsplit) * gv.hs +
                              (int64_t)(t0 + st * GB) * gv.ls;
                     q.vec = rows_aligned16(q.base, gv.ls);
                     q.rscale = wC[hl];
                   },
                   seg_k),
        seg_stager(TrStager<SPLIT, carried_t<T>>(lds.bh, lds.bl, nullptr, N, N - nt * GB, P, nullptr, nullptr, false, tid),
                   [&](TrStager<SPLIT, carried_t<T>> &q, int hl) {
                     q.base = carried_states<T>(p) + state_off(hl);
                     q.vec = rows_aligned16(q.base, N);
                   },
                   seg_k),
        tid, [&](int k0) {
          if ((k0 + GK) % seg_k != 0) return;
          // a head is complete: sum_n dC_h[l, n] C[l, n] goes to its ddA_cumsum row, dC_h to the sum
#pragma unroll
          for (int tm = 0; tm < 2; ++tm)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              float rs = accH.v[tm][0][r] * cr[tm][0][r] + accH.v[tm][1][r] * cr[tm][1][r];
              rs += dpp_f<DPP_ROW_SHR + 1>(0.f, rs);
              rs += dpp_f<DPP_ROW_SHR + 2>(0.f, rs);
              rs += dpp_f<DPP_ROW_SHR + 4>(0.f, rs);
              rs += dpp_f<DPP_ROW_SHR + 8>(0.f, rs);
              if (i == 15) dda_s[wn][k0 / seg_k][wm * 32 + tm * 16 + gq * 4 + r] = rs;
            }
#pragma unroll
          for (int ii = 0; ii < 2; ++ii)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              accC.v[ii][j] += accH.v[ii][j];
              accH.v[ii][j] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        });
    acc_foreach(accC, tid, [&](int m, int n, float v) {
      const int l = st * GB + m, nn = nt * GB + n;
      if (l < qlim && nn < N) acc_add<DET ? 1 : 0>(p.dC32, p.det_dC, (((int64_t)b * L + t0 + l) * G + g) * N + nn, v, det_scale_of(p));
      return v;
    });
    __syncthreads();
    for (int idx = tid; idx < nh * GB; idx += 256) {
      const int hl = idx / GB, r = idx % GB, l = st * GB + r;
      const float d = dda_s[0][hl][r] + dda_s[1][hl][r];
      if (l < qlim && d != 0.f)
        acc_add<DET ? 1 : 0>(p.ddA_cumsum, p.det_ddA_cumsum, chunk_off(p, b, g * hpg + hs + hl * nsplit, c) + l, d, det_scale_of(p));
    }
  }
}

template <typename T, bool SPLIT, bool DET> __global__ __launch_bounds__(256, 4) void bwd_dBC_state_kernel(const SsdParams p) {
  dBC_state_body<T, SPLIT, DET, 3>(p);
}
template <typename T, bool SPLIT, bool DET> __global__ __launch_bounds__(256, 4) void bwd_dC_state_kernel(const SsdParams p) {
  dBC_state_body<T, SPLIT, DET, 2>(p);
}

// The dB product alone with a 64 x 128 tile per workgroup (whole 128-state blocks, headdim in whole
// k steps, aligned x): k runs through (head, p) as above.
template <typename T, bool SPLIT, bool DET> __global__ __launch_bounds__(256) void bwd_dB_state_wide_kernel(const SsdParams p) {
  constexpr int MAXH = 8;
  __shared__ GemmLdsWide<SPLIT> lds;
  __shared__ float wB[MAXH][GB];
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads, G = p.ngroups;
  const int ntn = N / WB;
  const Block3 blk = xcd_block();
  const int nst = gridDim.x / ntn;
  const int st = blk.x % nst, nt = blk.x / nst;
  const int hpg = H / G, nsplit = head_splits(hpg);
  const int c = blk.y, bg = blk.z / nsplit, hs = blk.z % nsplit, b = bg / G, g = bg % G;
  const int nh = hs < hpg ? (hpg - hs + nsplit - 1) / nsplit : 0;
  const int t0 = c * Q, qlim = min(Q, L - t0);
  if (st * GB >= qlim || nh == 0) return;
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  for (int idx = tid; idx < nh * GB; idx += 256) {
    const int hl = idx / GB, r = idx % GB, s = st * GB + r, h = g * hpg + hs + hl * nsplit;
    float vb = 0.f;
    if (s < qlim) {
      const float *dA = chunk_row(p.dA_cumsum, p, b, h, c);
      bool okb = true;
      if (seq) {
        const int last = seq[qlim - 1];
        okb = last >= 0 && seq[s] == last;
      }
      if (okb) vb = fast_exp(fminf(dA[Q - 1] - dA[s], 0.f)) * chunk_row(p.dt_out, p, b, h, c)[s];
    }
    wB[hl][r] = vb;
  }
  GemmAccWide accB;
  accB.zero();
  auto sa = seg_stager(KcStager<SPLIT, T>(lds.ah, lds.al, nullptr, p.x_ls, qlim - st * GB, P, nullptr, nullptr, true, tid),
                       [&](KcStager<SPLIT, T> &q, int hl) {
                         q.base = static_cast<const T *>(p.x) + b * p.x_bs + (g * hpg + hs + hl * nsplit) * p.x_hs +
                                  (int64_t)(t0 + st * GB) * p.x_ls;
                         q.rscale = wB[hl];
                       },
                       P);
  auto sb = seg_stager(WideTrStager<SPLIT, carried_t<T>, WB>(lds.bh, lds.bl, nullptr, N, WB, nullptr, tid),
                       [&](WideTrStager<SPLIT, carried_t<T>, WB> &q, int hl) {
                         q.base = carried_dstates<T>(p) + (((int64_t)b * p.nchunks + c) * H + g * hpg + hs + hl * nsplit) * P * N + nt * WB;
                       },
                       P);
  block_gemm_wide<SPLIT, true>(accB, lds, nh * P, sa, sb, tid);  // the first barrier inside publishes wB
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1, i = lane & 15, gq = lane >> 4;
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int s = st * GB + wm * 32 + tm * 16 + gq * 4 + r;
      if (s >= qlim) continue;
      const int64_t row = (((int64_t)b * L + t0 + s) * G + g) * N + nt * WB + wn * 64 + i;
#pragma unroll
      for (int tn = 0; tn < 4; ++tn) acc_add<DET ? 1 : 0>(p.dB32, p.det_dB, row + tn * 16, accB.v[tm][tn][r], det_scale_of(p));
    }
}

// The dC product alone with a 64 x 128 tile per workgroup (same conditions, aligned g rows); the row sums
// of the tile against C after each head give the heads' ddA_cumsum rows.
template <typename T, bool SPLIT, bool DET> __global__ __launch_bounds__(256, 4) void bwd_dC_state_wide_kernel(const SsdParams p) {
  constexpr int MAXH = 8;
  __shared__ GemmLdsWide<SPLIT> lds;
  __shared__ float wC[MAXH][GB];
  __shared__ float dda_s[2][MAXH][GB];  // the running ddA_cumsum row sums after each head, per half of the tile's columns, flushed at the end:
                                        // a global atomic per head would sit in the memory queue in front of the next loads
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads, G = p.ngroups;
  const int ntn = N / WB;
  const Block3 blk = xcd_block();
  const int nst = gridDim.x / ntn;
  const int st = blk.x % nst, nt = blk.x / nst;
  const int hpg = H / G, nsplit = head_splits(hpg);
  const int c = blk.y, bg = blk.z / nsplit, hs = blk.z % nsplit, b = bg / G, g = bg % G;
  const int nh = hs < hpg ? (hpg - hs + nsplit - 1) / nsplit : 0;
  const int t0 = c * Q, qlim = min(Q, L - t0);
  if (st * GB >= qlim || nh == 0) return;
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  const View4 gv = g_view(p);
  for (int idx = tid; idx < nh * GB; idx += 256) {
    const int hl = idx / GB, r = idx % GB, s = st * GB + r, h = g * hpg + hs + hl * nsplit;
    float vc = 0.f;
    if (s < qlim) {
      const bool okc = !seq || seq[s] == (c > 0 ? seq[-1] : 0);
      if (okc) vc = fast_exp(chunk_row(p.dA_cumsum, p, b, h, c)[s]);
    }
    wC[hl][r] = vc;
  }
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1, i = lane & 15, gq = lane >> 4;
  // C at this lane's 32 accumulator positions (shared by the heads of the group); 16-bit inputs stay packed in
  // pairs, which keeps the kernel at four workgroups per CU without spills
  constexpr bool PK = sizeof(T) == 2;
  const int64_t Cb = b * p.C_bs + g * p.C_gs;
  uint32_t crp[2][2][4] = {};
  float crf[2][4][4];
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int l = st * GB + wm * 32 + tm * 16 + gq * 4 + r;
#pragma unroll
      for (int tn = 0; tn < 4; ++tn) {
        const int64_t at = Cb + (int64_t)(t0 + l) * p.C_ls + nt * WB + wn * 64 + tn * 16 + i;
        if constexpr (PK) {
          const uint32_t raw = l < qlim ? (uint32_t) reinterpret_cast<const uint16_t *>(p.C)[at] : 0u;
          crp[tm][tn >> 1][r] |= raw << (16 * (tn & 1));
        } else {
          crf[tm][tn][r] = l < qlim ? ldg<T>(p.C, at) : 0.f;
        }
      }
    }
  auto cr = [&](int tm, int tn, int r) -> float {
    if constexpr (PK) {
      const uint32_t w = crp[tm][tn >> 1][r];
      if constexpr (DT<T>::id == MAMBA_BF16) return (tn & 1) ? bf16_hi(w) : bf16_lo(w);
      else return (tn & 1) ? f16_hi(w) : f16_lo(w);
    } else {
      return crf[tm][tn][r];
    }
  };
  // One accumulator runs through the heads (at most 8 per workgroup); a head's share of the row sums is the
  // difference of the running row sums after it and after the head before.
  GemmAccWide acc;
  acc.zero();
  auto sa = seg_stager(KcStager<SPLIT, T>(lds.ah, lds.al, nullptr, gv.ls, qlim - st * GB, P, nullptr, nullptr, true, tid),
                       [&](KcStager<SPLIT, T> &q, int hl) {
                         q.base = static_cast<const T *>(gv.ptr) + b * gv.bs + (g * hpg + hs + hl * nsplit) * gv.hs +
                                  (int64_t)(t0 + st * GB) * gv.ls;
                         q.rscale = wC[hl];
                       },
                       P);
  auto sb = seg_stager(WideTrStager<SPLIT, carried_t<T>, WB>(lds.bh, lds.bl, nullptr, N, WB, nullptr, tid),
                       [&](WideTrStager<SPLIT, carried_t<T>, WB> &q, int hl) {
                         q.base = carried_states<T>(p) + (((int64_t)b * p.nchunks + c) * H + g * hpg + hs + hl * nsplit) * P * N + nt * WB;
                       },
                       P);
  // (one pair of stagers: the kernel has no registers to spare for a second)
  block_gemm_wide<SPLIT, false>(acc, lds, nh * P, sa, sb, tid, [&](int k0) {  // the first barrier inside publishes wC
    if ((k0 + GK) % P != 0) return;
    const int hl = k0 / P;
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float rs = 0.f;
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) rs = __builtin_fmaf(acc.v[tm][tn][r], cr(tm, tn, r), rs);
        rs += dpp_f<DPP_ROW_SHR + 1>(0.f, rs);
        rs += dpp_f<DPP_ROW_SHR + 2>(0.f, rs);
        rs += dpp_f<DPP_ROW_SHR + 4>(0.f, rs);
        rs += dpp_f<DPP_ROW_SHR + 8>(0.f, rs);
        if (i == 15) dda_s[wn][hl][wm * 32 + tm * 16 + gq * 4 + r] = rs;
      }
  });
  __syncthreads();
  for (int idx = tid; idx < nh * GB; idx += 256) {
    const int hl = idx / GB, r = idx % GB, l = st * GB + r;
    const float d = dda_s[0][hl][r] + dda_s[1][hl][r] - (hl > 0 ? dda_s[0][hl - 1][r] + dda_s[1][hl - 1][r] : 0.f);
    if (l < qlim && d != 0.f)
      acc_add<DET ? 1 : 0>(p.ddA_cumsum, p.det_ddA_cumsum, chunk_off(p, b, g * hpg + hs + hl * nsplit, c) + l, d, det_scale_of(p));
  }
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int l = st * GB + wm * 32 + tm * 16 + gq * 4 + r;
      if (l >= qlim) continue;
      const int64_t row = (((int64_t)b * L + t0 + l) * G + g) * N + nt * WB + wn * 64 + i;
#pragma unroll
      for (int tn = 0; tn < 4; ++tn) acc_add<DET ? 1 : 0>(p.dC32, p.det_dC, row + tn * 16, acc.v[tm][tn][r], det_scale_of(p));
    }
}

// ------------------------------------------------------------------ dCB
// dCB[b, c, g, l, s] = sum_{h in group} (sum_p g[l, p] x[s, p]) dt_s exp(a_l - a_s)   for l >= s in
// one sequence.  One workgroup per (batch, chunk, group, lower-triangular 64 x 64 tile pair) loops
// over the heads of the group with the sum in registers.  Per head, w = (head's term) * CB gives
// the in-chunk share of ddA_cumsum: + row sums at l, - column sums at s.
// FORM_CB: no CB buffer (p.CB null), the workgroup forms its tile of C B^T itself.
constexpr int DCB_MAXH = 16;  // heads per workgroup (dcb_head_splits keeps it at or below 16)
struct DcbShared {
  GemmLds lds;
  float hA_l[2][GB], hA_s[2][GB], hdt[2][GB];  // per-head rows, double-buffered over the head loop
  // the heads' ddA_cumsum shares (row sums per column half, column sums per row half), flushed at the end: a
  // global atomic per head would sit in the memory queue in front of the next head's loads
  float rs_s[2][DCB_MAXH][GB], cs_s[2][DCB_MAXH][GB];
};
// The tile pair (lt, st) of one workgroup.  BELOW: lt > st, the whole tile lies below the diagonal and the decay is
// factored; the kernel holds both forms as separate bodies, so that each keeps its own registers.
// FASTP (32 or 64 = headdim; bf16 operands on 16-byte aligned rows, no integer shadows): the heads' products run in a
// loop of their own instead of the general k pipeline -- a head's two 64 x headdim tiles go from memory to registers
// to LDS in 16-byte pieces at offsets computed once, one barrier pair and headdim / 32 MFMAs per 16 x 16 tile and
// head, the next head's tiles in flight under the weights.
// lp: this workgroup owns its tile, and the next stage takes it as bf16 (what its MFMA operand would round the fp32
// tile to anyway): the tile is stored as bf16, packed at the start of the dCB buffer.
template <typename T, bool SPLIT, bool DET, bool FORM_CB, bool BELOW, int FASTP>
DEVI void dcb_tile(const SsdParams &p, DcbShared &sh, const Block3 blk, const int lt, const int st, const bool lp) {
  GemmLds &lds = sh.lds;
  auto &hA_l = sh.hA_l;
  auto &hA_s = sh.hA_s;
  auto &hdt = sh.hdt;
  auto &rs_s = sh.rs_s;
  auto &cs_s = sh.cs_s;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int i = lane & 15, gq = lane >> 4;
  const int Q = p.chunk_size, L = p.seqlen, P = p.headdim, H = p.nheads, G = p.ngroups;
  const int hpg = H / G, nsplit = dcb_head_splits(hpg);
  const int c = blk.y, bg = blk.z / nsplit, hs = blk.z % nsplit, b = bg / G, g = bg % G;
  const int t0 = c * Q, qlim = min(Q, L - t0);
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  const View4 gv = g_view(p);
  const int64_t dCB_off = (((int64_t)b * p.nchunks + c) * G + g) * Q * Q;
  // This lane's 16 accumulator positions: CB there (the same for every head) and the causal /
  // same-sequence mask, kept as zeros in cbr and a bit per position.  Without a CB buffer (p.CB null: the caller
  // skipped ssd_bmm_chunk_fwd, see ssd_bwd_overwrites) the workgroup forms its tile of C B^T itself, with the same
  // pipeline, before the heads' products.
  float cbr[2][2][4];
  uint32_t live = 0;
  GemmAcc sum, acc;
  sum.zero();
  acc.zero();
  if constexpr (FORM_CB) {
    const T *Cl = static_cast<const T *>(p.C) + b * p.C_bs + g * p.C_gs + (int64_t)(t0 + lt * GB) * p.C_ls;
    const T *Bsr = static_cast<const T *>(p.B) + b * p.B_bs + g * p.B_gs + (int64_t)(t0 + st * GB) * p.B_ls;
    bool formed = false;
    if constexpr (FASTP != 0) {
      // The tile of C B^T the way the heads' products are formed below: FASTP states at a time, a 64 x FASTP piece of
      // the C rows and of the B rows from memory to LDS in 16-byte pieces, one barrier pair per piece.
      if (p.dstate % FASTP == 0 && rows_aligned16(Cl, p.C_ls) && rows_aligned16(Bsr, p.B_ls) && p.C_ls < (1 << 21) && p.B_ls < (1 << 21)) {
        constexpr int PITCH = FASTP + 8, NP = FASTP / 32, KS = FASTP / 32;
        uint16_t *ca = reinterpret_cast<uint16_t *>(&lds), *ba = ca + GB * PITCH;
        typedef const GLOBAL_AS char *gptr;
        uint32_t coff[NP], boff[NP];
        int loff[NP];
#pragma unroll
        for (int q = 0; q < NP; ++q) {
          const int id = tid + q * 256, r = id / (FASTP / 8), c8 = id % (FASTP / 8);
          // from the chunk's first row (rows past the end of the sequence re-read its last row: never negative)
          coff[q] = (uint32_t)(min(lt * GB + r, qlim - 1) * (int)p.C_ls + c8 * 8) * 2u;
          boff[q] = (uint32_t)(min(st * GB + r, qlim - 1) * (int)p.B_ls + c8 * 8) * 2u;
          loff[q] = r * PITCH + c8 * 8;
        }
        u32x4 cr[NP], br[NP];
        const T *Cc = static_cast<const T *>(p.C) + b * p.C_bs + g * p.C_gs + (int64_t)t0 * p.C_ls;
        const T *Bc = static_cast<const T *>(p.B) + b * p.B_bs + g * p.B_gs + (int64_t)t0 * p.B_ls;
        auto fetch_cb = [&](int n0) {
#pragma unroll
          for (int q = 0; q < NP; ++q) {
            cr[q] = *(const GLOBAL_AS u32x4 *)((gptr)(Cc + n0) + coff[q]);
            br[q] = *(const GLOBAL_AS u32x4 *)((gptr)(Bc + n0) + boff[q]);
          }
        };
        fetch_cb(0);
#pragma unroll 1
        for (int n0 = 0; n0 < p.dstate; n0 += FASTP) {
          lds_barrier();
#pragma unroll
          for (int q = 0; q < NP; ++q) {
            *reinterpret_cast<u32x4 *>(ca + loff[q]) = cr[q];
            *reinterpret_cast<u32x4 *>(ba + loff[q]) = br[q];
          }
          lds_barrier();
          fetch_cb(min(n0 + FASTP, p.dstate - FASTP));
#pragma unroll
          for (int kk = 0; kk < KS; ++kk) {
            bf16x8_t af[2], bfr[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
              af[t] = *reinterpret_cast<const bf16x8_t *>(&ca[(wm * 32 + t * 16 + i) * PITCH + kk * 32 + gq * 8]);
              bfr[t] = *reinterpret_cast<const bf16x8_t *>(&ba[(wn * 32 + t * 16 + i) * PITCH + kk * 32 + gq * 8]);
            }
#pragma unroll
            for (int tm = 0; tm < 2; ++tm)
#pragma unroll
              for (int tn = 0; tn < 2; ++tn)
                acc.v[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[tm], bfr[tn], acc.v[tm][tn], 0, 0, 0);
          }
        }
        formed = true;
      }
    }
    if (!formed)
      block_gemm_pipe<SPLIT>(
          acc, lds, 0, p.dstate,
          KcStager<SPLIT, T>(lds.ah, lds.al, Cl, p.C_ls, qlim - lt * GB, p.dstate, nullptr, nullptr, rows_aligned16(Cl, p.C_ls), tid),
          KcStager<SPLIT, T>(lds.bh, lds.bl, Bsr, p.B_ls, qlim - st * GB, p.dstate, nullptr, nullptr, rows_aligned16(Bsr, p.B_ls), tid),
          tid);
  }
  const float *CB = FORM_CB ? nullptr : p.CB + (((int64_t)b * p.nchunks + c) * G + g) * Q * Q;
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int l = lt * GB + wm * 32 + tm * 16 + gq * 4 + r, s = st * GB + wn * 32 + tn * 16 + i;
        const bool ok = l < qlim && s <= l && (!seq || seq[l] == seq[s]);
        if constexpr (FORM_CB) {
          cbr[tm][tn][r] = ok ? acc.v[tm][tn][r] : 0.f;
          acc.v[tm][tn][r] = 0.f;
        } else {
          cbr[tm][tn][r] = ok ? CB[(int64_t)l * Q + s] : 0.f;
        }
        live |= (uint32_t)ok << ((tm * 2 + tn) * 4 + r);
      }
  // One pipeline over the heads of this workgroup: k runs over (head, p), a head's product is
  // finished, weighted and added to the sum at its last k step, and the loads of the next head are
  // already in flight then.
  const int nh = (hpg - hs + nsplit - 1) / nsplit;
  const int seg_k = (P + GK - 1) / GK * GK;
  auto load_rows = [&](int hl, int par) {  // rows of head hl into buffer par; published by the next step's barriers
    const int h = g * hpg + hs + hl * nsplit;
    const float *dA = chunk_row(p.dA_cumsum, p, b, h, c);
    const float *dt = chunk_row(p.dt_out, p, b, h, c);
    // On the diagonal tiles the exponents' rows are kept times log2(e): the decay of an element is then one v_exp_f32
    // of a difference.  Below the diagonal every l lies after every s, and the decay is taken apart at the l tile's
    // first position, exp(a_l - a_ref) * exp(a_ref - a_s) with both exponents <= 0: the rows hold the two factors
    // (one exponential per row and head instead of one per element), the second one times dt_s.
    if constexpr (BELOW) {
      const float a_ref = dA[lt * GB] * kLog2e;
      if (tid < GB) hA_l[par][tid] = lt * GB + tid < Q ? fast_exp2(fminf(dA[lt * GB + tid] * kLog2e - a_ref, 0.f)) : 0.f;
      else if (tid < 2 * GB) hA_s[par][tid - GB] = dt[st * GB + tid - GB] * fast_exp2(fminf(a_ref - dA[st * GB + tid - GB] * kLog2e, 0.f));
      return;
    }
    if (tid < GB) hA_l[par][tid] = lt * GB + tid < Q ? dA[lt * GB + tid] * kLog2e : 0.f;
    else if (tid < 2 * GB) hA_s[par][tid - GB] = st * GB + tid - GB < Q ? dA[st * GB + tid - GB] * kLog2e : 0.f;
    else if (tid < 3 * GB) hdt[par][tid - 2 * GB] = st * GB + tid - 2 * GB < Q ? dt[st * GB + tid - 2 * GB] : 0.f;
  };
  load_rows(0, 0);
  // d = a head's dCB term (added to sum); w = d * CB, whose row / column sums go to ddA
  auto weigh_head = [&](int hl) {
    const int par = hl & 1;
    float a_s[2], dt_s[2] = {0.f, 0.f}, csum[2] = {0.f, 0.f};
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
      a_s[tn] = hA_s[par][wn * 32 + tn * 16 + i];
      if (!BELOW) dt_s[tn] = hdt[par][wn * 32 + tn * 16 + i];
    }
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = wm * 32 + tm * 16 + gq * 4 + r;
        const float a_l = hA_l[par][m];
        float rsum = 0.f;
#pragma unroll
        for (int tn = 0; tn < 2; ++tn) {
          // (not masked here: cbr is zero at the masked positions, so w is, and sum is masked once at the end)
          const float d = BELOW ? acc.v[tm][tn][r] * a_s[tn] * a_l
                                : acc.v[tm][tn][r] * dt_s[tn] * fast_exp2(fminf(a_l - a_s[tn], 0.f));
          acc.v[tm][tn][r] = 0.f;
          sum.v[tm][tn][r] += d;
          const float w = d * cbr[tm][tn][r];
          rsum += w;
          csum[tn] += w;
        }
        rsum += dpp_f<DPP_ROW_SHR + 1>(0.f, rsum);
        rsum += dpp_f<DPP_ROW_SHR + 2>(0.f, rsum);
        rsum += dpp_f<DPP_ROW_SHR + 4>(0.f, rsum);
        rsum += dpp_f<DPP_ROW_SHR + 8>(0.f, rsum);
        if (i == 15) rs_s[wn][hl][m] = rsum;
      }
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
      float cs = csum[tn];
      cs += __shfl_xor(cs, 16, 64);
      cs += __shfl_xor(cs, 32, 64);
      if (gq == 0) cs_s[wm][hl][wn * 32 + tn * 16 + i] = cs;
    }
  };
  if constexpr (FASTP != 0) {
    constexpr int PITCH = FASTP + 8, NP = FASTP / 32, KS = FASTP / 32;  // LDS row pitch; pieces per thread and tile; k slices
    static_assert(2 * GB * PITCH * sizeof(uint16_t) <= sizeof(GemmLds), "both tiles fit in the pipeline's LDS");
    uint16_t *ga = reinterpret_cast<uint16_t *>(&lds), *xa = ga + GB * PITCH;
    typedef const GLOBAL_AS char *gptr;
    // this thread's pieces of a head's tiles: byte offsets from the chunk's first row (rows past the end of the
    // sequence re-read its last row; what they produce is masked), the same for every head
    uint32_t goff[NP], xoff[NP];
    int loff[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int id = tid + q * 256, r = id / (FASTP / 8), c8 = id % (FASTP / 8);
      goff[q] = (uint32_t)(min(lt * GB + r, qlim - 1) * (int)gv.ls + c8 * 8) * 2u;
      xoff[q] = (uint32_t)(min(st * GB + r, qlim - 1) * (int)p.x_ls + c8 * 8) * 2u;
      loff[q] = r * PITCH + c8 * 8;
    }
    u32x4 gr[NP], xr[NP];
    // the first head's rows, and the distance to the next head of this workgroup's list
    const int h0 = g * hpg + hs;
    const gptr gb0 = (gptr)(static_cast<const T *>(gv.ptr) + b * gv.bs + h0 * gv.hs + (int64_t)t0 * gv.ls);
    const gptr xb0 = (gptr)(static_cast<const T *>(p.x) + b * p.x_bs + h0 * p.x_hs + (int64_t)t0 * p.x_ls);
    const int64_t gstep = (int64_t)nsplit * gv.hs * 2, xstep = (int64_t)nsplit * p.x_hs * 2;
    auto fetch = [&](int hl) {
      const gptr gb = gb0 + hl * gstep, xb = xb0 + hl * xstep;
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        gr[q] = *(const GLOBAL_AS u32x4 *)(gb + goff[q]);
        xr[q] = *(const GLOBAL_AS u32x4 *)(xb + xoff[q]);
      }
    };
    fetch(0);
#pragma unroll 1
    for (int hl = 0; hl < nh; ++hl) {
      lds_barrier();  // every wave is done with the previous head's tiles and rows
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        *reinterpret_cast<u32x4 *>(ga + loff[q]) = gr[q];
        *reinterpret_cast<u32x4 *>(xa + loff[q]) = xr[q];
      }
      load_rows(min(hl + 1, nh - 1), (hl + 1) & 1);  // (after the last head: its own rows again, into the idle buffer)
      lds_barrier();
      fetch(min(hl + 1, nh - 1));
      bf16x8_t af[2][KS], bfr[2][KS];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
          af[t][kk] = *reinterpret_cast<const bf16x8_t *>(&ga[(wm * 32 + t * 16 + i) * PITCH + kk * 32 + gq * 8]);
          bfr[t][kk] = *reinterpret_cast<const bf16x8_t *>(&xa[(wn * 32 + t * 16 + i) * PITCH + kk * 32 + gq * 8]);
        }
#pragma unroll
      for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int tn = 0; tn < 2; ++tn) {
          f32x4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int kk = 0; kk < KS; ++kk) v = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[tm][kk], bfr[tn][kk], v, 0, 0, 0);
          acc.v[tm][tn] = v;
        }
      weigh_head(hl);
    }
  } else
  // A = g rows (l, k = p), B = x rows (s, k = p): both k-contiguous
  block_gemm_pipe<SPLIT>(
      acc, lds, 0, nh * seg_k,
      seg_stager(KcStager<SPLIT, T>(lds.ah, lds.al, nullptr, gv.ls, qlim - lt * GB, P, nullptr, nullptr, false, tid),
                 [&](KcStager<SPLIT, T> &q, int hl) {
                   q.base = static_cast<const T *>(gv.ptr) + b * gv.bs + (g * hpg + hs + hl * nsplit) * gv.hs +
                            (int64_t)(t0 + lt * GB) * gv.ls;
                   q.vec = rows_aligned16(q.base, gv.ls);
                 },
                 seg_k),
      seg_stager(KcStager<SPLIT, T>(lds.bh, lds.bl, nullptr, p.x_ls, qlim - st * GB, P, nullptr, nullptr, false, tid),
                 [&](KcStager<SPLIT, T> &q, int hl) {
                   q.base = static_cast<const T *>(p.x) + b * p.x_bs + (g * hpg + hs + hl * nsplit) * p.x_hs +
                            (int64_t)(t0 + st * GB) * p.x_ls;
                   q.vec = rows_aligned16(q.base, p.x_ls);
                 },
                 seg_k),
      tid, [&](int k0) {
        const int hl = k0 / seg_k;
        // the buffer written here was last read one step ago, before this step's barriers
        if (k0 % seg_k == 0 && hl + 1 < nh) load_rows(hl + 1, (hl + 1) & 1);
        if ((k0 + GK) % seg_k != 0) return;
        weigh_head(hl);
      });
  __syncthreads();
  for (int idx = tid; idx < nh * GB; idx += 256) {
    const int hl = idx / GB, r = idx % GB;
    const int64_t dda = chunk_off(p, b, g * hpg + hs + hl * nsplit, c);
    const float row = rs_s[0][hl][r] + rs_s[1][hl][r], col = cs_s[0][hl][r] + cs_s[1][hl][r];
    if (lt * GB + r < Q && row != 0.f) acc_add<DET ? 1 : 0>(p.ddA_cumsum, p.det_ddA_cumsum, dda + lt * GB + r, row, det_scale_of(p));
    if (st * GB + r < Q && col != 0.f) acc_add<DET ? 1 : 0>(p.ddA_cumsum, p.det_ddA_cumsum, dda + st * GB + r, -col, det_scale_of(p));
  }
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (!((live >> ((tm * 2 + tn) * 4 + r)) & 1)) sum.v[tm][tn][r] = 0.f;  // causal / same-sequence mask
  // Several workgroups (head lists) add into one tile: dCB starts zeroed.  One list per group: this workgroup owns the
  // tile and stores it whole, zeros included, so the caller need not clear dCB (the later stages read these tiles only).
  const bool own_tile = !DET && nsplit == 1;
  acc_foreach(sum, tid, [&](int m, int n, float v) {
    const int l = lt * GB + m, s = st * GB + n;
    if (l < Q && s < Q) {
      if (own_tile && lp) st1<bf16_t>(reinterpret_cast<bf16_t *>(p.dCB) + dCB_off + (int64_t)l * Q + s, v);
      else if (own_tile) p.dCB[dCB_off + (int64_t)l * Q + s] = v;
      else if (v != 0.f) acc_add<DET ? 1 : 0>(p.dCB, p.det_dCB, dCB_off + (int64_t)l * Q + s, v, det_scale_of(p));
    }
    return v;
  });
}

template <typename T, bool SPLIT, bool DET, bool FORM_CB = false>
__global__ __launch_bounds__(256, 4) void bwd_dcb_kernel(const SsdParams p) {
  __shared__ DcbShared sh;
  const Block3 blk = xcd_block();
  int lt = 0, rem = blk.x;
  while (rem > lt) { rem -= lt + 1; ++lt; }
  const int st = rem;
  if (lt != st)
    dcb_tile<T, SPLIT, DET, FORM_CB, true, 0>(p, sh, blk, lt, st, false);
  else
    dcb_tile<T, SPLIT, DET, FORM_CB, false, 0>(p, sh, blk, lt, st, false);
}
// bf16 operands on 16-byte aligned rows of FASTP = 32 or 64 values, no integer shadows
template <bool FORM_CB, int FASTP>
__global__ __launch_bounds__(256, 4) void bwd_dcb_rows_kernel(const SsdParams p, const int lp) {
  __shared__ DcbShared sh;
  const Block3 blk = xcd_block();
  int lt = 0, rem = blk.x;
  while (rem > lt) { rem -= lt + 1; ++lt; }
  const int st = rem;
  if (lt != st)
    dcb_tile<bf16_t, false, false, FORM_CB, true, FASTP>(p, sh, blk, lt, st, lp != 0);
  else
    dcb_tile<bf16_t, false, false, FORM_CB, false, FASTP>(p, sh, blk, lt, st, lp != 0);
}

// ------------------------------------------------------------- bmm bwd
// dC32[l, n] += sum_{s <= l} dCB[l, s] B[s, n];   dB32[s, n] += sum_{l >= s} dCB[l, s] C[l, n]
template <typename T, bool SPLIT> __global__ __launch_bounds__(256) void bmm_chunk_bwd_kernel(const SsdParams p) {
  __shared__ GemmLds lds;
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, G = p.ngroups;
  const int ntn = cdiv(N, GB);
  const int mt = blockIdx.x / ntn, nt = blockIdx.x % ntn;
  const int c = blockIdx.y, b = blockIdx.z / G, g = blockIdx.z % G;
  const int t0 = c * Q, qlim = min(Q, L - t0);
  const float *dCB = p.dCB + (((int64_t)b * p.nchunks + c) * G + g) * Q * Q;
  const int64_t Cb = b * p.C_bs + g * p.C_gs, Bb = b * p.B_bs + g * p.B_gs;
  {
    GemmAcc acc;
    acc.zero();
    // dCB is zero above the diagonal (never written), so no mask is needed here.
    // A = dCB rows (l, k = s): k-contiguous fp32; B = B^T (rows n, k = s): row-contiguous
    const float *da = dCB + (int64_t)mt * GB * Q;
    const T *Ba = static_cast<const T *>(p.B) + Bb + (int64_t)t0 * p.B_ls + nt * GB;
    const bool va = rows_aligned16(da, Q), vb = rows_aligned16(Ba, p.B_ls);
    const int kend = min((mt + 1) * GB, qlim);
    block_gemm_pipe<SPLIT>(
        acc, lds, 0, kend,
        KcStager<SPLIT, float>(lds.ah, lds.al, da, Q, qlim - mt * GB, kend, nullptr, nullptr, va, tid),
        TrStager<SPLIT, T>(lds.bh, lds.bl, Ba, p.B_ls, N - nt * GB, kend, nullptr, nullptr, vb, tid),
        tid);
    acc_foreach(acc, tid, [&](int m, int n, float v) {
      const int l = mt * GB + m, nn = nt * GB + n;
      if (l < qlim && nn < N) p.dC32[(((int64_t)b * L + t0 + l) * G + g) * N + nn] += v;
      return v;
    });
  }
  {
    GemmAcc acc;
    acc.zero();
    // A = dCB^T (rows s, k = l): row-contiguous fp32; B = C^T (rows n, k = l): row-contiguous
    const float *da = dCB + mt * GB;
    const T *Ca = static_cast<const T *>(p.C) + Cb + (int64_t)t0 * p.C_ls + nt * GB;
    const bool va = rows_aligned16(da, Q), vb = rows_aligned16(Ca, p.C_ls);
    block_gemm_pipe<SPLIT>(
        acc, lds, mt * GB, qlim,
        TrStager<SPLIT, float>(lds.ah, lds.al, da, Q, qlim - mt * GB, qlim, nullptr, nullptr, va, tid),
        TrStager<SPLIT, T>(lds.bh, lds.bl, Ca, p.C_ls, N - nt * GB, qlim, nullptr, nullptr, vb, tid),
        tid);
    acc_foreach(acc, tid, [&](int m, int n, float v) {
      const int s = mt * GB + m, nn = nt * GB + n;
      if (s < qlim && nn < N) p.dB32[(((int64_t)b * L + t0 + s) * G + g) * N + nn] += v;
      return v;
    });
  }
}

// The same two products on 64 x 128 tiles (whole 128-state blocks, chunks of whole k steps, 16-byte aligned B / C
// rows): half the workgroups, each k step of dCB staged once for twice the columns.
// LP: dCB holds bf16 tiles (packed at the start of the buffer; see dcb_tile), which go to LDS as they are.
// which: 0 = both products, one after the other; 1 = the dC product only; 2 = the dB product only (the two read
// different operands and write different sums: dealt to two workgroups they halve a workgroup's serial work where
// the tiles alone do not fill the chip).
template <typename T, bool SPLIT, bool LP = false>
DEVI void bmm_chunk_bwd_wide_body(const SsdParams &p, int bx, int by, int bz, int which = 0) {
  using CBT = std::conditional_t<LP, bf16_t, float>;
  __shared__ GemmLdsWide<SPLIT> lds;
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, G = p.ngroups;
  const int ntn = N / WB;
  const int mt = bx / ntn, nt = bx % ntn;
  const int c = by, b = bz / G, g = bz % G;
  const int t0 = c * Q, qlim = min(Q, L - t0);
  if (mt * GB >= qlim) return;
  const CBT *dCB = reinterpret_cast<const CBT *>(p.dCB) + (((int64_t)b * p.nchunks + c) * G + g) * Q * Q;
  const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1, i = lane & 15, gq = lane >> 4;
  // dst[(row of the chunk) * G * N + column] += tile.  This stage is the last one to add into dB32 / dC32 and its
  // tiles cover every row once: with `fin` set the sum leaves here in the operands' dtype as well (dB / dC), and no
  // separate conversion pass over the fp32 sums is needed.
  auto add_tile = [&](const GemmAccWide &acc, float *dst, void *fin) {
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = mt * GB + wm * 32 + tm * 16 + gq * 4 + r;
        if (m >= qlim) continue;
        const int64_t at = (((int64_t)b * L + t0 + m) * G + g) * N + nt * WB + wn * 64 + i;
        float *row = dst + at;
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) {
          const float v = row[tn * 16] + acc.v[tm][tn][r];
          if (fin) st1<T>(static_cast<T *>(fin) + at + tn * 16, v);  // the finished sum: nobody reads the fp32 one
          else row[tn * 16] = v;
        }
      }
  };
  if (which != 2) {
    // dC: A = dCB rows (l, k = s), k-contiguous fp32, s up to the end of the l tile; B = B rows (k = s, n)
    GemmAccWide acc;
    acc.zero();
    const int kend = min((mt + 1) * GB, qlim);
    KcStager<SPLIT, CBT> sa(lds.ah, lds.al, dCB + (int64_t)mt * GB * Q, Q, qlim - mt * GB, kend, nullptr, nullptr, true, tid);
    const T *Ba = static_cast<const T *>(p.B) + b * p.B_bs + g * p.B_gs + (int64_t)t0 * p.B_ls + nt * WB;
    WideTrStager<SPLIT, T, WB> sb(lds.bh, lds.bl, Ba, p.B_ls, WB, nullptr, tid);
    block_gemm_wide<SPLIT>(acc, lds, kend, sa, sb, tid);
    add_tile(acc, p.dC32, p.dC);
  }
  if (which == 0) lds_barrier();  // the first product's last operand reads end before the second one's first commit
  if (which != 1) {
    // dB: A = dCB^T (rows s, k = l from the s tile on), row-contiguous fp32; B = C rows (k = l, n)
    GemmAccWide acc;
    acc.zero();
    const int k0 = mt * GB;
    WideTrStager<SPLIT, CBT, 64> sa(lds.ah, lds.al, dCB + (int64_t)k0 * Q + mt * GB, Q, min(GB, Q - mt * GB), nullptr, tid);
    const T *Ca = static_cast<const T *>(p.C) + b * p.C_bs + g * p.C_gs + (int64_t)(t0 + k0) * p.C_ls + nt * WB;
    WideTrStager<SPLIT, T, WB> sb(lds.bh, lds.bl, Ca, p.C_ls, WB, nullptr, tid);
    block_gemm_wide<SPLIT>(acc, lds, qlim - k0, sa, sb, tid);
    add_tile(acc, p.dB32, p.dB);
  }
}

template <typename T, bool SPLIT> __global__ __launch_bounds__(256) void bmm_chunk_bwd_wide_kernel(const SsdParams p) {
  bmm_chunk_bwd_wide_body<T, SPLIT>(p, blockIdx.x, blockIdx.y, blockIdx.z);
}

// --------------------------------------------------------- cumsum bwd
// One workgroup per (batch, chunk, 16 heads); thread tid handles position Q-1-tid, so that the
// reverse running sum of dL/da over the chunk (-> dL/d(dt A)) is a forward wave scan.  Then the
// chain through A, the clamp, softplus and the bias; dA and ddt_bias are reduced per workgroup.

DEVI float wave_incl_sum(float x) {
  x += dpp_f<DPP_ROW_SHR + 1>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 2>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 4>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 8>(0.f, x);
  x += dpp_f<DPP_ROW_BCAST15, 0xa>(0.f, x);
  x += dpp_f<DPP_ROW_BCAST31, 0xc>(0.f, x);
  return x;
}

constexpr int CSB_HT = 4;  // heads per workgroup in the backward kernel (more, smaller workgroups)

DEVI void chunk_cumsum_bwd_body(const SsdParams &p, int bx, int by, int bz) {
  __shared__ float wtot[4][CSB_HT], part[2][4][CSB_HT];
  const int H = p.nheads, Q = p.chunk_size, L = p.seqlen;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l = Q - 1 - tid;
  const int c = bx, h0 = by * CSB_HT, b = bz;
  const int t = c * Q + l;
  const bool inq = l >= 0, live = inq && t < L;
  const int lc = max(l, 0), tc = min(c * Q + lc, L - 1);  // clamped: every load below is unconditional
  // all loads first
  float g[CSB_HT], o[CSB_HT], d[CSB_HT], raw[CSB_HT], A[CSB_HT], bias[CSB_HT];
#pragma unroll
  for (int i = 0; i < CSB_HT; ++i) {
    const int h = min(h0 + i, H - 1);
    g[i] = chunk_row(p.ddA_cumsum, p, b, h, c)[lc];
    o[i] = chunk_row(p.ddt_out, p, b, h, c)[lc];
    d[i] = chunk_row(p.dt_out, p, b, h, c)[lc];
    raw[i] = ld_dyn(p.dt, b * p.dt_bs + (int64_t)tc * p.dt_ls + h * p.dt_hs, p.dt_dtype);
    A[i] = static_cast<const float *>(p.A)[h];
    bias[i] = p.dt_bias ? static_cast<const float *>(p.dt_bias)[h] : 0.f;
  }
  float run[CSB_HT];
#pragma unroll
  for (int i = 0; i < CSB_HT; ++i) {
    run[i] = wave_incl_sum((h0 + i < H && inq) ? g[i] : 0.f);
    if (lane == 63) wtot[wave][i] = run[i];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < CSB_HT; ++i) {
    const int h = h0 + i;
    float r = run[i];
    for (int w = 0; w < wave; ++w) r += wtot[w][i];
    float dAterm = 0.f, ddt = 0.f;
    if (h < H && live) {
      ddt = __builtin_fmaf(r, A[i], o[i]);
      dAterm = r * d[i];
      const float x = raw[i] + bias[i];
      const float v = p.dt_softplus ? softplus_f(x) : x;
      if (v < p.dt_min || v > p.dt_max) ddt = 0.f;
      if (p.dt_softplus && x <= 20.f) ddt *= sigmoid_f(x);
      st_dyn(p.ddt, ((int64_t)b * L + t) * H + h, p.dt_dtype, ddt);
    }
    dAterm = wave_sum_to_last(dAterm);
    ddt = wave_sum_to_last(ddt);
    if (lane == 63) {
      part[0][wave][i] = dAterm;
      part[1][wave][i] = ddt;
    }
  }
  // one atomic per workgroup and head: adds to one address serialise in L2
  __syncthreads();
  if (tid < 2 * CSB_HT) {
    const int which = tid / CSB_HT, i = tid % CSB_HT, h = h0 + i;
    const float v = part[which][0][i] + part[which][1][i] + part[which][2][i] + part[which][3][i];
    if (h < H) {
      if (which == 0) acc_add(p.dA, p.det_dA, h, v, det_scale_of(p));
      else if (p.ddt_bias) acc_add(p.ddt_bias, p.det_ddt_bias, h, v, det_scale_of(p));
    }
  }
}

__global__ __launch_bounds__(256) void chunk_cumsum_bwd_kernel(const SsdParams p) {
  chunk_cumsum_bwd_body(p, blockIdx.x, blockIdx.y, blockIdx.z);
}

// The last two stages read disjoint results of the stages before them (dCB; ddA_cumsum and ddt_out) and neither
// fills the chip for long: one launch deals the wide-tile bmm workgroups first and the cumsum workgroups behind them.
template <typename T, bool SPLIT, bool LP = false>
__global__ __launch_bounds__(256) void bmm_cumsum_bwd_kernel(const SsdParams p, int n_bmm, int bmm_x, int bmm_y, int cs_x, int cs_y, int split) {
  const int id = blockIdx.x;
  if (id < n_bmm) {
    // split: two workgroups per tile, one per product, neighbours in launch order (they share the dCB tile)
    const int t = split ? id >> 1 : id, which = split ? 1 + (id & 1) : 0;
    bmm_chunk_bwd_wide_body<T, SPLIT, LP>(p, t % bmm_x, (t / bmm_x) % bmm_y, t / (bmm_x * bmm_y), which);
  } else {
    const int k = id - n_bmm;
    chunk_cumsum_bwd_body(p, k % cs_x, (k / cs_x) % cs_y, k / (cs_x * cs_y));
  }
}

int check_bwd(const SsdParams *p) {
  if (!p || !p->x || !p->dt || !p->A || !p->B || !p->C || !p->dout) return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->seqlen <= 0 || p->nheads <= 0 || p->headdim <= 0 || p->dstate <= 0 || p->ngroups <= 0 ||
      p->chunk_size <= 0 || p->nheads % p->ngroups != 0)
    return MAMBA_E_BADARG;
  if (p->nchunks != (p->seqlen + p->chunk_size - 1) / p->chunk_size) return MAMBA_E_BADARG;
  if (p->chunk_size > 256 || p->dstate > 256 || p->headdim > 256) return MAMBA_E_UNSUPPORTED;
  if ((int64_t)p->batch * p->nheads > 65535 || p->nchunks > 65535) return MAMBA_E_UNSUPPORTED;
  if (p->dtype != MAMBA_F32 && p->dtype != MAMBA_BF16 && p->dtype != MAMBA_F16) return MAMBA_E_BADARG;
  if (!p->dt_out || !p->dA_cumsum || !p->ddA_cumsum || !p->ddt_out || !p->dCB || !p->dB32 || !p->dC32 ||
      !p->dx || !p->ddt || !p->dA)
    return MAMBA_E_BADARG;  // (CB may be null: ssd_bwd_dcb then forms its tiles itself; the tiled dx kernel refuses)
  // the carried states and their gradients: bf16 buffers next to bf16 operands, the fp32 ones otherwise
  if (p->dtype == MAMBA_BF16) {
    if (!p->states_lp || !p->dstates_lp) return MAMBA_E_BADARG;
    if ((reinterpret_cast<uintptr_t>(p->states_lp) | reinterpret_cast<uintptr_t>(p->dstates_lp)) & 15) return MAMBA_E_BADARG;
  } else if (!p->states || !p->dstates) {
    return MAMBA_E_BADARG;
  }
  if (p->z && (!p->dz || !p->gbuf || !p->out_x)) return MAMBA_E_BADARG;
  if (!p->z && !p->out) return MAMBA_E_BADARG;
  if (p->D && !p->dD) return MAMBA_E_BADARG;
  return MAMBA_OK;
}
int launched() { return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH; }

#define SSD_DISPATCH(KERNEL, GRID)                                                                   \
  switch (p->dtype) {                                                                                \
    case MAMBA_BF16: hipLaunchKernelGGL((KERNEL<bf16_t, false>), GRID, dim3(256), 0, s, *p); break;  \
    case MAMBA_F16: hipLaunchKernelGGL((KERNEL<f16_t, true>), GRID, dim3(256), 0, s, *p); break;     \
    default: hipLaunchKernelGGL((KERNEL<float, true>), GRID, dim3(256), 0, s, *p); break;            \
  }

// the same for kernels compiled per summation mode (float atomics / fixed-point integer atomics)
#define SSD_DISPATCH_DET(KERNEL, GRID)                                                                          \
  if (p->det_scale) {                                                                                           \
    switch (p->dtype) {                                                                                         \
      case MAMBA_BF16: hipLaunchKernelGGL((KERNEL<bf16_t, false, true>), GRID, dim3(256), 0, s, *p); break;     \
      case MAMBA_F16: hipLaunchKernelGGL((KERNEL<f16_t, true, true>), GRID, dim3(256), 0, s, *p); break;        \
      default: hipLaunchKernelGGL((KERNEL<float, true, true>), GRID, dim3(256), 0, s, *p); break;               \
    }                                                                                                           \
  } else {                                                                                                      \
    switch (p->dtype) {                                                                                         \
      case MAMBA_BF16: hipLaunchKernelGGL((KERNEL<bf16_t, false, false>), GRID, dim3(256), 0, s, *p); break;    \
      case MAMBA_F16: hipLaunchKernelGGL((KERNEL<f16_t, true, false>), GRID, dim3(256), 0, s, *p); break;       \
      default: hipLaunchKernelGGL((KERNEL<float, true, false>), GRID, dim3(256), 0, s, *p); break;              \
    }                                                                                                           \
  }

inline int tiles(int n) { return (n + GB - 1) / GB; }

}  // namespace

static int ssd_bwd_dz_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check_bwd(p);
  if (rc) return rc;
  if (!p->z && !p->D) return MAMBA_OK;  // neither a gate nor a skip term: nothing to compute
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((p->seqlen + 63) / 64, p->nheads, p->batch);
  switch (p->dtype) {
    case MAMBA_BF16: hipLaunchKernelGGL(bwd_dz_kernel<bf16_t>, grid, dim3(256), 0, s, *p); break;
    case MAMBA_F16: hipLaunchKernelGGL(bwd_dz_kernel<f16_t>, grid, dim3(256), 0, s, *p); break;
    default: hipLaunchKernelGGL(bwd_dz_kernel<float>, grid, dim3(256), 0, s, *p); break;
  }
  return launched();
}

static int ssd_bwd_dstates_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check_bwd(p);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  {
    const bool g_ok = p->z ? (p->headdim % 8 == 0 && reinterpret_cast<uintptr_t>(p->gbuf) % 16 == 0)
                           : wide_operand_ok(p->dout, p->dtype, p->dout_bs, p->dout_ls, p->dout_hs);
    const bool wide = p->dstate % WB == 0 && p->headdim % 8 == 0 && whole_k_steps(p) && g_ok &&
                      wide_operand_ok(p->C, p->dtype, p->C_bs, p->C_ls, p->C_gs);
    if (wide) {
      dim3 grid(tiles(p->headdim) * (p->dstate / WB), p->nchunks, p->batch * p->nheads);
      SSD_DISPATCH(bwd_dstates_wide_kernel, grid)
      return launched();
    }
  }
  dim3 grid(tiles(p->headdim) * tiles(p->dstate), p->nchunks, p->batch * p->nheads);
  SSD_DISPATCH(bwd_dstates_kernel, grid)
  return launched();
}

static int ssd_state_passing_bwd_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check_bwd(p);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int PN = p->headdim * p->dstate;
  auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool lp = p->dtype == MAMBA_BF16;
  const bool vec = PN % 4 == 0 && al16(p->dfinal_states) && al16(p->dinitial_states) &&
                   (lp ? true : al16(p->states) && al16(p->dstates));
  const size_t tbytes = (size_t)p->nchunks * 5 * sizeof(float);  // decay factors + the four waves' partial sums
  const bool table = tbytes <= SPB_TABLE_BYTES;
  if (vec) {
    dim3 grid((PN / 4 + 255) / 256, p->nheads, p->batch);
    if (table && PN % 1024 == 0) {
      if (lp) hipLaunchKernelGGL((state_passing_bwd_kernel<4, bf16_t, true, true>), grid, dim3(256), tbytes, s, *p);
      else hipLaunchKernelGGL((state_passing_bwd_kernel<4, float, true, true>), grid, dim3(256), tbytes, s, *p);
    } else if (table) {
      if (lp) hipLaunchKernelGGL((state_passing_bwd_kernel<4, bf16_t, true>), grid, dim3(256), tbytes, s, *p);
      else hipLaunchKernelGGL((state_passing_bwd_kernel<4, float, true>), grid, dim3(256), tbytes, s, *p);
    } else {
      if (lp) hipLaunchKernelGGL((state_passing_bwd_kernel<4, bf16_t, false>), grid, dim3(256), 0, s, *p);
      else hipLaunchKernelGGL((state_passing_bwd_kernel<4, float, false>), grid, dim3(256), 0, s, *p);
    }
  } else {
    dim3 grid((PN + 255) / 256, p->nheads, p->batch);
    if (lp) hipLaunchKernelGGL((state_passing_bwd_kernel<1, bf16_t, false>), grid, dim3(256), 0, s, *p);
    else hipLaunchKernelGGL((state_passing_bwd_kernel<1, float, false>), grid, dim3(256), 0, s, *p);
  }
  return launched();
}

// Without a gate dD is sum g x with g = dout, and the fused dx kernel holds both operands: where it runs and D is
// one value per head it adds dD up on its way, and the pass of bwd_dz_kernel over dout and x is not needed.
static bool dD_with_dx(const SsdParams *p) {
  return !p->z && p->D && p->dD && !p->D_has_hdim && ssd_bwd_dx_fused_supported(p);
}

static int ssd_bwd_dx_with(const SsdParams *p, mamba_stream_t stream, bool sum_dD) {
  int rc = check_bwd(p);
  if (rc) return rc;
  if (p->dx_ls < (int64_t)p->headdim || p->dx_hs < (int64_t)p->headdim) return MAMBA_E_BADARG;  // strides not filled in
  hipStream_t s = static_cast<hipStream_t>(stream);
  // bf16 on the common shapes: the fused kernel, which forms C B^T itself (p->CB is not read); else the tiled one
  rc = ssd_bwd_dx_fused_launch(p, s, sum_dD);
  if (rc != MAMBA_E_UNSUPPORTED) return rc;
  if (sum_dD) return MAMBA_E_UNSUPPORTED;  // dD_with_dx promised the fused kernel
  if (!p->CB) return MAMBA_E_BADARG;  // the tiled kernel reads C B^T
  dim3 grid(tiles(p->chunk_size) * tiles(p->headdim), p->nchunks, p->batch * p->nheads);
  SSD_DISPATCH_DET(bwd_dx_kernel, grid)
  return launched();
}
static int ssd_bwd_dx_one(const SsdParams *p, mamba_stream_t stream) { return ssd_bwd_dx_with(p, stream, false); }

static int ssd_bwd_dBC_state_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check_bwd(p);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // bf16 on the common shapes: the kernels that keep a head's operands in LDS; else the tiled ones
  rc = ssd_bwd_dbc_fused_launch(p, s);
  if (rc != MAMBA_E_UNSUPPORTED) return rc;
  const int zdim = p->batch * p->ngroups * head_splits(p->nheads / p->ngroups);
  dim3 grid(tiles(p->chunk_size) * tiles(p->dstate), p->nchunks, zdim);
  // whole 128-state blocks, headdim in whole k steps, aligned x rows: the dB product runs on wide tiles
  const bool wide = p->dstate % WB == 0 && p->headdim % GK == 0 &&
                    wide_operand_ok(p->x, p->dtype, p->x_bs, p->x_ls, p->x_hs);
  if (wide) {
    dim3 gridw(tiles(p->chunk_size) * (p->dstate / WB), p->nchunks, zdim);
    const bool g_ok = p->z ? (p->headdim % 8 == 0 && reinterpret_cast<uintptr_t>(p->gbuf) % 16 == 0)
                           : wide_operand_ok(p->dout, p->dtype, p->dout_bs, p->dout_ls, p->dout_hs);
    if (g_ok) {
      SSD_DISPATCH_DET(bwd_dC_state_wide_kernel, gridw)
    } else {
      SSD_DISPATCH_DET(bwd_dC_state_kernel, grid)
    }
    SSD_DISPATCH_DET(bwd_dB_state_wide_kernel, gridw)
    return launched();
  }
  SSD_DISPATCH_DET(bwd_dBC_state_kernel, grid)
  return launched();
}

// The head loop of its own in the dCB stage: bf16 operands on 16-byte aligned rows of 32 or 64 values, no integer
// shadows.
static bool dcb_rows_ok(const SsdParams *p) {
  const void *gp = p->z ? p->gbuf : p->dout;
  const int64_t g_ls = p->z ? (int64_t)p->nheads * p->headdim : p->dout_ls, g_hs = p->z ? p->headdim : p->dout_hs,
                g_bs = p->z ? (int64_t)p->seqlen * p->nheads * p->headdim : p->dout_bs;
  return p->dtype == MAMBA_BF16 && !p->det_scale && (p->headdim == 32 || p->headdim == 64) && gp && aligned(gp, 16) &&
         aligned(p->x, 16) && !(g_ls % 8 || g_hs % 8 || g_bs % 8) && !(p->x_ls % 8 || p->x_hs % 8 || p->x_bs % 8) &&
         g_ls < (1 << 21) && p->x_ls < (1 << 21);
}
static bool bmm_bwd_wide_ok(const SsdParams *p);
// Inside ssd_combined_bwd the dCB tiles pass from the dCB stage to the bmm stage as bf16 where one workgroup owns each
// tile and the bmm stage's operand is bf16 anyway (the stages on their own keep the fp32 tiles their interface names).
static int64_t bmm_cumsum_workgroups(const SsdParams *p);
static bool dcb_tiles_lp(const SsdParams *p) {
  return dcb_rows_ok(p) && p->dCB && dcb_head_splits(p->nheads / p->ngroups) == 1 && bmm_bwd_wide_ok(p) &&
         bmm_cumsum_workgroups(p) <= 0x7fffffff;  // (the one-launch form of the last two stages is the reader)
}

static int ssd_bwd_dcb_one(const SsdParams *p, mamba_stream_t stream, bool lp) {
  int rc = check_bwd(p);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int nt = tiles(p->chunk_size);
  dim3 grid(nt * (nt + 1) / 2, p->nchunks, p->batch * p->ngroups * dcb_head_splits(p->nheads / p->ngroups));
  if (dcb_rows_ok(p)) {
    const int lpi = lp ? 1 : 0;
    if (p->headdim == 64) {
      if (p->CB) hipLaunchKernelGGL((bwd_dcb_rows_kernel<false, 64>), grid, dim3(256), 0, s, *p, lpi);
      else hipLaunchKernelGGL((bwd_dcb_rows_kernel<true, 64>), grid, dim3(256), 0, s, *p, lpi);
    } else {
      if (p->CB) hipLaunchKernelGGL((bwd_dcb_rows_kernel<false, 32>), grid, dim3(256), 0, s, *p, lpi);
      else hipLaunchKernelGGL((bwd_dcb_rows_kernel<true, 32>), grid, dim3(256), 0, s, *p, lpi);
    }
    return launched();
  }
  if (!p->CB) {  // the workgroups form their tiles of C B^T themselves (default mode only: ssd_bwd_overwrites)
    if (p->det_scale) return MAMBA_E_BADARG;
    switch (p->dtype) {
      case MAMBA_BF16: hipLaunchKernelGGL((bwd_dcb_kernel<bf16_t, false, false, true>), grid, dim3(256), 0, s, *p); break;
      case MAMBA_F16: hipLaunchKernelGGL((bwd_dcb_kernel<f16_t, true, false, true>), grid, dim3(256), 0, s, *p); break;
      default: hipLaunchKernelGGL((bwd_dcb_kernel<float, true, false, true>), grid, dim3(256), 0, s, *p); break;
    }
    return launched();
  }
  SSD_DISPATCH_DET(bwd_dcb_kernel, grid)
  return launched();
}

static int ssd_bwd_dcb_stage(const SsdParams *p, mamba_stream_t stream) { return ssd_bwd_dcb_one(p, stream, false); }

static int ssd_bmm_chunk_bwd_one(const SsdParams *p_in, mamba_stream_t stream) {
  int rc = check_bwd(p_in);
  if (rc) return rc;
  // the stage on its own only adds into dB32 / dC32; dB / dC are written by ssd_combined_bwd, whose last stage this is
  SsdParams q = *p_in;
  q.dB = q.dC = nullptr;
  const SsdParams *p = &q;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (p->dstate % WB == 0 && p->chunk_size % GB == 0 && whole_k_steps(p) &&
      wide_operand_ok(p->B, p->dtype, p->B_bs, p->B_ls, p->B_gs) && wide_operand_ok(p->C, p->dtype, p->C_bs, p->C_ls, p->C_gs) &&
      reinterpret_cast<uintptr_t>(p->dCB) % 16 == 0) {
    dim3 gridw(tiles(p->chunk_size) * (p->dstate / WB), p->nchunks, p->batch * p->ngroups);
    SSD_DISPATCH(bmm_chunk_bwd_wide_kernel, gridw)
    return launched();
  }
  dim3 grid(tiles(p->chunk_size) * tiles(p->dstate), p->nchunks, p->batch * p->ngroups);
  SSD_DISPATCH(bmm_chunk_bwd_kernel, grid)
  return launched();
}

static int ssd_chunk_cumsum_bwd_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check_bwd(p);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(p->nchunks, (p->nheads + CSB_HT - 1) / CSB_HT, p->batch);
  hipLaunchKernelGGL(chunk_cumsum_bwd_kernel, grid, dim3(256), 0, s, *p);
  return launched();
}

extern "C" int ssd_det_convert(const int64_t *shadow, float *dst, int64_t n, const float *det_scale, mamba_stream_t stream) {
  if (n == 0) return MAMBA_OK;
  if (!shadow || !dst || !det_scale || n < 0 || (n + 255) / 256 > 0x7fffffff) return MAMBA_E_BADARG;
  hipLaunchKernelGGL(det_convert_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     shadow, dst, n, det_scale);
  return launched();
}

static bool bmm_bwd_wide_ok(const SsdParams *p) {
  return p->dstate % WB == 0 && p->chunk_size % GB == 0 && whole_k_steps(p) &&
         wide_operand_ok(p->B, p->dtype, p->B_bs, p->B_ls, p->B_gs) && wide_operand_ok(p->C, p->dtype, p->C_bs, p->C_ls, p->C_gs) &&
         reinterpret_cast<uintptr_t>(p->dCB) % 16 == 0;
}

// dst[i] = T(src[i]): the fp32 sums of dB / dC in the operands' dtype, for the paths whose last stage does not
// write them itself
template <typename T> __global__ __launch_bounds__(256) void cast_sum_kernel(const float *__restrict__ src, T *__restrict__ dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) st1<T>(dst + i, src[i]);
}
static int cast_sums(const SsdParams *p, mamba_stream_t stream) {
  const int64_t n = (int64_t)p->batch * p->seqlen * p->ngroups * p->dstate;
  if ((!p->dB && !p->dC) || n == 0) return MAMBA_OK;
  if ((n + 255) / 256 > 0x7fffffff) return MAMBA_E_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((n + 255) / 256));
  for (int k = 0; k < 2; ++k) {
    void *dst = k ? p->dC : p->dB;
    const float *src = k ? p->dC32 : p->dB32;
    if (!dst) continue;
    switch (p->dtype) {
      case MAMBA_BF16: hipLaunchKernelGGL(cast_sum_kernel<bf16_t>, grid, dim3(256), 0, s, src, static_cast<bf16_t *>(dst), n); break;
      case MAMBA_F16: hipLaunchKernelGGL(cast_sum_kernel<f16_t>, grid, dim3(256), 0, s, src, static_cast<f16_t *>(dst), n); break;
      default: hipLaunchKernelGGL(cast_sum_kernel<float>, grid, dim3(256), 0, s, src, static_cast<float *>(dst), n); break;
    }
  }
  return launched();
}

// The last two stages as one launch where the bmm stage runs on wide tiles, else one after the other.  Either way
// dB / dC (when the caller passes them) hold the finished sums in the operands' dtype afterwards.
static int64_t bmm_cumsum_workgroups(const SsdParams *p) {
  return (int64_t)tiles(p->chunk_size) * (p->dstate / WB) * p->nchunks * p->batch * p->ngroups +
         (int64_t)p->nchunks * ((p->nheads + CSB_HT - 1) / CSB_HT) * p->batch;
}
static int bmm_and_cumsum_bwd(const SsdParams *p, mamba_stream_t stream, bool lp = false) {
  int rc = check_bwd(p);
  if (rc) return rc;
  const int64_t bmm_x = tiles(p->chunk_size) * (p->dstate / WB), bmm_y = p->nchunks, bmm_z = (int64_t)p->batch * p->ngroups;
  const int64_t cs_x = p->nchunks, cs_y = (p->nheads + CSB_HT - 1) / CSB_HT, cs_z = p->batch;
  // few tiles (fewer than four workgroups per CU): a workgroup per product instead of one per tile
  const int split = bmm_x * bmm_y * bmm_z < 4 * (int64_t)cu_count() ? 1 : 0;
  const int64_t n_bmm = bmm_x * bmm_y * bmm_z * (split ? 2 : 1), total = n_bmm + cs_x * cs_y * cs_z;
  if (bmm_bwd_wide_ok(p) && p->dCB && total <= 0x7fffffff) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid((unsigned)total);
#define SSD_LAUNCH_BMM_CS(T, SPLIT) \
  hipLaunchKernelGGL((bmm_cumsum_bwd_kernel<T, SPLIT>), grid, dim3(256), 0, s, *p, (int)n_bmm, (int)bmm_x, (int)bmm_y, (int)cs_x, (int)cs_y, split)
    switch (p->dtype) {
      case MAMBA_BF16:
        if (lp) hipLaunchKernelGGL((bmm_cumsum_bwd_kernel<bf16_t, false, true>), grid, dim3(256), 0, s, *p, (int)n_bmm, (int)bmm_x, (int)bmm_y, (int)cs_x, (int)cs_y, split);
        else SSD_LAUNCH_BMM_CS(bf16_t, false);
        break;
      case MAMBA_F16: SSD_LAUNCH_BMM_CS(f16_t, true); break;
      default: SSD_LAUNCH_BMM_CS(float, true); break;
    }
#undef SSD_LAUNCH_BMM_CS
    return launched();
  }
  if ((rc = ssd_bmm_chunk_bwd(p, stream))) return rc;
  if ((rc = ssd_chunk_cumsum_bwd(p, stream))) return rc;
  return cast_sums(p, stream);
}

// The first two stages: one kernel where the gate's pass over dout, z and the pre-gate output can feed the
// state-gradient product directly (bf16 operands, one 128-state tile, whole k steps, 16-byte aligned rows), else
// ssd_bwd_dz and ssd_bwd_dstates.
static int dz_and_dstates(const SsdParams *p, mamba_stream_t stream) {
  int rc = check_bwd(p);
  if (rc) return rc;
  auto rows16 = [&](const void *q, int64_t bs, int64_t ls, int64_t hs) {
    return q && reinterpret_cast<uintptr_t>(q) % 16 == 0 && bs % 8 == 0 && ls % 8 == 0 && hs % 8 == 0;
  };
  const bool fused = p->z && p->out_x && p->dz && p->gbuf && p->dtype == MAMBA_BF16 && p->dstates_lp &&
                     p->dstate == WB && p->headdim % 8 == 0 && whole_k_steps(p) &&
                     rows16(p->dout, p->dout_bs, p->dout_ls, p->dout_hs) && rows16(p->z, p->z_bs, p->z_ls, p->z_hs) &&
                     rows16(p->out_x, p->out_bs, p->out_ls, p->out_hs) && rows16(p->x, p->x_bs, p->x_ls, p->x_hs) &&
                     rows16(p->dz, 0, 0, 0) && rows16(p->gbuf, 0, 0, 0) &&
                     wide_operand_ok(p->C, p->dtype, p->C_bs, p->C_ls, p->C_gs);
  if (fused) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(tiles(p->headdim), p->nchunks, p->batch * p->nheads);
    hipLaunchKernelGGL(bwd_dz_dstates_kernel<bf16_t>, grid, dim3(256), 0, s, *p);
    return launched();
  }
  if (!dD_with_dx(p) && (rc = ssd_bwd_dz(p, stream))) return rc;
  return ssd_bwd_dstates(p, stream);
}

static int ssd_combined_bwd_one(const SsdParams *p, mamba_stream_t stream) {
  int rc;
  if (p && p->det_scale) {
    // deterministic mode: every shared sum goes through its integer shadow
    if (!p->det_ddA_cumsum || !p->det_ddt_out || !p->det_dCB || !p->det_dB || !p->det_dC || !p->det_dA ||
        (p->D && !p->det_dD) || (p->ddt_bias && !p->det_ddt_bias))
      return MAMBA_E_BADARG;
    const int64_t rows = (int64_t)p->batch * p->nheads * p->nchunks * p->chunk_size;
    const int64_t bc = (int64_t)p->batch * p->seqlen * p->ngroups * p->dstate;
    const int64_t cb = (int64_t)p->batch * p->nchunks * p->ngroups * p->chunk_size * p->chunk_size;
    if ((rc = dz_and_dstates(p, stream))) return rc;
    if ((rc = ssd_state_passing_bwd(p, stream))) return rc;
    if ((rc = ssd_bwd_dBC_state(p, stream))) return rc;
    if ((rc = ssd_bwd_dx_with(p, stream, dD_with_dx(p)))) return rc;
    if ((rc = ssd_bwd_dcb(p, stream))) return rc;
    // every term of these sums is in: shadows -> the float buffers their readers take
    if ((rc = ssd_det_convert(p->det_dCB, p->dCB, cb, p->det_scale, stream))) return rc;
    if ((rc = ssd_det_convert(p->det_dB, p->dB32, bc, p->det_scale, stream))) return rc;
    if ((rc = ssd_det_convert(p->det_dC, p->dC32, bc, p->det_scale, stream))) return rc;
    if ((rc = ssd_det_convert(p->det_ddA_cumsum, p->ddA_cumsum, rows, p->det_scale, stream))) return rc;
    if ((rc = ssd_det_convert(p->det_ddt_out, p->ddt_out, rows, p->det_scale, stream))) return rc;
    if (p->D && (rc = ssd_det_convert(p->det_dD, p->dD, p->D_has_hdim ? (int64_t)p->nheads * p->headdim : p->nheads,
                                      p->det_scale, stream)))
      return rc;
    if ((rc = bmm_and_cumsum_bwd(p, stream))) return rc;  // bmm: one workgroup per output tile, plain adds
    if ((rc = ssd_det_convert(p->det_dA, p->dA, p->nheads, p->det_scale, stream))) return rc;
    if (p->ddt_bias) return ssd_det_convert(p->det_ddt_bias, p->ddt_bias, p->nheads, p->det_scale, stream);
    return MAMBA_OK;
  }
  if ((rc = dz_and_dstates(p, stream))) return rc;
  if ((rc = ssd_state_passing_bwd(p, stream))) return rc;
  // dC reads the forward states, which the state-passing kernel has just read, and dB and dx the dstates it has just
  // written: in this order each finds them in the last-level cache
  if ((rc = ssd_bwd_dBC_state(p, stream))) return rc;
  if ((rc = ssd_bwd_dx_with(p, stream, dD_with_dx(p)))) return rc;
  const bool lp = dcb_tiles_lp(p);
  if ((rc = ssd_bwd_dcb_one(p, stream, lp))) return rc;
  return bmm_and_cumsum_bwd(p, stream, lp);
}

extern "C" int ssd_bwd_overwrites(const SsdParams *p) {
  if (!p || check_bwd(p) != MAMBA_OK || p->det_scale || (int64_t)p->batch * p->nheads > SSD_MAX_GRID_ROWS) return 0;
  int flags = 0;
  if (dcb_head_splits(p->nheads / p->ngroups) == 1) flags |= SSD_OVERWRITES_DCB;
  if (ssd_bwd_dbc_fused_owns(p)) flags |= SSD_OVERWRITES_DBC;
  // CB: only the dCB stage and the tiled dx kernel read it.  Where the fused dx kernel runs and a group is one head
  // list (so that each tile of C B^T would be formed once), the dCB stage can form its tiles itself.
  if (dcb_head_splits(p->nheads / p->ngroups) == 1 && ssd_bwd_dx_fused_supported(p)) flags |= SSD_BWD_FORMS_CB;
  return flags;
}

// Public entry points: the whole problem in one go when one launch can index it, else in slices of batch rows.
extern "C" int ssd_bwd_dz(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_bwd_dz_one); }
extern "C" int ssd_bwd_dstates(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_bwd_dstates_one); }
extern "C" int ssd_state_passing_bwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_state_passing_bwd_one); }
extern "C" int ssd_bwd_dx(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_bwd_dx_one); }
extern "C" int ssd_bwd_dBC_state(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_bwd_dBC_state_one); }
extern "C" int ssd_bwd_dcb(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_bwd_dcb_stage); }
extern "C" int ssd_bmm_chunk_bwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_bmm_chunk_bwd_one); }
extern "C" int ssd_chunk_cumsum_bwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_chunk_cumsum_bwd_one); }
extern "C" int ssd_combined_bwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_combined_bwd_one); }
