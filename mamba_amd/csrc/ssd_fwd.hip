// Mamba-2 SSD forward for gfx950: chunk_cumsum, chunk_state, state_passing,
// bmm (C B^T) and chunk_scan.  The three dense contractions run on bf16 MFMA
// through the block-GEMM core of ssd_common.hpp; the other two are small
// streaming kernels.
#include "ssd_common.hpp"

namespace {

// ------------------------------------------------------------ chunk_cumsum
// One workgroup per (batch, chunk, 4 heads); thread = position inside the chunk, so loads of
// dt (head-contiguous) are 4 consecutive elements per thread and the stores of dt_out / dA_cumsum
// (position-contiguous) are coalesced.  (The kernel is a chain of short latencies, so it wants many small
// workgroups: 15.5 us with 16 heads per workgroup at batch 4 x 16 chunks x 80 heads, 11.1 with 4, 10.2 with 2.)  dt -> (+bias, softplus, clamp), zero past the end of the
// sequence; dA_cumsum = running sum of dt * A over the chunk (wave DPP scan + cross-wave offsets).
constexpr int CS_HT = 4;

DEVI float wave_incl_sum(float x) {
  x += dpp_f<DPP_ROW_SHR + 1>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 2>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 4>(0.f, x);
  x += dpp_f<DPP_ROW_SHR + 8>(0.f, x);
  x += dpp_f<DPP_ROW_BCAST15, 0xa>(0.f, x);
  x += dpp_f<DPP_ROW_BCAST31, 0xc>(0.f, x);
  return x;
}

__global__ __launch_bounds__(256) void chunk_cumsum_fwd_kernel(const SsdParams p) {
  __shared__ float wtot[4][CS_HT];
  const int H = p.nheads, nc = p.nchunks, Q = p.chunk_size;
  const int l = threadIdx.x, lane = l & 63, wave = l >> 6;
  const int c = blockIdx.x, h0 = blockIdx.y * CS_HT, b = blockIdx.z;
  const int t = c * Q + l;
  const bool live = l < Q && t < p.seqlen;
  float dtv[CS_HT], cs[CS_HT];
#pragma unroll
  for (int i = 0; i < CS_HT; ++i) {
    const int h = h0 + i;
    float dt = 0.f, A = 0.f;
    if (h < H) {
      A = static_cast<const float *>(p.A)[h];
      if (live) {
        dt = ld_dyn(p.dt, b * p.dt_bs + (int64_t)t * p.dt_ls + h * p.dt_hs, p.dt_dtype);
        if (p.dt_bias) dt += static_cast<const float *>(p.dt_bias)[h];
        if (p.dt_softplus) dt = softplus_f(dt);
        dt = fminf(fmaxf(dt, p.dt_min), p.dt_max);
      }
    }
    dtv[i] = dt;
    cs[i] = wave_incl_sum(dt * A);
    if (lane == 63) wtot[wave][i] = cs[i];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < CS_HT; ++i) {
    const int h = h0 + i;
    float off = 0.f;
    for (int w = 0; w < wave; ++w) off += wtot[w][i];
    if (h < H && l < Q) {
      const int64_t o = (((int64_t)b * H + h) * nc + c) * Q + l;
      p.dt_out[o] = dtv[i];
      p.dA_cumsum[o] = cs[i] + off;
    }
  }
}

DEVI bool seq_same(const int32_t *seq, int a, int b) { return seq[a] == seq[b]; }

// --------------------------------------------------------------- bmm (CB)
// CB[b, c, g, l, s] = sum_n C[l, n] B[s, n] for s-tiles at or below the l-tile,
// zeroed where seq_idx differs.
template <typename T, bool SPLIT> __global__ __launch_bounds__(256) void bmm_chunk_fwd_kernel(const SsdParams p) {
  __shared__ GemmLds lds;
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, G = p.ngroups;
  // blockIdx.x enumerates the lower-triangular tile pairs (mt >= nt)
  int mt = 0, rem = blockIdx.x;
  while (rem > mt) { rem -= mt + 1; ++mt; }
  const int nt = rem;
  const int c = blockIdx.y, b = blockIdx.z / G, g = blockIdx.z % G;
  const int t0 = c * Q;
  const int64_t Cb = b * p.C_bs + g * p.C_gs, Bb = b * p.B_bs + g * p.B_gs;
  GemmAcc acc;
  acc.zero();
  const int qlim = min(Q, L - t0);
  const T *Ca = static_cast<const T *>(p.C) + Cb + (int64_t)(t0 + mt * GB) * p.C_ls;
  const T *Ba = static_cast<const T *>(p.B) + Bb + (int64_t)(t0 + nt * GB) * p.B_ls;
  const bool va = rows_aligned16(Ca, p.C_ls), vb = rows_aligned16(Ba, p.B_ls);
  block_gemm_pipe<SPLIT>(
      acc, lds, 0, N,
      KcStager<SPLIT, T>(lds.ah, lds.al, Ca, p.C_ls, qlim - mt * GB, N, nullptr, nullptr, va, tid),
      KcStager<SPLIT, T>(lds.bh, lds.bl, Ba, p.B_ls, qlim - nt * GB, N, nullptr, nullptr, vb, tid),
      tid);
  float *CB = p.CB + (((int64_t)b * p.nchunks + c) * G + g) * Q * Q;
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  acc_foreach(acc, tid, [&](int m, int n, float v) {
    const int l = mt * GB + m, s = nt * GB + n;
    if (l < Q && s < Q) {
      float o = v;
      if (seq && (t0 + l >= L || t0 + s >= L || seq[l] != seq[s])) o = 0.f;
      CB[(int64_t)l * Q + s] = o;
    }
    return v;
  });
}

// ------------------------------------------------------------ chunk_state
// states[b, c, h, p, n] = sum_s x[s, p] B[s, n] exp(a_last - a_s) dt_s over the
// positions s of the chunk that belong to the sequence of its last position.
template <typename T, bool SPLIT> __global__ __launch_bounds__(256) void chunk_state_fwd_kernel(const SsdParams p) {
  __shared__ GemmLds lds;
  __shared__ float w[256];
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads;
  const int ntn = cdiv(N, GB);
  const Block3 blk = xcd_block_heads(H);  // the tiles of one (chunk, head) share its x / g rows: same L2
  const int pt = blk.x / ntn, nt = blk.x % ntn;
  const int c = blk.y, b = blk.z / H, h = blk.z % H;
  const int g = h / (H / p.ngroups);
  const int t0 = c * Q;
  const int qlim = min(Q, L - t0);
  const float *dA = p.dA_cumsum + (((int64_t)b * H + h) * p.nchunks + c) * Q;
  const float *dt = p.dt_out + (((int64_t)b * H + h) * p.nchunks + c) * Q;
  const float a_last = dA[Q - 1];
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  for (int s = tid; s < Q; s += 256) {
    float v = 0.f;
    if (s < qlim) {
      bool ok = true;
      if (seq) {
        const int last = seq[qlim - 1];
        ok = last >= 0 && seq[s] == last;
      }
      if (ok) v = fast_exp(fminf(a_last - dA[s], 0.f)) * dt[s];
    }
    w[s] = v;
  }
  const int64_t xb = b * p.x_bs + h * p.x_hs, Bb = b * p.B_bs + g * p.B_gs;
  GemmAcc acc;
  acc.zero();
  // A = x^T (rows p, k = position), B = (B w)^T (rows n, k = position): both row-contiguous sources
  const T *xa = static_cast<const T *>(p.x) + xb + (int64_t)t0 * p.x_ls + pt * GB;
  const T *Ba = static_cast<const T *>(p.B) + Bb + (int64_t)t0 * p.B_ls + nt * GB;
  const bool va = rows_aligned16(xa, p.x_ls), vb = rows_aligned16(Ba, p.B_ls);
  block_gemm_pipe<SPLIT>(  // the first barrier inside publishes w
      acc, lds, 0, qlim,
      TrStager<SPLIT, T>(lds.ah, lds.al, xa, p.x_ls, P - pt * GB, qlim, nullptr, nullptr, va, tid),
      TrStager<SPLIT, T>(lds.bh, lds.bl, Ba, p.B_ls, N - nt * GB, qlim, w, nullptr, vb, tid),
      tid);
  float *st = p.states + (((int64_t)b * p.nchunks + c) * H + h) * P * N;
  acc_foreach(acc, tid, [&](int m, int n, float v) {
    const int pp = pt * GB + m, nn = nt * GB + n;
    if (pp < P && nn < N) st[(int64_t)pp * N + nn] = v;
    return v;
  });
}

// The same product with a 64 x 128 tile per workgroup, for whole 128-state blocks of aligned operands
// and chunks that are whole k steps.
template <typename T, bool SPLIT> __global__ __launch_bounds__(256) void chunk_state_fwd_wide_kernel(const SsdParams p) {
  __shared__ GemmLdsWide<SPLIT> lds;
  __shared__ float w[256];
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads;
  const int ntn = N / WB;
  const Block3 blk = xcd_block_heads(H);
  const int pt = blk.x / ntn, nt = blk.x % ntn;
  const int c = blk.y, b = blk.z / H, h = blk.z % H;
  const int g = h / (H / p.ngroups);
  const int t0 = c * Q;
  const int qlim = min(Q, L - t0);
  const float *dA = p.dA_cumsum + (((int64_t)b * H + h) * p.nchunks + c) * Q;
  const float *dt = p.dt_out + (((int64_t)b * H + h) * p.nchunks + c) * Q;
  const float a_last = dA[Q - 1];
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  for (int s = tid; s < Q; s += 256) {
    float v = 0.f;
    if (s < qlim) {
      bool ok = true;
      if (seq) {
        const int last = seq[qlim - 1];
        ok = last >= 0 && seq[s] == last;
      }
      if (ok) v = fast_exp(fminf(a_last - dA[s], 0.f)) * dt[s];
    }
    w[s] = v;
  }
  const T *xa = static_cast<const T *>(p.x) + b * p.x_bs + h * p.x_hs + (int64_t)t0 * p.x_ls + pt * GB;
  const T *Ba = static_cast<const T *>(p.B) + b * p.B_bs + g * p.B_gs + (int64_t)t0 * p.B_ls + nt * WB;
  GemmAccWide acc;
  acc.zero();
  WideTrStager<SPLIT, T, 64> sa(lds.ah, lds.al, xa, p.x_ls, P - pt * GB, nullptr, tid);
  WideTrStager<SPLIT, T, WB> sb(lds.bh, lds.bl, Ba, p.B_ls, WB, w, tid);
  block_gemm_wide<SPLIT>(acc, lds, qlim, sa, sb, tid);  // the first barrier inside publishes w
  float *st = p.states + (((int64_t)b * p.nchunks + c) * H + h) * P * N;
  store_wide_rows(acc, lds, st + (int64_t)pt * GB * N + nt * WB, N, P - pt * GB, tid);
}

// ---------------------------------------------------- chunk_state_varlen
// Packed batch (batch 1): state at the last position of every sequence i = [cu[i], cu[i+1]).
// out[i, h, p, n] = sum_{k in the last chunk, k >= start} x[k, p] B[k, n] exp(a_end - a_k) dt_k
//                 + exp(a_end) states[c, h, p, n] if the sequence began before that chunk,
// with `states` the state entering each chunk.  Empty sequences give zeros.
template <typename T, bool SPLIT>
__global__ __launch_bounds__(256) void chunk_state_varlen_kernel(const SsdParams p, const int32_t *cu, float *out) {
  __shared__ GemmLds lds;
  __shared__ float w[256];
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, P = p.headdim, H = p.nheads;
  const int ntn = cdiv(N, GB);
  const int pt = blockIdx.x / ntn, nt = blockIdx.x % ntn;
  const int i = blockIdx.y, h = blockIdx.z;
  const int g = h / (H / p.ngroups);
  const int start = cu[i], end = min(cu[i + 1], p.seqlen);
  float *dst = out + ((int64_t)i * H + h) * P * N;
  GemmAcc acc;
  acc.zero();
  if (end > start) {
    const int c = (end - 1) / Q, t0 = c * Q;
    const int kstart = max(start - t0, 0), kend = end - t0;
    const float *dA = p.dA_cumsum + ((int64_t)h * p.nchunks + c) * Q;
    const float *dt = p.dt_out + ((int64_t)h * p.nchunks + c) * Q;
    const float a_end = dA[kend - 1];
    for (int k = tid; k < Q; k += 256)
      w[k] = (k >= kstart && k < kend) ? fast_exp(fminf(a_end - dA[k], 0.f)) * dt[k] : 0.f;
    const T *xa = static_cast<const T *>(p.x) + h * p.x_hs + (int64_t)t0 * p.x_ls + pt * GB;
    const T *Ba = static_cast<const T *>(p.B) + g * p.B_gs + (int64_t)t0 * p.B_ls + nt * GB;
    const bool va = rows_aligned16(xa, p.x_ls), vb = rows_aligned16(Ba, p.B_ls);
    block_gemm_pipe<SPLIT>(  // the first barrier inside publishes w
        acc, lds, kstart / GK * GK, kend,
        TrStager<SPLIT, T>(lds.ah, lds.al, xa, p.x_ls, P - pt * GB, kend, nullptr, nullptr, va, tid),
        TrStager<SPLIT, T>(lds.bh, lds.bl, Ba, p.B_ls, N - nt * GB, kend, w, nullptr, vb, tid),
        tid);
    if (start < t0) {
      const carried_t<T> *Hc = carried_states<T>(p) + ((int64_t)c * H + h) * P * N;
      const float sc = fast_exp(a_end);
      acc_foreach(acc, tid, [&](int m, int n, float v) {
        const int pp = pt * GB + m, nn = nt * GB + n;
        return (pp < P && nn < N) ? __builtin_fmaf(sc, ld1<carried_t<T>>(Hc + (int64_t)pp * N + nn), v) : v;
      });
    }
  }
  acc_foreach(acc, tid, [&](int m, int n, float v) {
    const int pp = pt * GB + m, nn = nt * GB + n;
    if (pp < P && nn < N) dst[(int64_t)pp * N + nn] = v;
    return v;
  });
}

// ---------------------------------------------------------- state_passing
// In place over `states`: slot c receives the state ENTERING chunk c; the state
// after the last chunk goes to final_states.  A thread owns W consecutive elements of the
// (headdim x dstate) state; the chunk loop is a serial recurrence, so the local states of the
// next SP_PF chunks are always in flight (the compiler cannot hoist those loads over the in-place
// stores by itself).  TABLE: the per-chunk decay factors are put in LDS before the loop; read one by one inside
// it they are scalar loads, each waited for with everything else the scalar unit has in flight, and with few rows
// per chunk (one long packed batch) that wait was the time of a step.
constexpr int SP_PF = 4;
constexpr size_t SP_TABLE_BYTES = 32768;

template <int W> struct VecF;
template <> struct VecF<1> {
  float v[1];
  DEVI void load(const float *p) { v[0] = *p; }
  DEVI void store(float *p) const { *p = v[0]; }
};
template <> struct VecF<4> {
  float v[4];
  DEVI void load(const float *p) {
    const f32x4 t = *reinterpret_cast<const f32x4 *>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  DEVI void store(float *p) const { *reinterpret_cast<f32x4 *>(p) = f32x4{v[0], v[1], v[2], v[3]}; }
};

// CT float: in place, slot c of `states` receives the state entering chunk c.  CT bf16_t: that state goes to
// states_lp in bf16 and `states` is only read.
template <int W, typename CT, bool TABLE> __global__ __launch_bounds__(256) void state_passing_fwd_kernel(const SsdParams p) {
  extern __shared__ float sp_decay[];
  const int PN = p.headdim * p.dstate, H = p.nheads, nc = p.nchunks, Q = p.chunk_size, L = p.seqlen;
  const int e = (blockIdx.x * 256 + threadIdx.x) * W;
  const int h = blockIdx.y, b = blockIdx.z;
  const float *dA = p.dA_cumsum + ((int64_t)b * H + h) * nc * Q;
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L : nullptr;
  auto decay_of = [&](int c) {  // carried-state factor of chunk c: 0 across a sequence boundary
    float scale = fast_exp(dA[c * Q + Q - 1]);
    if (seq) {
      const int seq_new = seq[min((c + 1) * Q, L) - 1], seq_prev = c > 0 ? seq[c * Q - 1] : 0;
      if (seq_new != seq_prev) scale = 0.f;
    }
    return scale;
  };
  if constexpr (TABLE) {
    for (int c = threadIdx.x; c < nc; c += 256) sp_decay[c] = decay_of(c);
    lds_barrier();
  }
  if (e >= PN) return;
  auto decay = [&](int c) { return TABLE ? sp_decay[c] : decay_of(c); };
  VecF<W> s;
#pragma unroll
  for (int i = 0; i < W; ++i) s.v[i] = 0.f;
  if (p.initial_states) s.load(p.initial_states + ((int64_t)b * H + h) * PN + e);
  auto slot = [&](int c) { return p.states + (((int64_t)b * nc + c) * H + h) * PN + e; };
  VecF<W> local[SP_PF];
  float scale[SP_PF];
#pragma unroll
  for (int j = 0; j < SP_PF; ++j) {
    local[j].load(slot(min(j, nc - 1)));
    scale[j] = decay(min(j, nc - 1));
  }
  // one chunk, its local state in slot j of the prefetch; `more`: request chunk c + SP_PF into the slot
  auto step = [&](int c, int j, bool more) {
    if constexpr (std::is_same_v<CT, float>) {
      s.store(slot(c));
    } else {
      CT *o = static_cast<CT *>(p.states_lp) + (((int64_t)b * nc + c) * H + h) * PN + e;
      if constexpr (W == 4) {
        *reinterpret_cast<u32x2 *>(o) = u32x2{pack_bf16(s.v[0], s.v[1]), pack_bf16(s.v[2], s.v[3])};
      } else {
        st1<CT>(o, s.v[0]);
      }
    }
    const VecF<W> loc = local[j];
    const float sc = scale[j];
    if (more) {  // past the last chunk the loads repeat it and nobody uses them: no branch, so no register copies
                 // (which would wait for the loads in flight) where the paths meet
      const int cn = min(c + SP_PF, nc - 1);
      local[j].load(slot(cn));
      scale[j] = decay(cn);
    }
#pragma unroll
    for (int i = 0; i < W; ++i) s.v[i] = __builtin_fmaf(sc, s.v[i], loc.v[i]);
  };
  // whole groups of SP_PF chunks without a branch inside, then the chunks left over from what the slots hold
  int c0 = 0;
  for (; c0 + SP_PF <= nc; c0 += SP_PF) {
#pragma unroll
    for (int j = 0; j < SP_PF; ++j) step(c0 + j, j, true);
  }
#pragma unroll
  for (int j = 0; j < SP_PF - 1; ++j)
    if (c0 + j < nc) step(c0 + j, j, false);
  s.store(p.final_states + ((int64_t)b * H + h) * PN + e);
}

// ------------------------------------------- chunk states and state passing in one pass
// bf16, headdim 64, 128 states, chunks of Q = 32 R positions that tile the sequence: one workgroup per (batch, head)
// walks the sequence once.  Per chunk it forms the chunk's own state (the product of chunk_state_fwd_wide_kernel,
// a 64 x 128 tile, k = position), writes the state ENTERING the chunk (bf16, what the scan and the backward pass
// read) and carries H <- decay_c H + S_c in fp32 registers; after the last chunk H is final_states.  The fp32
// per-chunk states never exist in memory (configuration 2: 168 MB written and read again), and the recurrence over
// the chunks costs no pass of its own.  With few workgroups (batch x heads) the loads must be deep instead: R pairs
// of stagers hold the operands of the next R steps -- one chunk ahead -- and no branch surrounds a load or a store
// of the walk, so each step waits for exactly its own operands.  The per-position weights w_s of chunk c + 1 are
// computed while chunk c is multiplied (two tables in LDS), the per-chunk decay factors once at the start.
constexpr int CSP_MAX_CHUNKS = 2048;
template <int R, bool HAS_SEQ> __global__ __launch_bounds__(256) void chunk_state_passing_fwd_kernel(const SsdParams p) {
  using T = bf16_t;
  using SA = WideTrStager<false, T, 64>;
  using SB = WideTrStager<false, T, WB>;
  constexpr int Q = 32 * R, P = 64, N = WB;
  static_assert(Q <= 256, "one table entry per thread");
  __shared__ GemmLdsWide<false> lds;
  __shared__ float wtab[2][Q];
  __shared__ float dec[CSP_MAX_CHUNKS];
  const int tid = threadIdx.x;
  const int L = p.seqlen, H = p.nheads, nc = p.nchunks;
  const int h = blockIdx.x, b = blockIdx.y;
  const int g = h / (H / p.ngroups);
  const float *dA = p.dA_cumsum + ((int64_t)b * H + h) * nc * Q;
  const float *dtp = p.dt_out + ((int64_t)b * H + h) * nc * Q;
  const int32_t *seq = HAS_SEQ ? p.seq_idx + (int64_t)b * L : nullptr;
  for (int c = tid; c < nc; c += 256) {  // carried-state factor of chunk c: 0 across a sequence boundary
    float scale = fast_exp(dA[c * Q + Q - 1]);
    if (HAS_SEQ) {
      const int seq_new = seq[(c + 1) * Q - 1], seq_prev = c > 0 ? seq[c * Q - 1] : 0;
      if (seq_new != seq_prev) scale = 0.f;
    }
    dec[c] = scale;
  }
  // w_s = dt_s exp(a_last - a_s) for the positions of the chunk's last sequence, else 0; entry min(tid, Q - 1)
  const int ts = min(tid, Q - 1);
  float t_a, t_alast, t_dt;
  int t_sid = 0, t_slast = 0;
  auto table_request = [&](int c) {
    t_a = *(const GLOBAL_AS float *)(dA + c * Q + ts);
    t_alast = *(const GLOBAL_AS float *)(dA + c * Q + Q - 1);
    t_dt = *(const GLOBAL_AS float *)(dtp + c * Q + ts);
    if (HAS_SEQ) {
      t_sid = *(const GLOBAL_AS int32_t *)(seq + c * Q + ts);
      t_slast = *(const GLOBAL_AS int32_t *)(seq + c * Q + Q - 1);
    }
  };
  auto table_write = [&](int c) {
    float v = fast_exp(fminf(t_alast - t_a, 0.f)) * t_dt;
    if (HAS_SEQ && !(t_slast >= 0 && t_sid == t_slast)) v = 0.f;
    if (tid < Q) wtab[c & 1][tid] = v;
  };
  table_request(0);
  table_write(0);

  // H in the accumulator layout: rows 32 wm + 16 tm + 4 g + r, columns 64 wn + 16 tn + i
  GemmAccWide Hs, acc;
  Hs.zero();
  if (p.initial_states) {
    const int lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1, i = lane & 15, gq = lane >> 4;
    const float *init = p.initial_states + ((int64_t)b * H + h) * P * N;
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int tn = 0; tn < 4; ++tn)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          Hs.v[tm][tn][r] = init[(wm * 32 + tm * 16 + gq * 4 + r) * N + wn * 64 + tn * 16 + i];
  }

  const T *xa = static_cast<const T *>(p.x) + b * p.x_bs + h * p.x_hs;
  const T *Ba = static_cast<const T *>(p.B) + b * p.B_bs + g * p.B_gs;
  SA sa[R];
  SB sb[R];
  {
    const SA sa0(lds.ah, lds.al, xa, p.x_ls, P, nullptr, tid);
    const SB sb0(lds.bh, lds.bl, Ba, p.B_ls, WB, wtab[0], tid);
#pragma unroll
    for (int j = 0; j < R; ++j) {
      sa[j] = sa0;
      sb[j] = sb0;
      sa[j].template fetch<true>(j * GK);
      sb[j].template fetch<true>(j * GK);
      // the requests leave in the order the walk consumes them: the waits in the loop are counted from the order
      // on either way into it, and the compiler would otherwise issue these independent loads last pair first
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  bf16_t *carried = static_cast<bf16_t *>(p.states_lp) + ((int64_t)b * nc * H + h) * P * N;
#pragma unroll 1
  for (int c = 0; c < nc; ++c) {
    table_request(min(c + 1, nc - 1));
    acc.zero();
    const float *ks = &wtab[c & 1][0] - c * Q;  // the stagers index their weights by position in the sequence
#pragma unroll
    for (int j = 0; j < R; ++j) {
      sb[j].kscale = ks;
      wide_step(acc, lds, c * Q + j * GK, sa[j], sb[j], min(c * Q + (j + R) * GK, L - GK), tid);
    }
    table_write(c + 1);  // read from the next step's first barrier on; last read two chunks ago
    store_wide_rows<false, bf16_t, false>(Hs, lds, carried + (int64_t)c * H * P * N, N, P, tid);
    const float d = dec[c];
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int tn = 0; tn < 4; ++tn) Hs.v[tm][tn] = Hs.v[tm][tn] * d + acc.v[tm][tn];
  }
  store_wide_rows<false, float, false>(Hs, lds, p.final_states + ((int64_t)b * H + h) * P * N, N, P, tid);
}

// ------------------------------------------------------------- chunk_scan
// out[l, p] = exp(a_l) [seq_l == seq before the chunk] sum_n C[l, n] Hc[p, n]
//           + sum_{s <= l} CB[l, s] exp(a_l - a_s) dt_s x[s, p] + D x[l, p];   out *= silu(z)
template <typename T, bool SPLIT> __global__ __launch_bounds__(256) void chunk_scan_fwd_kernel(const SsdParams p) {
  __shared__ GemmLds lds;
  __shared__ float a_s[256], dt_s[256], rscale[GB];
  const int tid = threadIdx.x;
  const int Q = p.chunk_size, N = p.dstate, L = p.seqlen, P = p.headdim, H = p.nheads, G = p.ngroups;
  const int ntp = cdiv(P, GB);
  const int mt = blockIdx.x / ntp, pt = blockIdx.x % ntp;
  const int c = blockIdx.y, b = blockIdx.z / H, h = blockIdx.z % H;
  const int g = h / (H / G);
  const int t0 = c * Q;
  const int qlim = min(Q, L - t0);
  const float *dA = p.dA_cumsum + (((int64_t)b * H + h) * p.nchunks + c) * Q;
  const float *dt = p.dt_out + (((int64_t)b * H + h) * p.nchunks + c) * Q;
  const int32_t *seq = p.seq_idx ? p.seq_idx + (int64_t)b * L + t0 : nullptr;
  for (int s = tid; s < Q; s += 256) {
    a_s[s] = dA[s];
    dt_s[s] = dt[s];
  }
  if (tid < GB) {
    const int l = mt * GB + tid;
    float sc = 0.f;
    if (l < qlim) {
      bool ok = true;
      if (seq) {
        const int prev = c > 0 ? seq[-1] : 0;
        ok = seq[l] == prev;
      }
      if (ok) sc = fast_exp(dA[l]);
    }
    rscale[tid] = sc;
  }
  const int64_t xb = b * p.x_bs + h * p.x_hs, Cb = b * p.C_bs + g * p.C_gs;
  const carried_t<T> *Hc = carried_states<T>(p) + (((int64_t)b * p.nchunks + c) * H + h) * P * N;
  const float *CB = p.CB + (((int64_t)b * p.nchunks + c) * G + g) * Q * Q;
  GemmAcc acc;
  acc.zero();
  {  // carried state -> outputs
    auto fa = [&](int r, int k) {  // (l, n)
      const int l = mt * GB + r;
      return (l < qlim && k < N) ? ldg<T>(p.C, Cb + (int64_t)(t0 + l) * p.C_ls + k) : 0.f;
    };
    auto fb = [&](int r, int k) {  // (p, n)
      const int pp = pt * GB + r;
      return (pp < P && k < N) ? ld1<carried_t<T>>(Hc + (int64_t)pp * N + k) : 0.f;
    };
    block_gemm<SPLIT, true, true>(acc, lds, 0, N, fa, fb, tid);
    acc_foreach(acc, tid, [&](int m, int n, float v) { return v * rscale[m]; });
  }
  {  // inside the chunk, causal
    const int kmax = min((mt + 1) * GB, qlim);
    auto fa = [&](int r, int k) {  // (l, s)
      const int l = mt * GB + r;
      if (l >= qlim || k > l) return 0.f;
      return CB[(int64_t)l * Q + k] * fast_exp(fminf(a_s[l] - a_s[k], 0.f)) * dt_s[k];
    };
    auto fb = [&](int r, int k) {  // (p, s)
      const int pp = pt * GB + r;
      return (pp < P && k < qlim) ? ldg<T>(p.x, xb + (int64_t)(t0 + k) * p.x_ls + pp) : 0.f;
    };
    block_gemm<SPLIT, true, false>(acc, lds, 0, kmax, fa, fb, tid);
  }
  const float *Dp = static_cast<const float *>(p.D);
  acc_foreach(acc, tid, [&](int m, int n, float v) {
    const int l = mt * GB + m, pp = pt * GB + n;
    if (l >= qlim || pp >= P) return v;
    float o = v;
    if (Dp) {
      const float d = p.D_has_hdim ? Dp[h * P + pp] : Dp[h];
      o = __builtin_fmaf(d, ldg<T>(p.x, xb + (int64_t)(t0 + l) * p.x_ls + pp), o);
    }
    const int64_t oi = b * p.out_bs + (int64_t)(t0 + l) * p.out_ls + h * p.out_hs + pp;
    if (p.z) {
      if (p.out_x) stg<T>(p.out_x, oi, o);
      const float z = ldg<T>(p.z, b * p.z_bs + (int64_t)(t0 + l) * p.z_ls + h * p.z_hs + pp);
      o *= z * sigmoid_f(z);
    }
    stg<T>(p.out, oi, o);
    return v;
  });
}

// ------------------------------------------------------------------ launch
int check(const SsdParams *p) {
  if (!p || !p->x || !p->dt || !p->A || !p->B || !p->C) return MAMBA_E_BADARG;
  if (p->batch <= 0 || p->seqlen <= 0 || p->nheads <= 0 || p->headdim <= 0 || p->dstate <= 0 || p->ngroups <= 0 ||
      p->chunk_size <= 0)
    return MAMBA_E_BADARG;
  if (p->nheads % p->ngroups != 0) return MAMBA_E_BADARG;
  if (p->nchunks != (p->seqlen + p->chunk_size - 1) / p->chunk_size) return MAMBA_E_BADARG;
  if (p->chunk_size > 256 || p->dstate > 256 || p->headdim > 256) return MAMBA_E_UNSUPPORTED;
  if ((int64_t)p->batch * p->nheads > 65535 || p->nchunks > 65535) return MAMBA_E_UNSUPPORTED;
  if (p->dtype != MAMBA_F32 && p->dtype != MAMBA_BF16 && p->dtype != MAMBA_F16) return MAMBA_E_BADARG;
  if (p->dt_dtype != MAMBA_F32 && p->dt_dtype != MAMBA_BF16 && p->dt_dtype != MAMBA_F16) return MAMBA_E_BADARG;
  return MAMBA_OK;
}
int launched() { return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH; }

#define SSD_DISPATCH(KERNEL, GRID)                                                                   \
  switch (p->dtype) {                                                                                \
    case MAMBA_BF16: hipLaunchKernelGGL((KERNEL<bf16_t, false>), GRID, dim3(256), 0, s, *p); break;  \
    case MAMBA_F16: hipLaunchKernelGGL((KERNEL<f16_t, true>), GRID, dim3(256), 0, s, *p); break;     \
    default: hipLaunchKernelGGL((KERNEL<float, true>), GRID, dim3(256), 0, s, *p); break;            \
  }

}  // namespace

static int ssd_chunk_cumsum_fwd_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check(p);
  if (rc) return rc;
  if (!p->dt_out || !p->dA_cumsum) return MAMBA_E_BADARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(p->nchunks, (p->nheads + CS_HT - 1) / CS_HT, p->batch);
  hipLaunchKernelGGL(chunk_cumsum_fwd_kernel, grid, dim3(256), 0, s, *p);
  return launched();
}

static int ssd_bmm_chunk_fwd_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check(p);
  if (rc) return rc;
  if (!p->CB) return MAMBA_E_BADARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int nt = (p->chunk_size + GB - 1) / GB;
  dim3 grid(nt * (nt + 1) / 2, p->nchunks, p->batch * p->ngroups);
  SSD_DISPATCH(bmm_chunk_fwd_kernel, grid)
  return launched();
}

static int ssd_chunk_state_fwd_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check(p);
  if (rc) return rc;
  if (!p->states || !p->dt_out || !p->dA_cumsum) return MAMBA_E_BADARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  {
    // whole 128-state blocks, 16-byte aligned x / B rows, headdim in whole groups of 8, whole k steps
    const bool wide = p->dstate % WB == 0 && p->headdim % 8 == 0 && whole_k_steps(p) &&
                      wide_operand_ok(p->x, p->dtype, p->x_bs, p->x_ls, p->x_hs) &&
                      wide_operand_ok(p->B, p->dtype, p->B_bs, p->B_ls, p->B_gs);
    if (wide) {
      dim3 grid(((p->headdim + GB - 1) / GB) * (p->dstate / WB), p->nchunks, p->batch * p->nheads);
      SSD_DISPATCH(chunk_state_fwd_wide_kernel, grid)
      return launched();
    }
  }
  dim3 grid(((p->headdim + GB - 1) / GB) * ((p->dstate + GB - 1) / GB), p->nchunks, p->batch * p->nheads);
  SSD_DISPATCH(chunk_state_fwd_kernel, grid)
  return launched();
}

extern "C" int ssd_chunk_state_varlen(const SsdParams *p, const int32_t *cu_seqlens, int nseq, float *varlen_states,
                                      mamba_stream_t stream) {
  int rc = check(p);
  if (rc) return rc;
  if (!p->dt_out || !p->dA_cumsum || !cu_seqlens || !varlen_states) return MAMBA_E_BADARG;
  if (!(p->dtype == MAMBA_BF16 ? p->states_lp : (void *)p->states)) return MAMBA_E_BADARG;  // the carried states
  if (p->batch != 1 || nseq < 0 || nseq > 65535) return MAMBA_E_BADARG;
  if (nseq == 0) return MAMBA_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(((p->headdim + GB - 1) / GB) * ((p->dstate + GB - 1) / GB), nseq, p->nheads);
  switch (p->dtype) {
    case MAMBA_BF16:
      hipLaunchKernelGGL((chunk_state_varlen_kernel<bf16_t, false>), grid, dim3(256), 0, s, *p, cu_seqlens, varlen_states);
      break;
    case MAMBA_F16:
      hipLaunchKernelGGL((chunk_state_varlen_kernel<f16_t, true>), grid, dim3(256), 0, s, *p, cu_seqlens, varlen_states);
      break;
    default:
      hipLaunchKernelGGL((chunk_state_varlen_kernel<float, true>), grid, dim3(256), 0, s, *p, cu_seqlens, varlen_states);
      break;
  }
  return launched();
}

static int ssd_state_passing_fwd_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check(p);
  if (rc) return rc;
  if (!p->states || !p->final_states || !p->dA_cumsum) return MAMBA_E_BADARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int PN = p->headdim * p->dstate;
  auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool lp = p->dtype == MAMBA_BF16;
  if (lp && !p->states_lp) return MAMBA_E_BADARG;
  const size_t tbytes = (size_t)p->nchunks * sizeof(float);
  const bool table = tbytes <= SP_TABLE_BYTES;
  if (PN % 4 == 0 && al16(p->states) && al16(p->final_states) && al16(p->initial_states) && al16(p->states_lp)) {
    dim3 grid((PN / 4 + 255) / 256, p->nheads, p->batch);
    if (table) {
      if (lp) hipLaunchKernelGGL((state_passing_fwd_kernel<4, bf16_t, true>), grid, dim3(256), tbytes, s, *p);
      else hipLaunchKernelGGL((state_passing_fwd_kernel<4, float, true>), grid, dim3(256), tbytes, s, *p);
    } else {
      if (lp) hipLaunchKernelGGL((state_passing_fwd_kernel<4, bf16_t, false>), grid, dim3(256), 0, s, *p);
      else hipLaunchKernelGGL((state_passing_fwd_kernel<4, float, false>), grid, dim3(256), 0, s, *p);
    }
  } else {
    dim3 grid((PN + 255) / 256, p->nheads, p->batch);
    if (lp) hipLaunchKernelGGL((state_passing_fwd_kernel<1, bf16_t, false>), grid, dim3(256), 0, s, *p);
    else hipLaunchKernelGGL((state_passing_fwd_kernel<1, float, false>), grid, dim3(256), 0, s, *p);
  }
  return launched();
}

static int ssd_chunk_scan_fwd_one(const SsdParams *p, mamba_stream_t stream) {
  int rc = check(p);
  if (rc) return rc;
  if (!p->CB || !p->out || !p->dt_out || !p->dA_cumsum) return MAMBA_E_BADARG;
  if (!(p->dtype == MAMBA_BF16 ? p->states_lp : (void *)p->states)) return MAMBA_E_BADARG;  // the carried states
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(((p->chunk_size + GB - 1) / GB) * ((p->headdim + GB - 1) / GB), p->nchunks, p->batch * p->nheads);
  SSD_DISPATCH(chunk_scan_fwd_kernel, grid)
  return launched();
}

// chunk_state + state_passing in one launch (chunk_state_passing_fwd_kernel): the shapes it is compiled for, whole
// chunks, 16-byte aligned operands.
static bool chunk_state_passing_shapes_ok(const SsdParams *p) {
  auto al16 = [](const void *q) { return q && (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  return p->dtype == MAMBA_BF16 && p->headdim == 64 && p->dstate == WB && (p->chunk_size == 256 || p->chunk_size == 128) &&
         p->seqlen % p->chunk_size == 0 && p->nchunks <= CSP_MAX_CHUNKS && p->nheads <= 65535 && p->batch <= 65535 &&
         al16(p->states_lp) && al16(p->final_states) && p->dt_out && p->dA_cumsum &&
         wide_operand_ok(p->x, p->dtype, p->x_bs, p->x_ls, p->x_hs) && wide_operand_ok(p->B, p->dtype, p->B_bs, p->B_ls, p->B_gs);
}
// The combined forward pass takes it where there are enough (batch, head) pairs for one workgroup each to keep the
// chip busy: a workgroup takes ~3.7 us per chunk of 256 whatever their number (its LDS traffic per k step is that of
// chunk_state_fwd_wide_kernel, and that is what bounds both), the two-kernel path ~24 ns per (batch, head, chunk).
// Measured at 80 heads x 4096 positions, walk / two kernels: batch 2 61 / 51 us, batch 3 65 / 95, batch 4 95 / 128
// (320 workgroups on 256 CUs: a quarter of the CUs do double duty), batch 8 169 / 252; one packed row of 64 heads x
// 32768 positions 436 / 195.
static bool chunk_state_passing_pays(const SsdParams *p) {
  return chunk_state_passing_shapes_ok(p) && (int64_t)p->batch * p->nheads >= cu_count() * 3 / 4;
}
extern "C" int ssd_chunk_state_passing_fwd(const SsdParams *p, mamba_stream_t stream) {
  int rc = check(p);
  if (rc) return rc;
  if (!chunk_state_passing_shapes_ok(p)) return MAMBA_E_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(p->nheads, p->batch);
  if (p->chunk_size == 256) {
    if (p->seq_idx) hipLaunchKernelGGL((chunk_state_passing_fwd_kernel<8, true>), grid, dim3(256), 0, s, *p);
    else hipLaunchKernelGGL((chunk_state_passing_fwd_kernel<8, false>), grid, dim3(256), 0, s, *p);
  } else {
    if (p->seq_idx) hipLaunchKernelGGL((chunk_state_passing_fwd_kernel<4, true>), grid, dim3(256), 0, s, *p);
    else hipLaunchKernelGGL((chunk_state_passing_fwd_kernel<4, false>), grid, dim3(256), 0, s, *p);
  }
  return launched();
}

static int ssd_combined_fwd_one(const SsdParams *p, mamba_stream_t stream) {
  int rc;
  if ((rc = ssd_chunk_cumsum_fwd(p, stream))) return rc;
  if (check(p) == MAMBA_OK && chunk_state_passing_pays(p)) {
    if ((rc = ssd_chunk_state_passing_fwd(p, stream))) return rc;
  } else {
    if ((rc = ssd_chunk_state_fwd(p, stream))) return rc;
    if ((rc = ssd_state_passing_fwd(p, stream))) return rc;
  }
  if (ssd_chunk_scan_fwd_fused_supported(p)) return ssd_chunk_scan_fwd_fused(p, stream);
  if ((rc = ssd_bmm_chunk_fwd(p, stream))) return rc;
  return ssd_chunk_scan_fwd(p, stream);
}

// Public entry points: the whole problem in one go when one launch can index it, else in slices of batch rows.
extern "C" int ssd_chunk_cumsum_fwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_chunk_cumsum_fwd_one); }
extern "C" int ssd_bmm_chunk_fwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_bmm_chunk_fwd_one); }
extern "C" int ssd_chunk_state_fwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_chunk_state_fwd_one); }
extern "C" int ssd_state_passing_fwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_state_passing_fwd_one); }
extern "C" int ssd_chunk_scan_fwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_chunk_scan_fwd_one); }
extern "C" int ssd_combined_fwd(const SsdParams *p, mamba_stream_t stream) { return ssd_sliced(p, stream, ssd_combined_fwd_one); }
