// Library-level entry points of libmamba_gfx950.so: queries, error strings and
// a graph-capturable zero fill.
#include "common.hpp"

namespace {
__global__ __launch_bounds__(256) void zero_kernel(uint32_t *p, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = 0u;
}
__global__ __launch_bounds__(256) void copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src[i];
}
// Eight independent chains of v_mfma_f32_16x16x32_bf16 per wave on register operands: the rate the matrix
// cores sustain with nothing else in the way (no LDS, no memory), as a yardstick for the GEMM kernels.
typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(256) void mfma_probe_kernel(float *sink, int iters) {
  const int lane = threadIdx.x & 63;
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  const s16x8 ai = {(short)(0x3f80 + lane), 0x3f80, 0x3f00, 0x3e80, 0x3f80, 0x3f00, 0x3e80, 0x3f80};
  const s16x8 bi = {0x3f80, (short)(0x3f00 + lane), 0x3f80, 0x3e80, 0x3f00, 0x3f80, 0x3e80, 0x3f00};
  const probe_bf16x8 a = __builtin_bit_cast(probe_bf16x8, ai), b = __builtin_bit_cast(probe_bf16x8, bi);
  f32x4 acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) s += acc[j].x + acc[j].y + acc[j].z + acc[j].w;
  if (s == -1.f) sink[0] = s;  // never true: keeps the loop alive
}
// Sixteen independent chains of v_fma_f32 per lane on register operands: the rate at which the vector ALUs
// issue fp32 instructions with nothing else in the way, as a yardstick for the scan kernels.
__global__ __launch_bounds__(256) void valu_probe_kernel(float *sink, int iters) {
  float a[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) a[j] = 1.f + 0.001f * (float)((threadIdx.x + j) & 31);
  const float m = 0.99999f, c = 1e-6f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
      for (int j = 0; j < 16; ++j) a[j] = __builtin_fmaf(a[j], m, c);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) s += a[j];
  if (s == -1.f) sink[0] = s;  // never true: keeps the loop alive
}
// A bare pass over (batch, position, head, 64 values) 16-bit tensors in the order the SSD kernels visit them: one
// workgroup per (batch, 256 positions, head) reads the 128-byte rows of NI tensors and writes those of two, 32
// positions per step with two steps in flight, and the heads of a (batch, chunk) are neighbours in launch order on
// one XCD.  No arithmetic to speak of, no LDS, no barrier: its rate is what this layout allows a kernel that touches
// every row once (a row of one head is 128 bytes, the next position's row lies nheads * 128 bytes further).
struct RowsProbeArgs {
  const uint16_t *in[4];
  uint16_t *out[2];
  int nheads, nchunks;
};
template <int NI> __global__ __launch_bounds__(256) void rows_probe_kernel(const RowsProbeArgs a) {
  const int t = threadIdx.x;
  const int n = gridDim.x, k = blockIdx.x;
  const int lid = n % 8 == 0 ? (k % 8) * (n / 8) + k / 8 : k;
  const int h = lid % a.nheads, c = (lid / a.nheads) % a.nchunks, b = lid / (a.nheads * a.nchunks);
  const int64_t row = (int64_t)a.nheads * 64;
  const int64_t base = ((int64_t)b * a.nchunks + c) * 256 * row + h * 64 + (t & 7) * 8 + (int64_t)(t >> 3) * row;
  constexpr int PF = 2, STEPS = 8;
  u32x4 q[PF][NI];
#pragma unroll
  for (int s = 0; s < PF; ++s)
#pragma unroll
    for (int i = 0; i < NI; ++i) q[s][i] = *reinterpret_cast<const u32x4 *>(a.in[i] + base + (int64_t)s * 32 * row);
#pragma unroll
  for (int st = 0; st < STEPS; ++st) {
    const int s = st % PF;
    u32x4 x = q[s][0], y = q[s][NI - 1];
#pragma unroll
    for (int i = 1; i < NI - 1; ++i) {
      if (i & 1) x ^= q[s][i];
      else y += q[s][i];
    }
    if (st + PF < STEPS) {
#pragma unroll
      for (int i = 0; i < NI; ++i) q[s][i] = *reinterpret_cast<const u32x4 *>(a.in[i] + base + (int64_t)(st + PF) * 32 * row);
    }
    const int64_t o = base + (int64_t)st * 32 * row;
    *reinterpret_cast<u32x4 *>(a.out[0] + o) = x;
    *reinterpret_cast<u32x4 *>(a.out[1] + o) = y;
  }
}
}  // namespace

extern "C" int64_t mamba_hip_rows_probe(const void *const *in, int n_in, void *const *out, int batch, int seqlen,
                                        int nheads, mamba_stream_t stream) {
  if (!in || !out || (n_in != 2 && n_in != 4) || batch <= 0 || nheads <= 0 || seqlen <= 0 || seqlen % 256) return MAMBA_E_BADARG;
  RowsProbeArgs a;
  for (int i = 0; i < 4; ++i) {
    a.in[i] = static_cast<const uint16_t *>(in[i < n_in ? i : 0]);
    if (!a.in[i] || (reinterpret_cast<uintptr_t>(a.in[i]) & 15)) return MAMBA_E_BADARG;
  }
  for (int i = 0; i < 2; ++i) {
    a.out[i] = static_cast<uint16_t *>(out[i]);
    if (!a.out[i] || (reinterpret_cast<uintptr_t>(a.out[i]) & 15)) return MAMBA_E_BADARG;
  }
  a.nheads = nheads, a.nchunks = seqlen / 256;
  const int64_t wgs = (int64_t)batch * a.nchunks * nheads;
  if (wgs > 0x7fffffff) return MAMBA_E_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (n_in == 4)
    hipLaunchKernelGGL(rows_probe_kernel<4>, dim3((unsigned)wgs), dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL(rows_probe_kernel<2>, dim3((unsigned)wgs), dim3(256), 0, s, a);
  if (hipGetLastError() != hipSuccess) return MAMBA_E_LAUNCH;
  return (int64_t)(n_in + 2) * batch * seqlen * nheads * 64 * 2;  // bytes this launch reads and writes
}

extern "C" int64_t mamba_hip_valu_probe(float *sink, int iters, int blocks, mamba_stream_t stream) {
  if (!sink || iters <= 0 || blocks <= 0) return MAMBA_E_BADARG;
  hipLaunchKernelGGL(valu_probe_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), sink, iters);
  if (hipGetLastError() != hipSuccess) return MAMBA_E_LAUNCH;
  return (int64_t)blocks * 256 * iters * 64;  // per-lane fma instructions of this launch
}

extern "C" int64_t mamba_hip_mfma_probe(float *sink, int iters, int blocks, mamba_stream_t stream) {
  if (!sink || iters <= 0 || blocks <= 0) return MAMBA_E_BADARG;
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), sink, iters);
  if (hipGetLastError() != hipSuccess) return MAMBA_E_LAUNCH;
  return (int64_t)blocks * 4 * iters * 8 * (2LL * 16 * 16 * 32);  // flops of this launch
}

extern "C" int mamba_hip_copy(void *dst, const void *src, int64_t nbytes, mamba_stream_t stream) {
  if (nbytes == 0) return MAMBA_OK;
  if (!dst || !src || nbytes < 0 || (nbytes & 15) || (reinterpret_cast<uintptr_t>(dst) & 15) ||
      (reinterpret_cast<uintptr_t>(src) & 15))
    return MAMBA_E_BADARG;
  const int64_t n = nbytes / 16;
  if ((n + 255) / 256 > 0x7fffffff) return MAMBA_E_UNSUPPORTED;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), n);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}

int mamba1_scan_tile(bool a_complex);  // mamba1_scan.hip

extern "C" int mamba_hip_query(int what) {
  switch (what) {
    case MAMBA_Q_ABI_VERSION: return 14;
    case MAMBA_Q_SCAN_TILE: return mamba1_scan_tile(false);
    case MAMBA_Q_SCAN_TILE_COMPLEX: return mamba1_scan_tile(true);
    case MAMBA_Q_MAX_DSTATE: return 256;
    case MAMBA_Q_SSD_MAX_DSTATE: return 256;
    case MAMBA_Q_SSD_MAX_HEADDIM: return 256;
    default: return MAMBA_E_BADARG;
  }
}

extern "C" const char *mamba_hip_strerror(int code) {
  switch (code) {
    case MAMBA_OK: return "success";
    case MAMBA_E_BADARG: return "bad argument (null pointer or inconsistent sizes)";
    case MAMBA_E_UNSUPPORTED: return "unsupported shape or dtype for this build";
    case MAMBA_E_LAUNCH: return "kernel launch failed";
    default: return "unknown error code";
  }
}

extern "C" int mamba_hip_zero(void *ptr, int64_t nbytes, mamba_stream_t stream) {
  if (nbytes == 0) return MAMBA_OK;
  if (!ptr || nbytes < 0 || (nbytes & 3) || (reinterpret_cast<uintptr_t>(ptr) & 3)) return MAMBA_E_BADARG;
  const int64_t n = nbytes / 4;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(zero_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<uint32_t *>(ptr), n);
  return hipGetLastError() == hipSuccess ? MAMBA_OK : MAMBA_E_LAUNCH;
}
