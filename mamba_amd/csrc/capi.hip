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
}  // namespace

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
    case MAMBA_Q_ABI_VERSION: return 12;
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
