// Pieces shared by the Mamba-1 scan kernels (mamba1_scan.hip, mamba1_scan_bwd_mx.hip): the tile constants,
// the staging of the B / C rows of a tile in LDS, row loads, and the channel geometry of a workgroup.
#pragma once
#include "common.hpp"

namespace {

constexpr int KI = 8;             // items per lane
constexpr int RL = 16;            // lanes per channel (one DPP row)
constexpr int ROWS = 4;           // channels per wave
constexpr int TILE = RL * KI;     // sequence positions per tile
constexpr int TILE_COMPLEX = 512; // tile of the complex kernels (mamba1_scan_complex.hip)
constexpr int NB16 = 16;          // states staged per LDS block
constexpr int NWAVES = 8;
constexpr int NTHREADS = NWAVES * 64;
constexpr int PASS_CH = NWAVES * ROWS;         // channels of a workgroup per pass
constexpr int BC_FLOATS = NB16 * TILE;         // one staged operand
constexpr int ACC_PITCH = TILE * ROWS;         // floats per state row of a dB / dC accumulator
constexpr int ACC_FLOATS = NB16 * ACC_PITCH;   // one accumulator: [n][half][lane][4]
constexpr int MAX_DSTATE = 256;
constexpr int MAX_PASSES = 8;

// B or C rows n0..n0+15 of the tile starting at t0 -> LDS as fp32, laid out [n][half][c][4] (c = the
// lane's place in its row) so that a lane reads its 8 items with two 16-byte LDS loads.
// BC: bit 0 set = B is not staged (input-independent), bit 1 = C likewise.
template <typename T, bool VEC, int BC>
DEVI void stage_bc(float *Bs, float *Cs, const T *Bg, int64_t B_ns, const T *Cg, int64_t C_ns, int n0, int N, int t0,
                   int L, int tid) {
  constexpr int FIRST = (BC & 1) ? NB16 * RL : 0, LAST = (BC & 2) ? NB16 * RL : 2 * NB16 * RL;
  if constexpr (BC == 3) {
    return;  // nothing is staged
  } else {
    const int unit = FIRST + tid;  // one 8-item unit per thread: 2 operands x 16 states x 16 segments
    if (unit >= LAST) return;
    const int which = unit >> 8, n = (unit >> 4) & 15, j = unit & 15;
    float v[8];
    if constexpr (VEC) {
      // from a clamped (valid) address, masked afterwards
      Pack8<T> raw;
      const int nc = min(n0 + n, N - 1), t = min(t0 + KI * j, L - KI);
      raw.load((which ? Cg + (int64_t)nc * C_ns : Bg + (int64_t)nc * B_ns) + t);
      raw.unpack(v);
      const bool ok = n0 + n < N && t0 + KI * j < L;
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = ok ? v[i] : 0.f;
    } else {
      const int t = t0 + KI * j;
      const T *src = (which ? Cg + (int64_t)(n0 + n) * C_ns : Bg + (int64_t)(n0 + n) * B_ns) + t;
      const int nvalid = (n0 + n < N) ? min(max(L - t, 0), KI) : 0;
      ld8_guard<T, false>(src, nvalid, 0.f, v);
    }
    float *dst = (which ? Cs : Bs) + n * TILE + j * 4;
    *reinterpret_cast<f32x4 *>(dst) = f32x4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4 *>(dst + 4 * RL) = f32x4{v[4], v[5], v[6], v[7]};
  }
}

// The 8 items of one (batch, channel) row owned by this lane, as stored: VEC reads 16 bytes from a
// clamped position (the caller masks lanes past the end), else element by element.
template <typename T, bool VEC> DEVI void load_items(Pack8<T> &k, const T *row, int tl, int L, int nvalid) {
  if constexpr (VEC) {
    k.load_global(row + min(tl, L - KI));
  } else {
    float v[8];
    ld8_guard<T, false>(row + tl, nvalid, 0.f, v);
    k.pack(v);
  }
}

// 8 floats of a [half][slot][4] LDS row: a slot's two 16-byte halves lie HALF_STRIDE floats apart
template <int HALF_STRIDE> DEVI void lds_st8(float *base, int slot, const float (&v)[8]) {
  *reinterpret_cast<f32x4 *>(base + slot * 4) = f32x4{v[0], v[1], v[2], v[3]};
  *reinterpret_cast<f32x4 *>(base + HALF_STRIDE + slot * 4) = f32x4{v[4], v[5], v[6], v[7]};
}
template <int HALF_STRIDE> DEVI void lds_ld8(const float *base, int slot, float (&o)[8]) {
  const f32x4 lo = *reinterpret_cast<const f32x4 *>(base + slot * 4);
  const f32x4 hi = *reinterpret_cast<const f32x4 *>(base + HALF_STRIDE + slot * 4);
  o[0] = lo.x; o[1] = lo.y; o[2] = lo.z; o[3] = lo.w;
  o[4] = hi.x; o[5] = hi.y; o[6] = hi.z; o[7] = hi.w;
}

// The 8 items of B (or C) for state n of channel d: from the staged tile, or, when the operand is an
// input-independent (dim, dstate) fp32 matrix, its one value for every position (0 for padded states).
template <int CONST>
DEVI void load_bc(float (&v)[8], const float *staged, const void *mat, int d, int N, int n_abs, int n_loc, int c) {
  if constexpr (CONST != 0) {
    const float x = n_abs < N ? static_cast<const float *>(mat)[(int64_t)d * N + n_abs] : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = x;
  } else {
    lds_ld8<4 * RL>(staged + n_loc * TILE, c, v);
  }
}

// Where a workgroup's channels lie: workgroup cb of group g takes `passes` passes of PASS_CH channels.
struct Geo {
  int g, cb, b, Dg, dend, ntiles, cblocks;
};
DEVI Geo geometry(const MambaScanParams &p, int passes) {
  Geo q;
  q.Dg = p.dim / p.ngroups;
  q.cblocks = (q.Dg + PASS_CH * passes - 1) / (PASS_CH * passes);
  q.g = blockIdx.x / q.cblocks;
  q.cb = blockIdx.x % q.cblocks;
  q.b = blockIdx.y;
  q.dend = (q.g + 1) * q.Dg;
  q.ntiles = (p.seqlen + TILE - 1) / TILE;
  return q;
}

// Row starts of one channel of the workgroup, kept in LDS: every (tile, pass) step needs nine
// addresses per lane, and as kernel arguments next to the loop state they did not fit the scalar
// registers (each step then re-read hundreds of spilled scalars through v_readlane).  Pointers read back
// from LDS carry no address space, so the rows are accessed through the helpers that name the global one.
template <typename T> struct BwdRow {
  const T *u, *delta, *dout, *z;
  T *du, *ddelta, *dz, *out_z;
  const float *ckpt;  // tile 0 of this channel
  float D, bias;
};

// 32 bytes per thread that nobody reads: a lane with nothing to store (past the end of the sequence, no z)
// stores there instead of branching around the store.  Shared by all workgroups.
static __device__ __align__(16) float bwd_spare[NTHREADS * 8];

}  // namespace
