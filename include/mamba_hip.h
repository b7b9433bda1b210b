/*
 * C ABI of libmamba_gfx950.so: hand-written HIP kernels (gfx950 / CDNA4) for
 * Mamba's scan hot path.  Plain pointers and sizes only; no torch types.
 *
 * Conventions
 *  - every pointer is a device pointer unless stated otherwise;
 *  - the caller owns and allocates every buffer (outputs and workspaces);
 *    the library never allocates or frees device memory;
 *  - strides are in ELEMENTS of the tensor's dtype; the sequence (or the
 *    innermost) dimension must have stride 1 where stated;
 *  - kernels are launched on `stream` and never synchronise with the host;
 *  - return value: 0 on success, a negative MAMBA_E_* code otherwise
 *    (mamba_hip_strerror() gives the text).  Nothing throws.
 */
#ifndef MAMBA_HIP_H_
#define MAMBA_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *mamba_stream_t; /* hipStream_t */

enum {
  MAMBA_OK = 0,
  MAMBA_E_BADARG = -1,      /* null pointer / inconsistent sizes */
  MAMBA_E_UNSUPPORTED = -2, /* valid request this build has no kernel for */
  MAMBA_E_LAUNCH = -3       /* hipGetLastError() != hipSuccess after launch */
};

enum { MAMBA_F32 = 0, MAMBA_BF16 = 1, MAMBA_F16 = 2 };

/* mamba_hip_query(what) */
enum {
  MAMBA_Q_ABI_VERSION = 0,
  MAMBA_Q_SCAN_TILE = 1,      /* sequence positions per checkpoint tile of the Mamba-1 scan */
  MAMBA_Q_MAX_DSTATE = 2,     /* largest d_state the Mamba-1 scan accepts */
  MAMBA_Q_SSD_MAX_DSTATE = 3, /* largest d_state of the SSD kernels */
  MAMBA_Q_SSD_MAX_HEADDIM = 4,
  MAMBA_Q_SCAN_TILE_COMPLEX = 5 /* the same for a complex A */
};

int mamba_hip_query(int what);
const char *mamba_hip_strerror(int code);

/* Fills `nbytes` (multiple of 4) of device memory with zero using a kernel, so
 * that it can be recorded into a HIP graph. */
int mamba_hip_zero(void *ptr, int64_t nbytes, mamba_stream_t stream);

/* Plain device-to-device copy of `nbytes` (multiple of 16, 16-byte aligned pointers), one 16-byte
 * element per thread.  It is the streaming yardstick the profiles are calibrated against: its HBM
 * traffic is exactly 2 * nbytes. */
int mamba_hip_copy(void *dst, const void *src, int64_t nbytes, mamba_stream_t stream);

/* Measurement yardstick for the GEMM kernels: launches `blocks` workgroups of 4 waves, each wave running
 * `iters` rounds of eight independent v_mfma_f32_16x16x32_bf16 on register operands (no LDS, no memory).
 * Returns the floating-point operations of the launch (> 0), or an error code (< 0).  `sink` is one float
 * of device memory that is never written. */
int64_t mamba_hip_mfma_probe(float *sink, int iters, int blocks, mamba_stream_t stream);

/* Measurement yardstick for the SSD kernels, whose operands are (batch, seqlen, nheads, 64) 16-bit tensors of which a
 * workgroup visits one head's 128-byte rows: a bare pass in that order, one workgroup per (batch, 256 positions,
 * head), which reads every row of `n_in` (2 or 4) such tensors and writes every row of the two tensors `out`
 * (xor / sum of the inputs; no LDS, no barrier, two steps of 32 positions in flight).  Its rate is what the layout
 * allows a kernel that touches each row once.  seqlen must be a multiple of 256, all pointers 16-byte aligned.
 * Returns the bytes the launch reads and writes (> 0), or an error code (< 0).  No counterpart in the reference. */
int64_t mamba_hip_rows_probe(const void *const *in, int n_in, void *const *out, int batch, int seqlen, int nheads,
                             mamba_stream_t stream);

/* Measurement yardstick for the scan kernels, whose time is fp32 vector-ALU issue: launches `blocks` workgroups of
 * 4 waves, each lane running `iters` rounds of 64 v_fma_f32 in sixteen independent chains on register operands.
 * Returns the per-lane instructions of the launch (> 0), or an error code (< 0).  `sink` as above. */
int64_t mamba_hip_valu_probe(float *sink, int iters, int blocks, mamba_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Mamba-1 selective scan.
 * Replaces selective_scan_cuda.fwd / .bwd
 * (reference csrc/selective_scan/selective_scan.cpp:226 and :338, params
 * struct csrc/selective_scan/selective_scan.h:7 and :52).
 *
 *   delta' = softplus(delta + delta_bias)            (each part optional)
 *   h[t,n] = exp(delta'[t] A[d,n]) h[t-1,n] + delta'[t] B[t,n] u[t]
 *   y[t]   = sum_n C[t,n] h[t,n] + D[d] u[t]
 *   out[t] = y[t] * silu(z[t])   (when z != NULL, else y[t])
 *
 * u, delta, z, out (and dout, du, ddelta, dz, out_z) are (batch, dim, seqlen)
 * of `dtype`, seqlen stride 1.  B, C are (batch, ngroups, dstate, seqlen) of
 * `dtype`, seqlen stride 1; channel d uses group d / (dim / ngroups).
 * A is (dim, dstate) fp32 contiguous; D, delta_bias are (dim) fp32 or NULL.
 * With bc_const bit 0 (bit 1) set, B (C) is instead a contiguous (dim, dstate) fp32
 * matrix used at every position (the reference's is_variable_B / is_variable_C false,
 * csrc/selective_scan/selective_scan.cpp:254-255); its strides are ignored and
 * ngroups describes the other operand (1 when both are matrices).
 *
 * With a_complex set (the reference's complex64 A, selective_scan.cpp:236,:312) the state is
 * complex: A is (dim, dstate, 2) fp32 (re, im); per-position B, C are (batch, ngroups, dstate,
 * 2 * seqlen) of `dtype` with (re, im) pairs interleaved along the last axis; input-independent
 * B, C are (dim, dstate, 2) fp32; out = 2 Re <h, C> (+ D u, gate); ckpt gains a trailing
 * dimension of 2, and so do dA_part and the dB32 / dC32 of input-independent operands, while the
 * dB32 / dC32 of per-position operands are (batch, ngroups, dstate, 2 * seqlen).
 *
 * ckpt is (batch, dim, ntiles, dstate) fp32 contiguous with
 * ntiles = ceil(seqlen / MAMBA_Q_SCAN_TILE) (MAMBA_Q_SCAN_TILE_COMPLEX with a complex A): the
 * state h after the last position of each tile.  ckpt[:, :, ntiles-1, :] is the final state.  The
 * backward pass re-computes the states inside a tile from ckpt.
 *
 * Backward: no float atomics are used for a real A, so every gradient repeats bit for bit from run to
 * run (the reference's deterministic mode, mamba_ssm/utils/determinism.py:21-27, is the only mode); with a
 * complex A the det_* fields at the end of the struct select it.
 * ------------------------------------------------------------------------- */
typedef struct MambaScanParams {
  int32_t batch, dim, seqlen, dstate, ngroups;
  int32_t dtype; /* MAMBA_F32 / MAMBA_BF16 / MAMBA_F16 */
  int32_t delta_softplus;
  int32_t bc_const; /* bit 0: B is an input-independent (dim, dstate) fp32 matrix; bit 1: C likewise */
  int32_t a_complex; /* 1: complex A (see above) */
  int32_t reserved0;

  const void *u, *delta, *A, *B, *C;
  const void *D, *z, *delta_bias; /* nullable */
  void *out;                      /* forward only */
  float *ckpt;                    /* forward: written; backward: read */

  int64_t u_bs, u_ds;         /* batch / dim stride */
  int64_t delta_bs, delta_ds;
  int64_t z_bs, z_ds;
  int64_t out_bs, out_ds;
  int64_t B_bs, B_gs, B_ns; /* batch / group / state stride */
  int64_t C_bs, C_gs, C_ns;

  /* ---- backward only (ignored by mamba1_scan_fwd) ---- */
  const void *dout;
  void *du, *ddelta;
  void *dz;    /* required iff z != NULL; may be a strided view */
  void *out_z; /* nullable: when set (and z != NULL) the gated output is re-computed into it */
  /* fp32 workspaces, contents ignored on entry.  dB32, dC32: (batch, ngroups, nparts, dstate, seqlen)
   * contiguous and 16-byte aligned, nparts = mamba1_scan_bwd_nparts(p): one partial sum per workgroup,
   * which the call then adds up in a fixed order into dB / dC below (with a complex A: nparts = 1 and
   * a last axis of 2 * seqlen).  dA_part: (batch, dim, dstate), dD_part, ddelta_bias_part:
   * (batch, dim) -- written, the caller sums them over batch.  For an input-independent B (C),
   * dB32 (dC32) is instead (batch, dim, dstate) partials, written like dA_part, and dB (dC) is unused. */
  float *dB32, *dC32, *dA_part, *dD_part, *ddelta_bias_part;
  int64_t dout_bs, dout_ds;
  int64_t du_bs, du_ds;
  int64_t ddelta_bs, ddelta_ds;
  int64_t dz_bs, dz_ds;
  int64_t outz_bs, outz_ds;
  /* gradients of per-position B and C: (batch, ngroups, dstate, seqlen) of `dtype`, contiguous
   * ((..., 2 * seqlen) with a complex A) */
  void *dB, *dC;
  /* ---- deterministic backward with a complex A (all null: float atomics there; a real A needs none of this, its
   * backward pass has no atomics) ----
   * The complex kernels add every channel's dB / dC terms into one sum per (batch, group, state, position).  With
   * det_scale set (device, {s, 1 / s}, s a power of two chosen by the caller as for SsdParams.det_scale) every term
   * is multiplied by s, rounded to an integer and added with a 64-bit integer atomic into det_dB / det_dC, int64
   * shadows of dB32 / dC32 (same shape, zero on entry; used for per-position operands only); the call converts them
   * into dB32 / dC32 before it forms dB / dC.  Counterpart of the reference's deterministic mode,
   * mamba_ssm/utils/determinism.py:21-27. */
  const float *det_scale;
  int64_t *det_dB, *det_dC;
} MambaScanParams;

int mamba1_scan_fwd(const MambaScanParams *p, mamba_stream_t stream);
int mamba1_scan_bwd(const MambaScanParams *p, mamba_stream_t stream);
/* Number of per-workgroup partials the backward call writes into dB32 / dC32 for these sizes on the
 * current device (> 0), or an error code.  Uses batch, dim, seqlen, dstate, ngroups, bc_const, a_complex. */
int mamba1_scan_bwd_nparts(const MambaScanParams *p);

/* No counterpart in the reference.  For callers that cannot allocate device memory -- code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc: mamba1_scan_fwd with the tile
 * checkpoints kept in a fixed buffer inside the library (MAMBA_NOALLOC_SCRATCH_BYTES per GPU, held until
 * the process ends) instead of a caller workspace.  p->ckpt is ignored; `last_state`
 * (nullable) is (batch, dim, dstate) fp32 contiguous ((batch, dim, dstate, 2) with a complex A) and
 * receives the state after the last position.  Allocates and frees nothing.  Requests whose checkpoints
 * batch * dim * ceil(seqlen / tile) * dstate (* 2 if complex) * 4 bytes exceed the buffer
 * return MAMBA_E_UNSUPPORTED.  Every call on a GPU uses that GPU's one buffer: calls that overlap on one
 * GPU (two streams, two threads) race and must be serialised by the caller.  The buffer's address is
 * looked up on the first call on a device; mamba_hip_init() does that ahead of time for the current
 * device (call it before capturing a graph). */
#define MAMBA_NOALLOC_SCRATCH_BYTES (32 << 20)
int mamba_hip_init(void);
int mamba1_scan_fwd_noalloc(const MambaScanParams *p, float *last_state, mamba_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Single-token decode: one step of the recurrence, in place on `state`.
 * Replaces the Triton kernel behind selective_state_update
 * (reference mamba_ssm/ops/triton/selective_state_update.py:24 kernel, :135
 * host function):
 *   dt' = softplus(dt + dt_bias)                (each part optional)
 *   state[b,h,p,n] = state * exp(A[h,p,n] dt'[b,h,p]) + B[b,g,n] dt' x[b,h,p]
 *   out[b,h,p] = sum_n state[b,h,p,n] C[b,g,n] + D[h,p] x[b,h,p];  out *= silu(z)
 * Every tensor is addressed through element strides, so stride-0 (expanded)
 * dt / A / dt_bias / D are accepted as they are.  Each operand has its own
 * dtype code (MAMBA_F32/BF16/F16); the arithmetic is fp32.
 * `state` has state_rows rows (>= batch when state_batch_indices is null: entry b uses row b).
 * state_batch_indices (int32, nullable): row of `state` used by batch entry b;
 * an index outside [0, state_rows) is a padding entry: its state is untouched and out = 0.
 * ------------------------------------------------------------------------- */
typedef struct MambaStepParams {
  int32_t batch, nheads, dim, dstate, ngroups;
  int32_t dt_softplus;
  int32_t state_dtype, x_dtype /* x, z, out */, dt_dtype, dt_bias_dtype, A_dtype, bc_dtype /* B, C */, D_dtype;
  int32_t state_rows; /* rows of `state` (its leading extent) */
  void *state;
  const void *x, *dt, *A, *B, *C;
  const void *D, *z, *dt_bias; /* nullable */
  void *out;
  const int32_t *state_batch_indices; /* nullable */
  int64_t state_bs, state_hs, state_ps, state_ns;
  int64_t x_bs, x_hs, x_ps;
  int64_t dt_bs, dt_hs, dt_ps;
  int64_t dt_bias_hs, dt_bias_ps;
  int64_t A_hs, A_ps, A_ns;
  int64_t B_bs, B_gs, B_ns;
  int64_t C_bs, C_gs, C_ns;
  int64_t D_hs, D_ps;
  int64_t z_bs, z_hs, z_ps;
  int64_t out_bs, out_hs, out_ps;
} MambaStepParams;

int ssm_state_update(const MambaStepParams *p, mamba_stream_t stream);

/* ------------------------------------------------------------------------- *
 * One generated token of a Mamba-2 mixer in ONE launch: the decode step of the depthwise convolution
 * over the x / B / C channels followed by the state update, i.e. the pair of calls
 *   xBC = causal_conv1d_update(xBC, conv_state, conv_weight, conv_bias, activation)
 *   y   = selective_state_update(ssm_state, x, dt, A, B, C, D, z, dt_bias, dt_softplus=True)
 * of the reference's step() (mamba_ssm/modules/mamba2.py:298-336).  At generation batches of 1-8 the two
 * kernels are launch-bound; fused, the step is one kernel that reads each state once.
 *   xBC        : (batch, conv_dim) of ssm.x_dtype, channels contiguous, conv_dim = nheads * dim + 2 * ngroups * dstate,
 *                laid out [x (nheads * dim) | B (ngroups * dstate) | C (ngroups * dstate)]
 *   conv_state : (conv_state_rows >= batch, conv_dim, state_len) of ssm.x_dtype through element strides, updated in place
 *                to the last state_len positions of [conv_state, xBC]; width - 1 <= state_len <= 4
 *   conv_weight: (conv_dim, width) of conv_weight_dtype, contiguous; conv_bias: (conv_dim) of the same dtype, nullable;
 *                width 2..4
 *   sync       : int32 (mamba2_decode_step_sync_ints(p)), all zero on entry and again on return (the workgroups of a
 *                (batch entry, group) count themselves off here; the last one shifts the conv state of the group's
 *                shared B / C channels once every other one has read it).  Calls that share `sync` must not overlap.
 * `ssm` describes the state update as for ssm_state_update; its x, B, C pointers and strides are ignored (the
 * convolution's outputs take their place), dt / A / dt_bias / D must be per head (stride 0 along dim and dstate:
 * the tie_hdim form of the reference's step), bc_dtype = x_dtype, and state_batch_indices must be null.
 * Returns MAMBA_E_UNSUPPORTED for anything outside this form (the caller then makes the two calls).
 * ------------------------------------------------------------------------- */
typedef struct MambaDecodeStepParams {
  MambaStepParams ssm;
  int32_t conv_dim, width, state_len, silu;
  int32_t conv_state_rows;
  int32_t conv_weight_dtype; /* dtype code of conv_weight and conv_bias (MAMBA_F32 = 0 / MAMBA_BF16 / MAMBA_F16) */
  const void *xBC;
  void *conv_state;
  const void *conv_weight;
  const void *conv_bias; /* nullable */
  int32_t *sync;
  int64_t xBC_bs;
  int64_t cs_bs, cs_cs, cs_ls; /* conv_state strides: row, channel, position */
} MambaDecodeStepParams;

int64_t mamba2_decode_step_sync_ints(const MambaDecodeStepParams *p); /* needs ssm.batch, nheads, ngroups, dim, dstate */
int mamba2_decode_step(const MambaDecodeStepParams *p, mamba_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Mamba-2 SSD (chunked state-space-dual scan).
 * Replaces the Triton kernels launched by _mamba_chunk_scan_combined_fwd / _bwd
 * (reference mamba_ssm/ops/triton/ssd_combined.py:343 and :397), i.e.
 * ssd_chunk_state.py (_chunk_cumsum_fwd :718, _chunk_state_fwd :812, ...),
 * ssd_state_passing.py (:196, :227), ssd_bmm.py (:165, :213) and
 * ssd_chunk_scan.py (:1259 ...).
 *
 * Shapes (b batch, L seqlen, H nheads, P headdim, G ngroups, N dstate,
 * Q chunk_size, c = nchunks = ceil(L / Q)):
 *   x, z, out, out_x, dout, dx, dz : (b, L, H, P) of `dtype`, P stride 1
 *   B, C, dB, dC                   : (b, L, G, N) of `dtype`, N stride 1
 *   dt, ddt                        : (b, L, H) of `dt_dtype`
 *   A, dt_bias                     : (H) fp32;  D: (H) or (H, P) fp32 (D_has_hdim)
 *   seq_idx                        : (b, L) int32, contiguous, nullable
 *   initial_states                 : (b, H, P, N) fp32 contiguous, nullable
 * fp32 workspaces, contiguous:
 *   dt_out, dA_cumsum              : (b, H, c, Q)
 *   states                         : (b, c, H, P, N)  chunk-local states after
 *                                    ssd_chunk_state_fwd; state ENTERING each
 *                                    chunk after ssd_state_passing_fwd (in place)
 *   final_states                   : (b, H, P, N)
 *   CB                             : (b, c, G, Q, Q)  only entries s <= l of
 *                                    row l / column s are defined
 * ------------------------------------------------------------------------- */
typedef struct SsdParams {
  int32_t batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks;
  int32_t dtype, dt_dtype;
  int32_t dt_softplus, D_has_hdim;
  float dt_min, dt_max;

  const void *x, *dt, *A, *B, *C;
  const void *D, *z, *dt_bias;          /* nullable */
  const float *initial_states;          /* nullable */
  const int32_t *seq_idx;               /* nullable */
  void *out;
  void *out_x;                          /* pre-gate output, written iff z != NULL; nullable (forward only: the backward pass reads it) */
  float *dt_out, *dA_cumsum, *states, *final_states, *CB;

  int64_t x_bs, x_ls, x_hs;
  int64_t z_bs, z_ls, z_hs;
  int64_t out_bs, out_ls, out_hs;       /* out and out_x share strides */
  int64_t B_bs, B_ls, B_gs;
  int64_t C_bs, C_ls, C_gs;
  int64_t dt_bs, dt_ls, dt_hs;

  /* ---- backward only ---- */
  const void *dout;
  const float *dfinal_states;           /* nullable, (b, H, P, N) */
  void *dx, *dz;                        /* `dtype`, (b, L, H, P): dz contiguous, dx with the strides below */
  void *ddt;                            /* `dt_dtype`, contiguous (b, L, H) */
  void *dB, *dC;                        /* `dtype`, contiguous (b, L, G, N); nullable: when set, ssd_combined_bwd leaves the
                                           finished sums of dB32 / dC32 here in the operands' dtype (its last stage writes
                                           them, so no conversion pass over the fp32 sums is needed) */
  float *dA, *ddt_bias;                 /* (H) fp32, zero on entry */
  float *dD;                            /* (H) or (H, P) fp32, zero on entry */
  float *dinitial_states;               /* nullable, (b, H, P, N) fp32 */
  /* fp32 workspaces: */
  float *dstates;                       /* (b, c, H, P, N) */
  float *ddA_cumsum;                    /* (b, H, c, Q), zero on entry */
  float *ddt_out;                       /* (b, H, c, Q), zero on entry */
  float *dCB;                           /* (b, c, G, Q, Q), zero on entry unless ssd_bwd_overwrites() has
                                           SSD_OVERWRITES_DCB (one workgroup then owns each tile and stores it).  A
                                           workspace: after ssd_bwd_dcb it holds fp32 tiles; what ssd_combined_bwd
                                           leaves in it is unspecified (bf16 tiles where it hands them on as such) */
  float *dB32, *dC32;                   /* (b, L, G, N), zero on entry unless ssd_bwd_overwrites() has
                                           SSD_OVERWRITES_DBC (the first stage that touches them then stores them).  With
                                           dB / dC set the finished sums are only in dB / dC */
  void *gbuf;                           /* (b, L, H, P) of `dtype`: dout * silu(z); used iff z != NULL */
  int64_t dout_bs, dout_ls, dout_hs;
  int64_t dx_bs, dx_ls, dx_hs;          /* dx may be a slice of a wider buffer; unit headdim stride */
  /* ---- deterministic backward (all null: float atomics, whose order changes the last bits from run to run) ----
   * det_scale: device, {s, 1 / s} with s a power of two chosen by the caller from the size of the upstream gradients
   * (2^30 / 2^floor(log2(max |dout|)) keeps ~9 decimal digits below that maximum and 9 above it).  Every term of a
   * sum that several workgroups share is multiplied by s, rounded to an integer and added with a 64-bit integer
   * atomic into the sum's shadow; integer adds are associative, so the sum does not depend on their order.  The
   * shadows have the shapes of dD, ddA_cumsum, ddt_out, dCB, dB32, dC32, dA, ddt_bias and are zero on entry;
   * ssd_combined_bwd converts each into its float buffer (ssd_det_convert) before that buffer's first reader runs.
   * Counterpart of the reference's deterministic mode, mamba_ssm/utils/determinism.py:21-27. */
  const float *det_scale;
  int64_t *det_dD, *det_ddA_cumsum, *det_ddt_out, *det_dCB, *det_dB, *det_dC, *det_dA, *det_ddt_bias;
  /* With dtype MAMBA_BF16 the states carried between chunks and their gradients pass between the kernels in bf16
   * (the matrix products take only the bf16 part of them anyway; the reference hands them on in the operands' dtype
   * too, ssd_combined.py:384-386 out_dtype=C.dtype and :455-466 dstates_dtype=x.dtype), both (b, c, H, P, N):
   *   states_lp   written by ssd_state_passing_fwd (`states` then keeps the chunks' own states and is not needed
   *               afterwards) or by ssd_chunk_state_passing_fwd (`states` is then not written at all), read by the scan, ssd_chunk_state_varlen, ssd_state_passing_bwd and ssd_bwd_dBC_state;
   *   dstates_lp  takes the place of `dstates` in every backward stage.
   * Required (non-NULL) for MAMBA_BF16, ignored for the other dtypes, which keep the fp32 `states` (in place) and
   * `dstates`. */
  void *states_lp, *dstates_lp;
} SsdParams;

/* forward stages, in launch order */
int ssd_chunk_cumsum_fwd(const SsdParams *p, mamba_stream_t stream);
int ssd_chunk_state_fwd(const SsdParams *p, mamba_stream_t stream);
int ssd_state_passing_fwd(const SsdParams *p, mamba_stream_t stream);
int ssd_bmm_chunk_fwd(const SsdParams *p, mamba_stream_t stream);
int ssd_chunk_scan_fwd(const SsdParams *p, mamba_stream_t stream);
/* chunk_scan with the C B^T contraction fused in (CB is neither read nor written): bf16,
 * headdim 32/64, dstate 64/128, chunk_size 64/128/256, 16-byte aligned rows.
 * ssd_chunk_scan_fwd_fused_supported returns 1 when it applies. */
int ssd_chunk_scan_fwd_fused_supported(const SsdParams *p);
int ssd_chunk_scan_fwd_fused(const SsdParams *p, mamba_stream_t stream);
/* ssd_chunk_state_fwd and ssd_state_passing_fwd in one launch, for MAMBA_BF16 with headdim 64, dstate 128,
 * chunk_size 128 / 256, seqlen a multiple of chunk_size and 16-byte aligned x / B rows; MAMBA_E_UNSUPPORTED otherwise.
 * One workgroup per (batch, head) walks the sequence: writes states_lp (the state entering each chunk) and
 * final_states, reads dt_out / dA_cumsum, initial_states, seq_idx; `states` is not touched.  Replaces the pair
 * _chunk_state_fwd + _state_passing_fwd of mamba_ssm/ops/triton/ssd_combined.py:375-382. */
int ssd_chunk_state_passing_fwd(const SsdParams *p, mamba_stream_t stream);
/* cumsum; chunk_state + state_passing (in one launch, ssd_chunk_state_passing_fwd, where it applies and batch x heads
 * is at least three quarters of the compute units); then the fused scan when supported, else bmm + chunk_scan */
int ssd_combined_fwd(const SsdParams *p, mamba_stream_t stream);
/* Packed batch (p->batch == 1): the state after the last position of each of the nseq sequences
 * [cu_seqlens[i], cu_seqlens[i+1]) into varlen_states (nseq, H, P, N) fp32.  Needs dt_out,
 * dA_cumsum and states (entering each chunk) of a forward pass whose seq_idx matches cu_seqlens.
 * Replaces chunk_state_varlen, mamba_ssm/ops/triton/ssd_chunk_state.py:1018. */
int ssd_chunk_state_varlen(const SsdParams *p, const int32_t *cu_seqlens, int nseq, float *varlen_states,
                           mamba_stream_t stream);

/* Backward.  Inputs: the forward inputs, dout, dfinal_states, the saved pre-gate
 * output in out_x (z != NULL) or out (z == NULL), and the forward workspaces
 * dt_out, dA_cumsum, CB, states re-computed by the forward stages 1-4.
 * ssd_combined_bwd runs, in order:
 *   ssd_bwd_dz        dz, gbuf = dout silu(z), dD
 *   ssd_bwd_dstates   dstates[c] = direct gradient of the state entering chunk c
 *                     (for bf16 with a gate, 128 states and 16-byte aligned rows ssd_combined_bwd runs these two
 *                     stages as one kernel: the pass that makes gbuf feeds the product; same outputs)
 *   ssd_state_passing_bwd  reverse recurrence over chunks (in place on dstates -> gradient
 *                     of the chunk-local states), dinitial_states, ddA_cumsum at chunk ends
 *   ssd_bwd_dBC_state state-path parts of dB32 / dC32
 *   ssd_bwd_dx        dx, ddt_out (direct part) and the matching ddA_cumsum terms.  For bf16 with headdim
 *                     32 / 64, dstate 64 / 128, chunk 64 / 128 / 256 and 16-byte aligned rows it forms C B^T
 *                     itself from B and C (CB is not read); every other problem reads CB
 *   ssd_bwd_dcb       dCB
 *   ssd_bmm_chunk_bwd dB32 / dC32 += dCB contractions
 *   ssd_chunk_cumsum_bwd  ddt, dA, ddt_bias from ddA_cumsum and ddt_out
 *                     (ssd_combined_bwd deals the workgroups of these last two stages to one launch where the bmm
 *                     stage runs on its 64 x 128 tiles: they read disjoint results of the stages before them)
 * ddA_cumsum holds the gradient with respect to the cumulative sums a_l; the last
 * stage turns it into the gradient of the per-position dt * A. */
int ssd_bwd_dz(const SsdParams *p, mamba_stream_t stream);
/* What the caller may leave out for the backward pass of this (completely filled, CB apart) problem: which of the sum
 * buffers the kernels write whole instead of adding into, so that they may be handed over uncleared, and whether CB
 * is needed at all: a set of the flags below; 0 in the deterministic mode, for a problem run in batch slices, or for
 * a bad argument.  Clearing a buffer that is reported here is harmless.  No
 * counterpart in the reference, whose Triton kernels write partial sums to fresh buffers and add them up with
 * torch (mamba_ssm/ops/triton/ssd_combined.py:441-509). */
#define SSD_OVERWRITES_DCB 1 /* dCB: at most 16 heads per group */
#define SSD_OVERWRITES_DBC 2 /* dB32 and dC32: one workgroup of the state-path stage holds all heads of a group */
#define SSD_BWD_FORMS_CB 4   /* not about clearing: the backward pass does not need CB from the caller (who may skip
                                ssd_bmm_chunk_fwd and pass CB = NULL): the dCB stage forms its tiles of C B^T itself and
                                the dx stage runs its fused kernel.  Passing CB anyway is always correct. */
int ssd_bwd_overwrites(const SsdParams *p);
/* dst[i] = shadow[i] / s for i < n (det_scale = {s, 1 / s} on the device): the step between the stages of a
 * deterministic backward pass that ssd_combined_bwd inserts by itself */
int ssd_det_convert(const int64_t *shadow, float *dst, int64_t n, const float *det_scale, mamba_stream_t stream);
int ssd_bwd_dstates(const SsdParams *p, mamba_stream_t stream);
int ssd_state_passing_bwd(const SsdParams *p, mamba_stream_t stream);
int ssd_bwd_dx(const SsdParams *p, mamba_stream_t stream);
int ssd_bwd_dBC_state(const SsdParams *p, mamba_stream_t stream);
int ssd_bwd_dcb(const SsdParams *p, mamba_stream_t stream);
int ssd_bmm_chunk_bwd(const SsdParams *p, mamba_stream_t stream);
int ssd_chunk_cumsum_bwd(const SsdParams *p, mamba_stream_t stream);
int ssd_combined_bwd(const SsdParams *p, mamba_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Depthwise causal 1-D convolution in front of the scans.  The reference calls the
 * separate causal_conv1d package for it (causal_conv1d_fn / causal_conv1d_cuda:
 * call sites mamba_ssm/ops/selective_scan_interface.py:224,:307,
 * mamba_ssm/ops/triton/ssd_combined.py:845,:920, mamba_ssm/modules/mamba2.py:236) and
 * falls back to nn.Conv1d(groups = channels, padding = width - 1)[..., :L]
 * (mamba_ssm/modules/mamba_simple.py:168-169):
 *   out[b, c, l] = act(bias[c] + sum_k weight[c, k] x[b, c, l - (width - 1) + k])
 * with x = 0 before position 0 and, when seq_idx is given, for taps whose position
 * has another sequence id than l.  x, out, dout, dx are of `dtype` and addressed through
 * (batch, channel, position) element strides; either the position stride or the
 * channel stride of all of them must be 1 (the two layouts of the callers).  weight
 * (dim, width), bias (dim), dweight, dbias are fp32 contiguous; dweight and dbias MUST be
 * zero on entry (the kernels add into them).  width is 2, 3 or 4.
 * The backward pass re-computes the pre-activation from x.
 * ------------------------------------------------------------------------- */
typedef struct CausalConvParams {
  int32_t batch, dim, seqlen, width;
  int32_t dtype; /* MAMBA_F32 / MAMBA_BF16 / MAMBA_F16 */
  int32_t silu;  /* 1: SiLU after the convolution */
  int32_t reserved0, reserved1;
  const void *x;
  const float *weight;
  const float *bias;      /* nullable */
  const int32_t *seq_idx; /* nullable, (batch, seqlen) contiguous */
  void *out;              /* forward only */
  int64_t x_bs, x_cs, x_ls; /* batch / channel / position stride */
  int64_t out_bs, out_cs, out_ls;
  /* ---- backward only ---- */
  const void *dout;
  void *dx;
  float *dweight;
  float *dbias; /* nullable */
  int64_t dout_bs, dout_cs, dout_ls;
  int64_t dx_bs, dx_cs, dx_ls;
  /* deterministic backward (all null: float atomics): fixed-point scale {s, 1 / s} on the device and int64 shadows
   * of dweight (dim, width) and dbias (dim), zero on entry; the caller converts them with ssd_det_convert */
  const float *det_scale;
  int64_t *det_dweight, *det_dbias;
} CausalConvParams;

int causal_conv1d_fwd(const CausalConvParams *p, mamba_stream_t stream);
int causal_conv1d_bwd(const CausalConvParams *p, mamba_stream_t stream);

/* -------------------------------------------------------------------------
 * Causal conv1d, decode step: with xn = [conv_state, x] along the position axis,
 *   out[b, c, t] = act(bias[c] + sum_k weight[c, k] * xn[b, c, state_len + t - (width-1) + k]),
 *   conv_state[b, c, :] <- the last state_len positions of xn      (in place)
 * Replaces the causal_conv1d package's causal_conv1d_update as the reference calls it
 * (mamba_ssm/modules/mamba2.py:298-304, mamba_ssm/modules/mamba_simple.py:223-229) and the
 * roll + insert + dot it falls back to (mamba2.py:291-296).
 * x, out: (batch, dim, seqlen) of `dtype`, any strides; conv_state: (rows, dim, state_len) of
 * `state_dtype`, any strides, state_len >= width - 1; conv_state_indices (nullable): int32 (batch,),
 * row of conv_state per batch entry; outside [0, state_rows) = padding entry (state untouched,
 * out = 0).
 * ------------------------------------------------------------------------- */
typedef struct CausalConvUpdateParams {
  int32_t batch, dim, seqlen, width, state_len;
  int32_t dtype, state_dtype;
  int32_t silu;
  int32_t state_rows; /* rows of conv_state; an index outside [0, state_rows) is a padding entry */
  int32_t weight_dtype; /* dtype code of weight and bias (MAMBA_F32 = 0 / MAMBA_BF16 / MAMBA_F16) */
  const void *x;
  void *conv_state;
  const void *weight; /* (dim, width) of weight_dtype, contiguous */
  const void *bias;   /* nullable; (dim) of weight_dtype */
  void *out;
  const int32_t *conv_state_indices; /* nullable */
  int64_t x_bs, x_cs, x_ls;
  int64_t out_bs, out_cs, out_ls;
  int64_t state_bs, state_cs, state_ls;
  const int32_t *cache_seqlens; /* nullable; (batch): conv_state is a circular buffer, entry b has seen cache_seqlens[b]
                                   positions, position t lives in slot t % state_len; nothing is shifted */
} CausalConvUpdateParams;

int causal_conv1d_update(const CausalConvUpdateParams *p, mamba_stream_t stream);

/* -------------------------------------------------------------------------
 * Convolution states of the sequences of one packed row:
 *   states[s, c, j] = x[cu_seqlens[s+1] - state_len + j, c], 0 before the start of sequence s.
 * Replaces causal_conv1d.causal_conv1d_varlen.causal_conv1d_varlen_states as called at
 * mamba_ssm/modules/mamba2.py:225-227 (per sequence it is the F.pad of :221).
 * x: (total, dim); cu_seqlens: int32 (nseq + 1); states: (nseq, dim, state_len); all of `dtype`.
 * ------------------------------------------------------------------------- */
typedef struct CausalConvVarlenParams {
  int32_t nseq, dim, total, state_len;
  int32_t dtype;
  int32_t reserved;
  const void *x;
  const int32_t *cu_seqlens;
  void *states;
  int64_t x_ls, x_cs;
  int64_t states_bs, states_cs, states_ls;
} CausalConvVarlenParams;

int causal_conv1d_varlen_states(const CausalConvVarlenParams *p, mamba_stream_t stream);

/* -------------------------------------------------------------------------
 * Gated LayerNorm / RMSNorm over groups of channels: the epilogue of the Mamba-2 block between
 * the chunked scan and the output projection.  Replaces the Triton launches of
 * mamba_ssm/ops/triton/layernorm_gated.py:108 (_layer_norm_fwd) and :271 (_layer_norm_bwd),
 * called from mamba_ssm/modules/mamba2.py:242 and mamba_ssm/ops/triton/ssd_combined.py:872-874.
 *   x' = norm_before_gate ? x : x * silu(z);   y = (x' - mean) * rstd * weight + bias;
 *   out = norm_before_gate ? y * silu(z) : y;  statistics per (row, group), mean = 0 when is_rms.
 * x, z, out, dy, dx, dz are (rows, dim) with unit channel stride and the given row strides, all
 * of `dtype`; weight / bias are fp32 (dim); mean / rstd are fp32 (rows, dim / group_size), written
 * by the forward call and read by the backward call (mean may be null when is_rms).
 * Backward: dw_part / db_part are caller-provided fp32 (nparts, dim) workspaces (any nparts in
 * 1..65536; a team of 8 .. 1024 threads, the smallest power of two with 16 * threads >= group_size (128
 * skipped), works on each (group, part), and a few thousand teams fill the GPU); dweight / dbias are
 * overwritten with their sums.  group_size <= 32768.
 * ------------------------------------------------------------------------- */
typedef struct NormGatedParams {
  int32_t rows, dim, group_size;
  int32_t dtype; /* MAMBA_F32 / MAMBA_BF16 / MAMBA_F16 */
  int32_t is_rms;
  int32_t norm_before_gate;
  int32_t nparts; /* backward only */
  float eps;
  const void *x;
  const void *z; /* nullable: no gate */
  const float *weight;
  const float *bias; /* nullable */
  void *out;         /* forward only */
  float *mean;       /* nullable when is_rms */
  float *rstd;
  int64_t x_rs, z_rs, out_rs;
  /* ---- backward only ---- */
  const void *dy;
  void *dx;
  void *dz; /* null iff z is null */
  float *dweight;
  float *dbias; /* null iff bias is null */
  float *dw_part;
  float *db_part; /* null iff bias is null */
  int64_t dy_rs, dx_rs, dz_rs;
} NormGatedParams;

int norm_gated_fwd(const NormGatedParams *p, mamba_stream_t stream);
int norm_gated_bwd(const NormGatedParams *p, mamba_stream_t stream);

/* -------------------------------------------------------------------------
 * LayerNorm / RMSNorm of (x + residual) with the sum handed on: the norm in front of every mixer
 * of the reference's Block (mamba_ssm/modules/block.py:57-66).  Replaces the Triton launches of
 * mamba_ssm/ops/triton/layer_norm.py:291 (_layer_norm_fwd) and :589 (_layer_norm_bwd) for the
 * arguments the Block uses (residual, prenorm, residual_in_fp32) and, through the optional fields at
 * the end of the struct, for the rest of that operator (rowscale, dropout, the second input x1 and the
 * second set of norm parameters weight1 / bias1; layer_norm.py:130-237 forward, :393-518 backward).
 *   forward:  s = drop(x * rowscale) + drop1(x1) + residual;  residual_out = s;
 *             out = (s - mean) * rstd * weight + bias;  out1 = (s - mean) * rstd * weight1 + bias1
 *   backward: d = d_norm(dy, dy1) + dresidual is the gradient of s, written as dresidual_in (res_dtype);
 *             dx = drop'(d) * rowscale and dx1 = drop1'(d) (dtype); without the optional parts dx = d
 * drop keeps an element with probability 1 - dropout_p and scales it by 1 / (1 - dropout_p); the draw is a
 * function of (seeds[0] for x, seeds[1] for x1; row; channel) that the backward call repeats, and the
 * forward call writes it out as bytes (1 = kept) where mask / mask1 are given.
 * x, out, dy, dx are (rows, dim) of `dtype`; residual, residual_out, dresidual, dresidual_in of
 * `res_dtype` (equal to dtype, or fp32); unit channel stride, row strides given.  In the backward
 * call `x` is the summed input the forward call wrote (residual_out, or x itself when there was
 * neither a residual nor a residual_out), of res_dtype.  weight / bias fp32 (dim); mean / rstd fp32
 * (rows), mean nullable when is_rms.  dw_part / db_part: fp32 (nparts, dim) workspaces, any nparts
 * in 1..65536; dweight / dbias are overwritten with the sums.  dim <= 32768.
 * ------------------------------------------------------------------------- */
typedef struct NormResidualParams {
  int32_t rows, dim;
  int32_t dtype, res_dtype;
  int32_t is_rms;
  int32_t nparts; /* backward only */
  float eps;
  int32_t reserved;
  const void *x;
  const void *residual; /* forward, nullable */
  const float *weight;
  const float *bias;  /* nullable */
  void *out;          /* forward only */
  void *residual_out; /* forward, nullable */
  float *mean;        /* nullable when is_rms */
  float *rstd;
  int64_t x_rs, residual_rs, out_rs, residual_out_rs;
  /* ---- backward only ---- */
  const void *dy;
  const void *dresidual; /* nullable */
  void *dx;
  void *dresidual_in; /* nullable */
  float *dweight;
  float *dbias; /* null iff bias is null */
  float *dw_part;
  float *db_part; /* null iff bias is null */
  int64_t dy_rs, dresidual_rs, dx_rs, dresidual_in_rs;
  /* ---- optional parts, all null / 0 when unused ---- */
  const void *x1;        /* (rows, dim) of dtype; not together with rowscale */
  const float *rowscale; /* (rows) */
  const int64_t *seeds;  /* 2 device words, required when dropout_p > 0 */
  uint8_t *mask;         /* forward, nullable: (rows, dim) bytes, dense */
  uint8_t *mask1;        /* forward, nullable: the same for x1 */
  const float *weight1;  /* (dim) */
  const float *bias1;    /* (dim), nullable */
  void *out1;            /* forward, required with weight1 */
  const void *dy1;       /* backward, required with weight1 */
  void *dx1;             /* backward, required with x1 */
  float *dweight1;       /* backward, required with weight1, like dweight */
  float *dbias1;         /* null iff bias1 is null */
  float *dw1_part;       /* (nparts, dim) workspaces like dw_part / db_part */
  float *db1_part;
  int64_t x1_rs, out1_rs, dy1_rs, dx1_rs;
  float dropout_p;
  int32_t reserved2;
} NormResidualParams;

int norm_residual_fwd(const NormResidualParams *p, mamba_stream_t stream);
int norm_residual_bwd(const NormResidualParams *p, mamba_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MAMBA_HIP_H_ */
