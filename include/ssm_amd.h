/*
 * ssm_amd.h - C ABI of the MI355X (gfx950) operator backend.
 *
 * Every entry point takes a pointer to a plain argument struct (device
 * pointers, sizes, enums) and a HIP stream passed as void*; it validates the
 * arguments on the host, enqueues its kernels on that stream and returns
 * SSM_OK or a negative ssm_status without synchronising.  No entry point
 * throws, and none keeps state between calls except the lazily raised
 * dynamic-LDS limit of a kernel.  Tensors are dense row-major with the shapes
 * given in the comments; "io dtype" is the activation dtype (fp32, bf16 or
 * fp16) and all arithmetic accumulates in fp32.
 *
 * The reference (b-vitamins/ssm) has no C interface: its operator boundary is
 * the Python module `ssm.ops`, and the calls a compiled backend receives from
 * it are the attribute calls listed in src/ssm/ops/__init__.py.  Each entry
 * point below names the reference call it stands behind.
 */
#ifndef SSM_AMD_H
#define SSM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SSM_AMD_ABI_VERSION 8

typedef enum ssm_status {
  SSM_OK = 0,
  SSM_ERR_NULL_POINTER = -1,   /* a required pointer is NULL */
  SSM_ERR_BAD_SHAPE = -2,      /* a size is <= 0 or sizes are inconsistent */
  SSM_ERR_BAD_DTYPE = -3,      /* unknown or unsupported dtype enum */
  SSM_ERR_BAD_KIND = -4,       /* unknown projection / layout / activation enum */
  SSM_ERR_ALIGNMENT = -5,      /* pointer not aligned to its element size */
  SSM_ERR_TOO_LARGE = -6,      /* a size exceeds what the kernels index */
  SSM_ERR_LAUNCH = -7,         /* the HIP runtime refused the launch */
  SSM_ERR_WORKSPACE = -8       /* workspace missing or too small */
} ssm_status;

typedef enum ssm_dtype { SSM_F32 = 0, SSM_BF16 = 1, SSM_F16 = 2 } ssm_dtype;

/* How a B / C projection of the selective scan is laid out. */
typedef enum ssm_proj_kind {
  SSM_PROJ_DN = 0,    /* (D, N)       shared by batch and time */
  SSM_PROJ_BDN = 1,   /* (B, D, N)    per batch row, constant in time */
  SSM_PROJ_BGNL = 2   /* (B, G, N, L) grouped and time-varying; channel d reads group d / (D/G) */
} ssm_proj_kind;

/* SSM_LAYOUT_ROWS_TO_BCL (the convolution only): x is a (B,C,L)-shaped view of memory laid out as rows of
 * channels, one row per time step (`x_row_stride` elements apart, `x_batch_stride` between batch rows) -- what the
 * reference's blocks pass (src/ssm/modules/mamba1.py:209-215, mamba2.py:159-165: `projected.permute(0, 2, 1)`);
 * y and dout are dense (B,C,L), dx is written as dense (B,L,C) rows. */
typedef enum ssm_layout { SSM_LAYOUT_BCL = 0, SSM_LAYOUT_BLC = 1, SSM_LAYOUT_ROWS_TO_BCL = 2 } ssm_layout;
typedef enum ssm_activation { SSM_ACT_IDENTITY = 0, SSM_ACT_SILU = 1 } ssm_activation;

int ssm_amd_abi_version(void);
/* Static, human-readable text for a status code. */
const char *ssm_amd_status_string(int status);
/* Detail of the last failing call on this thread ("" if none). */
const char *ssm_amd_last_error(void);

/* ------------------------------------------------------------------------
 * selective scan, forward.
 *   delta' = softplus(delta + dt_bias)            (both optional)
 *   h_t    = exp(delta'_t A) h_{t-1} + delta'_t u_t B_t ,  h_{-1} = 0
 *   y_t    = <h_t, C_t> + D u_t ;  y_t *= silu(z_t)
 * Stands behind `selective_scan(u, delta, A, B, C, D, z, dt_bias, softplus,
 * return_last_state)` as invoked at src/ssm/ops/__init__.py:1289-1303
 * (semantics: src/ssm/ops/python/reference.py:87-194).
 * ---------------------------------------------------------------------- */
typedef struct ssm_scan_fwd_args {
  const void *u;          /* (B, D, L) io dtype */
  const void *delta;      /* (B, D, L) io dtype */
  const void *z;          /* (B, D, L) io dtype, or NULL */
  const float *A;         /* (D, N) fp32 */
  const void *Bproj;      /* see b_kind, bc dtype */
  const void *Cproj;      /* see c_kind, bc dtype */
  const float *Dskip;     /* (D,) fp32, or NULL */
  const float *dt_bias;   /* (D,) fp32, or NULL */
  void *out;              /* (B, D, L) io dtype */
  void *last_state;       /* (B, D, N) io dtype, or NULL */
  float *chunk_states;    /* (B, D, ceil(L / ssm_scan_chunk_len()), N) fp32, or NULL: the state
                             entering each chunk, which ssm_scan_bwd restarts from */
  int32_t batch, dim, seqlen, nstate;
  int32_t io_dtype;       /* ssm_dtype of u, delta, z, out, last_state */
  int32_t bc_dtype;       /* ssm_dtype of Bproj and Cproj */
  int32_t b_kind, c_kind; /* ssm_proj_kind */
  int32_t b_groups, c_groups; /* G for SSM_PROJ_BGNL (must divide D), else ignored */
  int32_t delta_softplus; /* 0 / 1 */
  int32_t reserved;       /* must be 0 */
} ssm_scan_fwd_args;

int ssm_scan_fwd(const ssm_scan_fwd_args *args, void *hip_stream);
/* Time steps per checkpointed chunk (the granularity of chunk_states). */
int ssm_scan_chunk_len(void);

/* ------------------------------------------------------------------------
 * selective scan, backward.  Recomputes the states from `chunk_states` (as
 * written by ssm_scan_fwd with the same inputs) and returns the gradients of
 * every input for an upstream gradient `dout` (and optionally one for the
 * last state).  Stands behind `selective_scan_backward(grad_out,
 * grad_last_state, u, delta, A, B, C, D, z, dt_bias, softplus, ...)` as
 * invoked at src/ssm/ops/__init__.py:351-471 (formulas:
 * src/ssm/ops/cpu/selective_scan.cpp:393-532).  nstate <= 16 per call.
 * dB / dC have the shape of Bproj / Cproj and are fp32; results are
 * bit-reproducible (no atomics).
 * ---------------------------------------------------------------------- */
typedef struct ssm_scan_bwd_args {
  const void *u, *delta, *z;      /* (B, D, L) io dtype; z may be NULL */
  const void *dout;               /* (B, D, L) io dtype */
  const float *A;                 /* (D, N) */
  const void *Bproj, *Cproj;      /* as in the forward call, bc dtype */
  const float *Dskip, *dt_bias;   /* (D,) or NULL */
  const float *dlast_state;       /* (B, D, N) fp32 gradient of last_state, or NULL */
  const float *chunk_states;      /* from ssm_scan_fwd */
  void *du, *ddelta, *dz;         /* (B, D, L) io dtype; dz NULL iff z NULL */
  float *dA;                      /* (D, N) */
  void *dB, *dC;                  /* shape of Bproj / Cproj, float32 unless dbc_dtype says otherwise */
  float *dD, *ddt_bias;           /* (D,) or NULL */
  void *workspace;                /* ssm_scan_bwd_workspace_bytes(), 256-byte aligned */
  size_t workspace_bytes;
  int32_t batch, dim, seqlen, nstate;
  int32_t io_dtype, bc_dtype;
  int32_t b_kind, c_kind, b_groups, c_groups;
  int32_t delta_softplus;
  int32_t reserved;               /* must be 0 */
  int32_t dbc_dtype;              /* element type of dB and dC: SSM_F32 (= 0), or bc_dtype in a call that
                                     ssm_scan_bwd_per_row_workspace_bytes() accepts */
} ssm_scan_bwd_args;

size_t ssm_scan_bwd_workspace_bytes(int batch, int dim, int seqlen, int nstate, int b_kind, int c_kind,
                                    int b_groups, int c_groups);
/* Projections of their own per channel -- B and C of shape (B, D, N, L), i.e. b_groups == c_groups == dim, the form
 * of the reference's own Mamba1 module (src/ssm/modules/mamba1.py:229-246) -- in aligned rows of whole 8-step
 * runs: nothing sums over channels, dB and dC are written straight to their place (in float32 or, on request, in
 * the projections' type) and the call needs only this much workspace.  0: not such a call; it then needs
 * ssm_scan_bwd_workspace_bytes() and writes dB and dC in float32. */
size_t ssm_scan_bwd_per_row_workspace_bytes(const ssm_scan_bwd_args *args);
int ssm_scan_bwd(const ssm_scan_bwd_args *args, void *hip_stream);

/* ------------------------------------------------------------------------
 * selective state update for one token (decode step); `state` is updated in
 * place.  Stands behind `selective_state_step(state, x, dt, A, B, C, D, z,
 * dt_bias, softplus)` as invoked at src/ssm/ops/__init__.py:1395-1409
 * (semantics: src/ssm/ops/python/reference.py:197-309).  The grouped
 * projection form (B, G, N) is passed as SSM_PROJ_BGNL with L = 1.
 * ---------------------------------------------------------------------- */
typedef struct ssm_state_step_args {
  void *state;            /* (B, D, N) state dtype, read and written */
  const void *x;          /* (B, D) io dtype */
  const void *dt;         /* (B, D) io dtype */
  const void *z;          /* (B, D) io dtype, or NULL */
  const float *A;         /* (D, N) fp32 */
  const void *Bproj;      /* (D,N) | (B,D,N) | (B,G,N), bc dtype */
  const void *Cproj;
  const float *Dskip;     /* (D,) fp32 or NULL */
  const float *dt_bias;   /* (D,) fp32 or NULL */
  void *out;              /* (B, D) io dtype */
  int32_t batch, dim, nstate;
  int32_t state_dtype, io_dtype, bc_dtype;
  int32_t b_kind, c_kind, b_groups, c_groups;
  int32_t dt_softplus;
  /* Elements between consecutive batch rows of z and of grouped (B,G,N) projections, for rows that are slices of
   * wider rows (a decoding block's projected row); 0 = dense.  The rows themselves are contiguous. */
  int64_t z_batch_stride, b_batch_stride, c_batch_stride;
} ssm_state_step_args;

int ssm_state_step(const ssm_state_step_args *args, void *hip_stream);

/* Backward of the state update.  Stands behind the backend call
 * `selective_state_step_backward(grad_out, grad_state, state, x, dt, A, B, C, D,
 * z, dt_bias, softplus)` made at src/ssm/ops/__init__.py:654-668 (nine
 * gradients; formulas follow src/ssm/ops/cpu/state_step.cpp's backward).
 * `state` is the state BEFORE the step; `grad_state` is the gradient with
 * respect to the updated state. */
typedef struct ssm_state_step_bwd_args {
  const void *grad_out;    /* (B, D) io dtype, or NULL (zero) */
  const void *grad_state;  /* (B, D, N) state dtype, or NULL (zero) */
  const void *state;       /* (B, D, N) state dtype */
  const void *x, *dt;      /* (B, D) io dtype */
  const void *z;           /* (B, D) io dtype, or NULL */
  const float *A;          /* (D, N) fp32 */
  const void *Bproj, *Cproj; /* as in ssm_state_step_args */
  const float *Dskip;      /* (D,) fp32 or NULL */
  const float *dt_bias;    /* (D,) fp32 or NULL */
  void *dstate;            /* (B, D, N) state dtype */
  void *dx, *ddt;          /* (B, D) io dtype */
  void *dz;                /* (B, D) io dtype; given exactly when z is */
  float *dA;               /* (D, N) */
  float *dB, *dC;          /* fp32, shaped like Bproj / Cproj */
  float *dD, *ddt_bias;    /* (D,) or NULL */
  void *workspace;         /* ssm_state_step_bwd_workspace_bytes() bytes */
  size_t workspace_bytes;
  int32_t batch, dim, nstate;
  int32_t state_dtype, io_dtype, bc_dtype;
  int32_t b_kind, c_kind, b_groups, c_groups;
  int32_t dt_softplus;
} ssm_state_step_bwd_args;

size_t ssm_state_step_bwd_workspace_bytes(int batch, int dim, int nstate);
int ssm_state_step_bwd(const ssm_state_step_bwd_args *args, void *hip_stream);

/* ------------------------------------------------------------------------
 * fused decode step: roll the causal-conv window, apply the depthwise conv and
 * its activation to the new input, then run the selective state update on the
 * result - one launch per token.  It covers what `Mamba1.step` does with
 * separate tensor ops at src/ssm/modules/mamba1.py:345-353 (window roll, tap
 * sum, SiLU) followed by `selective_state_step` (:370-381) for callers whose
 * dt, B and C do not depend on the conv output of the same step.
 * `step.x` is the raw (pre-conv) input; `step.state` is the SSM state.
 * ---------------------------------------------------------------------- */
typedef struct ssm_decode_step_args {
  ssm_state_step_args step;
  void *conv_state;          /* (B, D, K) io dtype, rolled in place: [..., 1:] moves left, x appended */
  const float *conv_weight;  /* (D, K) fp32 */
  const float *conv_bias;    /* (D,) fp32 or NULL */
  void *conv_out;            /* (B, D) io dtype or NULL: activated conv output */
  int32_t conv_width;        /* K */
  int32_t conv_activation;   /* ssm_activation */
} ssm_decode_step_args;

int ssm_decode_step(const ssm_decode_step_args *args, void *hip_stream);

/* One decoding step of a Mamba-2 (SSD) block on cached states.  No counterpart in the reference (its
 * `Mamba2` module, /root/reference/src/ssm/modules/mamba2.py:20-140, has no cached step): this is the
 * single-token selective_state_step above (reference.py:197-309) with per-head step, decay and skip, preceded
 * by the depthwise convolution of the x | B | C columns on their cached windows, for the block that
 * configuration 4 describes.  The row of the input projection is consumed in place: z | xBC | dt with
 * d_inner = heads * headdim, 2 * groups * nstate and heads columns.
 *   xBC <- silu(conv(window rolled by one, xBC) + bias)          (window updated in place)
 *   dt = softplus(dt + dt_bias) if dt_softplus;  S <- exp(dt A) S + dt x (x) B;  y = S C + D x;  y *= silu(z) if gate */
typedef struct ssm_mamba2_decode_args {
  const void *zxbcdt;        /* (B, 2*d_inner + 2*G*N + H) io dtype */
  void *conv_state;          /* (B, d_inner + 2*G*N, K) io dtype: last K inputs per channel, oldest first; in place */
  const float *conv_weight;  /* (d_inner + 2*G*N, K) fp32 */
  const float *conv_bias;    /* (d_inner + 2*G*N,) fp32 or NULL */
  float *xbc;                /* (B, d_inner + 2*G*N) fp32: activated conv output (needed as workspace) */
  float *ssm_state;          /* (B, H, P, N) fp32, in place */
  const float *A;            /* (H,) */
  const float *Dskip;        /* (H,) or (H, P) if d_per_p, or NULL */
  const float *dt_bias;      /* (H,) or NULL */
  void *y;                   /* (B, d_inner) io dtype */
  int32_t batch, heads, headdim, groups, nstate, conv_width;
  int32_t io_dtype, d_per_p, dt_softplus, gate;
} ssm_mamba2_decode_args;
int ssm_mamba2_decode_step(const ssm_mamba2_decode_args *args, void *hip_stream);

/* The convolution part of a decoding step on its own: the new input x enters the cached window, which moves
 * on by one, and out = act(bias + sum_k weight[:, k] * window[:, :, k]).  It replaces the window roll, tap sum
 * and SiLU that `Mamba1.step` spells out with tensor ops at src/ssm/modules/mamba1.py:345-353, for blocks
 * whose dt, B and C are projections of this very output (so that ssm_decode_step does not apply). */
typedef struct ssm_conv1d_update_args {
  const void *x;             /* (B, C) io dtype; row b starts x_row_stride * b elements in */
  void *conv_state;          /* (B, C, K) io dtype: last K inputs per channel, oldest first; in place */
  const float *weight;       /* (C, K) fp32 */
  const float *bias;         /* (C,) fp32 or NULL */
  void *out;                 /* (B, C) io dtype */
  int64_t x_row_stride;      /* >= channels */
  int32_t batch, channels, width;
  int32_t io_dtype;          /* ssm_dtype */
  int32_t activation;        /* ssm_activation */
} ssm_conv1d_update_args;
int ssm_conv1d_update(const ssm_conv1d_update_args *args, void *hip_stream);

/* ------------------------------------------------------------------------
 * diagonal chunk scan: the operator the reference calls `ssd_chunk_scan`
 * (an element-wise recurrence per (batch, head, p); chunking does not change
 * the result).  Stands behind `ssd_chunk_scan(X, dt, A, B, C, chunk_size, D,
 * z, seq_lens, cu_seqlens, initial_states)` as invoked at
 * src/ssm/ops/__init__.py:1516-1531 (semantics: reference.py:312-463).
 * ---------------------------------------------------------------------- */
typedef enum ssm_chunk_kind {
  SSM_CHUNK_HP = 0,    /* (H, P) */
  SSM_CHUNK_BHP = 1,   /* (B, H, P) */
  SSM_CHUNK_BLHP = 2   /* (B, L, H, P) */
} ssm_chunk_kind;

typedef struct ssm_dscan_fwd_args {
  const void *X;              /* (B, L, H, P) x dtype */
  const void *dt;             /* (B, L, H) dt dtype; used as given */
  const float *A;             /* (H, P) if a_per_p else (H,) */
  const void *Bproj, *Cproj;  /* see b_kind / c_kind, bc dtype */
  const float *Dskip;         /* (H, P) if d_per_p else (H,), or NULL */
  const void *z;              /* (B, L, H, P) if z_per_p else (B, L, H), z dtype, or NULL */
  const void *initial_states; /* (B, H, P) init dtype, or NULL */
  const int32_t *seq_lens;    /* (B,) valid steps per batch row (device memory), or NULL */
  void *Y;                    /* (B, L, H, P) x dtype; rows at or beyond seq_lens[b] are zero */
  void *workspace;            /* ssm_dscan_fwd_workspace_bytes() bytes */
  size_t workspace_bytes;
  int32_t batch, seqlen, heads, proj;
  int32_t x_dtype, dt_dtype, bc_dtype, z_dtype, init_dtype;
  int32_t b_kind, c_kind;     /* ssm_chunk_kind */
  int32_t a_per_p, d_per_p, z_per_p;
  float *round_states;        /* optional output (B, ceil(L/64), H*P) fp32: the state entering every 64 steps, which
                                 ssm_dscan_bwd_args.round_states takes; only for calls for which
                                 ssm_dscan_fwd_one_pass() is non-zero (an error otherwise); or NULL */
} ssm_dscan_fwd_args;

size_t ssm_dscan_fwd_workspace_bytes(int batch, int seqlen, int heads, int proj);
int ssm_dscan_fwd(const ssm_dscan_fwd_args *args, void *hip_stream);
/* Non-zero when the call described (pointers included: alignment counts) runs the kernel that reads every input
 * once; only that kernel can fill round_states.  No counterpart in the reference. */
int ssm_dscan_fwd_one_pass(const ssm_dscan_fwd_args *args);

/* Backward of the diagonal chunk scan.  Stands behind the backend call
 * `ssd_chunk_scan_backward(grad_out, X, dt, A, B, C, D, z, seq_lens, cu_seqlens,
 * initial_states)` made at src/ssm/ops/__init__.py:869-884 (eight gradients:
 * X, dt, A, B, C, D, z, initial_states).  Parameter gradients are fp32 and have
 * the shape of the parameter; dX and dz have the dtype of X and z. */
typedef struct ssm_dscan_bwd_args {
  const void *grad_y;         /* (B, L, H, P) x dtype */
  const void *X, *dt;         /* as in ssm_dscan_fwd_args */
  const float *A;
  const void *Bproj, *Cproj;
  const float *Dskip;
  const void *z;
  const void *initial_states;
  const int32_t *seq_lens;
  void *dX;                   /* (B, L, H, P) x dtype */
  float *ddt;                 /* (B, L, H) */
  float *dA;                  /* (H, P) if a_per_p else (H,) */
  void *dB, *dC;              /* shaped like Bproj / Cproj; fp32 (see grads_in_io_dtype) */
  float *dD;                  /* (H, P) if d_per_p else (H,), or NULL */
  void *dz;                   /* shaped like z; fp32 (see grads_in_io_dtype); given exactly when z is */
  float *dinitial_states;     /* (B, H, P) fp32 or NULL */
  void *workspace;            /* ssm_dscan_bwd_workspace_bytes() bytes */
  size_t workspace_bytes;
  int32_t batch, seqlen, heads, proj;
  int32_t x_dtype, dt_dtype, bc_dtype, z_dtype, init_dtype;
  int32_t b_kind, c_kind;
  int32_t a_per_p, d_per_p, z_per_p;
  int32_t grads_in_io_dtype;  /* non-zero: the gradients that have X's shape are written in their tensors' element
                                 types instead of fp32: dB / dC when the projection is per token (bc dtype), dz when
                                 the gate is per channel (z dtype); every other gradient stays fp32 */
  int32_t reserved;           /* must be 0 */
  const float *round_states;  /* optional: what ssm_dscan_fwd wrote for the same inputs; spares the backward its own
                                 forward sweep when it takes the one-pass kernels (ignored otherwise); or NULL */
} ssm_dscan_bwd_args;

size_t ssm_dscan_bwd_workspace_bytes(int batch, int seqlen, int heads, int proj);
int ssm_dscan_bwd(const ssm_dscan_bwd_args *args, void *hip_stream);

/* ------------------------------------------------------------------------
 * state-space duality (Mamba-2) operator family.  The reference has no code
 * for these; their semantics are fixed by the vectors it ships in
 * tests/mamba_reference_cases.json, recorded through the call sites in
 * scripts/refresh_mamba_goldens.py:430-486 (chunk_cumsum, chunk_state,
 * state_passing, chunk_scan), :591-604 (combined) and :680-705 (bmm_chunk).
 * Layouts: x, z, y (B,L,H,P); dt (B,L,H); A (H,); Bm, Cm (B,L,G,N);
 * dt_out, dA_cumsum (B,H,nc,Q) fp32; CB (B,nc,G,Q,Q); states (B,nc,H,P,N);
 * final_states (B,H,P,N) fp32; nc = ceil(L/Q).  Fields named `reserved`
 * must be 0.
 * ---------------------------------------------------------------------- */

typedef struct ssm_ssd_dims {
  int32_t batch, seqlen, heads, headdim, groups, nstate, chunk;
} ssm_ssd_dims;

typedef struct ssm_ssd_cumsum_args {
  const void *dt;           /* (B,L,H) dt dtype */
  const float *A;           /* (H,) */
  const float *dt_bias;     /* (H,) or NULL */
  float *dA_cumsum;         /* (B,H,nc,Q) */
  float *dt_out;            /* (B,H,nc,Q) */
  ssm_ssd_dims dims;        /* headdim, groups, nstate unused */
  int32_t dt_dtype, dt_softplus;
  float dt_min, dt_max;     /* clamp applied after softplus; use 0 and +inf for none */
} ssm_ssd_cumsum_args;
int ssm_ssd_chunk_cumsum(const ssm_ssd_cumsum_args *args, void *hip_stream);

typedef struct ssm_ssd_bmm_args {
  const void *a, *b;        /* (B,L,G,K) in dtype */
  const int32_t *seq_idx;   /* (B,L) or NULL: entries across sequences are zeroed */
  void *out;                /* (B,nc,G,Q,Q) out dtype: out[l][s] = <a_l, b_s> */
  int32_t batch, seqlen, groups, kdim, chunk;
  int32_t in_dtype, out_dtype, causal, reserved;
} ssm_ssd_bmm_args;
int ssm_ssd_bmm_chunk(const ssm_ssd_bmm_args *args, void *hip_stream);

typedef struct ssm_ssd_chunk_state_args {
  const void *Bm;           /* (B,L,G,N) b dtype */
  const void *x;            /* (B,L,H,P) x dtype */
  const float *dt;          /* (B,H,nc,Q) */
  const float *dA_cumsum;   /* (B,H,nc,Q) */
  void *states;             /* (B,nc,H,P,N) states dtype */
  void *workspace;          /* optional: ssm_ssd_chunk_state_workspace_bytes() bytes of device memory;
                               without it the MFMA kernel is not used */
  size_t workspace_bytes;
  ssm_ssd_dims dims;
  int32_t x_dtype, b_dtype, states_dtype, reserved;
  const int32_t *seq_idx;   /* (B,L) or NULL: steps of another sequence than the chunk's last step add nothing */
  const float *x_row_scale; /* (B,H,nc,Q) or NULL: x stands for x * scale rounded to x's dtype, as if that tensor had
                               been written first (the backward puts the step into the operand this way); only the
                               matrix-core kernel takes it, and only for bfloat16 x: an error otherwise */
  int32_t x_time_reversed;  /* nonzero: the call walks the sequence backwards in time (B, dt, dA_cumsum given reversed)
                               while x is given in forward time: step tau reads x's row L-1-tau, and no reversed copy
                               of x is needed.  Matrix-core kernel only: an error otherwise */
} ssm_ssd_chunk_state_args;
size_t ssm_ssd_chunk_state_workspace_bytes(const ssm_ssd_dims *dims);
int ssm_ssd_chunk_state(const ssm_ssd_chunk_state_args *args, void *hip_stream);

typedef struct ssm_ssd_state_passing_args {
  const void *states;        /* (B,nc,H,dim) states dtype: per-chunk contributions */
  const float *dA_chunk_last;/* (B,H,nc): dA_cumsum at the last step of each chunk */
  const float *initial_states; /* (B,H,dim) fp32 or NULL */
  void *states_out;          /* (B,nc,H,dim) states dtype: state entering each chunk */
  float *final_states;       /* (B,H,dim) */
  int32_t batch, nchunks, heads, dim;
  int32_t states_dtype;
  int32_t seqlen, chunk;     /* only read with seq_idx */
  const int32_t *seq_idx;    /* (B,L) or NULL: the carried state is dropped where the sequence id of a chunk's
                                last step differs from that of the chunk before (the initial state belongs to id 0) */
} ssm_ssd_state_passing_args;
int ssm_ssd_state_passing(const ssm_ssd_state_passing_args *args, void *hip_stream);

typedef struct ssm_ssd_chunk_scan_args {
  const void *CB;           /* (B,nc,G,Q,Q) cb dtype, lower triangle used */
  const void *Cm;           /* (B,L,G,N) c dtype */
  const void *x;            /* (B,L,H,P) x dtype */
  const void *z;            /* (B,L,H,P) z dtype or NULL */
  const void *prev_states;  /* (B,nc,H,P,N) states dtype: state entering each chunk */
  const float *dt, *dA_cumsum; /* (B,H,nc,Q) */
  const float *Dskip;       /* (H,P) if d_per_p else (H,), or NULL */
  void *y;                  /* (B,L,H,P) x dtype (float32 if y_f32) */
  ssm_ssd_dims dims;
  int32_t x_dtype, c_dtype, cb_dtype, states_dtype, z_dtype, d_per_p, reserved;
  const int32_t *seq_idx;   /* (B,L) or NULL: the entering state only reaches steps whose sequence id equals that of
                               the last step of the chunk before (id 0 for the first chunk); CB must have been
                               formed with the same seq_idx */
  int32_t y_f32;            /* nonzero: y is float32 whatever x's dtype is (the backward's running sums need the
                               passes' results unrounded); 0: y has x's dtype */
  const float *x_row_scale; /* (B,H,nc,Q) or NULL: as in ssm_ssd_chunk_state_args (the skip term D x is not scaled) */
  /* The gradient's time-reversed pass (x = dy reversed, B and C in each other's place) can finish dx in this kernel
   * instead of writing its result u (y may then be NULL): with t = L-1-tau the forward step of reversed row tau,
   *   dx_out[t] = dx_dt[t] u[tau] + dx_Dskip dy[t],  dx_xu[t] = sum_p dx_x[t] u[tau],
   *   dx_s1[t] = sum_p round(dx_dt[t] dx_x[t]) u[tau]      (rounded to x's dtype if dx_round_dtx)
   * -- what ssm_ssd_bwd_dx computes from u (there dy is taken before its rounding to the operand's type, here after).
   * Matrix-core kernel only: bfloat16 operands, float32 states, no z / Dskip / seq_idx; an error otherwise. */
  const void *dx_x;         /* (B,L,H,P) x dtype, forward time */
  const float *dx_dt;       /* (B,L,H) */
  const float *dx_Dskip;    /* (H,P) if dx_d_per_p else (H,), or NULL */
  void *dx_out;             /* (B,L,H,P) float32 if dx_out_f32 else x dtype; NULL: the ordinary call */
  float *dx_xu, *dx_s1;     /* (B,L,H) */
  int32_t dx_d_per_p, dx_out_f32, dx_round_dtx;
  int32_t x_time_reversed;  /* as in ssm_ssd_chunk_state_args (C, CB, prev_states, dt, dA_cumsum given reversed, y or dx_*
                               as without it); not together with Dskip */
} ssm_ssd_chunk_scan_args;
int ssm_ssd_chunk_scan(const ssm_ssd_chunk_scan_args *args, void *hip_stream);

/* State at the last step of each sequence of a packed batch row (batch = 1): sequence i covers steps
 * cu_seqlens[i] .. cu_seqlens[i+1]-1.  Takes the entering states of the chunks (formed with seq_idx, or from
 * anywhere if every sequence starts on a chunk boundary) and adds the steps of the last chunk that belong to the
 * sequence.  The entering state of the first chunk (the row's initial state) counts for the sequence that starts
 * at step 0.  Replaces the upstream routine the reference's vectors were made with
 * (`chunk_state_varlen`, reached through `mamba_chunk_scan_combined(..., cu_seqlens=, return_varlen_states=True)`
 * at /root/reference/scripts/refresh_mamba_goldens.py:618-632; vectors `ssd_combined.combined_varlen`). */
typedef struct ssm_ssd_chunk_state_varlen_args {
  const void *Bm;           /* (1,L,G,N) b dtype */
  const void *x;            /* (1,L,H,P) x dtype */
  const float *dt;          /* (1,H,nc,Q) */
  const float *dA_cumsum;   /* (1,H,nc,Q) */
  const void *chunk_states; /* (1,nc,H,P,N) states dtype: state entering each chunk */
  const int32_t *cu_seqlens;/* (nseq+1) on the device, increasing, first 0, last <= L */
  float *states;            /* (nseq,H,P,N) */
  ssm_ssd_dims dims;        /* batch must be 1 */
  int32_t nseq;
  int32_t x_dtype, b_dtype, states_dtype;
} ssm_ssd_chunk_state_varlen_args;
int ssm_ssd_chunk_state_varlen(const ssm_ssd_chunk_state_varlen_args *args, void *hip_stream);

/* The whole forward (chunk_cumsum, bmm_chunk, chunk_state, state_passing,
 * chunk_scan; combined call recorded at scripts/refresh_mamba_goldens.py:591-604)
 * as one pass over the sequence that keeps the running state on chip: the
 * per-chunk states never reach device memory.  Covers bf16 and fp16 tensors with
 * headdim 64, chunk in {64, 128, 256}, nstate in {64, 128} and
 * seqlen % chunk == 0; ssm_ssd_combined_supported() tells, other shapes go
 * through the five calls above.  A head with A > 0 is treated as those calls
 * treat it (decays inside a chunk bounded by 1, the carried state growing). */
typedef struct ssm_ssd_combined_args {
  const void *x;              /* (B,L,H,P) io dtype */
  const void *dt;             /* (B,L,H) dt dtype, before bias / softplus / clamp */
  const float *A;             /* (H,) */
  const float *dt_bias;       /* (H,) or NULL */
  const void *Bm, *Cm;        /* (B,L,G,N) io dtype */
  const float *Dskip;         /* (H,P) if d_per_p else (H,), or NULL */
  const void *z;              /* (B,L,H,P) io dtype or NULL */
  const float *initial_states;/* (B,H,P,N) fp32 or NULL */
  void *y;                    /* (B,L,H,P) io dtype */
  float *final_states;        /* (B,H,P,N) fp32 or NULL */
  void *workspace;            /* ssm_ssd_combined_workspace_bytes() bytes, 256-byte aligned */
  size_t workspace_bytes;
  ssm_ssd_dims dims;
  int32_t io_dtype;           /* SSM_BF16 or SSM_F16 */
  int32_t dt_dtype, dt_softplus, d_per_p;
  float dt_min, dt_max;       /* clamp applied after softplus; use 0 and +inf for none */
  const int32_t *seq_idx;     /* (B, L) sequence ids of a packed batch (first id 0), or NULL: no state and no
                                 in-chunk term crosses from one sequence into the next */
  int64_t b_row_stride, c_row_stride;  /* elements from one step's (G, N) block of Bm / Cm to the next step's; 0: dense
                                 (G * N).  Lets B and C be the two halves of one projected row, read in place; rows
                                 stay 16-byte aligned (a multiple of 8 elements) */
} ssm_ssd_combined_args;
int ssm_ssd_combined_supported(const ssm_ssd_dims *dims, int io_dtype);   /* 1 / 0 */
size_t ssm_ssd_combined_workspace_bytes(const ssm_ssd_dims *dims);
int ssm_ssd_combined_fwd(const ssm_ssd_combined_args *args, void *hip_stream);

/* Element-wise stages of the gradient of the combined forward.  The reference holds no code for them: its
 * fixture `ssd_combined.combined_full.gradients` (tests/mamba_reference_cases.json, written by
 * scripts/refresh_mamba_goldens.py:677-705) fixes the nine gradients, which the Python side of this package
 * forms from passes of the forward kernels with operands in other roles; these three launches replace the
 * tensor operations between those passes.  Rows are (batch, step, head) vectors of `headdim` channels;
 * `headdim` must be 4 * 2^k (at most 256).
 *   gate: dy = dout silu(z) (dout without z), written in `dy_dtype` in time order and, when `dy_rev` is
 *         given, reversed in time;  dz = dout (ypre + D x) silu'(z);  s2 = <dy as stored, ypre>;  dyx = <dy, x>
 *   dx:   dx = dt u + D dy,  xu = <x, u>,  s1 = <dt x (rounded to bfloat16 if round_bf16), u>, with u given
 *         reversed in time
 *   db:   dB[b][l][g][n] = sum_{h in group g} dt[b][l][h] v_rev[b][L-1-l][h][n] */
typedef struct ssm_ssd_bwd_gate_args {
  const void *dout;          /* (B, L, H, P) io dtype */
  const void *z;             /* (B, L, H, P) io dtype or NULL */
  const void *x;             /* (B, L, H, P) io dtype */
  const float *ypre;         /* (B, L, H, P) fp32: output before skip and gate */
  const float *Dskip;        /* (H,) or (H, P) if d_per_p, or NULL */
  void *dy;                  /* (B, L, H, P) dy_dtype */
  void *dy_rev;              /* (B, L, H, P) dy_dtype, time reversed, or NULL */
  void *dz;                  /* (B, L, H, P) fp32 (io_dtype with dz_in_io_dtype); NULL exactly when z is */
  float *s2;                 /* (B, L, H) fp32 */
  float *dyx;                /* (B, L, H) fp32 */
  int32_t batch, seqlen, heads, headdim;
  int32_t io_dtype;          /* ssm_dtype of dout, z, x */
  int32_t dy_dtype;          /* SSM_F32 or SSM_BF16 */
  int32_t d_per_p;
  const float *w_dy;         /* (B, L, H) fp32 or NULL: per-row weight of dy_w */
  const float *w_x;          /* (B, L, H) fp32 or NULL: per-row weight of x_w */
  void *dy_w;                /* (B, L, H, P) dy_dtype or NULL: dy as stored times w_dy (rows of the product for dC) */
  void *x_w;                 /* (B, L, H, P) dy_dtype or NULL: x times w_x (rows of the product for dB) */
  int32_t dz_in_io_dtype;    /* nonzero: dz is written in io_dtype instead of fp32 */
} ssm_ssd_bwd_gate_args;
int ssm_ssd_bwd_gate(const ssm_ssd_bwd_gate_args *args, void *hip_stream);

typedef struct ssm_ssd_bwd_dx_args {
  const void *dout;          /* (B, L, H, P) io dtype */
  const void *z;             /* (B, L, H, P) io dtype or NULL */
  const void *x;             /* (B, L, H, P) io dtype */
  const float *u_rev;        /* (B, L, H, P) fp32, time reversed */
  const float *dt;           /* (B, L, H) fp32: the step after bias, softplus and clamp */
  const float *Dskip;        /* (H,) or (H, P) if d_per_p, or NULL */
  void *dx;                  /* (B, L, H, P) fp32 (io_dtype with dx_in_io_dtype) */
  float *xu;                 /* (B, L, H) fp32 */
  float *s1;                 /* (B, L, H) fp32 */
  int32_t batch, seqlen, heads, headdim;
  int32_t io_dtype, d_per_p, round_bf16;
  int32_t dx_in_io_dtype;    /* nonzero: dx is written in io_dtype instead of fp32 */
} ssm_ssd_bwd_dx_args;
int ssm_ssd_bwd_dx(const ssm_ssd_bwd_dx_args *args, void *hip_stream);

typedef struct ssm_ssd_bwd_db_args {
  const float *v_rev;        /* (B, L, H, N) fp32, time reversed */
  const float *dt;           /* (B, L, H) fp32 */
  float *dB;                 /* (B, L, G, N) fp32 */
  int32_t batch, seqlen, heads, groups, nstate;
} ssm_ssd_bwd_db_args;
int ssm_ssd_bwd_db(const ssm_ssd_bwd_db_args *args, void *hip_stream);

/* The matrix both dB and dC of a chunk's own steps follow from (the "dCB" of the published backward,
 * state-spaces/mamba ssd_combined.py: _chunk_scan_bwd_dcb + _chunk_state_bwd_db folded over heads):
 *   dCB[b,c,g,l,s] = sum_{h in g} dt[s,h] exp(cs[l,h] - cs[s,h]) <dy[b,cQ+l,h,:], x[b,cQ+s,h,:]>  (s <= l, else 0)
 * so that dB[cQ+s] = sum_l dCB[l,s] C[cQ+l] and dC[cQ+l] = sum_s dCB[l,s] B[cQ+s] are plain matrix products.
 * bf16 operands, float32 result; headdim 32 or 64, chunk a multiple of 32 that divides seqlen. */
typedef struct ssm_ssd_bwd_dcb_args {
  const void *dy;            /* (B, L, H, P) bf16: gradient at the output before skip and gate */
  const void *x;             /* (B, L, H, P) bf16 */
  const float *dt;           /* (B, H, nc, Q) fp32: the step after bias, softplus and clamp */
  const float *dA_cumsum;    /* (B, H, nc, Q) fp32: running sums of dt * A inside each chunk */
  float *dCB;                /* (B, nc, G, Q, Q) fp32 */
  int32_t batch, seqlen, heads, headdim, groups, chunk;
} ssm_ssd_bwd_dcb_args;
int ssm_ssd_bwd_dcb(const ssm_ssd_bwd_dcb_args *args, void *hip_stream);

/* The states at the chunk boundaries, as the two products above want them, and the anchors of the running sum
 * behind ddt and dA: `entering_fwd[b,c]` is the state before chunk c (first pass), `entering_rev[b,r]` the adjoint
 * state before reversed chunk r (second pass), i.e. behind chunk nc-1-r in time order.  Writes both as bfloat16
 * with chunks in time order (rev_bf16[b,c] = entering_rev[b,nc-1-c]) and
 *   anchor[b,c-1,h] = <entering_rev[b,nc-c,h], entering_fwd[b,c,h]>   for c = 1..nc-1,
 * every input read once.  `dim` = headdim * nstate.  No counterpart in the reference (see ssm_ssd_bwd_gate). */
typedef struct ssm_ssd_bwd_states_args {
  const float *entering_fwd;   /* (B, nc, H, dim) fp32 */
  const float *entering_rev;   /* (B, nc, H, dim) fp32 */
  void *fwd_bf16;              /* (B, nc, H, dim) bf16 */
  void *rev_bf16;              /* (B, nc, H, dim) bf16 */
  float *anchor;               /* (B, nc-1, H) fp32; may be NULL when nc == 1 */
  int32_t batch, nchunks, heads, dim;
} ssm_ssd_bwd_states_args;
int ssm_ssd_bwd_states(const ssm_ssd_bwd_states_args *args, void *hip_stream);

/* out[row][:] = x[row][:] * w[row], the product formed in float32 and rounded once to `out_dtype`: the operand
 * dt x of the backward's first pass.  `cols` a multiple of 4.  No counterpart in the reference. */
typedef struct ssm_ssd_scale_rows_args {
  const void *x;             /* (rows, cols) x_dtype */
  const float *w;            /* (rows,) fp32 */
  void *out;                 /* (rows, cols) out_dtype */
  int64_t rows;
  int32_t cols;
  int32_t x_dtype, out_dtype;   /* out_dtype: SSM_F32 or SSM_BF16 */
} ssm_ssd_scale_rows_args;
int ssm_ssd_scale_rows(const ssm_ssd_scale_rows_args *args, void *hip_stream);

/* What the gradient of the combined forward derives from the raw steps alone, in one launch (whole chunks):
 *   dt_out / dt_rows  the effective step (bias, softplus, clamp), chunked (B, H, nc, Q) and by rows (B, L, H)
 *   dA_cumsum         its running sum times A inside the chunk, as ssm_ssd_chunk_cumsum gives it
 *   dA_cumsum_rev     the same for the time-reversed sequence in which a step decays by the factor of the step that
 *                     follows it in time (position i of reversed chunk nc-1-c is step cQ + Q-1-i)
 *   w_dy[t] = exp(dA_cumsum at t),  w_x[t] = dt[t] * exp(dA_cumsum_rev at t's reversed position)
 * The published backward takes these inside its kernels (_chunk_scan_bwd_* of the mamba_ssm package the reference's
 * goldens come from, scripts/refresh_mamba_goldens.py:591-604); no single counterpart in the reference. */
typedef struct ssm_ssd_bwd_prep_args {
  const void *dt;            /* (B, L, H) dt_dtype: raw steps */
  const float *A;            /* (H,) */
  const float *dt_bias;      /* (H,) or NULL */
  float *dA_cumsum;          /* (B, H, nc, Q) */
  float *dt_out;             /* (B, H, nc, Q) */
  float *dA_cumsum_rev;      /* (B, H, nc, Q) */
  float *dt_rows;            /* (B, L, H) */
  float *w_dy;               /* (B, L, H) */
  float *w_x;                /* (B, L, H) */
  int32_t batch, seqlen, heads, chunk;
  int32_t dt_dtype, dt_softplus;
  float dt_min, dt_max;
} ssm_ssd_bwd_prep_args;
int ssm_ssd_bwd_prep(const ssm_ssd_bwd_prep_args *args, void *hip_stream);

/* The per-step scalars of the gradient of the combined forward (see ssm_ssd_bwd_gate), chunk by chunk:
 *   q[l]   = q_c + sum_{j<l in chunk} (s1[j] - s2[j]),  q_c = q0 for the first chunk and
 *            exp(dt A) at the chunk's first step (0 at the first step of a packed sequence) times anchor[c-1] after it
 *   ddt[l] = (A q[l] + xu[l]) * slope,  slope = sigmoid(raw) under softplus (else 1), 0 outside [dt_min, dt_max]
 *   dA_part[b,c,h] = sum_l dt[l] q[l],   dbias_part[b,c,h] = sum_l ddt[l]      (raw = dt_raw + dt_bias)
 * seqlen must be a multiple of chunk. */
typedef struct ssm_ssd_bwd_dt_args {
  const float *s1, *s2, *xu;       /* (B, L, H) fp32: outputs of ssm_ssd_bwd_dx / ssm_ssd_bwd_gate */
  const float *dt;                 /* (B, L, H) fp32: the step after bias, softplus and clamp */
  const void *dt_raw;              /* (B, L, H) dt_dtype: the step as given to the forward */
  const float *A;                  /* (H,) */
  const float *dt_bias;            /* (H,) or NULL */
  const float *q0;                 /* (B, H) or NULL (zero) */
  const float *anchor;             /* (B, nc-1, H); may be NULL with a single chunk */
  const uint8_t *first_step;       /* (B, L) nonzero at the first step of a packed sequence, or NULL */
  float *ddt;                      /* (B, L, H) fp32 */
  float *dA_part, *dbias_part;     /* (B, nc, H) fp32 */
  int32_t batch, seqlen, heads, chunk;
  int32_t dt_dtype, dt_softplus;
  float dt_min, dt_max;
} ssm_ssd_bwd_dt_args;
int ssm_ssd_bwd_dt(const ssm_ssd_bwd_dt_args *args, void *hip_stream);

/* ------------------------------------------------------------------------
 * depthwise causal conv1d (+ optional SiLU).
 * Forward stands behind `dw_causal_conv(x, weight, bias, activation)`
 * (src/ssm/ops/__init__.py:1594-1600; semantics reference.py:466-537);
 * backward behind `dw_causal_conv_backward(grad_out, x, weight, bias,
 * activation)` (formulas: src/ssm/ops/cpu/dw_causal_conv.cpp:161-204).
 * ---------------------------------------------------------------------- */

typedef struct ssm_conv1d_fwd_args {
  const void *x;          /* (B,C,L) or (B,L,C), io dtype */
  const float *weight;    /* (C, K) fp32 */
  const float *bias;      /* (C,) fp32 or NULL */
  void *y;                /* same layout and dtype as x (SSM_LAYOUT_ROWS_TO_BCL: dense (B,C,L)) */
  int32_t batch, channels, seqlen, width;
  int32_t io_dtype, layout, activation;
  int32_t pad0;
  int64_t x_batch_stride, x_row_stride;   /* elements; SSM_LAYOUT_ROWS_TO_BCL only, zero otherwise */
} ssm_conv1d_fwd_args;

int ssm_conv1d_fwd(const ssm_conv1d_fwd_args *args, void *hip_stream);

typedef struct ssm_conv1d_bwd_args {
  const void *x;          /* forward input */
  const void *dout;       /* gradient of y, same layout/dtype as x (SSM_LAYOUT_ROWS_TO_BCL: dense (B,C,L)) */
  const float *weight;
  const float *bias;      /* or NULL (needed to rebuild the pre-activation) */
  void *dx;               /* same layout/dtype as x (SSM_LAYOUT_ROWS_TO_BCL: dense (B,L,C) rows) */
  float *dweight;         /* (C, K) fp32 */
  float *dbias;           /* (C,) fp32 or NULL */
  void *workspace;        /* ssm_conv1d_bwd_workspace_bytes() bytes of device memory */
  size_t workspace_bytes;
  int32_t batch, channels, seqlen, width;
  int32_t io_dtype, layout, activation;
  int32_t pad0;
  int64_t x_batch_stride, x_row_stride;   /* elements; SSM_LAYOUT_ROWS_TO_BCL only, zero otherwise */
} ssm_conv1d_bwd_args;

size_t ssm_conv1d_bwd_workspace_bytes(int batch, int channels, int width);
int ssm_conv1d_bwd(const ssm_conv1d_bwd_args *args, void *hip_stream);

/* ------------------------------------------------------------------------
 * A dense (B,C,L) copy of a (B,C,L)-shaped view whose memory runs channels innermost (rows of channels, one row per
 * time step): what `tensor.contiguous()` does in the reference's Python path (src/ssm/ops/python/reference.py has no
 * layout demands, its kernels' wrappers call `.contiguous()`), and what the reference's blocks hand the scan --
 * `delta = F.linear(...).permute(0, 2, 1)`, `z = gate.permute(0, 2, 1)` (src/ssm/modules/mamba1.py:223-228).  The
 * scan walks time, so those views are copied; this entry point is that copy at the speed of the memory.
 * ---------------------------------------------------------------------- */
typedef struct ssm_rows_to_bcl_args {
  const void *src;          /* element (b, c, t) at src[b * src_batch_stride + t * src_row_stride + c] */
  void *dst;                /* (B, C, L) dense, same element size */
  int64_t src_batch_stride, src_row_stride;   /* elements; multiples of 4, rows do not overlap */
  int32_t batch, channels, seqlen;            /* channels a multiple of 4 */
  int32_t element_size;                       /* 2 or 4 bytes */
} ssm_rows_to_bcl_args;
int ssm_rows_to_bcl(const ssm_rows_to_bcl_args *args, void *hip_stream);

/* ------------------------------------------------------------------------
 * residual-add + LayerNorm / RMSNorm over the last axis of (rows, hidden).
 * Forward stands behind `fused_layer_norm(x, weight, bias, residual, is_rms,
 * eps, prenorm, residual_in_fp32)` (src/ssm/ops/__init__.py:1640-1652;
 * semantics reference.py:540-609) and can additionally emit the pre-norm sum
 * (`residual_out`) and the row statistics; backward stands behind
 * `fused_layer_norm_backward` (formulas: src/ssm/ops/cpu/layer_norm.cpp:277-336).
 * ---------------------------------------------------------------------- */
typedef struct ssm_norm_fwd_args {
  const void *x;            /* (rows, hidden) x dtype */
  const void *residual;     /* (rows, hidden) residual dtype, or NULL */
  const float *weight;      /* (hidden,) fp32 */
  const float *bias;        /* (hidden,) fp32 or NULL */
  void *y;                  /* (rows, hidden) x dtype */
  void *residual_out;       /* (rows, hidden) residual_out dtype, or NULL: x (+ residual if prenorm) */
  float *mean;              /* (rows,) or NULL (written as 0 for RMSNorm) */
  float *rstd;              /* (rows,) or NULL */
  int32_t rows, hidden;
  int32_t x_dtype, residual_dtype, residual_out_dtype;
  int32_t is_rms, prenorm;
  float eps;
} ssm_norm_fwd_args;

int ssm_norm_fwd(const ssm_norm_fwd_args *args, void *hip_stream);

typedef struct ssm_norm_bwd_args {
  const void *x;
  const void *residual;     /* or NULL */
  const void *dy;           /* (rows, hidden) x dtype */
  const float *weight;
  const float *mean;        /* (rows,) from the forward pass (ignored for RMSNorm) */
  const float *rstd;        /* (rows,) from the forward pass */
  void *dx;                 /* (rows, hidden) x dtype */
  void *dresidual;          /* (rows, hidden) residual dtype, or NULL */
  float *dweight;           /* (hidden,) fp32 */
  float *dbias;             /* (hidden,) fp32 or NULL */
  void *workspace;          /* ssm_norm_bwd_workspace_bytes() bytes of device memory */
  size_t workspace_bytes;
  int32_t rows, hidden;
  int32_t x_dtype, residual_dtype;
  int32_t is_rms, prenorm;
} ssm_norm_bwd_args;

size_t ssm_norm_bwd_workspace_bytes(int rows, int hidden);
int ssm_norm_bwd(const ssm_norm_bwd_args *args, void *hip_stream);

/* ssm_norm_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving or
 * training loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The partial column
 * sums go to a buffer of SSM_NORM_BWD_STATIC_BYTES that is part of the library's code object (each GPU the
 * library runs on holds one until the process ends) instead of `workspace`, whose two fields are ignored; the call
 * allocates and frees nothing, and its results are bit-identical to ssm_norm_bwd's.  Calls whose partial sums
 * do not fit -- min(1024, ceil(rows / 4)) x 2 x hidden floats for hidden <= 8192 -- return SSM_ERR_TOO_LARGE.
 * All calls on one GPU share the buffer: calls that overlap there (two streams, two threads) race; calls on one
 * stream are ordered and safe.  The first call on a device looks the buffer's address up and must not happen
 * while a stream is being captured. */
#define SSM_NORM_BWD_STATIC_BYTES (8u << 20)
int ssm_norm_bwd_static(const ssm_norm_bwd_args *args, void *hip_stream);

/* -------------------------------------------------------------------------
 * The five operators in double precision.
 *
 * The reference computes in the promoted type of its inputs (src/ssm/ops/python/reference.py:9-19, :135-137:
 * float64 tensors, or a float64 `A`, make float64 the compute type) and runs torch.autograd.gradcheck in float64
 * on the device against every operator of a compiled backend (tests/ops/test_backend_gradients.py:1172-1201
 * selective_scan, :1291-1321 selective_state_step, :1416-1447 ssd_chunk_scan, :1497-1517 dw_causal_conv,
 * :1578-1612 fused_layer_norm).  These entry points serve such calls: every tensor is `double`, all arithmetic is
 * double, nothing is allocated, results are the same bits on every run.  They are plain kernels (one thread per
 * independent recurrence), not tuned ones.
 *
 * Projections that the reference broadcasts are passed as views: a base pointer and element strides over the
 * full index space, 0 on a broadcast axis.  Gradients of such operands are written dense over the full index
 * space and summed over the broadcast axes by the caller; gradients of per-channel parameters are written as one
 * row per batch entry (`*_rows`) and summed over the batch by the caller.  Each struct serves the forward and
 * the backward entry; a forward call ignores the backward's fields.
 * ---------------------------------------------------------------------- */
typedef struct ssm_f64_scan_args {   /* reference.py:88-197 */
  const double *u, *delta;           /* (B, D, L) */
  const double *z;                   /* (B, D, L) or NULL */
  const double *A;                   /* (D, N) */
  const double *Bproj, *Cproj;       /* views over (B, D, N, L) */
  const double *Dskip, *dt_bias;     /* (D,) or NULL */
  double *out;                       /* (B, D, L) */
  double *last_state;                /* (B, D, N): the final state; required (it is the running state); the backward
                                        entry uses it as scratch */
  int64_t b_stride[4], c_stride[4];  /* element strides of Bproj / Cproj over (B, D, N, L) */
  /* backward */
  const double *dout;                /* (B, D, L) */
  const double *dlast_state;         /* (B, D, N) or NULL */
  double *states;                    /* scratch (B, D, L, N) */
  double *ypre;                      /* scratch (B, D, L) */
  double *du, *ddelta;               /* (B, D, L) */
  double *dz;                        /* (B, D, L); required with z */
  double *dA_rows;                   /* (B, D, N) */
  double *dB, *dC;                   /* dense (B, D, N, L) */
  double *dD_rows, *dbias_rows;      /* (B, D) or NULL */
  int32_t batch, dim, seqlen, nstate, delta_softplus;
} ssm_f64_scan_args;
int ssm_f64_scan_fwd(const ssm_f64_scan_args *args, void *hip_stream);
int ssm_f64_scan_bwd(const ssm_f64_scan_args *args, void *hip_stream);

typedef struct ssm_f64_step_args {   /* reference.py:200-312 */
  double *state;                     /* (B, D, N): updated in place by the forward; the state before the step for the backward */
  const double *x, *dt;              /* (B, D) */
  const double *z;                   /* (B, D) or NULL */
  const double *A;                   /* (D, N) */
  const double *Bproj, *Cproj;       /* views over (B, D, N) */
  const double *Dskip, *dt_bias;     /* (D,) or NULL */
  double *out;                       /* (B, D) */
  int64_t b_stride[3], c_stride[3];
  /* backward */
  const double *dout;                /* (B, D) or NULL */
  const double *dstate_new;          /* (B, D, N) gradient of the updated state, or NULL */
  double *dstate;                    /* (B, D, N) */
  double *dx, *ddt;                  /* (B, D); ddt is also the bias gradient's rows */
  double *dz;                        /* (B, D); required with z */
  double *dA_rows, *dB, *dC;         /* (B, D, N) */
  double *dD_rows;                   /* (B, D) or NULL */
  int32_t batch, dim, nstate, dt_softplus;
} ssm_f64_step_args;
int ssm_f64_state_step(const ssm_f64_step_args *args, void *hip_stream);
int ssm_f64_state_step_bwd(const ssm_f64_step_args *args, void *hip_stream);

typedef struct ssm_f64_dscan_args {  /* reference.py:315-480 */
  const double *X;                   /* (B, L, H, P) */
  const double *dt;                  /* (B, L, H) */
  const double *A;                   /* (H, P) */
  const double *Bproj, *Cproj;       /* views over (B, L, H, P) */
  const double *Dskip;               /* (H, P) or NULL */
  const double *z;                   /* view over (B, L, H, P), or NULL */
  const double *init;                /* (B, H, P) or NULL */
  const int32_t *lengths;            /* (B,) valid steps per row, or NULL */
  double *Y;                         /* (B, L, H, P) */
  int64_t b_stride[4], c_stride[4], z_stride[4];
  /* backward */
  const double *dY;                  /* (B, L, H, P) */
  double *states;                    /* scratch (B, L, H, P) */
  double *dX, *ddt_rows, *dB, *dC;   /* dense (B, L, H, P); ddt_rows is summed over P by the caller */
  double *dz;                        /* dense (B, L, H, P); required with z */
  double *dA_rows;                   /* (B, H, P) */
  double *dD_rows, *dinit;           /* (B, H, P) or NULL */
  int32_t batch, seqlen, heads, hdim;
} ssm_f64_dscan_args;
int ssm_f64_dscan_fwd(const ssm_f64_dscan_args *args, void *hip_stream);
int ssm_f64_dscan_bwd(const ssm_f64_dscan_args *args, void *hip_stream);

typedef struct ssm_f64_conv_args {   /* reference.py:483-533 */
  const double *x;                   /* view over (B, C, L): either layout */
  const double *weight;              /* (C, K) */
  const double *bias;                /* (C,) or NULL */
  double *y;                         /* view over (B, C, L) */
  int64_t x_stride[3], y_stride[3];
  /* backward */
  const double *dy;                  /* view over (B, C, L) */
  double *dx;                        /* view over (B, C, L) */
  int64_t dy_stride[3], dx_stride[3];
  double *dpre;                      /* scratch, dense (B, C, L) */
  double *dw;                        /* (C, K) */
  double *db;                        /* (C,) or NULL */
  int32_t batch, channels, seqlen, width, activation;   /* ssm_activation */
} ssm_f64_conv_args;
int ssm_f64_conv_fwd(const ssm_f64_conv_args *args, void *hip_stream);
int ssm_f64_conv_bwd(const ssm_f64_conv_args *args, void *hip_stream);

typedef struct ssm_f64_norm_args {   /* reference.py:536-609 */
  const double *x;                   /* (rows, hidden) */
  const double *residual;            /* (rows, hidden) or NULL */
  const double *weight;              /* (hidden,) */
  const double *bias;                /* (hidden,) or NULL */
  double *y;                         /* (rows, hidden) */
  double *residual_out;              /* (rows, hidden) or NULL: x (+ residual if prenorm) */
  double *mean, *rstd;               /* (rows,): written by the forward, read by the backward */
  /* backward */
  const double *dy;                  /* (rows, hidden) */
  double *dx;                        /* (rows, hidden) */
  double *dresidual;                 /* (rows, hidden) or NULL */
  double *dw;                        /* (hidden,) */
  double *db;                        /* (hidden,) or NULL */
  int64_t rows;
  int32_t hidden, is_rms, prenorm;
  double eps;
} ssm_f64_norm_args;
int ssm_f64_norm_fwd(const ssm_f64_norm_args *args, void *hip_stream);
int ssm_f64_norm_bwd(const ssm_f64_norm_args *args, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* SSM_AMD_H */
