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

#define SSM_AMD_ABI_VERSION 1

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
  int32_t batch, dim, seqlen, nstate;
  int32_t io_dtype;       /* ssm_dtype of u, delta, z, out, last_state */
  int32_t bc_dtype;       /* ssm_dtype of Bproj and Cproj */
  int32_t b_kind, c_kind; /* ssm_proj_kind */
  int32_t b_groups, c_groups; /* G for SSM_PROJ_BGNL (must divide D), else ignored */
  int32_t delta_softplus; /* 0 / 1 */
  int32_t tune_items;     /* 0 = automatic; else time steps per lane (4, 8 or 16) */
} ssm_scan_fwd_args;

int ssm_scan_fwd(const ssm_scan_fwd_args *args, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* SSM_AMD_H */
