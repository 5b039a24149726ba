// Parameter blocks shared by the state-space-duality (Mamba-2) kernels.
//
// Tensor layouts (row-major):
//   x, z, y        (B, L, H, P)        dt (B, L, H)       A (H,)
//   Bm, Cm         (B, L, G, N)        head h reads group h / (H/G)
//   dt_out, dA_cs  (B, H, nc, Q) fp32  (chunked step and its running sum times A)
//   CB             (B, nc, G, Q, Q)    CB[l][s] = <C_l, B_s>
//   states         (B, nc, H, P, N)    per-chunk contribution / state entering a chunk
//   final_states   (B, H, P, N) fp32
#pragma once
#include "common.hpp"

namespace ssm {

struct SsdDims {
  int batch, len, heads, hdim, groups, nstate, chunk, nchunks;
};

struct SsdCumsumParams {
  const void *dt;
  const float *A, *bias;
  float *dA_cs, *dt_out;
  SsdDims d;
  int dt_dtype, softplus;
  float dt_min, dt_max;
};

struct SsdBmmParams {
  const void *a, *b;          // (B, L, G, K)
  const int *seq_idx;         // (B, L) or null
  void *out;                  // (B, nc, G, Q, Q)
  int batch, len, groups, kdim, chunk, nchunks;
  int in_dtype, out_dtype, causal;
};

struct SsdStateParams {
  const void *Bm, *x;
  const float *dt, *dA_cs;
  void *states;
  void *scratch;              // optional device scratch for the MFMA path (transposed B)
  size_t scratch_bytes;
  SsdDims d;
  int x_dtype, b_dtype, states_dtype;
  const int *seq_idx;         // (B, L) or null
  const float *x_scale;       // (B, H, nc, Q) or null: x stands for x * scale rounded to x's type (matrix-core kernels only)
  int x_reversed;             // x is given in forward time while the call walks reversed time: step tau reads row L-1-tau
};

struct SsdPassParams {
  const void *states;         // (B, nc, H, dim)
  const float *dA_last;       // (B, H, nc)
  const float *init;          // (B, H, dim) or null
  void *out;                  // (B, nc, H, dim): state entering each chunk
  float *final_states;        // (B, H, dim)
  int batch, nchunks, heads, dim;
  int states_dtype;
  int len, chunk;             // only read with seq_idx
  const int *seq_idx;         // (B, L) or null
};

// In place of y, the matrix-core chunk_scan of the backward's time-reversed pass can finish dx itself: with u its
// own result at reversed step tau (forward step t = L-1-tau) and dy its operand x,
//   dx_t = dt_t u + D dy,   xu_t = sum_p x_t u,   s1_t = sum_p round(dt_t x_t) u
// (what ssm_ssd_bwd_dx computes from u written out in float32).
struct SsdDxEpilogue {
  const void *x;              // (B, L, H, P) of the pass's element type, forward time
  const float *dt;            // (B, L, H)
  const float *Dk;            // (H,) / (H, P) or null
  void *dx;                   // (B, L, H, P) float32 or the element type; null: no such epilogue
  float *xu, *s1;             // (B, L, H)
  int d_per_p, dx_f32, round_dtx;
};

struct SsdScanParams {
  const void *CB, *Cm, *x, *z, *prev;
  const float *dt, *dA_cs, *Dk;
  void *y;
  SsdDims d;
  int x_dtype, c_dtype, cb_dtype, states_dtype, z_dtype;
  int d_per_p;                // D is (H, P) instead of (H,)
  const int *seq_idx;         // (B, L) or null
  int y_dtype;                // x_dtype, or SSM_F32 on request
  const float *x_scale;       // (B, H, nc, Q) or null: x stands for x * scale rounded to x's type (matrix-core kernels only)
  SsdDxEpilogue dx;
  int x_reversed;             // as in SsdStateParams
};

__device__ __forceinline__ void store_any(void *p, int dtype, size_t i, float v) {
  if (dtype == SSM_F32) reinterpret_cast<float *>(p)[i] = v;
  else if (dtype == SSM_BF16) reinterpret_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else reinterpret_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
}

// exp(min(v, 0)): decay factors inside a chunk never exceed 1 when A <= 0; the
// clamp only matters for (unphysical) positive A and mirrors the published kernels.
__device__ __forceinline__ float decay_exp(float v) { return exp2_hw(fminf(v, 0.0f) * LOG2E); }

// ---- bf16 MFMA helpers (v_mfma_f32_32x32x16_bf16) ----
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

__device__ __forceinline__ f32x16_t mma(bf16x8_t a, bf16x8_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8_t load_frag(const void *p) { return *reinterpret_cast<const bf16x8_t *>(p); }

__device__ __forceinline__ bf16x8_t pack8(const float (&v)[8]) {
  bf16x8_t r;
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = (__bf16)v[j];
  return r;
}

__device__ __forceinline__ void unpack8(bf16x8_t r, float (&v)[8]) {
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (float)r[j];
}

// ---- the same for float16 operands (v_mfma_f32_32x32x16_f16), and the element type as a parameter ----
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;

__device__ __forceinline__ f32x16_t mma(f16x8_t a, f16x8_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ void unpack8(f16x8_t r, float (&v)[8]) {
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (float)r[j];
}
template <typename E> struct Vec8;
template <> struct Vec8<__bf16> { using type = bf16x8_t; };
template <> struct Vec8<_Float16> { using type = f16x8_t; };
template <typename E> using V8 = typename Vec8<E>::type;
template <typename E>
__device__ __forceinline__ V8<E> load_frag_e(const void *p) { return *reinterpret_cast<const V8<E> *>(p); }
// Four neighbouring 16-bit elements (8 bytes, 8-byte aligned) to and from float32.
template <typename E>
__device__ __forceinline__ void load4_e(const E *p, float (&v)[4]) {
  typedef __attribute__((__vector_size__(4 * sizeof(E)))) E vec4_t;
  const vec4_t r = *reinterpret_cast<const vec4_t *>(p);
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = (float)r[j];
}
template <typename E>
__device__ __forceinline__ void store4_e(E *p, const float (&v)[4]) {
  typedef __attribute__((__vector_size__(4 * sizeof(E)))) E vec4_t;
  vec4_t r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r[j] = (E)v[j];
  *reinterpret_cast<vec4_t *>(p) = r;
}
template <typename E>
__device__ __forceinline__ V8<E> pack8_e(const float (&v)[8]) {
  V8<E> r;
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = (E)v[j];
  return r;
}

// Row of C-layout register r for a lane in half g = lane / 32.
__device__ __forceinline__ int crow(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

// MFMA variants, defined in ssd_mfma.hip; return false when the shape is not covered.
bool ssd_bmm_mfma(const SsdBmmParams &p, hipStream_t s);
bool ssd_chunk_state_mfma(const SsdStateParams &p, hipStream_t s);
size_t ssd_chunk_state_scratch_bytes(const SsdDims &d);
bool ssd_chunk_scan_mfma(const SsdScanParams &p, hipStream_t s);
// Float32 matrix-core variants for all other dtypes and shapes, defined in ssd_tiled.hip; false when the
// chunk is too long for their LDS arrays.
bool ssd_bmm_tiled(const SsdBmmParams &p, hipStream_t s);
bool ssd_chunk_state_tiled(const SsdStateParams &p, hipStream_t s);
bool ssd_chunk_scan_tiled(const SsdScanParams &p, hipStream_t s);
void note_mfma_launch(int bits);   // recorded for ssm_ssd_mfma_launches()

}  // namespace ssm
