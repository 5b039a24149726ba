// Single-token selective state update (decode step) for gfx950.
//
//   dt'   = softplus(dt + dt_bias)
//   h'    = exp(dt' A) h + dt' x B          (state overwritten in place)
//   y     = <h', C> + D x ;  y *= silu(z)
//
// The op moves 2 * B*D*N state elements and little else, so it is laid out
// for HBM streaming: TPR lanes share one (batch, channel) row, each lane owns
// VEC consecutive state entries per trip (128-bit accesses when VEC = 4), and
// the partial dot products are combined with a butterfly inside the wave.
#include "common.hpp"

#include <type_traits>

namespace ssm {

struct StepParams {
  void *state;
  const void *x, *dt, *z, *Bp, *Cp;
  const float *A, *Dk, *bias;
  void *out;
  int batch, dim, nstate;
  int io_dtype, bc_dtype;
  int b_kind, c_kind, b_groups, c_groups;
  int softplus;
  int tpr_log2;   // lanes per row = 1 << tpr_log2
  long long z_bs, b_bs, c_bs;   // elements between batch rows of z and of grouped B / C (dense: dim, groups * nstate)
  // fused causal-conv front end (decode): x is the raw input, the conv window is rolled in place
  void *conv_state;          // (B, D, K) io dtype or null
  const float *conv_w;       // (D, K)
  const float *conv_b;       // (D,) or null
  void *conv_out;            // (B, D) io dtype or null: the activated conv output fed to the step
  int conv_k, conv_silu;
};

__device__ __forceinline__ void store_from_f32(void *p, int dtype, size_t i, float v) {
  if (dtype == SSM_F32) reinterpret_cast<float *>(p)[i] = v;
  else if (dtype == SSM_BF16) reinterpret_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else reinterpret_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
}

template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const T *p, float (&v)[VEC]) {
  Pack<T, VEC> raw = *reinterpret_cast<const Pack<T, VEC> *>(p);
#pragma unroll
  for (int i = 0; i < VEC; ++i) v[i] = to_f32(raw.v[i]);
}

template <int VEC>
__device__ __forceinline__ void load_vec_rt(const void *p, int dtype, size_t off, float (&v)[VEC]) {
  if (dtype == SSM_F32) load_vec<float, VEC>(reinterpret_cast<const float *>(p) + off, v);
  else if (dtype == SSM_BF16) load_vec<bf16_t, VEC>(reinterpret_cast<const bf16_t *>(p) + off, v);
  else load_vec<f16_t, VEC>(reinterpret_cast<const f16_t *>(p) + off, v);
}

// Accesses of the activations and projections.  io_t = void: the element type is looked up at run time
// (any mix of dtypes); otherwise x, dt, z, B, C, the conv window and the outputs all have type io_t and
// the reads of a thread are straight-line code that the compiler issues together.
template <typename io_t>
__device__ __forceinline__ float ld_io(const void *p, int dtype, size_t i) {
  if constexpr (std::is_void<io_t>::value) return load_as_f32(p, dtype, i);
  else return to_f32(reinterpret_cast<const io_t *>(p)[i]);
}
template <typename io_t>
__device__ __forceinline__ void st_io(void *p, int dtype, size_t i, float v) {
  if constexpr (std::is_void<io_t>::value) store_from_f32(p, dtype, i, v);
  else reinterpret_cast<io_t *>(p)[i] = from_f32<io_t>(v);
}
template <typename io_t, int VEC>
__device__ __forceinline__ void ld_vec_io(const void *p, int dtype, size_t off, float (&v)[VEC]) {
  if constexpr (std::is_void<io_t>::value) load_vec_rt<VEC>(p, dtype, off, v);
  else load_vec<io_t, VEC>(reinterpret_cast<const io_t *>(p) + off, v);
}
template <typename io_t>
__device__ __forceinline__ float round_io(float v, int dtype) {
  if constexpr (std::is_void<io_t>::value) {
    if (dtype == SSM_BF16) return to_f32(from_f32<bf16_t>(v));
    if (dtype == SSM_F16) return to_f32(from_f32<f16_t>(v));
    return v;
  } else {
    return to_f32(from_f32<io_t>(v));
  }
}

template <typename state_t, int VEC>
__global__ __launch_bounds__(256) void state_step_kernel(const StepParams p) {
  const int tpr = 1 << p.tpr_log2;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t row = gid >> p.tpr_log2;
  const int sub = (int)(gid & (tpr - 1));
  const size_t nrows = (size_t)p.batch * p.dim;
  const bool live = row < nrows;
  const size_t r = live ? row : 0;          // dead lanes shadow row 0 but never store
  const int b = (int)(r / p.dim), d = (int)(r % p.dim);
  const int N = p.nstate;

  size_t b_off, c_off;
  if (p.b_kind == SSM_PROJ_BGNL) b_off = (size_t)b * p.b_bs + (size_t)(d / (p.dim / p.b_groups)) * N;
  else b_off = ((p.b_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
  if (p.c_kind == SSM_PROJ_BGNL) c_off = (size_t)b * p.c_bs + (size_t)(d / (p.dim / p.c_groups)) * N;
  else c_off = ((p.c_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
  state_t *srow = reinterpret_cast<state_t *>(p.state) + r * N;
  const float *arow = p.A + (size_t)d * N;

  // The first trip's operands are requested before anything else: they do not depend on the
  // conv front end, and the compiler cannot move these reads above the window stores by itself.
  const int n_first = sub * VEC;
  const bool first_ok = n_first < N;
  float h0[VEC], a0[VEC], bv0[VEC], cv0[VEC];
  if (first_ok) {
    load_vec<state_t, VEC>(srow + n_first, h0);
    load_vec<float, VEC>(arow + n_first, a0);
    load_vec_rt<VEC>(p.Bp, p.bc_dtype, b_off + n_first, bv0);
    load_vec_rt<VEC>(p.Cp, p.bc_dtype, c_off + n_first, cv0);
  }

  float dtv = load_as_f32(p.dt, p.io_dtype, r);
  if (p.bias) dtv += p.bias[d];
  float xv = load_as_f32(p.x, p.io_dtype, r);
  const float zv = p.z ? load_as_f32(p.z, p.io_dtype, (size_t)b * p.z_bs + d) : 0.0f;
  if (p.softplus) dtv = softplus_f32(dtv);
  if (p.conv_state) {
    // window <- (window[1:], x); x <- act(bias + sum_k w[k] window[k]).  The row's lanes
    // share the taps; every lane loads before any lane of the row stores.
    const int K = p.conv_k;
    float part = 0.0f;
    for (int k0 = 0; k0 < K; k0 += tpr) {
      const int k = k0 + sub;
      float v = 0.0f;
      if (k < K) {
        v = (k < K - 1) ? load_as_f32(p.conv_state, p.io_dtype, r * K + k + 1) : xv;
        part = __builtin_fmaf(v, p.conv_w[(size_t)d * K + k], part);
      }
      if (live && k < K) store_from_f32(p.conv_state, p.io_dtype, r * K + k, v);
    }
    for (int m = tpr >> 1; m >= 1; m >>= 1) part += __shfl_xor(part, m, WAVE);
    if (p.conv_b) part += p.conv_b[d];
    xv = p.conv_silu ? silu_f32(part) : part;
    // the step consumes what a separate conv kernel would have written in the io dtype
    if (p.io_dtype == SSM_BF16) xv = to_f32(from_f32<bf16_t>(xv));
    else if (p.io_dtype == SSM_F16) xv = to_f32(from_f32<f16_t>(xv));
    if (p.conv_out && live && sub == 0) store_from_f32(p.conv_out, p.io_dtype, r, xv);
  }
  const float dx = dtv * xv;
  const float dt2 = dtv * LOG2E;

  float acc = 0.0f;
  for (int n0 = n_first; n0 < N; n0 += tpr * VEC) {
    float h[VEC], a[VEC], bv[VEC], cv[VEC];
    if (n0 == n_first) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        h[i] = h0[i]; a[i] = a0[i]; bv[i] = bv0[i]; cv[i] = cv0[i];
      }
    } else {
      load_vec<state_t, VEC>(srow + n0, h);
      load_vec<float, VEC>(arow + n0, a);
      load_vec_rt<VEC>(p.Bp, p.bc_dtype, b_off + n0, bv);
      load_vec_rt<VEC>(p.Cp, p.bc_dtype, c_off + n0, cv);
    }
    Pack<state_t, VEC> outv;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float hn = __builtin_fmaf(exp2_hw(dt2 * a[i]), h[i], dx * bv[i]);
      acc = __builtin_fmaf(hn, cv[i], acc);
      outv.v[i] = from_f32<state_t>(hn);
    }
    if (live) *reinterpret_cast<Pack<state_t, VEC> *>(srow + n0) = outv;
  }
  for (int m = tpr >> 1; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, WAVE);
  if (live && sub == 0) {
    float y = acc;
    if (p.Dk) y = __builtin_fmaf(p.Dk[d], xv, y);
    if (p.z) y *= silu_f32(zv);
    store_from_f32(p.out, p.io_dtype, r, y);
  }
}

// Variant for the common decode shapes (N = 4 * lanes-per-row, lanes-per-row in {4, 8, 16},
// batch divisible by RB): a thread keeps what depends only on the channel (its four entries of
// A, dt_bias, D, its conv tap) in registers and walks RB batch rows with them, which removes a
// third of the cache traffic (A is as large as the state) and most of the small reads.  The three
// per-row scalars x, dt, z are fetched by lanes 0, 1, 2 of the row with one instruction and
// shared through the wave.
template <typename state_t, typename io_t, bool CONV, int RB>
__global__ __launch_bounds__(256) void state_step_rb_kernel(const StepParams p) {
  constexpr int VEC = 4;
  const int tpr = 1 << p.tpr_log2;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t col = gid >> p.tpr_log2;
  const int sub = (int)(gid & (tpr - 1));
  const size_t ncols = (size_t)p.dim * (p.batch / RB);
  const bool live = col < ncols;
  const unsigned cc = live ? (unsigned)col : 0u;          // batch * dim < 2^27: 32-bit index arithmetic
  const int d = (int)(cc % (unsigned)p.dim), bg = (int)(cc / (unsigned)p.dim);
  const int N = p.nstate, n0 = sub * VEC;
  const int lane = lane_id(), base = lane & ~(tpr - 1);

  float a[VEC];
  load_vec<float, VEC>(p.A + (size_t)d * N + n0, a);
  const float bias = p.bias ? p.bias[d] : 0.0f;
  const float Dk = p.Dk ? p.Dk[d] : 0.0f;
  const int K = p.conv_k;
  float tap = 0.0f;
  if (CONV) {
    tap = p.conv_w[(size_t)d * K + min(sub, K - 1)];
    if (sub >= K) tap = 0.0f;
  }
  const float cbias = (CONV && p.conv_b) ? p.conv_b[d] : 0.0f;
  // every lane reads one of the row's scalars (lanes past the third repeat x): no lane-dependent branch
  const void *scal_ptr = sub == 1 ? p.dt : (sub == 2 && p.z ? p.z : p.x);
  const int bgrp = p.b_kind == SSM_PROJ_BGNL ? d / (p.dim / p.b_groups) : 0;
  const int cgrp = p.c_kind == SSM_PROJ_BGNL ? d / (p.dim / p.c_groups) : 0;
  const int win_k = min(sub + 1, max(K - 1, 0));

  float h[RB][VEC], bv[RB][VEC], cv[RB][VEC], scal[RB], win[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int b = bg * RB + rb;
    const size_t r = (size_t)b * p.dim + d;
    const size_t b_off = p.b_kind == SSM_PROJ_BGNL ? (size_t)b * p.b_bs + (size_t)bgrp * N
                                                    : ((p.b_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
    const size_t c_off = p.c_kind == SSM_PROJ_BGNL ? (size_t)b * p.c_bs + (size_t)cgrp * N
                                                    : ((p.c_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
    load_vec<state_t, VEC>(reinterpret_cast<const state_t *>(p.state) + r * N + n0, h[rb]);
    ld_vec_io<io_t, VEC>(p.Bp, p.bc_dtype, b_off + n0, bv[rb]);
    ld_vec_io<io_t, VEC>(p.Cp, p.bc_dtype, c_off + n0, cv[rb]);
    scal[rb] = ld_io<io_t>(scal_ptr, p.io_dtype, (sub == 2 && p.z) ? (size_t)b * p.z_bs + d : r);
    win[rb] = CONV ? ld_io<io_t>(p.conv_state, p.io_dtype, r * K + win_k) : 0.0f;
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int b = bg * RB + rb;
    const size_t r = (size_t)b * p.dim + d;
    float xv = __shfl(scal[rb], base, WAVE);
    float dtv = __shfl(scal[rb], base + 1, WAVE) + bias;
    const float zv = __shfl(scal[rb], base + 2, WAVE);
    if (p.softplus) dtv = softplus_f32(dtv);
    if (CONV) {
      // window <- (window[1:], x); x <- act(bias + sum_k w[k] window[k]); lane k of the row owns tap k
      const float v = sub + 1 < K ? win[rb] : xv;
      float part = sub < K ? v * tap : 0.0f;
      if (live && sub < K) st_io<io_t>(p.conv_state, p.io_dtype, r * K + sub, v);
      for (int m = tpr >> 1; m >= 1; m >>= 1) part += __shfl_xor(part, m, WAVE);
      part += cbias;
      xv = round_io<io_t>(p.conv_silu ? silu_f32(part) : part, p.io_dtype);
      if (p.conv_out && live && sub == 0) st_io<io_t>(p.conv_out, p.io_dtype, r, xv);
    }
    const float dx = dtv * xv, dt2 = dtv * LOG2E;
    float acc = 0.0f;
    Pack<state_t, VEC> outv;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float hn = __builtin_fmaf(exp2_hw(dt2 * a[i]), h[rb][i], dx * bv[rb][i]);
      acc = __builtin_fmaf(hn, cv[rb][i], acc);
      outv.v[i] = from_f32<state_t>(hn);
    }
    if (live) *reinterpret_cast<Pack<state_t, VEC> *>(reinterpret_cast<state_t *>(p.state) + r * N + n0) = outv;
    for (int m = tpr >> 1; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, WAVE);
    if (live && sub == 0) {
      float y = __builtin_fmaf(Dk, xv, acc);
      if (p.z) y *= silu_f32(zv);
      st_io<io_t>(p.out, p.io_dtype, r, y);
    }
  }
}

template <typename state_t, typename io_t, int RB>
static void launch_rb(const StepParams &p, unsigned grid, hipStream_t stream) {
  if (p.conv_state) hipLaunchKernelGGL((state_step_rb_kernel<state_t, io_t, true, RB>), dim3(grid), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((state_step_rb_kernel<state_t, io_t, false, RB>), dim3(grid), dim3(256), 0, stream, p);
}

template <typename state_t>
static int launch_step(const StepParams &p0, bool vec4, hipStream_t stream) {
  StepParams p = p0;
  const int vec = vec4 ? 4 : 1;
  const int per_row = (p.nstate + vec - 1) / vec;
  int lg = 0;
  while ((1 << lg) < per_row && lg < 4) ++lg;    // at most 16 lanes per row
  p.tpr_log2 = lg;
  if (vec4 && p.nstate == (4 << lg) && lg >= 2 && (!p.conv_state || p.conv_k <= (1 << lg))) {
    // four batch rows per thread when the batch allows it (and is large enough to fill the device that way),
    // one otherwise; float32 states with activations and projections of one type: element types known at
    // compile time
    const bool four = p.batch % 4 == 0 && (size_t)p.batch * p.dim >= 65536;
    const size_t threads_rb = ((size_t)p.dim * (four ? p.batch / 4 : p.batch)) << lg;
    const unsigned grid_rb = (unsigned)((threads_rb + 255) / 256);
    bool done = false;
    if constexpr (std::is_same<state_t, float>::value) {
      if (p.io_dtype == p.bc_dtype) {
        if (p.io_dtype == SSM_BF16) four ? launch_rb<state_t, bf16_t, 4>(p, grid_rb, stream) : launch_rb<state_t, bf16_t, 1>(p, grid_rb, stream);
        else if (p.io_dtype == SSM_F16) four ? launch_rb<state_t, f16_t, 4>(p, grid_rb, stream) : launch_rb<state_t, f16_t, 1>(p, grid_rb, stream);
        else four ? launch_rb<state_t, float, 4>(p, grid_rb, stream) : launch_rb<state_t, float, 1>(p, grid_rb, stream);
        done = true;
      }
    }
    if (!done) four ? launch_rb<state_t, void, 4>(p, grid_rb, stream) : launch_rb<state_t, void, 1>(p, grid_rb, stream);
    SSM_CHECK_LAUNCH("ssm_state_step");
    return SSM_OK;
  }
  const size_t threads = ((size_t)p.batch * p.dim) << lg;
  const unsigned grid = (unsigned)((threads + 255) / 256);
  if (vec4) hipLaunchKernelGGL((state_step_kernel<state_t, 4>), dim3(grid), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((state_step_kernel<state_t, 1>), dim3(grid), dim3(256), 0, stream, p);
  SSM_CHECK_LAUNCH("ssm_state_step");
  return SSM_OK;
}

}  // namespace ssm

static int run_state_step(const ssm_state_step_args *a, const ssm_decode_step_args *dec, void *hip_stream);

extern "C" int ssm_state_step(const ssm_state_step_args *a, void *hip_stream) {
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_state_step: args is NULL");
  return run_state_step(a, nullptr, hip_stream);
}

extern "C" int ssm_decode_step(const ssm_decode_step_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_decode_step: args is NULL");
  SSM_REQUIRE(a->conv_state && a->conv_weight, SSM_ERR_NULL_POINTER,
              "ssm_decode_step: conv_state and conv_weight are required");
  SSM_REQUIRE(a->conv_width > 0 && a->conv_width <= 64, SSM_ERR_BAD_SHAPE, "ssm_decode_step: conv_width=%d",
              a->conv_width);
  SSM_REQUIRE(a->conv_activation == SSM_ACT_IDENTITY || a->conv_activation == SSM_ACT_SILU, SSM_ERR_BAD_KIND,
              "ssm_decode_step: conv_activation=%d", a->conv_activation);
  return run_state_step(&a->step, a, hip_stream);
}

static int run_state_step(const ssm_state_step_args *a, const ssm_decode_step_args *dec, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a->state && a->x && a->dt && a->A && a->Bproj && a->Cproj && a->out, SSM_ERR_NULL_POINTER,
              "ssm_state_step: state, x, dt, A, Bproj, Cproj and out are required");
  SSM_REQUIRE(a->batch > 0 && a->dim > 0 && a->nstate > 0, SSM_ERR_BAD_SHAPE,
              "ssm_state_step: batch=%d dim=%d nstate=%d must all be positive", a->batch, a->dim, a->nstate);
  SSM_REQUIRE(valid_dtype(a->state_dtype) && valid_dtype(a->io_dtype) && valid_dtype(a->bc_dtype),
              SSM_ERR_BAD_DTYPE, "ssm_state_step: state_dtype=%d io_dtype=%d bc_dtype=%d", a->state_dtype,
              a->io_dtype, a->bc_dtype);
  auto kind_ok = [](int k) { return k == SSM_PROJ_DN || k == SSM_PROJ_BDN || k == SSM_PROJ_BGNL; };
  SSM_REQUIRE(kind_ok(a->b_kind) && kind_ok(a->c_kind), SSM_ERR_BAD_KIND, "ssm_state_step: b_kind=%d c_kind=%d",
              a->b_kind, a->c_kind);
  if (a->b_kind == SSM_PROJ_BGNL)
    SSM_REQUIRE(a->b_groups > 0 && a->dim % a->b_groups == 0, SSM_ERR_BAD_SHAPE,
                "ssm_state_step: b_groups=%d must divide dim=%d", a->b_groups, a->dim);
  if (a->c_kind == SSM_PROJ_BGNL)
    SSM_REQUIRE(a->c_groups > 0 && a->dim % a->c_groups == 0, SSM_ERR_BAD_SHAPE,
                "ssm_state_step: c_groups=%d must divide dim=%d", a->c_groups, a->dim);
  SSM_REQUIRE((size_t)a->batch * a->dim < ((size_t)1 << 27), SSM_ERR_TOO_LARGE, "ssm_state_step: too many rows");
  const int ss = dtype_size(a->state_dtype), es = dtype_size(a->io_dtype), bs = dtype_size(a->bc_dtype);
  SSM_REQUIRE(aligned_to(a->state, ss) && aligned_to(a->x, es) && aligned_to(a->dt, es) &&
                  aligned_to(a->out, es) && (!a->z || aligned_to(a->z, es)) && aligned_to(a->A, 4) &&
                  aligned_to(a->Bproj, bs) && aligned_to(a->Cproj, bs),
              SSM_ERR_ALIGNMENT, "ssm_state_step: a pointer is not aligned to its element size");

  StepParams p;
  p.state = a->state; p.x = a->x; p.dt = a->dt; p.z = a->z; p.Bp = a->Bproj; p.Cp = a->Cproj;
  p.A = a->A; p.Dk = a->Dskip; p.bias = a->dt_bias; p.out = a->out;
  p.batch = a->batch; p.dim = a->dim; p.nstate = a->nstate;
  p.io_dtype = a->io_dtype; p.bc_dtype = a->bc_dtype;
  p.b_kind = a->b_kind; p.c_kind = a->c_kind;
  p.b_groups = a->b_kind == SSM_PROJ_BGNL ? a->b_groups : 1;
  p.c_groups = a->c_kind == SSM_PROJ_BGNL ? a->c_groups : 1;
  p.softplus = a->dt_softplus ? 1 : 0;
  SSM_REQUIRE(a->z_batch_stride >= 0 && a->b_batch_stride >= 0 && a->c_batch_stride >= 0 &&
                  (a->z_batch_stride == 0 || a->z_batch_stride >= a->dim) &&
                  (a->b_batch_stride == 0 || (a->b_kind == SSM_PROJ_BGNL && a->b_batch_stride >= (long long)a->b_groups * a->nstate)) &&
                  (a->c_batch_stride == 0 || (a->c_kind == SSM_PROJ_BGNL && a->c_batch_stride >= (long long)a->c_groups * a->nstate)),
              SSM_ERR_BAD_SHAPE,
              "ssm_state_step: batch strides must hold a row (z: dim; B, C: groups * nstate, grouped projections only)");
  p.z_bs = a->z_batch_stride ? a->z_batch_stride : a->dim;
  p.b_bs = a->b_batch_stride ? a->b_batch_stride : (long long)p.b_groups * a->nstate;
  p.c_bs = a->c_batch_stride ? a->c_batch_stride : (long long)p.c_groups * a->nstate;
  p.tpr_log2 = 0;
  p.conv_state = nullptr; p.conv_w = nullptr; p.conv_b = nullptr; p.conv_out = nullptr; p.conv_k = 0; p.conv_silu = 0;
  if (dec) {
    SSM_REQUIRE(aligned_to(dec->conv_state, es) && (!dec->conv_out || aligned_to(dec->conv_out, es)),
                SSM_ERR_ALIGNMENT, "ssm_decode_step: a pointer is not aligned to its element size");
    p.conv_state = dec->conv_state; p.conv_w = dec->conv_weight; p.conv_b = dec->conv_bias;
    p.conv_out = dec->conv_out; p.conv_k = dec->conv_width; p.conv_silu = dec->conv_activation == SSM_ACT_SILU;
  }
  const bool vec4 = a->nstate % 4 == 0 && aligned_to(a->state, 4 * ss) && aligned_to(a->A, 16) &&
                    aligned_to(a->Bproj, 4 * bs) && aligned_to(a->Cproj, 4 * bs) && p.b_bs % 4 == 0 && p.c_bs % 4 == 0;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  switch (a->state_dtype) {
    case SSM_F32: return launch_step<float>(p, vec4, stream);
    case SSM_BF16: return launch_step<bf16_t>(p, vec4, stream);
    default: return launch_step<f16_t>(p, vec4, stream);
  }
}
