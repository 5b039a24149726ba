// Backward of the single-token selective state update.
//
// Forward (state_step.hip):  d' = softplus(dt + bias);  a_n = exp(d' A_n);
//   h'_n = a_n h_n + d' x B_n;   y0 = <h', C> + D x;   y = y0 silu(z)
// Given gy = dL/dy and gh' = dL/dh' (either may be absent):
//   g0    = gy silu(z)                       dz = gy y0 silu'(z)
//   gn_n  = gh'_n + g0 C_n                   dC_n = g0 h'_n
//   dh_n  = gn_n a_n                         dA_n = gn_n h_n a_n d'
//   dd'   = sum_n gn_n (h_n a_n A_n + x B_n) dB_n = gn_n d' x
//   dx    = g0 D + d' sum_n gn_n B_n         dD   = g0 x
//   ddt   = dd' sigmoid(dt + bias)  (softplus on; else dd')          dbias = ddt
// One thread per (batch, channel) row.  Parameter gradients are written as
// per-row partials and folded in a fixed order afterwards (no atomics).
#include "common.hpp"

#include <type_traits>

namespace ssm {

struct StepBwdParams {
  const void *gy, *gstate, *state, *x, *dt, *z, *Bp, *Cp;
  const float *A, *Dk, *bias;
  void *dstate, *dx, *ddt, *dz;
  float *pA, *pB, *pC, *pD, *pbias;     // per-row partials
  int batch, dim, nstate;
  int io_dtype, state_dtype, bc_dtype;
  int b_kind, c_kind, b_groups, c_groups;
  int softplus;
};

__device__ __forceinline__ void store_rt(void *p, int dtype, size_t i, float v) {
  if (dtype == SSM_F32) reinterpret_cast<float *>(p)[i] = v;
  else if (dtype == SSM_BF16) reinterpret_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else reinterpret_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
}

__global__ __launch_bounds__(256) void state_step_bwd_kernel(const StepBwdParams p) {
  const size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= (size_t)p.batch * p.dim) return;
  const int b = (int)(r / p.dim), d = (int)(r % p.dim);
  const int N = p.nstate;

  const float pre = load_as_f32(p.dt, p.io_dtype, r) + (p.bias ? p.bias[d] : 0.0f);
  const float step = p.softplus ? softplus_f32(pre) : pre;
  const float dstep_dpre = p.softplus ? (pre > 20.0f ? 1.0f : sigmoid_f32(pre)) : 1.0f;
  const float xv = load_as_f32(p.x, p.io_dtype, r);
  const float gy = p.gy ? load_as_f32(p.gy, p.io_dtype, r) : 0.0f;
  float gate = 1.0f, dgate = 0.0f;
  if (p.z) {
    const float zv = load_as_f32(p.z, p.io_dtype, r);
    const float sg = sigmoid_f32(zv);
    gate = zv * sg;
    dgate = sg * (1.0f + zv * (1.0f - sg));
  }
  const float g0 = gy * gate;

  size_t b_off, c_off;
  if (p.b_kind == SSM_PROJ_BGNL) b_off = ((size_t)b * p.b_groups + d / (p.dim / p.b_groups)) * N;
  else b_off = ((p.b_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
  if (p.c_kind == SSM_PROJ_BGNL) c_off = ((size_t)b * p.c_groups + d / (p.dim / p.c_groups)) * N;
  else c_off = ((p.c_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;

  float y0 = 0.0f, dstep = 0.0f, sum_gb = 0.0f;
  for (int n = 0; n < N; ++n) {
    const float h = load_as_f32(p.state, p.state_dtype, r * N + n);
    const float A = p.A[(size_t)d * N + n];
    const float Bn = load_as_f32(p.Bp, p.bc_dtype, b_off + n);
    const float Cn = load_as_f32(p.Cp, p.bc_dtype, c_off + n);
    const float a = exp2_hw(step * A * LOG2E);
    const float hn = __builtin_fmaf(a, h, step * xv * Bn);
    const float gn = (p.gstate ? load_as_f32(p.gstate, p.state_dtype, r * N + n) : 0.0f) + g0 * Cn;
    y0 = __builtin_fmaf(hn, Cn, y0);
    store_rt(p.dstate, p.state_dtype, r * N + n, gn * a);
    p.pA[r * N + n] = gn * h * a * step;
    p.pB[r * N + n] = gn * step * xv;
    p.pC[r * N + n] = g0 * hn;
    dstep = __builtin_fmaf(gn, __builtin_fmaf(h * a, A, xv * Bn), dstep);
    sum_gb = __builtin_fmaf(gn, Bn, sum_gb);
  }
  const float Dv = p.Dk ? p.Dk[d] : 0.0f;
  y0 = __builtin_fmaf(Dv, xv, y0);
  const float ddt = dstep * dstep_dpre;
  store_rt(p.dx, p.io_dtype, r, __builtin_fmaf(g0, Dv, step * sum_gb));
  store_rt(p.ddt, p.io_dtype, r, ddt);
  if (p.dz) store_rt(p.dz, p.io_dtype, r, gy * y0 * dgate);
  p.pD[r] = g0 * xv;
  p.pbias[r] = ddt;
}

// The same with one lane per (row, state) for N = 2^k <= 64: every access of the state-sized tensors is
// coalesced, the sums over a row's states are butterflies inside the wave.  io_t = void looks the element
// types up at run time; otherwise x, dt, z, B, C and the gradients of the activations have type io_t and
// the state tensors are float32, so that the reads are straight-line code issued together.
template <typename io_t>
__global__ __launch_bounds__(256) void state_step_bwd_lanes_kernel(const StepBwdParams p, const int lg) {
  constexpr bool RT = std::is_void<io_t>::value;
  using act_t = typename std::conditional<RT, float, io_t>::type;
  const int N = 1 << lg;
  const size_t rows = (size_t)p.batch * p.dim;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const bool live = gid < (rows << lg);
  const size_t g = live ? gid : 0;
  const unsigned r = (unsigned)(g >> lg);
  const int n = (int)(g & (size_t)(N - 1));
  const int b = (int)(r / (unsigned)p.dim), d = (int)(r % (unsigned)p.dim);
  const size_t b_off = p.b_kind == SSM_PROJ_BGNL ? ((size_t)b * p.b_groups + d / (p.dim / p.b_groups)) * N
                                                  : ((p.b_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
  const size_t c_off = p.c_kind == SSM_PROJ_BGNL ? ((size_t)b * p.c_groups + d / (p.dim / p.c_groups)) * N
                                                  : ((p.c_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
  auto act = [&](const void *q, size_t i) -> float {
    if constexpr (RT) return load_as_f32(q, p.io_dtype, i);
    else return to_f32(reinterpret_cast<const act_t *>(q)[i]);
  };
  auto proj = [&](const void *q, size_t i) -> float {
    if constexpr (RT) return load_as_f32(q, p.bc_dtype, i);
    else return to_f32(reinterpret_cast<const act_t *>(q)[i]);
  };
  auto st = [&](const void *q, size_t i) -> float {
    if constexpr (RT) return load_as_f32(q, p.state_dtype, i);
    else return reinterpret_cast<const float *>(q)[i];
  };
  // absent inputs read a present one and drop the value: no branch around a read
  const float dt_raw = act(p.dt, r), xv = act(p.x, r);
  const float gy_raw = act(p.gy ? p.gy : p.x, r), z_raw = act(p.z ? p.z : p.x, r);
  const float h = st(p.state, g), gs_raw = st(p.gstate ? p.gstate : p.state, g);
  const float A = p.A[(size_t)d * N + n], Bn = proj(p.Bp, b_off + n), Cn = proj(p.Cp, c_off + n);
  const float bias = p.bias ? p.bias[d] : 0.0f, Dv = p.Dk ? p.Dk[d] : 0.0f;

  const float pre = dt_raw + bias;
  const float step = p.softplus ? softplus_f32(pre) : pre;
  const float dstep_dpre = p.softplus ? (pre > 20.0f ? 1.0f : sigmoid_f32(pre)) : 1.0f;
  const float gy = p.gy ? gy_raw : 0.0f;
  float gate = 1.0f, dgate = 0.0f;
  if (p.z) {
    const float sg = sigmoid_f32(z_raw);
    gate = z_raw * sg;
    dgate = sg * (1.0f + z_raw * (1.0f - sg));
  }
  const float g0 = gy * gate;
  const float a = exp2_hw(step * A * LOG2E);
  const float hn = __builtin_fmaf(a, h, step * xv * Bn);
  const float gn = (p.gstate ? gs_raw : 0.0f) + g0 * Cn;
  float y0 = hn * Cn, dstep = gn * __builtin_fmaf(h * a, A, xv * Bn), sum_gb = gn * Bn;
  for (int m = N >> 1; m >= 1; m >>= 1) {
    y0 += __shfl_xor(y0, m, WAVE);
    dstep += __shfl_xor(dstep, m, WAVE);
    sum_gb += __shfl_xor(sum_gb, m, WAVE);
  }
  if (!live) return;
  if constexpr (RT) store_rt(p.dstate, p.state_dtype, g, gn * a);
  else reinterpret_cast<float *>(p.dstate)[g] = gn * a;
  p.pA[g] = gn * h * a * step;
  p.pB[g] = gn * step * xv;
  p.pC[g] = g0 * hn;
  if (n == 0) {
    y0 = __builtin_fmaf(Dv, xv, y0);
    const float ddt = dstep * dstep_dpre;
    const float dxv = __builtin_fmaf(g0, Dv, step * sum_gb);
    if constexpr (RT) {
      store_rt(p.dx, p.io_dtype, r, dxv);
      store_rt(p.ddt, p.io_dtype, r, ddt);
      if (p.dz) store_rt(p.dz, p.io_dtype, r, gy * y0 * dgate);
    } else {
      reinterpret_cast<act_t *>(p.dx)[r] = from_f32<act_t>(dxv);
      reinterpret_cast<act_t *>(p.ddt)[r] = from_f32<act_t>(ddt);
      if (p.dz) reinterpret_cast<act_t *>(p.dz)[r] = from_f32<act_t>(gy * y0 * dgate);
    }
    p.pD[r] = g0 * xv;
    p.pbias[r] = ddt;
  }
}

}  // namespace ssm

static size_t step_bwd_floats(int batch, int dim, int nstate) {
  return (size_t)batch * dim * (3 * (size_t)nstate + 2);
}

extern "C" size_t ssm_state_step_bwd_workspace_bytes(int batch, int dim, int nstate) {
  if (batch <= 0 || dim <= 0 || nstate <= 0) return 0;
  return step_bwd_floats(batch, dim, nstate) * sizeof(float);
}

extern "C" int ssm_state_step_bwd(const ssm_state_step_bwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_state_step_bwd: args is NULL");
  SSM_REQUIRE(a->state && a->x && a->dt && a->A && a->Bproj && a->Cproj && a->dstate && a->dx && a->ddt && a->dA &&
                  a->dB && a->dC,
              SSM_ERR_NULL_POINTER,
              "ssm_state_step_bwd: state, x, dt, A, Bproj, Cproj, dstate, dx, ddt, dA, dB and dC are required");
  SSM_REQUIRE((a->z != nullptr) == (a->dz != nullptr), SSM_ERR_NULL_POINTER,
              "ssm_state_step_bwd: dz must be given exactly when z is");
  SSM_REQUIRE(a->batch > 0 && a->dim > 0 && a->nstate > 0, SSM_ERR_BAD_SHAPE,
              "ssm_state_step_bwd: batch=%d dim=%d nstate=%d must all be positive", a->batch, a->dim, a->nstate);
  SSM_REQUIRE(valid_dtype(a->state_dtype) && valid_dtype(a->io_dtype) && valid_dtype(a->bc_dtype), SSM_ERR_BAD_DTYPE,
              "ssm_state_step_bwd: state_dtype=%d io_dtype=%d bc_dtype=%d", a->state_dtype, a->io_dtype, a->bc_dtype);
  auto kind_ok = [](int k) { return k == SSM_PROJ_DN || k == SSM_PROJ_BDN || k == SSM_PROJ_BGNL; };
  SSM_REQUIRE(kind_ok(a->b_kind) && kind_ok(a->c_kind), SSM_ERR_BAD_KIND, "ssm_state_step_bwd: b_kind=%d c_kind=%d",
              a->b_kind, a->c_kind);
  if (a->b_kind == SSM_PROJ_BGNL)
    SSM_REQUIRE(a->b_groups > 0 && a->dim % a->b_groups == 0, SSM_ERR_BAD_SHAPE,
                "ssm_state_step_bwd: b_groups=%d must divide dim=%d", a->b_groups, a->dim);
  if (a->c_kind == SSM_PROJ_BGNL)
    SSM_REQUIRE(a->c_groups > 0 && a->dim % a->c_groups == 0, SSM_ERR_BAD_SHAPE,
                "ssm_state_step_bwd: c_groups=%d must divide dim=%d", a->c_groups, a->dim);
  SSM_REQUIRE((size_t)a->batch * a->dim < ((size_t)1 << 27), SSM_ERR_TOO_LARGE, "ssm_state_step_bwd: too many rows");
  const size_t need = step_bwd_floats(a->batch, a->dim, a->nstate) * sizeof(float);
  SSM_REQUIRE(a->workspace && a->workspace_bytes >= need && aligned_to(a->workspace, 4), SSM_ERR_WORKSPACE,
              "ssm_state_step_bwd: workspace of %zu bytes required", need);

  const size_t rows = (size_t)a->batch * a->dim, rn = rows * a->nstate;
  float *ws = reinterpret_cast<float *>(a->workspace);
  StepBwdParams p;
  p.gy = a->grad_out; p.gstate = a->grad_state; p.state = a->state; p.x = a->x; p.dt = a->dt; p.z = a->z;
  p.Bp = a->Bproj; p.Cp = a->Cproj; p.A = a->A; p.Dk = a->Dskip; p.bias = a->dt_bias;
  p.dstate = a->dstate; p.dx = a->dx; p.ddt = a->ddt; p.dz = a->dz;
  p.pA = ws; p.pB = ws + rn; p.pC = ws + 2 * rn; p.pD = ws + 3 * rn; p.pbias = ws + 3 * rn + rows;
  p.batch = a->batch; p.dim = a->dim; p.nstate = a->nstate;
  p.io_dtype = a->io_dtype; p.state_dtype = a->state_dtype; p.bc_dtype = a->bc_dtype;
  p.b_kind = a->b_kind; p.c_kind = a->c_kind;
  p.b_groups = a->b_kind == SSM_PROJ_BGNL ? a->b_groups : 1;
  p.c_groups = a->c_kind == SSM_PROJ_BGNL ? a->c_groups : 1;
  p.softplus = a->dt_softplus ? 1 : 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  int lg = 0;
  while ((1 << lg) < a->nstate) ++lg;
  if ((1 << lg) == a->nstate && lg <= 6) {
    const dim3 grid((unsigned)(((rows << lg) + 255) / 256));
    const bool typed = a->state_dtype == SSM_F32 && a->io_dtype == a->bc_dtype;
    if (typed && a->io_dtype == SSM_BF16) hipLaunchKernelGGL(state_step_bwd_lanes_kernel<bf16_t>, grid, dim3(256), 0, s, p, lg);
    else if (typed && a->io_dtype == SSM_F16) hipLaunchKernelGGL(state_step_bwd_lanes_kernel<f16_t>, grid, dim3(256), 0, s, p, lg);
    else if (typed && a->io_dtype == SSM_F32) hipLaunchKernelGGL(state_step_bwd_lanes_kernel<float>, grid, dim3(256), 0, s, p, lg);
    else hipLaunchKernelGGL(state_step_bwd_lanes_kernel<void>, grid, dim3(256), 0, s, p, lg);
  } else {
    hipLaunchKernelGGL(state_step_bwd_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, s, p);
  }
  SSM_CHECK_LAUNCH("ssm_state_step_bwd");

  const int Bn = a->batch, D = a->dim, N = a->nstate;
  launch_fold_rows(p.pA, a->dA, Bn, (size_t)D * N, s);
  if (a->dD) launch_fold_rows(p.pD, a->dD, Bn, (size_t)D, s);
  if (a->ddt_bias) launch_fold_rows(p.pbias, a->ddt_bias, Bn, (size_t)D, s);
  auto fold_proj = [&](int kind, int groups, const float *partial, float *out) {
    if (kind == SSM_PROJ_BGNL) launch_fold_sum(partial, out, (size_t)Bn * groups, D / groups, (size_t)N, s);
    else if (kind == SSM_PROJ_BDN) launch_fold_rows(partial, out, 1, (size_t)Bn * D * N, s);
    else launch_fold_rows(partial, out, Bn, (size_t)D * N, s);
  };
  fold_proj(a->b_kind, p.b_groups, p.pB, a->dB);
  fold_proj(a->c_kind, p.c_groups, p.pC, a->dC);
  SSM_CHECK_LAUNCH("ssm_state_step_bwd(fold)");
  return SSM_OK;
}
