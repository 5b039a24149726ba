// Backward of the diagonal chunked scan (the reference's `ssd_chunk_scan`).
//
// Forward per (batch, head, p) channel, t < len(batch):
//   a_t = exp(dt_t A);  s_t = a_t s_{t-1} + dt_t B_t X_t;  y0_t = s_t C_t + D X_t;  y_t = y0_t silu(z_t)
// Backward, with gy = dL/dy and lambda_t = dL/ds_t (lambda past the end is 0):
//   g0_t = gy_t silu(z_t)                     dz_t = gy_t y0_t silu'(z_t)
//   lambda_t = lambda_{t+1} a_{t+1} + g0_t C_t
//   dC_t = g0_t s_t       dD += g0_t X_t      dX_t = g0_t D + lambda_t dt_t B_t      dB_t = lambda_t dt_t X_t
//   ddt_t += lambda_t (s_{t-1} a_t A + B_t X_t)                 dA += lambda_t s_{t-1} a_t dt_t
//   dinit = lambda_0 a_0
// One thread per channel: a forward sweep stores the states, a reverse sweep
// consumes them.  Everything that is a sum over channels, batch or time beyond
// the thread's own loop is written as a partial and folded in a fixed order.
#include "common.hpp"

namespace ssm {

constexpr int DB_THREADS = 256;

struct DscanBwdParams {
  const void *gy, *X, *dt, *Bp, *Cp, *z, *init;
  const float *A, *Dk;
  const int *lengths;
  void *dX;                       // (B,L,H,P) x dtype
  float *states;                  // (B,L,HP) scratch
  float *ddt_p;                   // (B,L,HP) partial of ddt (summed over p afterwards)
  float *dz_p;                    // (B,L,HP): dz itself when z is per channel, else a partial
  float *dB_t, *dC_t;             // (B,L,HP) when the projection is time-varying, else null
  float *pA, *pD, *pB, *pC;       // (B,HP) sums over time
  float *dinit;                   // (B,HP) or null
  int batch, len, heads, proj;
  int x_dtype, dt_dtype, bc_dtype, z_dtype, init_dtype;
  int a_stride_p, d_stride_p;
  long long b_stride_b, b_stride_t, c_stride_b, c_stride_t;
  int z_per_p;
};

__device__ __forceinline__ void db_store(void *p, int dtype, size_t i, float v) {
  if (dtype == SSM_F32) reinterpret_cast<float *>(p)[i] = v;
  else if (dtype == SSM_BF16) reinterpret_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else reinterpret_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
}

__global__ __launch_bounds__(DB_THREADS) void dscan_bwd_kernel(const DscanBwdParams p) {
  const int HP = p.heads * p.proj;
  const int hp = blockIdx.x * DB_THREADS + threadIdx.x;
  if (hp >= HP) return;
  const int b = blockIdx.y;
  const int h = hp / p.proj, pp = hp % p.proj;
  const int valid = p.lengths ? min(max(p.lengths[b], 0), p.len) : p.len;
  const float A = p.A[(size_t)h * (p.a_stride_p ? p.proj : 1) + (p.a_stride_p ? pp : 0)];
  const float Dk = p.Dk ? p.Dk[(size_t)h * (p.d_stride_p ? p.proj : 1) + (p.d_stride_p ? pp : 0)] : 0.0f;
  const size_t row0 = (size_t)b * p.len;
  const float s_init = p.init ? load_as_f32(p.init, p.init_dtype, (size_t)b * HP + hp) : 0.0f;

  // forward sweep: states[t] = s_t
  float s = s_init;
  for (int t = 0; t < valid; ++t) {
    const float dtv = load_as_f32(p.dt, p.dt_dtype, (row0 + t) * p.heads + h);
    const float xv = load_as_f32(p.X, p.x_dtype, (row0 + t) * HP + hp);
    const float bv = load_as_f32(p.Bp, p.bc_dtype, (size_t)(b * p.b_stride_b + t * p.b_stride_t) + hp);
    s = __builtin_fmaf(exp2_hw(dtv * A * LOG2E), s, dtv * bv * xv);
    p.states[(row0 + t) * HP + hp] = s;
  }
  // steps past the end contribute nothing
  for (int t = valid; t < p.len; ++t) {
    const size_t xi = (row0 + t) * HP + hp;
    db_store(p.dX, p.x_dtype, xi, 0.0f);
    p.ddt_p[xi] = 0.0f;
    if (p.dz_p) p.dz_p[xi] = 0.0f;
    if (p.dB_t) p.dB_t[xi] = 0.0f;
    if (p.dC_t) p.dC_t[xi] = 0.0f;
  }

  // reverse sweep
  float lam_next_a = 0.0f;          // lambda_{t+1} a_{t+1}
  float accA = 0.0f, accD = 0.0f, accB = 0.0f, accC = 0.0f;
  for (int t = valid - 1; t >= 0; --t) {
    const size_t xi = (row0 + t) * HP + hp;
    const float dtv = load_as_f32(p.dt, p.dt_dtype, (row0 + t) * p.heads + h);
    const float xv = load_as_f32(p.X, p.x_dtype, xi);
    const float bv = load_as_f32(p.Bp, p.bc_dtype, (size_t)(b * p.b_stride_b + t * p.b_stride_t) + hp);
    const float cv = load_as_f32(p.Cp, p.bc_dtype, (size_t)(b * p.c_stride_b + t * p.c_stride_t) + hp);
    const float st = p.states[xi];
    const float sprev = t > 0 ? p.states[xi - HP] : s_init;
    const float a = exp2_hw(dtv * A * LOG2E);
    const float gy = load_as_f32(p.gy, p.x_dtype, xi);
    float g0 = gy;
    if (p.z) {
      const size_t zi = p.z_per_p ? xi : (row0 + t) * p.heads + h;
      const float zv = load_as_f32(p.z, p.z_dtype, zi);
      const float sg = sigmoid_f32(zv);
      const float y0 = __builtin_fmaf(st, cv, Dk * xv);
      p.dz_p[xi] = gy * y0 * sg * (1.0f + zv * (1.0f - sg));
      g0 = gy * zv * sg;
    }
    const float lam = __builtin_fmaf(g0, cv, lam_next_a);
    db_store(p.dX, p.x_dtype, xi, __builtin_fmaf(g0, Dk, lam * dtv * bv));
    p.ddt_p[xi] = lam * __builtin_fmaf(sprev * a, A, bv * xv);
    const float gB = lam * dtv * xv, gC = g0 * st;
    if (p.dB_t) p.dB_t[xi] = gB; else accB += gB;
    if (p.dC_t) p.dC_t[xi] = gC; else accC += gC;
    accA = __builtin_fmaf(lam * sprev, a * dtv, accA);
    accD = __builtin_fmaf(g0, xv, accD);
    lam_next_a = lam * a;
  }
  const size_t bi = (size_t)b * HP + hp;
  p.pA[bi] = accA;
  p.pD[bi] = accD;
  p.pB[bi] = accB;
  p.pC[bi] = accC;
  if (p.dinit) p.dinit[bi] = lam_next_a;
}

}  // namespace ssm

// Workspace (floats): states, ddt partial, dz partial, dB/dC time-varying copies are outputs
// themselves; then four (B,HP) partials.
static size_t dscan_bwd_floats(int batch, int seqlen, int heads, int proj) {
  const size_t blhp = (size_t)batch * seqlen * heads * proj, bhp = (size_t)batch * heads * proj;
  return 3 * blhp + 4 * bhp;
}

extern "C" size_t ssm_dscan_bwd_workspace_bytes(int batch, int seqlen, int heads, int proj) {
  if (batch <= 0 || seqlen <= 0 || heads <= 0 || proj <= 0) return 0;
  return dscan_bwd_floats(batch, seqlen, heads, proj) * sizeof(float);
}

extern "C" int ssm_dscan_bwd(const ssm_dscan_bwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_dscan_bwd: args is NULL");
  SSM_REQUIRE(a->grad_y && a->X && a->dt && a->A && a->Bproj && a->Cproj && a->dX && a->ddt && a->dA && a->dB && a->dC,
              SSM_ERR_NULL_POINTER,
              "ssm_dscan_bwd: grad_y, X, dt, A, Bproj, Cproj, dX, ddt, dA, dB and dC are required");
  SSM_REQUIRE((a->z != nullptr) == (a->dz != nullptr), SSM_ERR_NULL_POINTER,
              "ssm_dscan_bwd: dz must be given exactly when z is");
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->proj > 0, SSM_ERR_BAD_SHAPE,
              "ssm_dscan_bwd: batch=%d seqlen=%d heads=%d proj=%d must all be positive", a->batch, a->seqlen, a->heads,
              a->proj);
  SSM_REQUIRE(valid_dtype(a->x_dtype) && valid_dtype(a->dt_dtype) && valid_dtype(a->bc_dtype) &&
                  (!a->z || valid_dtype(a->z_dtype)) && (!a->initial_states || valid_dtype(a->init_dtype)),
              SSM_ERR_BAD_DTYPE, "ssm_dscan_bwd: unsupported dtype");
  SSM_REQUIRE(a->batch < 65536, SSM_ERR_TOO_LARGE, "ssm_dscan_bwd: batch too large");
  SSM_REQUIRE((size_t)a->batch * a->seqlen * a->heads * a->proj < ((size_t)1 << 38), SSM_ERR_TOO_LARGE,
              "ssm_dscan_bwd: tensor too large");
  auto kind_ok = [](int k) { return k == SSM_CHUNK_HP || k == SSM_CHUNK_BHP || k == SSM_CHUNK_BLHP; };
  SSM_REQUIRE(kind_ok(a->b_kind) && kind_ok(a->c_kind), SSM_ERR_BAD_KIND, "ssm_dscan_bwd: b_kind=%d c_kind=%d",
              a->b_kind, a->c_kind);
  const size_t need = ssm_dscan_bwd_workspace_bytes(a->batch, a->seqlen, a->heads, a->proj);
  SSM_REQUIRE(a->workspace && a->workspace_bytes >= need && aligned_to(a->workspace, 4), SSM_ERR_WORKSPACE,
              "ssm_dscan_bwd: workspace of %zu bytes required", need);

  const int Bn = a->batch, L = a->seqlen, H = a->heads, P = a->proj;
  const long long HP = (long long)H * P;
  const size_t blhp = (size_t)Bn * L * HP, bhp = (size_t)Bn * HP;
  float *ws = reinterpret_cast<float *>(a->workspace);
  DscanBwdParams p{};
  p.gy = a->grad_y; p.X = a->X; p.dt = a->dt; p.Bp = a->Bproj; p.Cp = a->Cproj; p.z = a->z; p.init = a->initial_states;
  p.A = a->A; p.Dk = a->Dskip; p.lengths = a->seq_lens; p.dX = a->dX;
  p.states = ws; p.ddt_p = ws + blhp;
  const bool dz_direct = a->z && a->z_per_p;
  p.dz_p = !a->z ? nullptr : (dz_direct ? a->dz : ws + 2 * blhp);
  p.dB_t = a->b_kind == SSM_CHUNK_BLHP ? a->dB : nullptr;
  p.dC_t = a->c_kind == SSM_CHUNK_BLHP ? a->dC : nullptr;
  p.pA = ws + 3 * blhp; p.pD = p.pA + bhp; p.pB = p.pD + bhp; p.pC = p.pB + bhp;
  p.dinit = a->dinitial_states;
  p.batch = Bn; p.len = L; p.heads = H; p.proj = P;
  p.x_dtype = a->x_dtype; p.dt_dtype = a->dt_dtype; p.bc_dtype = a->bc_dtype; p.z_dtype = a->z_dtype;
  p.init_dtype = a->init_dtype;
  p.a_stride_p = a->a_per_p ? 1 : 0;
  p.d_stride_p = a->d_per_p ? 1 : 0;
  auto strides = [&](int kind, long long &sb, long long &st) {
    sb = kind == SSM_CHUNK_HP ? 0 : (kind == SSM_CHUNK_BHP ? HP : HP * L);
    st = kind == SSM_CHUNK_BLHP ? HP : 0;
  };
  strides(a->b_kind, p.b_stride_b, p.b_stride_t);
  strides(a->c_kind, p.c_stride_b, p.c_stride_t);
  p.z_per_p = a->z_per_p ? 1 : 0;

  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  const dim3 grid((unsigned)((HP + DB_THREADS - 1) / DB_THREADS), (unsigned)Bn);
  hipLaunchKernelGGL(dscan_bwd_kernel, grid, dim3(DB_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_dscan_bwd");

  // ddt (B,L,H) and, for a per-head gate, dz (B,L,H): sums over p
  launch_fold_sum(p.ddt_p, a->ddt, (size_t)Bn * L * H, P, 1, s);
  if (a->z && !dz_direct) launch_fold_sum(p.dz_p, a->dz, (size_t)Bn * L * H, P, 1, s);
  // sums over batch, then over p when the parameter is per head; `states` is free again and
  // serves as the (H,P) intermediate
  float *tmp = p.states;
  auto fold_param = [&](const float *partial, float *out, bool per_p) {
    if (per_p) launch_fold_rows(partial, out, Bn, (size_t)HP, s);
    else {
      launch_fold_rows(partial, tmp, Bn, (size_t)HP, s);
      launch_fold_sum(tmp, out, (size_t)H, P, 1, s);
    }
  };
  fold_param(p.pA, a->dA, a->a_per_p != 0);
  if (a->dD) fold_param(p.pD, a->dD, a->d_per_p != 0);
  auto fold_proj = [&](int kind, const float *partial, float *out) {
    if (kind == SSM_CHUNK_HP) launch_fold_rows(partial, out, Bn, (size_t)HP, s);
    else if (kind == SSM_CHUNK_BHP) launch_fold_rows(partial, out, 1, bhp, s);
  };
  fold_proj(a->b_kind, p.pB, a->dB);
  fold_proj(a->c_kind, p.pC, a->dC);
  SSM_CHECK_LAUNCH("ssm_dscan_bwd(fold)");
  return SSM_OK;
}
