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
// Time is cut into segments that run in parallel (as in the forward).  A first kernel folds every
// (segment, channel) into three numbers: the product of its decays, the state it would reach from zero,
// and the adjoint it would hand to the segment before it if nothing came in from the one after it
// (mu_t = lambda_t a_t obeys mu_t = a_t mu_{t+1} + a_t g0_t C_t, the same decays).  The main kernel
// rebuilds what enters a segment from both sides out of those folds, sweeps forward storing the
// states, then sweeps backward producing every gradient.  Sums over channels, batch, segments or time
// beyond a thread's own loop are written as partials and folded in a fixed order.
#include "common.hpp"

#include <type_traits>

namespace ssm {

constexpr int DB_THREADS = 256;
constexpr int DB_UNROLL = 8;          // time steps whose reads are in flight together

int dscan_segments(int batch, int len, int hp);   // dscan.hip: the forward's choice, reused here
// dscan.hip: the forward's one-pass walk reduced to the table of the states entering every 64 steps
void launch_dscan_round_states(const void *X, const void *dt, const void *Bproj, const float *A, const void *init,
                               int init_dtype, const int *lengths, float *round_states, int batch, int len, int heads,
                               int proj, int x_dtype, bool b_const, int bc_dtype, long long b_stride_b, bool a_per_p,
                               hipStream_t s);

struct DscanBwdParams {
  const void *gy, *X, *dt, *Bp, *Cp, *z, *init;
  const float *A, *Dk;
  const int *lengths;
  void *dX;                       // (B,L,H,P) x dtype
  float *states;                  // (B,L,HP) scratch
  float *ddt_p;                   // (B,L,HP) partial of ddt (summed over p afterwards); unused with ddt_direct
  float *ddt_direct;              // (B,L,H): written by the kernel when a head is exactly one wavefront
  void *dz_p;                     // (B,L,HP): dz itself when z is per channel (element type g_z_dtype), else a float32 partial
  float *dz_direct;               // (B,L,H): per-head gate and a head is one wavefront
  void *dB_t, *dC_t;              // (B,L,HP) when the projection is time-varying (element type g_bc_dtype), else null
  int g_bc_dtype, g_z_dtype;      // float32 unless the caller asked for gradients in the tensors' own types
  float *round_states;            // (B, ceil(L/64), HP): the state entering every 64 steps (one-pass kernels)
  float *fold;                    // (B, nseg, HP, 3): decay product, local state, local adjoint
  float *pA, *pD, *pB, *pC;       // (B, nseg, HP) sums over the segment's steps
  float *dinit;                   // (B,HP) or null
  int batch, len, heads, proj;
  int x_dtype, dt_dtype, bc_dtype, z_dtype, init_dtype;
  int a_stride_p, d_stride_p;
  long long b_stride_b, b_stride_t, c_stride_b, c_stride_t;
  int z_per_p;
  int seg_len, nseg;
};

__device__ __forceinline__ void db_store(void *p, int dtype, size_t i, float v) {
  if (dtype == SSM_F32) reinterpret_cast<float *>(p)[i] = v;
  else if (dtype == SSM_BF16) reinterpret_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else reinterpret_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
}

// io_t = void: element types looked up at run time; otherwise gy, X, B, C, z and dX are io_t and dt is
// float32, and the reads of a group of steps are straight-line code.
template <typename io_t>
__device__ __forceinline__ float db_load(const void *p, int dtype, size_t i) {
  if constexpr (std::is_void<io_t>::value) return load_as_f32(p, dtype, i);
  else return to_f32(reinterpret_cast<const io_t *>(p)[i]);
}
template <typename io_t>
__device__ __forceinline__ float db_load_dt(const void *p, int dtype, size_t i) {
  if constexpr (std::is_void<io_t>::value) return load_as_f32(p, dtype, i);
  else return reinterpret_cast<const float *>(p)[i];
}
template <typename io_t>
__device__ __forceinline__ void db_store_x(void *p, int dtype, size_t i, float v) {
  if constexpr (std::is_void<io_t>::value) db_store(p, dtype, i, v);
  else reinterpret_cast<io_t *>(p)[i] = from_f32<io_t>(v);
}

template <typename io_t>
__global__ __launch_bounds__(DB_THREADS) void dscan_bwd_fold_kernel(const DscanBwdParams p) {
  const int HP = p.heads * p.proj;
  const int hp = blockIdx.x * DB_THREADS + threadIdx.x;
  if (hp >= HP) return;
  const int seg = blockIdx.y, b = blockIdx.z;
  const int h = hp / p.proj, pp = hp % p.proj;
  const int valid = p.lengths ? min(max(p.lengths[b], 0), p.len) : p.len;
  const int t_begin = seg * p.seg_len;
  const int stop = min(min(p.len, t_begin + p.seg_len), valid);
  const float A2 = p.A[(size_t)h * (p.a_stride_p ? p.proj : 1) + (p.a_stride_p ? pp : 0)] * LOG2E;
  const size_t row0 = (size_t)b * p.len;
  float prod = 1.0f, s = 0.0f, M = 0.0f;
  for (int t0 = t_begin; t0 < stop; t0 += DB_UNROLL) {
    float dtv[DB_UNROLL], xv[DB_UNROLL], bv[DB_UNROLL], cv[DB_UNROLL], gv[DB_UNROLL], zv[DB_UNROLL];
#pragma unroll
    for (int j = 0; j < DB_UNROLL; ++j) {
      const int t = min(t0 + j, stop - 1);
      const size_t xi = (row0 + t) * HP + hp;
      dtv[j] = db_load_dt<io_t>(p.dt, p.dt_dtype, (row0 + t) * p.heads + h);
      xv[j] = db_load<io_t>(p.X, p.x_dtype, xi);
      bv[j] = db_load<io_t>(p.Bp, p.bc_dtype, (size_t)(b * p.b_stride_b + t * p.b_stride_t) + hp);
      cv[j] = db_load<io_t>(p.Cp, p.bc_dtype, (size_t)(b * p.c_stride_b + t * p.c_stride_t) + hp);
      gv[j] = db_load<io_t>(p.gy, p.x_dtype, xi);
      {
        // an absent gate reads X in its place (value dropped): no branch around the read
        const float zraw = db_load<io_t>(p.z ? p.z : p.X, p.z ? p.z_dtype : p.x_dtype, (p.z && !p.z_per_p) ? (row0 + t) * p.heads + h : xi);
        zv[j] = p.z ? zraw : 0.0f;
      }
    }
#pragma unroll
    for (int j = 0; j < DB_UNROLL; ++j) {
      if (t0 + j < stop) {
        const float a = exp2_hw(dtv[j] * A2);
        s = __builtin_fmaf(a, s, dtv[j] * bv[j] * xv[j]);
        prod *= a;                                          // product of the decays up to and including this step
        const float g0 = p.z ? gv[j] * zv[j] * sigmoid_f32(zv[j]) : gv[j];
        M = __builtin_fmaf(prod, g0 * cv[j], M);
      }
    }
  }
  float *f = p.fold + (((size_t)b * p.nseg + seg) * HP + hp) * 3;
  f[0] = prod;
  f[1] = s;
  f[2] = M;
}

template <typename io_t>
__global__ __launch_bounds__(DB_THREADS) void dscan_bwd_kernel(const DscanBwdParams p) {
  const int HP = p.heads * p.proj;
  const int hp = blockIdx.x * DB_THREADS + threadIdx.x;
  // whole wavefronts leave together (the sums over a head below use every lane of a wavefront)
  if (hp >= HP) return;
  const int seg = blockIdx.y, b = blockIdx.z;
  const int h = hp / p.proj, pp = hp % p.proj;
  const int valid = p.lengths ? min(max(p.lengths[b], 0), p.len) : p.len;
  const int t_begin = seg * p.seg_len;
  const int t_end = min(p.len, t_begin + p.seg_len);
  const int stop = min(t_end, valid);
  const float A = p.A[(size_t)h * (p.a_stride_p ? p.proj : 1) + (p.a_stride_p ? pp : 0)];
  const float A2 = A * LOG2E;
  const float Dk = p.Dk ? p.Dk[(size_t)h * (p.d_stride_p ? p.proj : 1) + (p.d_stride_p ? pp : 0)] : 0.0f;
  const size_t row0 = (size_t)b * p.len;
  const int lane = threadIdx.x & 63;

  // what enters the segment: the state from the left, the adjoint (times its decay) from the right
  float s_in = p.init ? load_as_f32(p.init, p.init_dtype, (size_t)b * HP + hp) : 0.0f;
  for (int j = 0; j < seg; ++j) {
    const float *f = p.fold + (((size_t)b * p.nseg + j) * HP + hp) * 3;
    s_in = __builtin_fmaf(f[0], s_in, f[1]);
  }
  float mu_in = 0.0f;
  for (int j = p.nseg - 1; j > seg; --j) {
    const float *f = p.fold + (((size_t)b * p.nseg + j) * HP + hp) * 3;
    mu_in = __builtin_fmaf(f[0], mu_in, f[2]);
  }

  // forward sweep: states[t] = s_t
  float s = s_in;
  for (int t0 = t_begin; t0 < stop; t0 += DB_UNROLL) {
    float dtv[DB_UNROLL], xv[DB_UNROLL], bv[DB_UNROLL];
#pragma unroll
    for (int j = 0; j < DB_UNROLL; ++j) {
      const int t = min(t0 + j, stop - 1);
      dtv[j] = db_load_dt<io_t>(p.dt, p.dt_dtype, (row0 + t) * p.heads + h);
      xv[j] = db_load<io_t>(p.X, p.x_dtype, (row0 + t) * HP + hp);
      bv[j] = db_load<io_t>(p.Bp, p.bc_dtype, (size_t)(b * p.b_stride_b + t * p.b_stride_t) + hp);
    }
#pragma unroll
    for (int j = 0; j < DB_UNROLL; ++j) {
      if (t0 + j < stop) {
        s = __builtin_fmaf(exp2_hw(dtv[j] * A2), s, dtv[j] * bv[j] * xv[j]);
        p.states[(row0 + t0 + j) * HP + hp] = s;
      }
    }
  }
  // steps past the end contribute nothing
  for (int t = max(stop, t_begin); t < t_end; ++t) {
    const size_t xi = (row0 + t) * HP + hp;
    db_store_x<io_t>(p.dX, p.x_dtype, xi, 0.0f);
    if (p.ddt_direct) { if (pp == 0) p.ddt_direct[(row0 + t) * p.heads + h] = 0.0f; }
    else p.ddt_p[xi] = 0.0f;
    if (p.dz_direct) { if (pp == 0) p.dz_direct[(row0 + t) * p.heads + h] = 0.0f; }
    else if (p.dz_p) db_store(p.dz_p, p.g_z_dtype, xi, 0.0f);
    if (p.dB_t) db_store(p.dB_t, p.g_bc_dtype, xi, 0.0f);
    if (p.dC_t) db_store(p.dC_t, p.g_bc_dtype, xi, 0.0f);
  }

  // reverse sweep
  float lam_next_a = mu_in;         // lambda_{t+1} a_{t+1}
  float accA = 0.0f, accD = 0.0f, accB = 0.0f, accC = 0.0f;
  for (int t1 = stop - 1; t1 >= t_begin; t1 -= DB_UNROLL) {
    float dtv[DB_UNROLL], xv[DB_UNROLL], bv[DB_UNROLL], cv[DB_UNROLL], gv[DB_UNROLL], zv[DB_UNROLL];
    float st[DB_UNROLL + 1];        // st[j] = s_{t1 - j}, st[UNROLL] = the state before the group's first step
#pragma unroll
    for (int j = 0; j < DB_UNROLL; ++j) {
      const int t = max(t1 - j, t_begin);
      const size_t xi = (row0 + t) * HP + hp;
      dtv[j] = db_load_dt<io_t>(p.dt, p.dt_dtype, (row0 + t) * p.heads + h);
      xv[j] = db_load<io_t>(p.X, p.x_dtype, xi);
      bv[j] = db_load<io_t>(p.Bp, p.bc_dtype, (size_t)(b * p.b_stride_b + t * p.b_stride_t) + hp);
      cv[j] = db_load<io_t>(p.Cp, p.bc_dtype, (size_t)(b * p.c_stride_b + t * p.c_stride_t) + hp);
      gv[j] = db_load<io_t>(p.gy, p.x_dtype, xi);
      {
        // an absent gate reads X in its place (value dropped): no branch around the read
        const float zraw = db_load<io_t>(p.z ? p.z : p.X, p.z ? p.z_dtype : p.x_dtype, (p.z && !p.z_per_p) ? (row0 + t) * p.heads + h : xi);
        zv[j] = p.z ? zraw : 0.0f;
      }
      st[j] = p.states[xi];
    }
    {
      const int t = t1 - DB_UNROLL;
      const float before = p.states[(row0 + max(t, t_begin)) * HP + hp];
      st[DB_UNROLL] = t >= t_begin ? before : s_in;
    }
#pragma unroll
    for (int j = 0; j < DB_UNROLL; ++j) {
      const int t = t1 - j;
      if (t >= t_begin) {                       // uniform over the workgroup
        const size_t xi = (row0 + t) * HP + hp;
        const float sprev = t > t_begin ? st[j + 1] : s_in;
        const float a = exp2_hw(dtv[j] * A2);
        float g0 = gv[j];
        if (p.z) {
          const float sg = sigmoid_f32(zv[j]);
          const float y0 = __builtin_fmaf(st[j], cv[j], Dk * xv[j]);
          const float dzv = gv[j] * y0 * sg * (1.0f + zv[j] * (1.0f - sg));
          if (p.dz_direct) {
            const float tot = wave_sum(dzv);
            if (lane == 0) p.dz_direct[(row0 + t) * p.heads + h] = tot;
          } else {
            db_store(p.dz_p, p.g_z_dtype, xi, dzv);
          }
          g0 = gv[j] * zv[j] * sg;
        }
        const float lam = __builtin_fmaf(g0, cv[j], lam_next_a);
        db_store_x<io_t>(p.dX, p.x_dtype, xi, __builtin_fmaf(g0, Dk, lam * dtv[j] * bv[j]));
        const float ddtv = lam * __builtin_fmaf(sprev * a, A, bv[j] * xv[j]);
        if (p.ddt_direct) {
          const float tot = wave_sum(ddtv);
          if (lane == 0) p.ddt_direct[(row0 + t) * p.heads + h] = tot;
        } else {
          p.ddt_p[xi] = ddtv;
        }
        const float gB = lam * dtv[j] * xv[j], gC = g0 * st[j];
        if (p.dB_t) db_store(p.dB_t, p.g_bc_dtype, xi, gB); else accB += gB;
        if (p.dC_t) db_store(p.dC_t, p.g_bc_dtype, xi, gC); else accC += gC;
        accA = __builtin_fmaf(lam * sprev, a * dtv[j], accA);
        accD = __builtin_fmaf(g0, xv[j], accD);
        lam_next_a = lam * a;
      }
    }
  }
  const size_t bi = ((size_t)b * p.nseg + seg) * HP + hp;
  p.pA[bi] = accA;
  p.pD[bi] = accD;
  p.pB[bi] = accB;
  p.pC[bi] = accC;
  if (p.dinit && seg == 0) p.dinit[(size_t)b * HP + hp] = lam_next_a;
}

}  // namespace ssm

#include "dscan_bwd_onepass.hpp"

// Workspace (floats): states, ddt partial, dz partial (dB/dC time-varying copies are outputs
// themselves); then per (batch, segment, channel) the three folds and four partial sums.
static void dscan_bwd_segments(int batch, int seqlen, int heads, int proj, int &seg_len, int &nseg) {
  nseg = ssm::dscan_segments(batch, seqlen, heads * proj);
  seg_len = (seqlen + nseg - 1) / nseg;
  nseg = (seqlen + seg_len - 1) / seg_len;
}
static size_t dscan_bwd_floats(int batch, int seqlen, int heads, int proj) {
  int seg_len, nseg;
  dscan_bwd_segments(batch, seqlen, heads, proj, seg_len, nseg);
  const size_t blhp = (size_t)batch * seqlen * heads * proj, bshp = (size_t)batch * nseg * heads * proj;
  return 3 * blhp + 7 * bshp;
}

extern "C" size_t ssm_dscan_bwd_workspace_bytes(int batch, int seqlen, int heads, int proj) {
  if (batch <= 0 || seqlen <= 0 || heads <= 0 || proj <= 0) return 0;
  return dscan_bwd_floats(batch, seqlen, heads, proj) * sizeof(float);
}

extern "C" int ssm_dscan_bwd(const ssm_dscan_bwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_dscan_bwd: args is NULL");
  SSM_CHECK_RESERVED("ssm_dscan_bwd", a);
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
  int seg_len, nseg;
  dscan_bwd_segments(Bn, L, H, P, seg_len, nseg);
  const size_t blhp = (size_t)Bn * L * HP, bhp = (size_t)Bn * HP, bshp = bhp * nseg;
  float *ws = reinterpret_cast<float *>(a->workspace);
  DscanBwdParams p{};
  p.gy = a->grad_y; p.X = a->X; p.dt = a->dt; p.Bp = a->Bproj; p.Cp = a->Cproj; p.z = a->z; p.init = a->initial_states;
  p.A = a->A; p.Dk = a->Dskip; p.lengths = a->seq_lens; p.dX = a->dX;
  p.states = ws; p.ddt_p = ws + blhp;
  const bool dz_direct = a->z && a->z_per_p;
  p.dz_p = !a->z ? nullptr : (dz_direct ? a->dz : (void *)(ws + 2 * blhp));
  p.dB_t = a->b_kind == SSM_CHUNK_BLHP ? a->dB : nullptr;
  p.dC_t = a->c_kind == SSM_CHUNK_BLHP ? a->dC : nullptr;
  const bool grads_io = a->grads_in_io_dtype != 0;
  p.g_bc_dtype = grads_io ? a->bc_dtype : SSM_F32;
  p.g_z_dtype = (grads_io && dz_direct) ? a->z_dtype : SSM_F32;
  p.fold = ws + 3 * blhp;
  p.pA = p.fold + 3 * bshp; p.pD = p.pA + bshp; p.pB = p.pD + bshp; p.pC = p.pB + bshp;
  p.dinit = a->dinitial_states;
  p.seg_len = seg_len; p.nseg = nseg;
  // a head of 64 channels is one wavefront: the sums over p are taken in the kernel
  const bool wave_heads = P == WAVE;
  p.ddt_direct = wave_heads ? a->ddt : nullptr;
  p.dz_direct = (wave_heads && a->z && !a->z_per_p) ? reinterpret_cast<float *>(a->dz) : nullptr;
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
  const dim3 grid((unsigned)((HP + DB_THREADS - 1) / DB_THREADS), (unsigned)nseg, (unsigned)Bn);
  const bool typed = a->dt_dtype == SSM_F32 && a->bc_dtype == a->x_dtype && (!a->z || a->z_dtype == a->x_dtype);
  // one pass: float32 dt, a gate of X's shape and type or none, a head's channels in 16, 32 or 64 lanes, and either
  // per-token B and C of X's type with per-head A and D, or B and C one value per channel (any type, gradients in
  // float32) with A and D per head or per channel
  const int vec = a->x_dtype == SSM_F32 ? 1 : 2;
  const size_t vbytes = (size_t)vec * dtype_size(a->x_dtype);
  const size_t gbytes = grads_io ? vbytes : (size_t)vec * 4;
  const int lph = P % vec == 0 ? P / vec : 0;
  const bool streamed = a->b_kind == SSM_CHUNK_BLHP && a->c_kind == SSM_CHUNK_BLHP && a->bc_dtype == a->x_dtype &&
                        !a->a_per_p && !a->d_per_p && aligned_to(a->Bproj, vbytes) && aligned_to(a->Cproj, vbytes) &&
                        aligned_to(a->dB, gbytes) && aligned_to(a->dC, gbytes);
  const bool constant = a->b_kind != SSM_CHUNK_BLHP && a->c_kind != SSM_CHUNK_BLHP &&
                        aligned_to(a->Bproj, dtype_size(a->bc_dtype)) && aligned_to(a->Cproj, dtype_size(a->bc_dtype)) &&
                        aligned_to(a->dB, 4) && aligned_to(a->dC, 4);
  const bool onepass = SSM_RESERVED(a) == 0 && a->batch < 65536 && (streamed || constant) && a->dt_dtype == SSM_F32 &&
                       (!a->z || (a->z_dtype == a->x_dtype && a->z_per_p)) && (lph == 16 || lph == 32 || lph == 64) &&
                       HP % (WAVE * vec) == 0 && (size_t)L * HP < ((size_t)1 << 30) && aligned_to(a->X, vbytes) &&
                       aligned_to(a->grad_y, vbytes) && aligned_to(a->dX, vbytes) &&
                       (!a->z || (aligned_to(a->z, vbytes) && aligned_to(a->dz, gbytes)));
  if (onepass) {
    const int rounds = (L + DBO_ROUND - 1) / DBO_ROUND;
    p.round_states = a->round_states ? const_cast<float *>(a->round_states) : ws;
    // per-channel sums of a batch row, (B, HP) each; those that are the caller's gradient already go there
    float *sums = ws + (size_t)Bn * rounds * HP;
    p.pA = sums;
    p.pD = sums + bhp;
    p.pB = (constant && a->b_kind == SSM_CHUNK_BHP) ? reinterpret_cast<float *>(a->dB) : sums + 2 * bhp;
    p.pC = (constant && a->c_kind == SSM_CHUNK_BHP) ? reinterpret_cast<float *>(a->dC) : sums + 3 * bhp;
    float *head_tmp = sums + 4 * bhp;                      // (HP) on the way to a per-head sum
    p.ddt_direct = a->ddt;
    if (a->round_states == nullptr)                      // no table from the forward: make it
      launch_dscan_round_states(a->X, a->dt, a->Bproj, a->A, a->initial_states, a->init_dtype, a->seq_lens, ws, Bn, L, H,
                                P, a->x_dtype, constant, a->bc_dtype, p.b_stride_b, a->a_per_p != 0, s);
    if (a->x_dtype == SSM_BF16) launch_bwd_onepass<bf16_t, 2>(p, grads_io, constant, s);
    else if (a->x_dtype == SSM_F16) launch_bwd_onepass<f16_t, 2>(p, grads_io, constant, s);
    else launch_bwd_onepass<float, 1>(p, grads_io, constant, s);
    SSM_CHECK_LAUNCH("ssm_dscan_bwd");
    if (!a->a_per_p && !a->d_per_p) {
      hipLaunchKernelGGL(dscan_bwd_head_sums_kernel, dim3(H), dim3(WAVE), 0, s, p.pA, p.pD, a->dA, a->dD, Bn, H, P);
    } else {
      auto param_sum = [&](const float *partial, float *out, bool per_p) {
        if (per_p) launch_fold_rows(partial, out, Bn, (size_t)HP, s);
        else {
          launch_fold_rows(partial, head_tmp, Bn, (size_t)HP, s);
          launch_fold_sum(head_tmp, out, (size_t)H, P, 1, s);
        }
      };
      param_sum(p.pA, a->dA, a->a_per_p != 0);
      if (a->dD) param_sum(p.pD, a->dD, a->d_per_p != 0);
    }
    if (constant && a->b_kind == SSM_CHUNK_HP) launch_fold_rows(p.pB, reinterpret_cast<float *>(a->dB), Bn, (size_t)HP, s);
    if (constant && a->c_kind == SSM_CHUNK_HP) launch_fold_rows(p.pC, reinterpret_cast<float *>(a->dC), Bn, (size_t)HP, s);
    SSM_CHECK_LAUNCH("ssm_dscan_bwd(sums)");
    return SSM_OK;
  } else {
#define SSM_DB_LAUNCH(T)                                                                       \
  {                                                                                            \
    if (nseg > 1) hipLaunchKernelGGL(dscan_bwd_fold_kernel<T>, grid, dim3(DB_THREADS), 0, s, p); \
    hipLaunchKernelGGL(dscan_bwd_kernel<T>, grid, dim3(DB_THREADS), 0, s, p);                  \
  }
  if (typed && a->x_dtype == SSM_BF16) SSM_DB_LAUNCH(bf16_t)
  else if (typed && a->x_dtype == SSM_F16) SSM_DB_LAUNCH(f16_t)
  else if (typed && a->x_dtype == SSM_F32) SSM_DB_LAUNCH(float)
  else SSM_DB_LAUNCH(void)
#undef SSM_DB_LAUNCH
  SSM_CHECK_LAUNCH("ssm_dscan_bwd");
  }

  // ddt (B,L,H) and, for a per-head gate, dz (B,L,H): sums over p, unless the kernel took them itself
  if (!p.ddt_direct) launch_fold_sum(p.ddt_p, a->ddt, (size_t)Bn * L * H, P, 1, s);
  if (a->z && !dz_direct && !p.dz_direct) launch_fold_sum(reinterpret_cast<const float *>(p.dz_p), reinterpret_cast<float *>(a->dz), (size_t)Bn * L * H, P, 1, s);
  // sums over batch and segments, then over p when the parameter is per head; `states` is free again
  // and serves as the (H,P) intermediate
  float *tmp = p.states;
  auto fold_param = [&](const float *partial, float *out, bool per_p) {
    if (per_p) launch_fold_rows(partial, out, Bn * nseg, (size_t)HP, s);
    else {
      launch_fold_rows(partial, tmp, Bn * nseg, (size_t)HP, s);
      launch_fold_sum(tmp, out, (size_t)H, P, 1, s);
    }
  };
  fold_param(p.pA, a->dA, a->a_per_p != 0);
  if (a->dD) fold_param(p.pD, a->dD, a->d_per_p != 0);
  auto fold_proj = [&](int kind, const float *partial, float *out) {
    if (kind == SSM_CHUNK_HP) launch_fold_rows(partial, out, Bn * nseg, (size_t)HP, s);
    else if (kind == SSM_CHUNK_BHP) launch_fold_sum(partial, out, (size_t)Bn, nseg, (size_t)HP, s);
  };
  fold_proj(a->b_kind, p.pB, reinterpret_cast<float *>(a->dB));
  fold_proj(a->c_kind, p.pC, reinterpret_cast<float *>(a->dC));
  SSM_CHECK_LAUNCH("ssm_dscan_bwd(fold)");
  return SSM_OK;
}
