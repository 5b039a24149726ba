// Selective scan, forward, for gfx950.
//
// One wavefront owns one (batch, channel) row.  Time is cut into chunks of
// T = 64*K steps; inside a chunk lane l owns the K consecutive steps
// [l*K, l*K+K).  For every state index n the lane folds its K steps into one
// affine map h -> P h + S, the 64 maps are composed with a DPP scan
// (row_shr 1/2/4/8, row_bcast 15/31), the state entering the lane is read from
// the previous lane, and the K steps are replayed from that state to emit
// y += h * C.  The running state of the row (one float per n) is carried from
// chunk to chunk in LDS and, after the last chunk, is the op's last_state.
//
// Time-varying B/C of one (batch, group) are shared by all channels of the
// group: the workgroup (up to 8 wavefronts = 8 channels of one group) stages
// them once per chunk in LDS as fp32, transposed so that a lane fetches the
// four values of four consecutive steps with one conflict-free 128-bit read.
#include "common.hpp"

namespace ssm {

constexpr int SCAN_NB = 16;          // state indices staged per pass
constexpr int SCAN_MAX_WAVES = 8;    // channels per workgroup
constexpr int SCAN_MAX_N = 256;      // state size limit (carry array)

struct ScanFwdParams {
  const void *u, *delta, *z, *Bp, *Cp;
  const float *A, *Dk, *bias;
  void *out, *last;
  int batch, dim, len, nstate;
  int bc_dtype;
  int b_kind, c_kind, b_groups, c_groups;
  int softplus;
  int vec_ok;     // rows of u/delta/z/out are 16-byte aligned
  int bc_vec_ok;  // rows of B/C allow 4-element vector loads
};

// Copy the [nn][T] slab of one time-varying projection into LDS as fp32.
// src_off is the element offset of (b, g, nb, 0); rows are `len` apart.
template <int K>
__device__ __forceinline__ void stage_tile(float *dst, const void *src, int dtype, size_t src_off,
                                           int len, int t0, int nn, bool vec_ok) {
  constexpr int T = WAVE * K;
  constexpr int QT = T / 4;
  for (int e = threadIdx.x; e < nn * QT; e += blockDim.x) {
    const int nl = e / QT;
    const int tl = (e % QT) * 4;
    const int t = t0 + tl;
    const size_t off = src_off + (size_t)nl * len + t;
    float4 v;
    if (vec_ok && t + 4 <= len) {
      if (dtype == SSM_F32) {
        v = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(src) + off);
      } else {
        const uint2 raw = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(src) + off);
        if (dtype == SSM_BF16) {
          v.x = __uint_as_float(raw.x << 16);
          v.y = __uint_as_float(raw.x & 0xffff0000u);
          v.z = __uint_as_float(raw.y << 16);
          v.w = __uint_as_float(raw.y & 0xffff0000u);
        } else {
          union { uint32_t u; _Float16 h[2]; } a, b;
          a.u = raw.x;
          b.u = raw.y;
          v.x = (float)a.h[0];
          v.y = (float)a.h[1];
          v.z = (float)b.h[0];
          v.w = (float)b.h[1];
        }
      }
    } else {
      v.x = (t + 0 < len) ? load_as_f32(src, dtype, off + 0) : 0.0f;
      v.y = (t + 1 < len) ? load_as_f32(src, dtype, off + 1) : 0.0f;
      v.z = (t + 2 < len) ? load_as_f32(src, dtype, off + 2) : 0.0f;
      v.w = (t + 3 < len) ? load_as_f32(src, dtype, off + 3) : 0.0f;
    }
    const int owner = tl / K;        // lane that owns these four steps
    const int item = tl % K;         // first of the four within the lane's run
    *reinterpret_cast<float4 *>(dst + nl * T + (item >> 2) * (WAVE * 4) + owner * 4) = v;
  }
}

template <typename io_t, int K>
__global__ __launch_bounds__(WAVE *SCAN_MAX_WAVES) void scan_fwd_kernel(const ScanFwdParams p) {
  constexpr int T = WAVE * K;
  extern __shared__ __align__(16) float tiles[];           // B tile [NB][T] then C tile [NB][T]
  __shared__ float carry[SCAN_MAX_WAVES][SCAN_MAX_N];

  const int rows = (int)(blockDim.x >> 6);
  const int wave = wave_id_uniform();
  const int lane = lane_id();
  const int blocks_per_batch = p.dim / rows;
  const int b = (int)blockIdx.x / blocks_per_batch;
  const int d0 = ((int)blockIdx.x % blocks_per_batch) * rows;
  const int d = d0 + wave;
  const int L = p.len, N = p.nstate;

  const size_t row = (size_t)b * p.dim + d;
  const io_t *u_row = reinterpret_cast<const io_t *>(p.u) + row * L;
  const io_t *dl_row = reinterpret_cast<const io_t *>(p.delta) + row * L;
  const io_t *z_row = p.z ? reinterpret_cast<const io_t *>(p.z) + row * L : nullptr;
  io_t *out_row = reinterpret_cast<io_t *>(p.out) + row * L;
  const float *A_row = p.A + (size_t)d * N;
  const float Dk = p.Dk ? p.Dk[d] : 0.0f;
  const float bias = p.bias ? p.bias[d] : 0.0f;
  const bool vec_ok = p.vec_ok != 0;

  const bool bvary = p.b_kind == SSM_PROJ_BGNL;
  const bool cvary = p.c_kind == SSM_PROJ_BGNL;
  float *Bs = tiles;
  float *Cs = tiles + (bvary ? SCAN_NB * T : 0);
  // element offset of this row's (or this group's) projection at n = 0, t = 0
  size_t b_off, c_off;
  if (bvary) b_off = ((size_t)b * p.b_groups + d0 / (p.dim / p.b_groups)) * (size_t)N * L;
  else b_off = ((p.b_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
  if (cvary) c_off = ((size_t)b * p.c_groups + d0 / (p.dim / p.c_groups)) * (size_t)N * L;
  else c_off = ((p.c_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;

  for (int n = lane; n < N; n += WAVE) carry[wave][n] = 0.0f;

  const int nchunks = (L + T - 1) / T;
  for (int c = 0; c < nchunks; ++c) {
    const int t0 = c * T;
    const int t = t0 + lane * K;

    float dl[K], du[K], y[K];
    {
      float uu[K];
      load_run<io_t, K>(u_row, t, L, vec_ok, uu);
      load_run<io_t, K>(dl_row, t, L, vec_ok, dl);
#pragma unroll
      for (int i = 0; i < K; ++i) {
        float dv = dl[i] + bias;
        if (p.softplus) dv = softplus_f32(dv);
        dv = (t + i < L) ? dv : 0.0f;      // steps past the end are the identity map
        dl[i] = dv;
        du[i] = dv * uu[i];
        y[i] = Dk * uu[i];
      }
    }
    float dsum = 0.0f;
#pragma unroll
    for (int i = 0; i < K; ++i) dsum += dl[i];

    for (int nb = 0; nb < N; nb += SCAN_NB) {
      const int nn = min(SCAN_NB, N - nb);
      if (bvary || cvary) {
        __syncthreads();   // every wave is done with the previous slab
        if (bvary) stage_tile<K>(Bs, p.Bp, p.bc_dtype, b_off + (size_t)nb * L, L, t0, nn, p.bc_vec_ok != 0);
        if (cvary) stage_tile<K>(Cs, p.Cp, p.bc_dtype, c_off + (size_t)nb * L, L, t0, nn, p.bc_vec_ok != 0);
        __syncthreads();
      }
      for (int nl = 0; nl < nn; ++nl) {
        const int n = nb + nl;
        const float A2 = A_row[n] * LOG2E;
        const float Bconst = bvary ? 0.0f : load_as_f32(p.Bp, p.bc_dtype, b_off + n);
        const float Cconst = cvary ? 0.0f : load_as_f32(p.Cp, p.bc_dtype, c_off + n);

        // fold the lane's K steps into (P, h): state_out = P * state_in + h
        float a[K], bx[K];
        float h = 0.0f;
#pragma unroll
        for (int q = 0; q < K / 4; ++q) {
          float4 bv;
          if (bvary) bv = *reinterpret_cast<const float4 *>(Bs + nl * T + q * (WAVE * 4) + lane * 4);
          else bv = make_float4(Bconst, Bconst, Bconst, Bconst);
          const float bq[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int i = q * 4 + j;
            a[i] = exp2_hw(dl[i] * A2);
            bx[i] = du[i] * bq[j];
            h = __builtin_fmaf(a[i], h, bx[i]);
          }
        }
        float P = exp2_hw(dsum * A2);
        wave_scan_affine(P, h);

        const float H = carry[wave][n];                       // row state entering the chunk
        float hs = __builtin_fmaf(wave_prev(P, 1.0f), H, wave_prev(h, 0.0f));   // entering this lane
        if (lane == WAVE - 1) carry[wave][n] = __builtin_fmaf(P, H, h);

        // replay the K steps from the true entering state
#pragma unroll
        for (int q = 0; q < K / 4; ++q) {
          float4 cv;
          if (cvary) cv = *reinterpret_cast<const float4 *>(Cs + nl * T + q * (WAVE * 4) + lane * 4);
          else cv = make_float4(Cconst, Cconst, Cconst, Cconst);
          const float cq[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int i = q * 4 + j;
            hs = __builtin_fmaf(a[i], hs, bx[i]);
            y[i] = __builtin_fmaf(hs, cq[j], y[i]);
          }
        }
      }
    }

    if (z_row) {
      float zz[K];
      load_run<io_t, K>(z_row, t, L, vec_ok, zz);
#pragma unroll
      for (int i = 0; i < K; ++i) y[i] *= silu_f32(zz[i]);
    }
    store_run<io_t, K>(out_row, t, L, vec_ok, y);
  }

  if (p.last) {
    io_t *last_row = reinterpret_cast<io_t *>(p.last) + row * N;
    for (int n = lane; n < N; n += WAVE) last_row[n] = from_f32<io_t>(carry[wave][n]);
  }
}

template <typename io_t, int K>
static int launch_scan_fwd(const ScanFwdParams &p, int rows, bool tiles, hipStream_t stream) {
  const size_t lds = tiles ? (size_t)((p.b_kind == SSM_PROJ_BGNL) + (p.c_kind == SSM_PROJ_BGNL)) * SCAN_NB *
                                 WAVE * K * sizeof(float)
                           : 0;
  auto kernel = scan_fwd_kernel<io_t, K>;
  if (allow_dynamic_lds(kernel, lds) != hipSuccess) {
    (void)hipGetLastError();
    set_error("ssm_scan_fwd: cannot reserve %zu bytes of LDS", lds);
    return SSM_ERR_LAUNCH;
  }
  const unsigned grid = (unsigned)((size_t)p.batch * (p.dim / rows));
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(WAVE * rows), lds, stream, p);
  SSM_CHECK_LAUNCH("ssm_scan_fwd");
  return SSM_OK;
}

template <typename io_t>
static int dispatch_items(const ScanFwdParams &p, int items, int rows, bool tiles, hipStream_t s) {
  switch (items) {
    case 4: return launch_scan_fwd<io_t, 4>(p, rows, tiles, s);
    case 8: return launch_scan_fwd<io_t, 8>(p, rows, tiles, s);
    case 16: return launch_scan_fwd<io_t, 16>(p, rows, tiles, s);
    default: set_error("ssm_scan_fwd: tune_items must be 0, 4, 8 or 16"); return SSM_ERR_BAD_KIND;
  }
}

static bool valid_kind(int k) { return k == SSM_PROJ_DN || k == SSM_PROJ_BDN || k == SSM_PROJ_BGNL; }

}  // namespace ssm

extern "C" int ssm_scan_fwd(const ssm_scan_fwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_scan_fwd: args is NULL");
  SSM_REQUIRE(a->u && a->delta && a->A && a->Bproj && a->Cproj && a->out, SSM_ERR_NULL_POINTER,
              "ssm_scan_fwd: u, delta, A, Bproj, Cproj and out are required");
  SSM_REQUIRE(a->batch > 0 && a->dim > 0 && a->seqlen > 0 && a->nstate > 0, SSM_ERR_BAD_SHAPE,
              "ssm_scan_fwd: batch=%d dim=%d seqlen=%d nstate=%d must all be positive", a->batch, a->dim,
              a->seqlen, a->nstate);
  SSM_REQUIRE(a->nstate <= SCAN_MAX_N, SSM_ERR_TOO_LARGE, "ssm_scan_fwd: nstate=%d exceeds %d", a->nstate,
              SCAN_MAX_N);
  SSM_REQUIRE(valid_dtype(a->io_dtype) && valid_dtype(a->bc_dtype), SSM_ERR_BAD_DTYPE,
              "ssm_scan_fwd: io_dtype=%d bc_dtype=%d", a->io_dtype, a->bc_dtype);
  SSM_REQUIRE(valid_kind(a->b_kind) && valid_kind(a->c_kind), SSM_ERR_BAD_KIND, "ssm_scan_fwd: b_kind=%d c_kind=%d",
              a->b_kind, a->c_kind);
  const bool bvary = a->b_kind == SSM_PROJ_BGNL, cvary = a->c_kind == SSM_PROJ_BGNL;
  if (bvary)
    SSM_REQUIRE(a->b_groups > 0 && a->dim % a->b_groups == 0, SSM_ERR_BAD_SHAPE,
                "ssm_scan_fwd: b_groups=%d must divide dim=%d", a->b_groups, a->dim);
  if (cvary)
    SSM_REQUIRE(a->c_groups > 0 && a->dim % a->c_groups == 0, SSM_ERR_BAD_SHAPE,
                "ssm_scan_fwd: c_groups=%d must divide dim=%d", a->c_groups, a->dim);
  const size_t rows_total = (size_t)a->batch * a->dim;
  SSM_REQUIRE(rows_total * (size_t)a->seqlen < ((size_t)1 << 40) && rows_total < ((size_t)1 << 31),
              SSM_ERR_TOO_LARGE, "ssm_scan_fwd: tensor too large");
  const int es = dtype_size(a->io_dtype), bs = dtype_size(a->bc_dtype);
  SSM_REQUIRE(aligned_to(a->u, es) && aligned_to(a->delta, es) && aligned_to(a->out, es) &&
                  (!a->z || aligned_to(a->z, es)) && (!a->last_state || aligned_to(a->last_state, es)) &&
                  aligned_to(a->Bproj, bs) && aligned_to(a->Cproj, bs) && aligned_to(a->A, 4) &&
                  (!a->Dskip || aligned_to(a->Dskip, 4)) && (!a->dt_bias || aligned_to(a->dt_bias, 4)),
              SSM_ERR_ALIGNMENT, "ssm_scan_fwd: a pointer is not aligned to its element size");

  ScanFwdParams p;
  p.u = a->u; p.delta = a->delta; p.z = a->z; p.Bp = a->Bproj; p.Cp = a->Cproj;
  p.A = a->A; p.Dk = a->Dskip; p.bias = a->dt_bias; p.out = a->out; p.last = a->last_state;
  p.batch = a->batch; p.dim = a->dim; p.len = a->seqlen; p.nstate = a->nstate;
  p.bc_dtype = a->bc_dtype;
  p.b_kind = a->b_kind; p.c_kind = a->c_kind;
  p.b_groups = bvary ? a->b_groups : 1; p.c_groups = cvary ? a->c_groups : 1;
  p.softplus = a->delta_softplus ? 1 : 0;
  p.vec_ok = ((size_t)a->seqlen * es) % 16 == 0 && aligned_to(a->u, 16) && aligned_to(a->delta, 16) &&
             aligned_to(a->out, 16) && (!a->z || aligned_to(a->z, 16));
  p.bc_vec_ok = a->seqlen % 4 == 0 && aligned_to(a->Bproj, 4 * bs) && aligned_to(a->Cproj, 4 * bs);

  // channels per workgroup: all must read the same B group and the same C group
  int per = a->dim;
  if (bvary) per = a->dim / a->b_groups;
  int per_c = cvary ? a->dim / a->c_groups : a->dim;
  int rows = SCAN_MAX_WAVES;
  while (rows > 1 && (per % rows != 0 || per_c % rows != 0 || a->dim % rows != 0)) rows >>= 1;

  int items = a->tune_items;
  if (items == 0) items = a->seqlen <= 256 ? 4 : 8;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  const bool tiles = bvary || cvary;
  switch (a->io_dtype) {
    case SSM_F32: return dispatch_items<float>(p, items, rows, tiles, stream);
    case SSM_BF16: return dispatch_items<bf16_t>(p, items, rows, tiles, stream);
    default: return dispatch_items<f16_t>(p, items, rows, tiles, stream);
  }
}
