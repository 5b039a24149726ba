// Residual-add + LayerNorm / RMSNorm, forward and backward, for gfx950.
//
//   v = x (+ residual when prenorm)           accumulated in fp32
//   LayerNorm: y = (v - mean) * rsqrt(var + eps) * w + b     (two-pass biased variance)
//   RMSNorm:   y = v * rsqrt(mean(v^2) + eps) * w + b
//   post-norm: y += residual
//
// One wavefront normalises one row and keeps the row in registers, so x and
// the residual are read from HBM exactly once and y / residual_out are written
// once; row statistics (mean, rstd) can be saved for the backward pass.
// Rows longer than the register budget (64 lanes * 32 values) fall back to a
// re-reading variant.
//
// Backward: a persistent grid walks rows; each wavefront produces dx (and
// dresidual) for its rows and accumulates dw/db columns in registers; per-wave
// partials are written once and folded by a second kernel in a fixed order.
#include "common.hpp"

#include <mutex>

#include <type_traits>

namespace ssm {

constexpr int LN_THREADS = 256;
constexpr int LN_WAVES = LN_THREADS / WAVE;

struct NormParams {
  const void *x, *res, *dy;
  const float *w, *b;
  void *y, *res_out, *dx, *dres;
  float *mean, *rstd;       // per row; fwd: optional outputs, bwd: required inputs (mean unused for RMS)
  float *partial;           // bwd: [nwaves_total][2][hidden]
  int rows, hidden;
  int x_dtype, res_dtype, res_out_dtype;
  int is_rms, prenorm;
  float eps;
};

__device__ __forceinline__ void store_f32_as(void *p, int dtype, size_t i, float v) {
  if (dtype == SSM_F32) reinterpret_cast<float *>(p)[i] = v;
  else if (dtype == SSM_BF16) reinterpret_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else reinterpret_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
}

// Row element j of lane `lane`, trip `k`: column = (k * 64 + lane) * VEC + i.
template <int VEC>
__device__ __forceinline__ void load_cols(const void *p, int dtype, size_t base, int col, int hidden, bool vec_ok,
                                          float (&v)[VEC]) {
  if (vec_ok && col + VEC <= hidden) {
    if (dtype == SSM_F32) {
      Pack<float, VEC> r = *reinterpret_cast<const Pack<float, VEC> *>(reinterpret_cast<const float *>(p) + base + col);
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] = r.v[i];
    } else if (dtype == SSM_BF16) {
      Pack<bf16_t, VEC> r = *reinterpret_cast<const Pack<bf16_t, VEC> *>(reinterpret_cast<const bf16_t *>(p) + base + col);
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] = to_f32(r.v[i]);
    } else {
      Pack<f16_t, VEC> r = *reinterpret_cast<const Pack<f16_t, VEC> *>(reinterpret_cast<const f16_t *>(p) + base + col);
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] = to_f32(r.v[i]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = (col + i < hidden) ? load_as_f32(p, dtype, base + col + i) : 0.0f;
  }
}

template <int VEC>
__device__ __forceinline__ void store_cols(void *p, int dtype, size_t base, int col, int hidden, bool vec_ok,
                                           const float (&v)[VEC]) {
  if (vec_ok && col + VEC <= hidden) {
    if (dtype == SSM_F32) {
      Pack<float, VEC> r;
#pragma unroll
      for (int i = 0; i < VEC; ++i) r.v[i] = v[i];
      *reinterpret_cast<Pack<float, VEC> *>(reinterpret_cast<float *>(p) + base + col) = r;
    } else if (dtype == SSM_BF16) {
      Pack<bf16_t, VEC> r;
#pragma unroll
      for (int i = 0; i < VEC; ++i) r.v[i] = from_f32<bf16_t>(v[i]);
      *reinterpret_cast<Pack<bf16_t, VEC> *>(reinterpret_cast<bf16_t *>(p) + base + col) = r;
    } else {
      Pack<f16_t, VEC> r;
#pragma unroll
      for (int i = 0; i < VEC; ++i) r.v[i] = from_f32<f16_t>(v[i]);
      *reinterpret_cast<Pack<f16_t, VEC> *>(reinterpret_cast<f16_t *>(p) + base + col) = r;
    }
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      if (col + i < hidden) store_f32_as(p, dtype, base + col + i, v[i]);
  }
}

// ------------------------------------------------------------------ forward

// A row is held in registers by one wavefront (WG = false: TRIPS * 64 * VEC >= hidden) or, for long rows, by
// the whole workgroup (WG = true: TRIPS * 256 * VEC >= hidden; sums over the row go through LDS).  VEC = 4
// keeps every access <= 16 bytes for all dtypes.
template <bool WG>
__device__ __forceinline__ float row_sum(float v, float *red) {
  v = wave_sum(v);
  if constexpr (WG) {
    const int wave = threadIdx.x >> 6;
    __syncthreads();                                   // the slots may still be read from the sum before
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    v = 0.0f;
#pragma unroll
    for (int w = 0; w < LN_WAVES; ++w) v += red[w];
  }
  return v;
}

template <int TRIPS, bool WG>
__global__ __launch_bounds__(LN_THREADS) void norm_fwd_kernel(const NormParams p, int vec_ok) {
  constexpr int VEC = 4;
  constexpr int OWNERS = WG ? LN_THREADS : WAVE;       // threads that share a row
  __shared__ float red[LN_WAVES];
  const int wave = threadIdx.x >> 6, lane = WG ? (int)threadIdx.x : (int)(threadIdx.x & 63);
  const int row = WG ? (int)blockIdx.x : (int)(blockIdx.x * LN_WAVES + wave);
  if (row >= p.rows) return;                           // whole workgroups in WG mode
  const int H = p.hidden;
  const size_t base = (size_t)row * H;
  const bool vok = vec_ok != 0;
  float v[TRIPS][VEC], r[TRIPS][VEC];
  float sum = 0.0f;
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int col = (k * OWNERS + lane) * VEC;
    load_cols<VEC>(p.x, p.x_dtype, base, col, H, vok, v[k]);
    if (p.res) {
      load_cols<VEC>(p.res, p.res_dtype, base, col, H, vok, r[k]);
      if (p.prenorm) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[k][i] += r[k][i];
      }
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) sum += v[k][i];
    if (p.res_out) store_cols<VEC>(p.res_out, p.res_out_dtype, base, col, H, vok, v[k]);
  }
  const float inv_h = 1.0f / (float)H;
  float mean = 0.0f;
  if (!p.is_rms) mean = row_sum<WG>(sum, red) * inv_h;
  float sq = 0.0f;
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int col = (k * OWNERS + lane) * VEC;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float c = (col + i < H) ? v[k][i] - mean : 0.0f;
      sq = __builtin_fmaf(c, c, sq);
    }
  }
  const float rstd = 1.0f / sqrtf(row_sum<WG>(sq, red) * inv_h + p.eps);
  if (lane == 0) {
    if (p.mean) p.mean[row] = mean;
    if (p.rstd) p.rstd[row] = rstd;
  }
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int col = (k * OWNERS + lane) * VEC;
    if (col >= H) continue;
    float wv[VEC], bv[VEC], out[VEC];
    load_cols<VEC>(p.w, SSM_F32, 0, col, H, vok, wv);
    if (p.b) load_cols<VEC>(p.b, SSM_F32, 0, col, H, vok, bv);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float o = (v[k][i] - mean) * rstd * wv[i];
      if (p.b) o += bv[i];
      if (p.res && !p.prenorm) o += r[k][i];
      out[i] = o;
    }
    store_cols<VEC>(p.y, p.x_dtype, base, col, H, vok, out);
  }
}

// The one-wavefront-per-row kernel with the element types known at compile time (XT: x and y; RT: residual
// and residual_out) for rows of a multiple of four columns with 16-byte aligned tensors.  Every read is
// unconditional - column indices are clamped into the row, an absent residual or bias reads a stand-in of
// the same type whose value is dropped - so a wavefront's reads are in flight together instead of one
// behind the other, which is what a call on a handful of rows (a decoding step) waits for.
template <typename T, int VEC>
__device__ __forceinline__ void ld_pack(const void *p, size_t i, float (&v)[VEC]) {
  const Pack<T, VEC> raw = *reinterpret_cast<const Pack<T, VEC> *>(reinterpret_cast<const T *>(p) + i);
#pragma unroll
  for (int j = 0; j < VEC; ++j) v[j] = to_f32(raw.v[j]);
}
template <typename T, int VEC>
__device__ __forceinline__ void st_pack(void *p, size_t i, const float (&v)[VEC]) {
  Pack<T, VEC> raw;
#pragma unroll
  for (int j = 0; j < VEC; ++j) raw.v[j] = from_f32<T>(v[j]);
  *reinterpret_cast<Pack<T, VEC> *>(reinterpret_cast<T *>(p) + i) = raw;
}

template <int TRIPS, bool WG, typename XT, typename RT>
__global__ __launch_bounds__(LN_THREADS) void norm_fwd_typed_kernel(const NormParams p) {
  constexpr int VEC = 4;
  constexpr int OWNERS = WG ? LN_THREADS : WAVE;       // threads that share a row
  __shared__ float red[LN_WAVES];
  const int wave = threadIdx.x >> 6, lane = WG ? (int)threadIdx.x : (int)(threadIdx.x & 63);
  const int row = WG ? (int)blockIdx.x : (int)(blockIdx.x * LN_WAVES + wave);
  if (row >= p.rows) return;                           // whole workgroups in WG mode
  const int H = p.hidden;
  const size_t base = (size_t)row * H;
  const bool has_res = p.res != nullptr, has_b = p.b != nullptr;
  // stand-ins of the right element type: residual_out (type RT) or, without one, x (then RT = XT)
  const void *resp = has_res ? p.res : (p.res_out ? (const void *)p.res_out : p.x);
  const float *bp = has_b ? p.b : p.w;
  float v[TRIPS][VEC], r[TRIPS][VEC];
  float sum = 0.0f;
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int colc = min((k * OWNERS + lane) * VEC, H - VEC);
    ld_pack<XT, VEC>(p.x, base + colc, v[k]);
  }
  if (has_res) {                 // one test in front of all of a row's residual reads, none between them
#pragma unroll
    for (int k = 0; k < TRIPS; ++k) ld_pack<RT, VEC>(resp, base + min((k * OWNERS + lane) * VEC, H - VEC), r[k]);
  } else {
#pragma unroll
    for (int k = 0; k < TRIPS; ++k)
#pragma unroll
      for (int i = 0; i < VEC; ++i) r[k][i] = 0.0f;
  }
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int col = (k * OWNERS + lane) * VEC;
    const bool live = col < H;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      if (p.prenorm) v[k][i] += r[k][i];
      if (!live) v[k][i] = 0.0f;
      sum += v[k][i];
    }
    if (p.res_out && live) st_pack<RT, VEC>(p.res_out, base + col, v[k]);
  }
  float wv[TRIPS][VEC], bv[TRIPS][VEC];
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int colc = min((k * OWNERS + lane) * VEC, H - VEC);
    ld_pack<float, VEC>(p.w, colc, wv[k]);
    ld_pack<float, VEC>(bp, colc, bv[k]);
  }
  const float inv_h = 1.0f / (float)H;
  float mean = 0.0f;
  if (!p.is_rms) mean = row_sum<WG>(sum, red) * inv_h;
  float sq = 0.0f;
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const bool live = (k * OWNERS + lane) * VEC < H;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float c = live ? v[k][i] - mean : 0.0f;
      sq = __builtin_fmaf(c, c, sq);
    }
  }
  const float rstd = 1.0f / sqrtf(row_sum<WG>(sq, red) * inv_h + p.eps);
  if (lane == 0) {
    if (p.mean) p.mean[row] = mean;
    if (p.rstd) p.rstd[row] = rstd;
  }
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int col = (k * OWNERS + lane) * VEC;
    float out[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float o = (v[k][i] - mean) * rstd * wv[k][i];
      if (has_b) o += bv[k][i];
      if (has_res && !p.prenorm) o += r[k][i];
      out[i] = o;
    }
    if (col < H) st_pack<XT, VEC>(p.y, base + col, out);
  }
}

template <typename XT, typename RT>
static void launch_norm_fwd_typed(const NormParams &p, int per_lane, unsigned grid, hipStream_t s) {
  const dim3 b(LN_THREADS);
  if (per_lane <= 4) hipLaunchKernelGGL((norm_fwd_typed_kernel<1, false, XT, RT>), dim3(grid), b, 0, s, p);
  else if (per_lane <= 8) hipLaunchKernelGGL((norm_fwd_typed_kernel<2, false, XT, RT>), dim3(grid), b, 0, s, p);
  else if (per_lane <= 12) hipLaunchKernelGGL((norm_fwd_typed_kernel<3, false, XT, RT>), dim3(grid), b, 0, s, p);
  else if (per_lane <= 16) hipLaunchKernelGGL((norm_fwd_typed_kernel<4, false, XT, RT>), dim3(grid), b, 0, s, p);
  // (a trip that holds no column still reads one: rows of 1280, 1536 and 1792 columns get trip counts of their own)
  else if (per_lane <= 20) hipLaunchKernelGGL((norm_fwd_typed_kernel<5, false, XT, RT>), dim3(grid), b, 0, s, p);
  else if (per_lane <= 24) hipLaunchKernelGGL((norm_fwd_typed_kernel<6, false, XT, RT>), dim3(grid), b, 0, s, p);
  else if (per_lane <= 28) hipLaunchKernelGGL((norm_fwd_typed_kernel<7, false, XT, RT>), dim3(grid), b, 0, s, p);
  else if (per_lane <= 32) hipLaunchKernelGGL((norm_fwd_typed_kernel<8, false, XT, RT>), dim3(grid), b, 0, s, p);
  else if (p.hidden <= 4096) hipLaunchKernelGGL((norm_fwd_typed_kernel<4, true, XT, RT>), dim3(p.rows), b, 0, s, p);
  else if (p.hidden <= 5120) hipLaunchKernelGGL((norm_fwd_typed_kernel<5, true, XT, RT>), dim3(p.rows), b, 0, s, p);
  else if (p.hidden <= 6144) hipLaunchKernelGGL((norm_fwd_typed_kernel<6, true, XT, RT>), dim3(p.rows), b, 0, s, p);
  else if (p.hidden <= 8192) hipLaunchKernelGGL((norm_fwd_typed_kernel<8, true, XT, RT>), dim3(p.rows), b, 0, s, p);
  else hipLaunchKernelGGL((norm_fwd_typed_kernel<16, true, XT, RT>), dim3(p.rows), b, 0, s, p);
}

// True when the call was taken by a typed kernel.
static bool norm_fwd_typed(const NormParams &p, int per_lane, unsigned grid, hipStream_t s) {
  if (p.hidden > 16384 || p.hidden < 4) return false;
  // residual and residual_out must agree on one type, float32 or that of x
  int rt = -1;
  if (p.res) rt = p.res_dtype;
  if (p.res_out) {
    if (rt >= 0 && p.res_out_dtype != rt) return false;
    rt = p.res_out_dtype;
  }
  if (rt < 0) rt = p.x_dtype;
  if (rt != SSM_F32 && rt != p.x_dtype) return false;
  const bool rf = rt == SSM_F32;
  if (p.x_dtype == SSM_BF16) rf ? launch_norm_fwd_typed<bf16_t, float>(p, per_lane, grid, s) : launch_norm_fwd_typed<bf16_t, bf16_t>(p, per_lane, grid, s);
  else if (p.x_dtype == SSM_F16) rf ? launch_norm_fwd_typed<f16_t, float>(p, per_lane, grid, s) : launch_norm_fwd_typed<f16_t, f16_t>(p, per_lane, grid, s);
  else launch_norm_fwd_typed<float, float>(p, per_lane, grid, s);
  return true;
}

// Any hidden size: three sweeps over the row from memory.
__global__ __launch_bounds__(LN_THREADS) void norm_fwd_long_kernel(const NormParams p) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int row = blockIdx.x * LN_WAVES + wave;
  if (row >= p.rows) return;
  const int H = p.hidden;
  const size_t base = (size_t)row * H;
  auto val = [&](int c) -> float {
    float v = load_as_f32(p.x, p.x_dtype, base + c);
    if (p.res && p.prenorm) v += load_as_f32(p.res, p.res_dtype, base + c);
    return v;
  };
  float sum = 0.0f;
  for (int c = lane; c < H; c += WAVE) sum += val(c);
  const float inv_h = 1.0f / (float)H;
  const float mean = p.is_rms ? 0.0f : wave_sum(sum) * inv_h;
  float sq = 0.0f;
  for (int c = lane; c < H; c += WAVE) {
    const float d = val(c) - mean;
    sq = __builtin_fmaf(d, d, sq);
  }
  const float rstd = 1.0f / sqrtf(wave_sum(sq) * inv_h + p.eps);
  if (lane == 0) {
    if (p.mean) p.mean[row] = mean;
    if (p.rstd) p.rstd[row] = rstd;
  }
  for (int c = lane; c < H; c += WAVE) {
    const float v = val(c);
    if (p.res_out) store_f32_as(p.res_out, p.res_out_dtype, base + c, v);
    float o = (v - mean) * rstd * p.w[c];
    if (p.b) o += p.b[c];
    if (p.res && !p.prenorm) o += load_as_f32(p.res, p.res_dtype, base + c);
    store_f32_as(p.y, p.x_dtype, base + c, o);
  }
}

// ----------------------------------------------------------------- backward

// Each wave handles rows wave_global, wave_global + nwaves, ...; columns are
// owned by (lane, trip) exactly as in the forward kernel.
// XT = void: element types looked up at run time.  Otherwise x, dy, dx have type XT, residual and dresidual
// type RT, rows are a multiple of four columns long and aligned, and all reads of a row are unconditional
// (clamped columns, a stand-in for an absent residual), i.e. in flight together.
template <int TRIPS, bool WG, typename XT = void, typename RT = void>
__global__ __launch_bounds__(LN_THREADS) void norm_bwd_kernel(const NormParams p, int vec_ok) {
  constexpr int VEC = 4;
  constexpr bool TYPED = !std::is_void<XT>::value;
  using xt = typename std::conditional<TYPED, XT, float>::type;
  using rt = typename std::conditional<TYPED, RT, float>::type;
  constexpr int OWNERS = WG ? LN_THREADS : WAVE;       // threads that share a row
  __shared__ float red[LN_WAVES];
  const int wave = threadIdx.x >> 6, lane = WG ? (int)threadIdx.x : (int)(threadIdx.x & 63);
  const int nwaves = WG ? (int)gridDim.x : (int)(gridDim.x * LN_WAVES);      // row owners in the grid
  const int gw = WG ? (int)blockIdx.x : (int)(blockIdx.x * LN_WAVES + wave);
  const int H = p.hidden;
  const bool vok = vec_ok != 0;
  const float inv_h = 1.0f / (float)H;
  float dw[TRIPS][VEC], db[TRIPS][VEC], wv[TRIPS][VEC];
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int col = (k * OWNERS + lane) * VEC;
    if constexpr (TYPED) ld_pack<float, VEC>(p.w, min(col, H - VEC), wv[k]);
    else load_cols<VEC>(p.w, SSM_F32, 0, col, H, vok, wv[k]);
#pragma unroll
    for (int i = 0; i < VEC; ++i) dw[k][i] = db[k][i] = 0.0f;
  }
  const bool has_add = p.res && p.prenorm;
  // typed reads of a residual that is absent (or not added: post-norm) go to memory of the same element type
  // and extent and are dropped: the residual itself if there is one, else dresidual, else x (then RT = XT)
  const void *resp = p.res ? p.res : (p.dres ? (const void *)p.dres : p.x);
  const float *meanp = p.is_rms ? p.rstd : p.mean;
  for (int row = gw; row < p.rows; row += nwaves) {
    const size_t base = (size_t)row * H;
    float mean = meanp[row];
    if (p.is_rms) mean = 0.0f;
    const float rstd = p.rstd[row];
    float xh[TRIPS][VEC], g[TRIPS][VEC], dyv[TRIPS][VEC];
    float s1 = 0.0f, s2 = 0.0f;     // sum g*xhat, sum g
    float vin[TRIPS][VEC], rin[TRIPS][VEC];
    if constexpr (TYPED) {
#pragma unroll
      for (int k = 0; k < TRIPS; ++k) {
        const int colc = min((k * OWNERS + lane) * VEC, H - VEC);
        ld_pack<xt, VEC>(p.x, base + colc, vin[k]);
        ld_pack<rt, VEC>(resp, base + colc, rin[k]);
        ld_pack<xt, VEC>(p.dy, base + colc, dyv[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < TRIPS; ++k) {
      const int col = (k * OWNERS + lane) * VEC;
      float v[VEC];
      if constexpr (TYPED) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = has_add ? vin[k][i] + rin[k][i] : vin[k][i];
      } else {
        load_cols<VEC>(p.x, p.x_dtype, base, col, H, vok, v);
        if (has_add) {
          float r[VEC];
          load_cols<VEC>(p.res, p.res_dtype, base, col, H, vok, r);
#pragma unroll
          for (int i = 0; i < VEC; ++i) v[i] += r[i];
        }
        load_cols<VEC>(p.dy, p.x_dtype, base, col, H, vok, dyv[k]);
      }
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const bool in = col + i < H;
        xh[k][i] = in ? (v[i] - mean) * rstd : 0.0f;
        g[k][i] = in ? dyv[k][i] * wv[k][i] : 0.0f;
        s1 = __builtin_fmaf(g[k][i], xh[k][i], s1);
        s2 += g[k][i];
        dw[k][i] = __builtin_fmaf(dyv[k][i], xh[k][i], dw[k][i]);
        db[k][i] += dyv[k][i];
      }
    }
    const float c1 = row_sum<WG>(s1, red) * inv_h;
    const float c2 = p.is_rms ? 0.0f : row_sum<WG>(s2, red) * inv_h;
#pragma unroll
    for (int k = 0; k < TRIPS; ++k) {
      const int col = (k * OWNERS + lane) * VEC;
      if (col >= H) continue;
      float dxv[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) dxv[i] = (g[k][i] - c2 - xh[k][i] * c1) * rstd;
      if constexpr (TYPED) {
        st_pack<xt, VEC>(p.dx, base + col, dxv);
        if (p.dres) st_pack<rt, VEC>(p.dres, base + col, p.prenorm ? dxv : dyv[k]);
      } else {
        store_cols<VEC>(p.dx, p.x_dtype, base, col, H, vok, dxv);
        if (p.dres) store_cols<VEC>(p.dres, p.res_dtype, base, col, H, vok, p.prenorm ? dxv : dyv[k]);
      }
    }
  }
  if constexpr (WG) {                                  // every thread owns its columns: the partial is complete
    float *pw = p.partial + (size_t)blockIdx.x * 2 * H;
#pragma unroll
    for (int k = 0; k < TRIPS; ++k) {
      const int col = (k * OWNERS + lane) * VEC;
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        if (col + i < H) {
          pw[col + i] = dw[k][i];
          pw[H + col + i] = db[k][i];
        }
    }
    return;
  }
  // one partial per workgroup: waves 1.. hand their column sums to wave 0 through LDS (fixed order)
  __shared__ float wsum[LN_WAVES - 1][2][WG ? 1 : TRIPS * WAVE * VEC];
  if (wave > 0) {
#pragma unroll
    for (int k = 0; k < TRIPS; ++k) {
      const int col = (k * OWNERS + lane) * VEC;
      *reinterpret_cast<float4 *>(&wsum[wave - 1][0][col]) = make_float4(dw[k][0], dw[k][1], dw[k][2], dw[k][3]);
      *reinterpret_cast<float4 *>(&wsum[wave - 1][1][col]) = make_float4(db[k][0], db[k][1], db[k][2], db[k][3]);
    }
  }
  __syncthreads();
  if (wave == 0) {
    float *pw = p.partial + (size_t)blockIdx.x * 2 * H;
#pragma unroll
    for (int k = 0; k < TRIPS; ++k) {
      const int col = (k * OWNERS + lane) * VEC;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float a = dw[k][i], b = db[k][i];
#pragma unroll
        for (int w = 0; w < LN_WAVES - 1; ++w) {
          a += wsum[w][0][col + i];
          b += wsum[w][1][col + i];
        }
        if (col + i < H) {
          pw[col + i] = a;
          pw[H + col + i] = b;
        }
      }
    }
  }
}

__global__ __launch_bounds__(LN_THREADS) void norm_bwd_long_kernel(const NormParams p) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int nwaves = gridDim.x * LN_WAVES;
  const int gw = blockIdx.x * LN_WAVES + wave;
  const int H = p.hidden;
  const float inv_h = 1.0f / (float)H;
  float *pw = p.partial + (size_t)gw * 2 * H;
  for (int c = lane; c < 2 * H; c += WAVE) pw[c] = 0.0f;
  for (int row = gw; row < p.rows; row += nwaves) {
    const size_t base = (size_t)row * H;
    const float mean = p.is_rms ? 0.0f : p.mean[row];
    const float rstd = p.rstd[row];
    auto xhat = [&](int c) -> float {
      float v = load_as_f32(p.x, p.x_dtype, base + c);
      if (p.res && p.prenorm) v += load_as_f32(p.res, p.res_dtype, base + c);
      return (v - mean) * rstd;
    };
    float s1 = 0.0f, s2 = 0.0f;
    for (int c = lane; c < H; c += WAVE) {
      const float dy = load_as_f32(p.dy, p.x_dtype, base + c);
      const float gg = dy * p.w[c];
      const float xh = xhat(c);
      s1 = __builtin_fmaf(gg, xh, s1);
      s2 += gg;
      pw[c] = __builtin_fmaf(dy, xh, pw[c]);
      pw[H + c] += dy;
    }
    const float c1 = wave_sum(s1) * inv_h;
    const float c2 = p.is_rms ? 0.0f : wave_sum(s2) * inv_h;
    for (int c = lane; c < H; c += WAVE) {
      const float dy = load_as_f32(p.dy, p.x_dtype, base + c);
      const float dxv = (dy * p.w[c] - c2 - xhat(c) * c1) * rstd;
      store_f32_as(p.dx, p.x_dtype, base + c, dxv);
      if (p.dres) store_f32_as(p.dres, p.res_dtype, base + c, p.prenorm ? dxv : dy);
    }
  }
}

// dw[c] = sum_w partial[w][0][c], db[c] = sum_w partial[w][1][c].  A workgroup takes 16 columns; its 256
// threads are 16 columns x 16 slices of the partials, summed in a fixed order (slice by slice, then over slices).
constexpr int FOLD_COLS = 16, FOLD_SLICES = LN_THREADS / FOLD_COLS;
__global__ __launch_bounds__(LN_THREADS) void norm_bwd_fold_kernel(const float *partial, float *dw, float *db,
                                                                    int nparts, int hidden) {
  __shared__ float sw_s[FOLD_SLICES][FOLD_COLS], sb_s[FOLD_SLICES][FOLD_COLS];
  const int cl = threadIdx.x % FOLD_COLS, sl = threadIdx.x / FOLD_COLS;
  const int c = blockIdx.x * FOLD_COLS + cl;
  float sw = 0.0f, sb = 0.0f;
  if (c < hidden) {
    // eight partials at a time: their reads are in flight together, the additions keep their order
    int w = sl;
    for (; w + 7 * FOLD_SLICES < nparts; w += 8 * FOLD_SLICES) {
      float a[8], b[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        a[k] = partial[(size_t)(w + k * FOLD_SLICES) * 2 * hidden + c];
        b[k] = partial[(size_t)(w + k * FOLD_SLICES) * 2 * hidden + hidden + c];
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        sw += a[k];
        sb += b[k];
      }
    }
    for (; w < nparts; w += FOLD_SLICES) {
      sw += partial[(size_t)w * 2 * hidden + c];
      sb += partial[(size_t)w * 2 * hidden + hidden + c];
    }
  }
  sw_s[sl][cl] = sw;
  sb_s[sl][cl] = sb;
  __syncthreads();
  if (sl == 0 && c < hidden) {
    float a = 0.0f, b = 0.0f;
    for (int j = 0; j < FOLD_SLICES; ++j) {
      a += sw_s[j][cl];
      b += sb_s[j][cl];
    }
    dw[c] = a;
    if (db) db[c] = b;
  }
}

static int norm_bwd_grid(int rows) {
  // persistent: at most 4 workgroups per CU on a 256-CU part, never more waves than rows
  const int want = (rows + LN_WAVES - 1) / LN_WAVES;
  return want < 1024 ? (want < 1 ? 1 : want) : 1024;
}

static int norm_check(const char *who, const void *x, const float *w, const void *y, int rows, int hidden,
                      int x_dtype, const void *res, int res_dtype) {
  SSM_REQUIRE(x && w && y, SSM_ERR_NULL_POINTER, "%s: x, weight and output are required", who);
  SSM_REQUIRE(rows > 0 && hidden > 0, SSM_ERR_BAD_SHAPE, "%s: rows=%d hidden=%d must be positive", who, rows, hidden);
  SSM_REQUIRE(valid_dtype(x_dtype) && (!res || valid_dtype(res_dtype)), SSM_ERR_BAD_DTYPE,
              "%s: x_dtype=%d residual_dtype=%d", who, x_dtype, res_dtype);
  SSM_REQUIRE((size_t)rows * hidden < ((size_t)1 << 40), SSM_ERR_TOO_LARGE, "%s: tensor too large", who);
  return SSM_OK;
}

}  // namespace ssm

extern "C" int ssm_norm_fwd(const ssm_norm_fwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_norm_fwd: args is NULL");
  int rc = norm_check("ssm_norm_fwd", a->x, a->weight, a->y, a->rows, a->hidden, a->x_dtype, a->residual,
                      a->residual_dtype);
  if (rc != SSM_OK) return rc;
  if (a->residual_out)
    SSM_REQUIRE(valid_dtype(a->residual_out_dtype), SSM_ERR_BAD_DTYPE, "ssm_norm_fwd: residual_out_dtype=%d",
                a->residual_out_dtype);
  NormParams p{};
  p.x = a->x; p.res = a->residual; p.w = a->weight; p.b = a->bias; p.y = a->y; p.res_out = a->residual_out;
  p.mean = a->mean; p.rstd = a->rstd;
  p.rows = a->rows; p.hidden = a->hidden;
  p.x_dtype = a->x_dtype; p.res_dtype = a->residual_dtype; p.res_out_dtype = a->residual_out_dtype;
  p.is_rms = a->is_rms ? 1 : 0; p.prenorm = a->prenorm ? 1 : 0; p.eps = a->eps;
  const int vec_ok = a->hidden % 4 == 0 && aligned_to(a->x, 16) && aligned_to(a->y, 16) &&
                     aligned_to(a->weight, 16) && (!a->bias || aligned_to(a->bias, 16)) &&
                     (!a->residual || aligned_to(a->residual, 16)) &&
                     (!a->residual_out || aligned_to(a->residual_out, 16));
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  const unsigned grid = (unsigned)((a->rows + LN_WAVES - 1) / LN_WAVES);
  const int per_lane = (a->hidden + WAVE - 1) / WAVE;
  if (vec_ok && norm_fwd_typed(p, per_lane, grid, s)) {
    SSM_CHECK_LAUNCH("ssm_norm_fwd");
    return SSM_OK;
  }
  if (per_lane <= 4) hipLaunchKernelGGL((norm_fwd_kernel<1, false>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (per_lane <= 8) hipLaunchKernelGGL((norm_fwd_kernel<2, false>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (per_lane <= 12) hipLaunchKernelGGL((norm_fwd_kernel<3, false>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (per_lane <= 16) hipLaunchKernelGGL((norm_fwd_kernel<4, false>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (per_lane <= 32) hipLaunchKernelGGL((norm_fwd_kernel<8, false>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (a->hidden <= 4096) hipLaunchKernelGGL((norm_fwd_kernel<4, true>), dim3(a->rows), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (a->hidden <= 8192) hipLaunchKernelGGL((norm_fwd_kernel<8, true>), dim3(a->rows), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (a->hidden <= 16384) hipLaunchKernelGGL((norm_fwd_kernel<16, true>), dim3(a->rows), dim3(LN_THREADS), 0, s, p, vec_ok);
  else hipLaunchKernelGGL(norm_fwd_long_kernel, dim3(grid), dim3(LN_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_norm_fwd");
  return SSM_OK;
}

namespace ssm {
template <typename XT, typename RT>
static void launch_norm_bwd_typed(const NormParams &p, int hidden, int grid, hipStream_t s) {
  const int per_lane = (hidden + WAVE - 1) / WAVE;
  const dim3 g(grid), b(LN_THREADS);
  if (per_lane <= 4) hipLaunchKernelGGL((norm_bwd_kernel<1, false, XT, RT>), g, b, 0, s, p, 1);
  else if (per_lane <= 8) hipLaunchKernelGGL((norm_bwd_kernel<2, false, XT, RT>), g, b, 0, s, p, 1);
  else if (per_lane <= 12) hipLaunchKernelGGL((norm_bwd_kernel<3, false, XT, RT>), g, b, 0, s, p, 1);
  else if (hidden <= 1024) hipLaunchKernelGGL((norm_bwd_kernel<1, true, XT, RT>), g, b, 0, s, p, 1);
  else if (hidden <= 2048) hipLaunchKernelGGL((norm_bwd_kernel<2, true, XT, RT>), g, b, 0, s, p, 1);
  // a thread's registers grow with the trips it is compiled for: the widths of common models (2560, 5120) get
  // their own count rather than the next power of two
  else if (hidden <= 3072) hipLaunchKernelGGL((norm_bwd_kernel<3, true, XT, RT>), g, b, 0, s, p, 1);
  else if (hidden <= 4096) hipLaunchKernelGGL((norm_bwd_kernel<4, true, XT, RT>), g, b, 0, s, p, 1);
  else if (hidden <= 5120) hipLaunchKernelGGL((norm_bwd_kernel<5, true, XT, RT>), g, b, 0, s, p, 1);
  else if (hidden <= 6144) hipLaunchKernelGGL((norm_bwd_kernel<6, true, XT, RT>), g, b, 0, s, p, 1);
  else hipLaunchKernelGGL((norm_bwd_kernel<8, true, XT, RT>), g, b, 0, s, p, 1);
}
}  // namespace ssm

extern "C" size_t ssm_norm_bwd_workspace_bytes(int rows, int hidden) {
  if (rows <= 0 || hidden <= 0) return 0;
  return (size_t)ssm::norm_bwd_grid(rows) * ssm::LN_WAVES * 2 * (size_t)hidden * sizeof(float);
}

namespace ssm {

// Partial column sums one call writes before the fold reads them: one per workgroup, or one per wave for rows
// beyond 8192 columns.
static size_t norm_bwd_partials(int rows, int hidden) {
  const size_t grid = (size_t)norm_bwd_grid(rows);
  return hidden <= 8192 ? grid : grid * LN_WAVES;
}

static int norm_bwd_check(const char *who, const ssm_norm_bwd_args *a) {
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "%s: args is NULL", who);
  int rc = norm_check(who, a->x, a->weight, a->dx, a->rows, a->hidden, a->x_dtype, a->residual, a->residual_dtype);
  if (rc != SSM_OK) return rc;
  SSM_REQUIRE(a->dy && a->rstd && a->dweight && (a->is_rms || a->mean), SSM_ERR_NULL_POINTER,
              "%s: dy, rstd, dweight (and mean for LayerNorm) are required", who);
  SSM_REQUIRE(!a->dresidual || a->residual, SSM_ERR_NULL_POINTER, "%s: dresidual needs residual", who);
  return SSM_OK;
}

// The launches of the backward pass; `partial` holds norm_bwd_partials() x 2 x hidden floats.
static int norm_bwd_launch(const ssm_norm_bwd_args *a, float *partial, void *hip_stream) {
  NormParams p{};
  p.x = a->x; p.res = a->residual; p.dy = a->dy; p.w = a->weight; p.dx = a->dx; p.dres = a->dresidual;
  p.mean = const_cast<float *>(a->mean); p.rstd = const_cast<float *>(a->rstd);
  p.partial = partial;
  p.rows = a->rows; p.hidden = a->hidden;
  p.x_dtype = a->x_dtype; p.res_dtype = a->residual_dtype;
  p.is_rms = a->is_rms ? 1 : 0; p.prenorm = a->prenorm ? 1 : 0;
  const int vec_ok = a->hidden % 4 == 0 && aligned_to(a->x, 16) && aligned_to(a->dy, 16) && aligned_to(a->dx, 16) &&
                     aligned_to(a->weight, 16) && (!a->residual || aligned_to(a->residual, 16)) &&
                     (!a->dresidual || aligned_to(a->dresidual, 16));
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  const int grid = norm_bwd_grid(a->rows);
  const int per_lane = (a->hidden + WAVE - 1) / WAVE;
  // typed kernels: one element type RT (float32 or that of x) for residual and dresidual
  const int rt = (a->residual || a->dresidual) ? a->residual_dtype : a->x_dtype;
  if (vec_ok && a->hidden >= 4 && a->hidden <= 8192 && (rt == SSM_F32 || rt == a->x_dtype)) {
    const bool rf = rt == SSM_F32;
    if (a->x_dtype == SSM_BF16) rf ? launch_norm_bwd_typed<bf16_t, float>(p, a->hidden, grid, s) : launch_norm_bwd_typed<bf16_t, bf16_t>(p, a->hidden, grid, s);
    else if (a->x_dtype == SSM_F16) rf ? launch_norm_bwd_typed<f16_t, float>(p, a->hidden, grid, s) : launch_norm_bwd_typed<f16_t, f16_t>(p, a->hidden, grid, s);
    else launch_norm_bwd_typed<float, float>(p, a->hidden, grid, s);
  }
  else if (per_lane <= 4) hipLaunchKernelGGL((norm_bwd_kernel<1, false>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (per_lane <= 8) hipLaunchKernelGGL((norm_bwd_kernel<2, false>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (per_lane <= 12) hipLaunchKernelGGL((norm_bwd_kernel<3, false>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (a->hidden <= 1024) hipLaunchKernelGGL((norm_bwd_kernel<1, true>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (a->hidden <= 2048) hipLaunchKernelGGL((norm_bwd_kernel<2, true>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (a->hidden <= 4096) hipLaunchKernelGGL((norm_bwd_kernel<4, true>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else if (a->hidden <= 8192) hipLaunchKernelGGL((norm_bwd_kernel<8, true>), dim3(grid), dim3(LN_THREADS), 0, s, p, vec_ok);
  else hipLaunchKernelGGL(norm_bwd_long_kernel, dim3(grid), dim3(LN_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_norm_bwd");
  const int nparts = a->hidden <= 8192 ? grid : grid * LN_WAVES;   // the long-row kernel writes one per wave
  hipLaunchKernelGGL(norm_bwd_fold_kernel, dim3((a->hidden + FOLD_COLS - 1) / FOLD_COLS), dim3(LN_THREADS), 0, s,
                     p.partial, a->dweight, a->dbias, nparts, a->hidden);
  SSM_CHECK_LAUNCH("ssm_norm_bwd(fold)");
  return SSM_OK;
}

// Device memory for the partial sums of ssm_norm_bwd_static: part of the code object, so every GPU that the
// library runs on holds its own copy from load to process end.  The name is a host-side handle only; the
// address on the current device comes from hipGetSymbolAddress and is kept per device.
constexpr size_t NORM_BWD_STATIC_FLOATS = SSM_NORM_BWD_STATIC_BYTES / sizeof(float);
static __device__ __align__(256) float scratch[NORM_BWD_STATIC_FLOATS];

constexpr int MAX_DEVICES = 64;
static std::mutex scratch_lock;
static float *scratch_on_device[MAX_DEVICES];

static int norm_bwd_scratch(float **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    set_error("ssm_norm_bwd_static: no usable current device (%s)", e == hipSuccess ? "index out of range" : hipGetErrorString(e));
    return SSM_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (!scratch_on_device[dev]) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      set_error("ssm_norm_bwd_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return SSM_ERR_LAUNCH;
    }
    scratch_on_device[dev] = reinterpret_cast<float *>(ptr);
  }
  *out = scratch_on_device[dev];
  return SSM_OK;
}

}  // namespace ssm

extern "C" int ssm_norm_bwd(const ssm_norm_bwd_args *a, void *hip_stream) {
  using namespace ssm;
  const int rc = norm_bwd_check("ssm_norm_bwd", a);
  if (rc != SSM_OK) return rc;
  SSM_REQUIRE(a->workspace && a->workspace_bytes >= ssm_norm_bwd_workspace_bytes(a->rows, a->hidden),
              SSM_ERR_WORKSPACE, "ssm_norm_bwd: workspace of %zu bytes required",
              ssm_norm_bwd_workspace_bytes(a->rows, a->hidden));
  return norm_bwd_launch(a, reinterpret_cast<float *>(a->workspace), hip_stream);
}

extern "C" int ssm_norm_bwd_static(const ssm_norm_bwd_args *a, void *hip_stream) {
  using namespace ssm;
  int rc = norm_bwd_check("ssm_norm_bwd_static", a);
  if (rc != SSM_OK) return rc;
  const size_t need = norm_bwd_partials(a->rows, a->hidden) * 2 * (size_t)a->hidden;
  SSM_REQUIRE(need <= NORM_BWD_STATIC_FLOATS, SSM_ERR_TOO_LARGE,
              "ssm_norm_bwd_static: rows=%d hidden=%d need %zu bytes of partial sums, the built-in buffer holds %zu; "
              "use ssm_norm_bwd with a workspace", a->rows, a->hidden, need * sizeof(float),
              (size_t)SSM_NORM_BWD_STATIC_BYTES);
  float *partial = nullptr;
  rc = norm_bwd_scratch(&partial);
  if (rc != SSM_OK) return rc;
  return norm_bwd_launch(a, partial, hip_stream);
}
