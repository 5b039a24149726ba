// Depthwise causal 1-D convolution (+ optional SiLU), forward and backward.
//
//   pre[b,c,t] = bias[c] + sum_k w[c,k] x[b,c,t-(K-1)+k]      (x = 0 for t < 0)
//   y          = silu(pre) or pre
//
// Pure streaming kernels: every thread owns one 16-byte run of the output
// (VEC elements) and rebuilds its input window from the 16-byte runs around
// it, so HBM sees each byte once and the overlap is served by L1/L2.
//   channels-first (B,C,L): runs are along time; one workgroup per (b,c) row.
//   channels-last  (B,L,C): runs are along channels; a thread slides over a
//                           strip of time steps keeping K rows in registers.
// Shapes the vector path cannot take (misaligned rows, K-1 > VEC) go through
// an element-wise kernel with explicit bounds.
//
// Backward recomputes pre (no activation is saved), forms g = dout*silu'(pre),
// emits dx = sum_k g[t+(K-1)-k] w[k] and per-row partial sums of dw/dbias that
// a second kernel folds over the batch in a fixed order (no atomics).
#include "common.hpp"

namespace ssm {

constexpr int CONV_TAPS = 5;           // widest kernel the vector paths take (K <= 5)
constexpr int CONV_THREADS = 256;
constexpr int CONV_WHOLE_BATCH_MIN_CHANNELS = 1024;   // (B,C,L) backward: from here on a workgroup per channel

// Taps in reverse order: wrev[m] multiplies x[t - m]; zero beyond the kernel width.
template <int TAPS>
__device__ __forceinline__ void load_taps(const float *w, int c, int K, float (&wrev)[TAPS]) {
#pragma unroll
  for (int m = 0; m < TAPS; ++m) wrev[m] = m < K ? w[(size_t)c * K + (K - 1 - m)] : 0.0f;
}

// The taps and the bias of VEC neighbouring channels from channel c0 on.  `wide`: the kernel is 4 wide and weight and
// bias start on 16-byte boundaries, c0 is a multiple of VEC: one 16-byte read per channel and one read for the
// biases instead of five 4-byte reads per channel (a thread that owns 8 steps of 4 channels otherwise issues more
// reads for its taps than for its rows).
template <int VEC, int TAPS>
__device__ __forceinline__ void load_taps_of(const float *w, const float *b, int c0, int K, bool wide,
                                             float (&wrev)[VEC][TAPS], float (&bias)[VEC]) {
  if (wide) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const Pack<float, 4> q = *reinterpret_cast<const Pack<float, 4> *>(w + (size_t)(c0 + i) * 4);
      wrev[i][0] = q.v[3]; wrev[i][1] = q.v[2]; wrev[i][2] = q.v[1]; wrev[i][3] = q.v[0];
#pragma unroll
      for (int m = 4; m < TAPS; ++m) wrev[i][m] = 0.0f;
    }
    if (b) {
      const Pack<float, VEC> q = *reinterpret_cast<const Pack<float, VEC> *>(b + c0);
#pragma unroll
      for (int i = 0; i < VEC; ++i) bias[i] = q.v[i];
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) bias[i] = 0.0f;
    }
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      bias[i] = b ? b[c0 + i] : 0.0f;
      load_taps(w, c0 + i, K, wrev[i]);
    }
  }
}

struct ConvParams {
  const void *x, *dout;
  const float *w, *bias;     // (C,K) fp32, (C,) fp32 or null
  void *y;                   // fwd: y ; bwd: dx
  float *partial;            // bwd: [B][C][K+1] partial sums (dw..., dbias)
  int batch, chans, len, K;
  int silu;
  long long x_bs, x_rs;      // rows-in kernels: elements between batch rows and between time steps of x
  int wide_taps;             // K == 4, weight and bias on 16-byte boundaries (see load_taps_of)
  float *dw, *dbias;         // (B,C,L) backward with `whole_batch`: the sums themselves instead of partials
  int whole_batch;           // (B,C,L) backward: a workgroup takes a channel's rows of every batch entry in turn
};

__device__ __forceinline__ float silu_grad(float pre) {
  const float s = sigmoid_f32(pre);
  return s * __builtin_fmaf(pre, 1.0f - s, 1.0f);
}

// A whole vector at element t of a row of `len` elements (a multiple of VEC, 16-byte aligned), zeros when
// the vector lies before or past the row: the read itself is unconditional (the index is clamped into the
// row), so several of them are in flight together instead of each waiting behind its own bounds check.
template <typename T, int VEC>
__device__ __forceinline__ void load_vec_or_zero(const T *row, int t, int len, float (&out)[VEC]) {
  const int tc = min(max(t, 0), len - VEC);
  const Pack<T, VEC> raw = *reinterpret_cast<const Pack<T, VEC> *>(row + tc);
  const bool in = t >= 0 && t < len;
#pragma unroll
  for (int i = 0; i < VEC; ++i) out[i] = in ? to_f32(raw.v[i]) : 0.0f;
}

template <typename T, int VEC>
__device__ __forceinline__ void store_vec(T *row, int t, const float (&v)[VEC]) {
  Pack<T, VEC> raw;
#pragma unroll
  for (int i = 0; i < VEC; ++i) raw.v[i] = from_f32<T>(v[i]);
  *reinterpret_cast<Pack<T, VEC> *>(row + t) = raw;
}

// ---------------------------------------------------------------- forward, (B,C,L)

// AL: rows (channel vectors) start on 16-byte boundaries and the row length (channel count) is a whole
// number of vectors; otherwise the same kernel reads and writes element by element.
template <typename T, bool AL, int TAPS>
__global__ __launch_bounds__(CONV_THREADS) void conv_fwd_cf_kernel(const ConvParams p) {
  constexpr int VEC = 16 / sizeof(T);
  const int row = blockIdx.x;                       // b * C + c
  const int c = row % p.chans;
  const T *xr = reinterpret_cast<const T *>(p.x) + (size_t)row * p.len;
  T *yr = reinterpret_cast<T *>(p.y) + (size_t)row * p.len;
  float wrev1[1][TAPS], bias1[1];
  load_taps_of<1, TAPS>(p.w, p.bias, c, p.K, p.wide_taps, wrev1, bias1);
  const float (&wrev)[TAPS] = wrev1[0];
  const float bias = bias1[0];
  for (int t0 = threadIdx.x * VEC; t0 < p.len; t0 += CONV_THREADS * VEC) {
    float win[2 * VEC];
    if constexpr (AL) {
      float prev[VEC], cur[VEC];
      load_vec_or_zero<T, VEC>(xr, t0 - VEC, p.len, prev);
      load_vec_or_zero<T, VEC>(xr, t0, p.len, cur);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        win[i] = prev[i];
        win[VEC + i] = cur[i];
      }
    } else {
      if (t0 > 0) {
        float prev[VEC];
        load_run<T, VEC>(xr, t0 - VEC, p.len, AL, prev);
#pragma unroll
        for (int i = 0; i < VEC; ++i) win[i] = prev[i];
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) win[i] = 0.0f;
      }
      float cur[VEC];
      load_run<T, VEC>(xr, t0, p.len, AL, cur);
#pragma unroll
      for (int i = 0; i < VEC; ++i) win[VEC + i] = cur[i];
    }
    float out[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float acc = bias;
#pragma unroll
      for (int m = 0; m < TAPS; ++m) acc = __builtin_fmaf(wrev[m], win[VEC + i - m], acc);
      out[i] = p.silu ? silu_f32(acc) : acc;
    }
    if constexpr (AL) store_vec<T, VEC>(yr, t0, out);
    else store_run<T, VEC>(yr, t0, p.len, AL, out);
  }
}

// Element-wise forward for any K / alignment, either layout.
template <typename T>
__global__ __launch_bounds__(CONV_THREADS) void conv_fwd_generic_kernel(const ConvParams p, int channels_last) {
  const size_t total = (size_t)p.batch * p.chans * p.len;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
    int b, c, t;
    if (channels_last) { c = (int)(e % p.chans); t = (int)((e / p.chans) % p.len); b = (int)(e / ((size_t)p.chans * p.len)); }
    else { t = (int)(e % p.len); c = (int)((e / p.len) % p.chans); b = (int)(e / ((size_t)p.chans * p.len)); }
    float acc = p.bias ? p.bias[c] : 0.0f;
    for (int k = 0; k < p.K; ++k) {
      const int ts = t - (p.K - 1) + k;
      if (ts < 0) continue;
      const size_t idx = channels_last ? ((size_t)b * p.len + ts) * p.chans + c : ((size_t)b * p.chans + c) * p.len + ts;
      acc = __builtin_fmaf(p.w[(size_t)c * p.K + k], to_f32(reinterpret_cast<const T *>(p.x)[idx]), acc);
    }
    reinterpret_cast<T *>(p.y)[e] = from_f32<T>(p.silu ? silu_f32(acc) : acc);
  }
}

// ---------------------------------------------------------------- forward, (B,L,C)

constexpr int CONV_CL_STRIP = 16;   // time steps per thread

// AL: rows (channel vectors) start on 16-byte boundaries and the row length (channel count) is a whole
// number of vectors; otherwise the same kernel reads and writes element by element.
constexpr int CONV_CL_FWD_BYTES = 8;   // bytes of channels per thread
template <typename T, bool AL, int TAPS>
__global__ __launch_bounds__(CONV_THREADS) void conv_fwd_cl_kernel(const ConvParams p) {
  constexpr int VEC = CONV_CL_FWD_BYTES / sizeof(T);
  const int cvecs = (p.chans + VEC - 1) / VEC;
  const int strips = (p.len + CONV_CL_STRIP - 1) / CONV_CL_STRIP;
  const size_t total = (size_t)p.batch * strips * cvecs;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int cv = (int)(gid % cvecs);
  const int strip = (int)((gid / cvecs) % strips);
  const int b = (int)(gid / ((size_t)cvecs * strips));
  const int c0 = cv * VEC;
  const int cw = min(VEC, p.chans - c0);          // channels of this vector that exist
  const int K = p.K;
  constexpr int HIST = TAPS - 1;
  float wrev[VEC][TAPS], bias[VEC];
  if constexpr (AL) load_taps_of<VEC, TAPS>(p.w, p.bias, c0, K, p.wide_taps, wrev, bias);
  else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      bias[i] = (p.bias && i < cw) ? p.bias[c0 + i] : 0.0f;
      load_taps(p.w, i < cw ? c0 + i : c0, K, wrev[i]);
    }
  }
  const T *xb = reinterpret_cast<const T *>(p.x) + (size_t)b * p.len * p.chans + c0;
  T *yb = reinterpret_cast<T *>(p.y) + (size_t)b * p.len * p.chans + c0;
  const int t_begin = strip * CONV_CL_STRIP;
  const int t_end = min(p.len, t_begin + CONV_CL_STRIP);
  if constexpr (AL) {
    // all rows of the strip and the K-1 before it are requested at once, unconditionally (row index clamped
    // into the sequence, rows before its start become zeros): one wait instead of one per step
    Pack<T, VEC> raw[HIST + CONV_CL_STRIP];
#pragma unroll
    for (int j = 0; j < HIST + CONV_CL_STRIP; ++j) {
      const int ts = t_begin - HIST + j;
      raw[j] = *reinterpret_cast<const Pack<T, VEC> *>(xb + (size_t)min(max(ts, 0), p.len - 1) * p.chans);
    }
#pragma unroll
    for (int j = 0; j < HIST; ++j) {
      if (t_begin - HIST + j < 0) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) raw[j].v[i] = from_f32<T>(0.0f);
      }
    }
#pragma unroll
    for (int s = 0; s < CONV_CL_STRIP; ++s) {
      if (t_begin + s >= t_end) break;
      float out[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float acc = bias[i];
#pragma unroll
        for (int m = 0; m < TAPS; ++m) acc = __builtin_fmaf(wrev[i][m], to_f32(raw[HIST + s - m].v[i]), acc);
        out[i] = p.silu ? silu_f32(acc) : acc;
      }
      store_vec<T, VEC>(yb + (size_t)(t_begin + s) * p.chans, 0, out);
    }
    return;
  }
  // hist[j] holds x at time (t - 1 - j); filled with the K-1 rows before the strip
  float hist[HIST][VEC];
#pragma unroll
  for (int j = 0; j < HIST; ++j) {
    const int ts = t_begin - 1 - j;
    float v[VEC];
    if (j < K - 1 && ts >= 0) load_run<T, VEC>(xb + (size_t)ts * p.chans, 0, cw, AL, v);
    else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] = 0.0f;
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) hist[j][i] = v[i];
  }
  for (int t = t_begin; t < t_end; ++t) {
    float cur[VEC], out[VEC];
    load_run<T, VEC>(xb + (size_t)t * p.chans, 0, cw, AL, cur);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float acc = __builtin_fmaf(wrev[i][0], cur[i], bias[i]);
#pragma unroll
      for (int j = 0; j < HIST; ++j) acc = __builtin_fmaf(wrev[i][j + 1], hist[j][i], acc);
      out[i] = p.silu ? silu_f32(acc) : acc;
    }
    store_run<T, VEC>(yb + (size_t)t * p.chans, 0, cw, AL, out);
#pragma unroll
    for (int j = HIST - 1; j > 0; --j)
#pragma unroll
      for (int i = 0; i < VEC; ++i) hist[j][i] = hist[j - 1][i];
#pragma unroll
    for (int i = 0; i < VEC; ++i) hist[0][i] = cur[i];
  }
}

// The same forward for aligned rows of sequences of at least a few strips: a thread walks CONV_CL_WALK strips in
// turn.  A launch of one strip per thread runs as a single round of waves that all read, then all compute, then
// all write.  Walking, a thread requests the rows of its next strip before it computes the present one and keeps
// the present strip's last K-1 rows as the next one's history (no row is read twice): 25.4 -> 24.1 us at
// 8 x 2048 x 1536 bf16, whatever the number of strips walked (2 to 16).  What remains is not the shape of the
// walk: the channels-first kernel does the same arithmetic per element in 19.5 us on rows that are contiguous
// in time.
constexpr int CONV_CL_WALK = 4, CONV_CL_WALK_STRIP = 8;   // strips of 8 steps: 24.1 us against 25.4 with 16 and 27.9 with 32
constexpr int CONV_CL_WALK_THREADS = 64;
template <typename T, int TAPS>
__global__ __launch_bounds__(CONV_CL_WALK_THREADS) void conv_fwd_cl_walk_kernel(const ConvParams p) {
  constexpr int VEC = CONV_CL_FWD_BYTES / sizeof(T);
  constexpr int HIST = TAPS - 1, S = CONV_CL_WALK_STRIP, SPAN = CONV_CL_WALK_STRIP * CONV_CL_WALK;
  const int cvecs = p.chans / VEC;
  const int spans = (p.len + SPAN - 1) / SPAN;
  const size_t total = (size_t)p.batch * spans * cvecs;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int cv = (int)(gid % cvecs);
  const int span = (int)((gid / cvecs) % spans);
  const int b = (int)(gid / ((size_t)cvecs * spans));
  const int c0 = cv * VEC;
  float wrev[VEC][TAPS], bias[VEC];
  load_taps_of<VEC, TAPS>(p.w, p.bias, c0, p.K, p.wide_taps, wrev, bias);
  const T *xb = reinterpret_cast<const T *>(p.x) + (size_t)b * p.len * p.chans + c0;
  T *yb = reinterpret_cast<T *>(p.y) + (size_t)b * p.len * p.chans + c0;
  const int t_first = span * SPAN;
  Pack<T, VEC> raw[HIST + S];
#pragma unroll
  for (int j = 0; j < HIST + S; ++j)
    raw[j] = *reinterpret_cast<const Pack<T, VEC> *>(xb + (size_t)min(max(t_first - HIST + j, 0), p.len - 1) * p.chans);
#pragma unroll
  for (int j = 0; j < HIST; ++j) {
    if (t_first - HIST + j < 0) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) raw[j].v[i] = from_f32<T>(0.0f);
    }
  }
#pragma unroll
  for (int w = 0; w < CONV_CL_WALK; ++w) {
    const int t_begin = t_first + w * S;
    Pack<T, VEC> nxt[S];
    if (w + 1 < CONV_CL_WALK) {
#pragma unroll
      for (int j = 0; j < S; ++j)
        nxt[j] = *reinterpret_cast<const Pack<T, VEC> *>(xb + (size_t)min(t_begin + S + j, p.len - 1) * p.chans);
    }
#pragma unroll
    for (int sidx = 0; sidx < S; ++sidx) {
      float out[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float acc = bias[i];
#pragma unroll
        for (int m = 0; m < TAPS; ++m) acc = __builtin_fmaf(wrev[i][m], to_f32(raw[HIST + sidx - m].v[i]), acc);
        out[i] = p.silu ? silu_f32(acc) : acc;
      }
      if (t_begin + sidx < p.len) store_vec<T, VEC>(yb + (size_t)(t_begin + sidx) * p.chans, 0, out);
    }
    if (w + 1 < CONV_CL_WALK) {
#pragma unroll
      for (int j = 0; j < HIST; ++j) raw[j] = raw[S + j];
#pragma unroll
      for (int j = 0; j < S; ++j) raw[HIST + j] = nxt[j];
    }
  }
}

// --------------------------------------------------------------- backward, (B,C,L)

// AL: rows (channel vectors) start on 16-byte boundaries and the row length (channel count) is a whole
// number of vectors; otherwise the same kernel reads and writes element by element.
template <typename T, bool AL, int TAPS>
__global__ __launch_bounds__(CONV_THREADS) void conv_bwd_cf_kernel(const ConvParams p) {
  constexpr int VEC = 16 / sizeof(T);
  __shared__ float red[CONV_THREADS / WAVE][TAPS + 1];
  const int c = blockIdx.x % p.chans;
  const int K = p.K;
  float wrev1[1][TAPS], bias1[1];
  load_taps_of<1, TAPS>(p.w, p.bias, c, K, p.wide_taps, wrev1, bias1);
  const float (&wrev)[TAPS] = wrev1[0];
  const float bias = bias1[0];
  float dwrev[TAPS], db = 0.0f;
#pragma unroll
  for (int m = 0; m < TAPS; ++m) dwrev[m] = 0.0f;

  // the rows of this workgroup: one (b, c) row, or with `whole_batch` channel c of every batch entry
  const int b_first = p.whole_batch ? 0 : (int)(blockIdx.x / p.chans);
  const int b_end = p.whole_batch ? p.batch : b_first + 1;
  for (int b = b_first; b < b_end; ++b) {
  const size_t row = (size_t)b * p.chans + c;
  const T *xr = reinterpret_cast<const T *>(p.x) + row * p.len;
  const T *gr = reinterpret_cast<const T *>(p.dout) + row * p.len;
  T *dxr = reinterpret_cast<T *>(p.y) + row * p.len;
  for (int t0 = threadIdx.x * VEC; t0 < p.len; t0 += CONV_THREADS * VEC) {
    // x over [t0-VEC, t0+2*VEC), dout over [t0, t0+2*VEC)
    float xw[3 * VEC], g[2 * VEC];
    if constexpr (AL) {
      float v0[VEC], v1[VEC], v2[VEC], g0[VEC], g1[VEC];
      load_vec_or_zero<T, VEC>(xr, t0 - VEC, p.len, v0);
      load_vec_or_zero<T, VEC>(xr, t0, p.len, v1);
      load_vec_or_zero<T, VEC>(xr, t0 + VEC, p.len, v2);
      load_vec_or_zero<T, VEC>(gr, t0, p.len, g0);
      load_vec_or_zero<T, VEC>(gr, t0 + VEC, p.len, g1);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        xw[i] = v0[i]; xw[VEC + i] = v1[i]; xw[2 * VEC + i] = v2[i];
        g[i] = g0[i]; g[VEC + i] = g1[i];
      }
    } else {
      float v[VEC];
      if (t0 > 0) load_run<T, VEC>(xr, t0 - VEC, p.len, AL, v);
      else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = 0.0f;
      }
#pragma unroll
      for (int i = 0; i < VEC; ++i) xw[i] = v[i];
      load_run<T, VEC>(xr, t0, p.len, AL, v);
#pragma unroll
      for (int i = 0; i < VEC; ++i) xw[VEC + i] = v[i];
      load_run<T, VEC>(xr, t0 + VEC, p.len, AL, v);       // zero past the end
#pragma unroll
      for (int i = 0; i < VEC; ++i) xw[2 * VEC + i] = v[i];
      load_run<T, VEC>(gr, t0, p.len, AL, v);
#pragma unroll
      for (int i = 0; i < VEC; ++i) g[i] = v[i];
      load_run<T, VEC>(gr, t0 + VEC, p.len, AL, v);
#pragma unroll
      for (int i = 0; i < VEC; ++i) g[VEC + i] = v[i];
    }
    if (p.silu) {
      // g <- dout * silu'(pre) on [t0, t0 + VEC + K - 1)
#pragma unroll
      for (int i = 0; i < 2 * VEC; ++i) {
        if (i < VEC + K - 1) {
          float pre = bias;
#pragma unroll
          for (int m = 0; m < TAPS; ++m) pre = __builtin_fmaf(wrev[m], xw[VEC + i - m], pre);
          g[i] *= silu_grad(pre);
        }
      }
    }
    float dx[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float acc = 0.0f;
#pragma unroll
      for (int m = 0; m < TAPS; ++m) acc = __builtin_fmaf(g[i + m], wrev[m], acc);
      dx[i] = acc;
      db += g[i];
#pragma unroll
      for (int m = 0; m < TAPS; ++m) dwrev[m] = __builtin_fmaf(g[i], xw[VEC + i - m], dwrev[m]);
    }
    if constexpr (AL) store_vec<T, VEC>(dxr, t0, dx);
    else store_run<T, VEC>(dxr, t0, p.len, AL, dx);
  }
  }
  // block reduction of dw[0..K) and db
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
  for (int m = 0; m < TAPS; ++m) {
    const float s = wave_sum(dwrev[m]);
    if (lane == 0) red[wave][m] = s;
  }
  {
    const float s = wave_sum(db);
    if (lane == 0) red[wave][TAPS] = s;
  }
  __syncthreads();
  if (threadIdx.x <= K) {
    // slot k < K holds dw[k] = dwrev[K-1-k]; slot K holds dbias
    const int src = threadIdx.x < K ? (K - 1 - (int)threadIdx.x) : TAPS;
    float s = 0.0f;
    for (int wv = 0; wv < CONV_THREADS / WAVE; ++wv) s += red[wv][src];
    if (!p.whole_batch) p.partial[(size_t)blockIdx.x * (K + 1) + threadIdx.x] = s;
    else if ((int)threadIdx.x < K) p.dw[(size_t)c * K + threadIdx.x] = s;
    else if (p.dbias) p.dbias[c] = s;
  }
}

// ---------------------------------------------------------------- backward, (B,L,C)
// A thread owns 16 bytes of channels over one time segment and walks it once: x and dout of a step are
// read, the pre-activation rebuilt from the last steps of x, the gradient g_t at the pre-activation kept
// for the next steps, and dx of three steps back (which needs g up to three steps ahead) written.  Sums
// for dw and dbias over the thread's own steps go out as one partial per (batch, segment).
constexpr int CONV_CL_SEGS = 32;    // time segments per batch row at most (the workspace is sized for it)

__host__ __device__ inline int conv_cl_seg_len(int len) {
  const int per = (len + CONV_CL_SEGS - 1) / CONV_CL_SEGS;
  return per < 16 ? 16 : per;
}

// AL: rows (channel vectors) start on 16-byte boundaries and the row length (channel count) is a whole
// number of vectors; otherwise the same kernel reads and writes element by element.
constexpr int CONV_CL_BWD_BYTES = 4;   // bytes of channels per thread: the walk keeps ~20 values per channel in registers
template <typename T, bool AL, int TAPS>
__global__ __launch_bounds__(CONV_THREADS) void conv_bwd_cl_kernel(const ConvParams p) {
  constexpr int VEC = CONV_CL_BWD_BYTES / sizeof(T);
  constexpr int HIST = TAPS - 1;
  const int cvecs = (p.chans + VEC - 1) / VEC;
  const int seg_len = conv_cl_seg_len(p.len);
  const int nseg = (p.len + seg_len - 1) / seg_len;
  const size_t total = (size_t)p.batch * nseg * cvecs;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int cv = (int)(gid % cvecs);
  const int seg = (int)((gid / cvecs) % nseg);
  const int b = (int)(gid / ((size_t)cvecs * nseg));
  const int c0 = cv * VEC;
  const int cw = min(VEC, p.chans - c0);          // channels of this vector that exist
  const int K = p.K;
  float wrev[VEC][TAPS], bias[VEC], dwr[VEC][TAPS], db[VEC];
  if constexpr (AL) load_taps_of<VEC, TAPS>(p.w, p.bias, c0, K, p.wide_taps, wrev, bias);
  else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      bias[i] = (p.bias && i < cw) ? p.bias[c0 + i] : 0.0f;
      load_taps(p.w, i < cw ? c0 + i : c0, K, wrev[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    db[i] = 0.0f;
#pragma unroll
    for (int m = 0; m < TAPS; ++m) dwr[i][m] = 0.0f;
  }
  const T *xb = reinterpret_cast<const T *>(p.x) + (size_t)b * p.len * p.chans + c0;
  const T *gb = reinterpret_cast<const T *>(p.dout) + (size_t)b * p.len * p.chans + c0;
  T *dxb = reinterpret_cast<T *>(p.y) + (size_t)b * p.len * p.chans + c0;
  const int t_begin = seg * seg_len;
  const int t_end = min(p.len, t_begin + seg_len);
  // xh[j] = x at time (t - 1 - j), gh[m] = g at time (t - 1 - m) once the step's own values are pushed
  float xh[HIST][VEC], gh[TAPS][VEC];
#pragma unroll
  for (int j = 0; j < HIST; ++j) {
    const int ts = t_begin - 1 - j;
    float v[VEC];
    if (ts >= 0) load_run<T, VEC>(xb + (size_t)ts * p.chans, 0, cw, AL, v);
    else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] = 0.0f;
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) xh[j][i] = v[i];
  }
#pragma unroll
  for (int m = 0; m < TAPS; ++m)
#pragma unroll
    for (int i = 0; i < VEC; ++i) gh[m][i] = 0.0f;

  const int t_last = t_end + HIST;                    // exclusive: dx of the last own step needs g three steps on
  // one step, given x_t and dout_t (ignored past the end of the sequence)
  auto step = [&](const int t, const float (&cur_in)[VEC], const float (&go)[VEC]) {
    float cur[VEC], g[VEC];
    if (t < p.len) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) cur[i] = cur_in[i];
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        g[i] = go[i];
        if (p.silu) {
          float pre = __builtin_fmaf(wrev[i][0], cur[i], bias[i]);
#pragma unroll
          for (int j = 0; j < HIST; ++j) pre = __builtin_fmaf(wrev[i][j + 1], xh[j][i], pre);
          g[i] *= silu_grad(pre);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) cur[i] = g[i] = 0.0f;
    }
    if (t < t_end) {                                  // own step: sums for dw (reversed taps) and dbias
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        db[i] += g[i];
        dwr[i][0] = __builtin_fmaf(g[i], cur[i], dwr[i][0]);
#pragma unroll
        for (int j = 0; j < HIST; ++j) dwr[i][j + 1] = __builtin_fmaf(g[i], xh[j][i], dwr[i][j + 1]);
      }
    }
    // push: gh[0] = g_t ... gh[3] = g_{t-3};  xh[0] = x_t ...
#pragma unroll
    for (int m = TAPS - 1; m > 0; --m)
#pragma unroll
      for (int i = 0; i < VEC; ++i) gh[m][i] = gh[m - 1][i];
#pragma unroll
    for (int i = 0; i < VEC; ++i) gh[0][i] = g[i];
#pragma unroll
    for (int j = HIST - 1; j > 0; --j)
#pragma unroll
      for (int i = 0; i < VEC; ++i) xh[j][i] = xh[j - 1][i];
#pragma unroll
    for (int i = 0; i < VEC; ++i) xh[0][i] = cur[i];
    // dx of the step three back: sum_j g_{t'+j} wrev[j] with t' = t - 3, i.e. g_{t'+j} = gh[3 - j]
    const int td = t - HIST;
    if (td >= t_begin) {
      float out[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < TAPS; ++j) acc = __builtin_fmaf(gh[HIST - j][i], wrev[i][j], acc);
        out[i] = acc;
      }
      store_run<T, VEC>(dxb + (size_t)td * p.chans, 0, cw, AL, out);
    }
  };
  if constexpr (AL) {
    // rows of a group of steps are requested together, unconditionally (row index clamped into the sequence)
    constexpr int GROUP = 8;
    for (int tg = t_begin; tg < t_last; tg += GROUP) {
      Pack<T, VEC> rx[GROUP], rg[GROUP];
#pragma unroll
      for (int j = 0; j < GROUP; ++j) {
        const size_t at = (size_t)min(tg + j, p.len - 1) * p.chans;
        rx[j] = *reinterpret_cast<const Pack<T, VEC> *>(xb + at);
        rg[j] = *reinterpret_cast<const Pack<T, VEC> *>(gb + at);
      }
#pragma unroll
      for (int j = 0; j < GROUP; ++j) {
        if (tg + j >= t_last) break;
        float cur[VEC], go[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          cur[i] = to_f32(rx[j].v[i]);
          go[i] = to_f32(rg[j].v[i]);
        }
        step(tg + j, cur, go);
      }
    }
  } else {
    for (int t = t_begin; t < t_last; ++t) {
      float cur[VEC], go[VEC];
      if (t < p.len) {
        load_run<T, VEC>(xb + (size_t)t * p.chans, 0, cw, AL, cur);
        load_run<T, VEC>(gb + (size_t)t * p.chans, 0, cw, AL, go);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) cur[i] = go[i] = 0.0f;
      }
      step(t, cur, go);
    }
  }
  // partial[(b * nseg + seg)][c][K + 1]: taps in the order of w, then the bias sum
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    if (i >= cw) break;
    float *part = p.partial + (((size_t)b * nseg + seg) * p.chans + c0 + i) * (K + 1);
#pragma unroll
    for (int m = 0; m < TAPS; ++m)
      if (m < K) part[K - 1 - m] = dwr[i][m];
    part[K] = db[i];
  }
}

// ------------------------------------------- rows of (B,L,C) in, (B,C,L) out (forward and backward)
// The reference's blocks hand the convolution a (B,C,L)-shaped view of a projection whose memory is (B,L,C') rows
// (src/ssm/modules/mamba1.py:209-215, mamba2.py:159-165: `projected.permute(0, 2, 1)`, in the first a half of a
// wider projection, so with gaps between the rows) and use the result as (B,C,L).  These kernels take that view
// as it lies instead of a transposed copy: a workgroup owns a tile of 64 channels x TT steps; its threads work
// with channels innermost (a thread: VEC neighbouring channels over 8 steps, the rows read straight from global
// memory, the lanes of a row on 128 or 256 contiguous bytes), and the turn to time innermost goes through LDS in
// 16-byte units of steps of one channel.  Unit u of the tile row of channel group g (the VEC channels of one thread)
// lies at unit (u ^ (g mod units per row)): the 16 lanes that hold one unit each for 16 channel groups, and the
// 16 lanes that move 16 neighbouring units of one row, both land on different bank groups (all 16, or 8 of them
// twice where a row has 8 units).
constexpr int CONV_TR_CH = 64, CONV_TR_STRIP = 8;
constexpr int CONV_TR_FWD_VEC = 4, CONV_TR_FWD_STEPS = 64;    // forward: 16 lanes x 8 strips
constexpr int CONV_TR_BWD_VEC = 2, CONV_TR_BWD_STEPS = 128, CONV_TR_BWD_STRIP = 16;   // backward: 32 lanes x 8 strips of 16 steps
constexpr int CONV_TR_THREADS = 256;
constexpr int CONV_TR_ALIGN = 4;                                // channels: count, strides and start of x are multiples
constexpr int CONV_TR_FWD_THREADS = (CONV_TR_CH / CONV_TR_FWD_VEC) * (CONV_TR_FWD_STEPS / CONV_TR_STRIP);
static_assert((CONV_TR_CH / CONV_TR_BWD_VEC) * (CONV_TR_BWD_STEPS / CONV_TR_BWD_STRIP) == CONV_TR_THREADS, "backward tile");

// AL: the rows of y (L elements each) start on 16-byte boundaries and L is a whole number of 16-byte units.
template <typename T, bool AL, int TAPS>
__global__ __launch_bounds__(CONV_TR_FWD_THREADS) void conv_fwd_tr_kernel(const ConvParams p) {
  constexpr int CH = CONV_TR_CH, TT = CONV_TR_FWD_STEPS, S = CONV_TR_STRIP, VEC = CONV_TR_FWD_VEC, HIST = TAPS - 1;
  constexpr int UNIT = 16 / sizeof(T), UPR = TT / UNIT, UPS = S / UNIT;   // elements per unit, units per row / strip
  constexpr int GROUPS = CH / VEC;
  __shared__ __attribute__((aligned(16))) T tile[CH * TT];
  const int ttiles = (p.len + TT - 1) / TT, ctiles = (p.chans + CH - 1) / CH;
  int bid = blockIdx.x;
  const int ct = bid % ctiles; bid /= ctiles;
  const int tt = bid % ttiles;
  const int b = bid / ttiles;
  const int cg = threadIdx.x % GROUPS, ts = threadIdx.x / GROUPS;
  const int c_own = ct * CH + cg * VEC;
  const int c0 = c_own < p.chans ? c_own : 0;        // the channel count is a multiple of VEC: a group is all in or all out
  const int t0 = tt * TT + ts * S;
  float wrev[VEC][TAPS], bias[VEC];
  load_taps_of<VEC, TAPS>(p.w, p.bias, c0, p.K, p.wide_taps, wrev, bias);
  const T *xb = reinterpret_cast<const T *>(p.x) + (size_t)b * p.x_bs + c0;
  Pack<T, VEC> raw[HIST + S];
#pragma unroll
  for (int j = 0; j < HIST + S; ++j)
    raw[j] = *reinterpret_cast<const Pack<T, VEC> *>(xb + (size_t)min(max(t0 - HIST + j, 0), p.len - 1) * p.x_rs);
#pragma unroll
  for (int j = 0; j < HIST; ++j) {
    if (t0 - HIST + j < 0) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) raw[j].v[i] = from_f32<T>(0.0f);
    }
  }
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    Pack<T, UNIT> col[UPS];
#pragma unroll
    for (int sidx = 0; sidx < S; ++sidx) {
      float acc = bias[i];
#pragma unroll
      for (int m = 0; m < TAPS; ++m) acc = __builtin_fmaf(wrev[i][m], to_f32(raw[HIST + sidx - m].v[i]), acc);
      col[sidx / UNIT].v[sidx % UNIT] = from_f32<T>(p.silu ? silu_f32(acc) : acc);
    }
    const int r = cg * VEC + i;
#pragma unroll
    for (int h = 0; h < UPS; ++h)
      *reinterpret_cast<Pack<T, UNIT> *>(tile + r * TT + ((ts * UPS + h) ^ (cg % UPR)) * UNIT) = col[h];
  }
  __syncthreads();
  T *yb = reinterpret_cast<T *>(p.y) + (size_t)b * p.chans * p.len;
  for (int v = threadIdx.x; v < CH * UPR; v += CONV_TR_FWD_THREADS) {
    const int r = v / UPR, u = v % UPR;
    const int c = ct * CH + r, t = tt * TT + u * UNIT;
    if (c >= p.chans || t >= p.len) continue;
    const Pack<T, UNIT> val = *reinterpret_cast<const Pack<T, UNIT> *>(tile + r * TT + (u ^ ((r / VEC) % UPR)) * UNIT);
    T *dst = yb + (size_t)c * p.len + t;
    if constexpr (AL) *reinterpret_cast<Pack<T, UNIT> *>(dst) = val;
    else {
#pragma unroll
      for (int e = 0; e < UNIT; ++e)
        if (t + e < p.len) dst[e] = val.v[e];
    }
  }
}

// Backward on the same kind of tile: dout (B,C,L) comes in through LDS (a tile's steps and one unit beyond them,
// zeros past the end of the sequence), x is read as rows, dx goes out as dense (B,L,C) rows.  A thread rebuilds the
// pre-activation at its 8 steps and the 4 after them (dx of a step takes g of the 4 steps that follow), so the
// transcendental work is 1.5 times the forward's; the kernel stays bound by its three streams.  A workgroup walks
// the tiles of one time segment (CONV_CL_SEGS segments per batch row at most) and leaves one partial sum of dw
// and dbias per segment.
__host__ __device__ inline int conv_tr_seg_tiles(int len) {
  const int tiles = (len + CONV_TR_BWD_STEPS - 1) / CONV_TR_BWD_STEPS;
  return (tiles + CONV_CL_SEGS - 1) / CONV_CL_SEGS;
}

template <typename T, bool AL, int TAPS>
__global__ __launch_bounds__(CONV_TR_THREADS) void conv_bwd_tr_kernel(const ConvParams p) {
  constexpr int CH = CONV_TR_CH, TT = CONV_TR_BWD_STEPS, S = CONV_TR_BWD_STRIP, VEC = CONV_TR_BWD_VEC, HIST = TAPS - 1;
  constexpr int UNIT = 16 / sizeof(T), UPR = TT / UNIT, UPS = S / UNIT;
  constexpr int GU = (S + HIST + UNIT - 1) / UNIT;      // units of dout a thread takes: its strip and 4 steps on
  constexpr int GROUPS = CH / VEC, GROUPS_PER_WAVE = GROUPS < WAVE ? GROUPS : WAVE;
  __shared__ __attribute__((aligned(16))) T gt[CH * TT];       // the tile's units, swizzled
  __shared__ __attribute__((aligned(16))) T gnext[CH * UNIT];  // per channel, the unit beyond the tile
  __shared__ float red[CONV_TR_THREADS / WAVE][CH][TAPS + 1];
  const int ttiles = (p.len + TT - 1) / TT, ctiles = (p.chans + CH - 1) / CH;
  const int seg_tiles = conv_tr_seg_tiles(p.len);
  const int nseg = (ttiles + seg_tiles - 1) / seg_tiles;
  int bid = blockIdx.x;
  const int seg = bid % nseg; bid /= nseg;
  const int ct = bid % ctiles;
  const int b = bid / ctiles;
  const int cg = threadIdx.x % GROUPS, ts = threadIdx.x / GROUPS;
  const int c_own = ct * CH + cg * VEC;
  const bool c_in = c_own < p.chans;
  const int c0 = c_in ? c_own : 0;
  const int K = p.K;
  float wrev[VEC][TAPS], bias[VEC], dwr[VEC][TAPS], db[VEC];
  load_taps_of<VEC, TAPS>(p.w, p.bias, c0, K, p.wide_taps, wrev, bias);
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    db[i] = 0.0f;
#pragma unroll
    for (int m = 0; m < TAPS; ++m) dwr[i][m] = 0.0f;
  }
  const T *xb = reinterpret_cast<const T *>(p.x) + (size_t)b * p.x_bs + c0;
  const T *gb = reinterpret_cast<const T *>(p.dout) + (size_t)b * p.chans * p.len;
  T *dxb = reinterpret_cast<T *>(p.y) + (size_t)b * p.len * p.chans + c0;

  const int tt_end = min(ttiles, (seg + 1) * seg_tiles);
  for (int tt = seg * seg_tiles; tt < tt_end; ++tt) {
    const int t0 = tt * TT + ts * S;
    // this thread's rows of x: 4 before the strip, the strip, 4 after it
    Pack<T, VEC> raw[HIST + S + HIST];
#pragma unroll
    for (int j = 0; j < HIST + S + HIST; ++j)
      raw[j] = *reinterpret_cast<const Pack<T, VEC> *>(xb + (size_t)min(max(t0 - HIST + j, 0), p.len - 1) * p.x_rs);
    // dout of the tile into LDS
    for (int v = threadIdx.x; v < CH * (UPR + 1); v += CONV_TR_THREADS) {
      const bool beyond = v >= CH * UPR;
      const int r = beyond ? v - CH * UPR : v / UPR, u = beyond ? UPR : v % UPR;
      const int c = ct * CH + r, t = tt * TT + u * UNIT;
      Pack<T, UNIT> val;
      if (c < p.chans && t < p.len) {
        const T *src = gb + (size_t)c * p.len + t;
        if constexpr (AL) val = *reinterpret_cast<const Pack<T, UNIT> *>(src);
        else {
#pragma unroll
          for (int e = 0; e < UNIT; ++e) val.v[e] = t + e < p.len ? src[e] : from_f32<T>(0.0f);
        }
      } else {
#pragma unroll
        for (int e = 0; e < UNIT; ++e) val.v[e] = from_f32<T>(0.0f);
      }
      if (!beyond) *reinterpret_cast<Pack<T, UNIT> *>(gt + r * TT + (u ^ ((r / VEC) % UPR)) * UNIT) = val;
      else *reinterpret_cast<Pack<T, UNIT> *>(gnext + r * UNIT) = val;
    }
#pragma unroll
    for (int j = 0; j < HIST; ++j) {
      if (t0 - HIST + j < 0) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) raw[j].v[i] = from_f32<T>(0.0f);
      }
    }
    __syncthreads();
    Pack<T, VEC> out[S];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const int r = cg * VEC + i;
      Pack<T, UNIT> gu[GU];
#pragma unroll
      for (int h = 0; h < GU; ++h) {
        const int u = ts * UPS + h;
        gu[h] = u < UPR ? *reinterpret_cast<const Pack<T, UNIT> *>(gt + r * TT + (u ^ (cg % UPR)) * UNIT)
                        : *reinterpret_cast<const Pack<T, UNIT> *>(gnext + r * UNIT);
      }
      float g[S + HIST];
#pragma unroll
      for (int j = 0; j < S + HIST; ++j) {
        g[j] = t0 + j < p.len ? to_f32(gu[j / UNIT].v[j % UNIT]) : 0.0f;
        if (p.silu && t0 + j < p.len) {
          float pre = bias[i];
#pragma unroll
          for (int m = 0; m < TAPS; ++m) pre = __builtin_fmaf(wrev[i][m], to_f32(raw[HIST + j - m].v[i]), pre);
          g[j] *= silu_grad(pre);
        }
      }
#pragma unroll
      for (int sidx = 0; sidx < S; ++sidx) {
        float acc = 0.0f;
#pragma unroll
        for (int m = 0; m < TAPS; ++m) acc = __builtin_fmaf(g[sidx + m], wrev[i][m], acc);
        out[sidx].v[i] = from_f32<T>(acc);
        db[i] += g[sidx];
#pragma unroll
        for (int m = 0; m < TAPS; ++m) dwr[i][m] = __builtin_fmaf(g[sidx], to_f32(raw[HIST + sidx - m].v[i]), dwr[i][m]);
      }
    }
    if (c_in) {
#pragma unroll
      for (int sidx = 0; sidx < S; ++sidx)
        if (t0 + sidx < p.len) *reinterpret_cast<Pack<T, VEC> *>(dxb + (size_t)(t0 + sidx) * p.chans) = out[sidx];
    }
    __syncthreads();                                      // the next tile's dout overwrites gt
  }
  // sums over the workgroup's strips: those of one wave through lane exchanges, the waves through LDS
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
#pragma unroll
    for (int m = 0; m <= TAPS; ++m) {
      float s = m < TAPS ? dwr[i][m] : db[i];
#pragma unroll
      for (int d = GROUPS_PER_WAVE; d < WAVE; d *= 2) s += __shfl_xor(s, d);
      if (lane < GROUPS_PER_WAVE) red[wave][cg * VEC + i][m] = s;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < CH * (K + 1); e += CONV_TR_THREADS) {
    const int r = e / (K + 1), k = e % (K + 1);
    const int c = ct * CH + r;
    if (c >= p.chans) continue;
    const int src = k < K ? K - 1 - k : TAPS;        // slot k < K holds dw[k] = dwrev[K-1-k]; slot K the bias sum
    float s = 0.0f;
#pragma unroll
    for (int wv = 0; wv < CONV_TR_THREADS / WAVE; ++wv) s += red[wv][r][src];
    p.partial[(((size_t)b * nseg + seg) * p.chans + c) * (K + 1) + k] = s;
  }
}

// Element-wise backward (any K / alignment, either layout): one thread per
// (b, c) row walks the row sequentially.  Slow path, correctness only.
template <typename T>
__global__ __launch_bounds__(CONV_THREADS) void conv_bwd_generic_kernel(const ConvParams p, int channels_last) {
  const int row = blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= p.batch * p.chans) return;
  const int b = row / p.chans, c = row % p.chans;
  const int K = p.K;
  auto at = [&](int t) -> size_t {
    return channels_last ? ((size_t)b * p.len + t) * p.chans + c : ((size_t)b * p.chans + c) * p.len + t;
  };
  const T *x = reinterpret_cast<const T *>(p.x);
  const T *go = reinterpret_cast<const T *>(p.dout);
  T *dx = reinterpret_cast<T *>(p.y);
  const float bias = p.bias ? p.bias[c] : 0.0f;
  auto gval = [&](int t) -> float {
    float g = to_f32(go[at(t)]);
    if (p.silu) {
      float pre = bias;
      for (int k = 0; k < K; ++k) {
        const int ts = t - (K - 1) + k;
        if (ts >= 0) pre = __builtin_fmaf(p.w[(size_t)c * K + k], to_f32(x[at(ts)]), pre);
      }
      g *= silu_grad(pre);
    }
    return g;
  };
  float *part = p.partial + (size_t)row * (K + 1);
  for (int k = 0; k <= K; ++k) part[k] = 0.0f;
  for (int t = 0; t < p.len; ++t) {
    const float g = gval(t);
    part[K] += g;
    for (int k = 0; k < K; ++k) {
      const int ts = t - (K - 1) + k;
      if (ts >= 0) part[k] = __builtin_fmaf(g, to_f32(x[at(ts)]), part[k]);
    }
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) {
      const int tg = t + (K - 1) - k;
      if (tg < p.len) acc = __builtin_fmaf(gval(tg), p.w[(size_t)c * K + k], acc);
    }
    dx[at(t)] = from_f32<T>(acc);
  }
}

// dw[c,k] = sum_b partial[b][c][k], dbias[c] = sum_b partial[b][c][K]; fixed order: a workgroup takes 16
// neighbouring outputs, its 256 threads are those outputs x 16 slices of the partials (slice s adds partials
// s, s + 16, ...), and the slices are added up in order.
constexpr int CONV_FOLD_COLS = 16, CONV_FOLD_SLICES = CONV_THREADS / CONV_FOLD_COLS;

__global__ __launch_bounds__(CONV_THREADS) void conv_bwd_fold_kernel(const float *partial, float *dw, float *dbias,
                                                                      int batch, int chans, int K) {
  __shared__ float part[CONV_FOLD_SLICES][CONV_FOLD_COLS];
  const int n = chans * (K + 1);
  const int col = threadIdx.x % CONV_FOLD_COLS, sl = threadIdx.x / CONV_FOLD_COLS;
  const int e = blockIdx.x * CONV_FOLD_COLS + col;
  float s = 0.0f;
  if (e < n) {
#pragma unroll 4
    for (int b = sl; b < batch; b += CONV_FOLD_SLICES) s += partial[(size_t)b * n + e];
  }
  part[sl][col] = s;
  __syncthreads();
  if (sl == 0 && e < n) {
    float t = 0.0f;
#pragma unroll
    for (int k = 0; k < CONV_FOLD_SLICES; ++k) t += part[k][col];
    const int c = e / (K + 1), k = e % (K + 1);
    if (k < K) dw[(size_t)c * K + k] = t;
    else if (dbias) dbias[c] = t;
  }
}

// Every vector kernel exists for 4 and for 5 taps: the widths up to 4 (4 is what the models use) skip the fifth
// multiply-add of each sum and, backward, the fourth step of look-ahead.
#define CONV_LAUNCH(kernel, targs, grid, block)                                                        \
  do {                                                                                                 \
    if (p.K <= 4) hipLaunchKernelGGL((kernel<targs, 4>), grid, block, 0, s, p);                        \
    else hipLaunchKernelGGL((kernel<targs, 5>), grid, block, 0, s, p);                                 \
  } while (0)
#define CONV_T_AL(al) T, al

template <typename T>
static int conv_fwd_typed(const ConvParams &p, int layout, bool vec_ok, hipStream_t s) {
  constexpr int VEC = 16 / sizeof(T);
  const size_t total = (size_t)p.batch * p.chans * p.len;
  const int channels_last = layout == SSM_LAYOUT_BLC;
  if (layout == SSM_LAYOUT_ROWS_TO_BCL) {
    const size_t blocks = (size_t)p.batch * ((p.chans + CONV_TR_CH - 1) / CONV_TR_CH) * ((p.len + CONV_TR_FWD_STEPS - 1) / CONV_TR_FWD_STEPS);
    if (p.len % VEC == 0) CONV_LAUNCH(conv_fwd_tr_kernel, CONV_T_AL(true), dim3((unsigned)blocks), dim3(CONV_TR_FWD_THREADS));
    else CONV_LAUNCH(conv_fwd_tr_kernel, CONV_T_AL(false), dim3((unsigned)blocks), dim3(CONV_TR_FWD_THREADS));
  } else if (p.K <= CONV_TAPS && !channels_last) {
    if (vec_ok && p.len % VEC == 0) CONV_LAUNCH(conv_fwd_cf_kernel, CONV_T_AL(true), dim3(p.batch * p.chans), dim3(CONV_THREADS));
    else CONV_LAUNCH(conv_fwd_cf_kernel, CONV_T_AL(false), dim3(p.batch * p.chans), dim3(CONV_THREADS));
  } else if (p.K <= CONV_TAPS && channels_last) {
    const int strips = (p.len + CONV_CL_STRIP - 1) / CONV_CL_STRIP;
    constexpr int VECF = CONV_CL_FWD_BYTES / sizeof(T);
    const size_t threads = (size_t)p.batch * strips * ((p.chans + VECF - 1) / VECF);
    const dim3 grid((unsigned)((threads + CONV_THREADS - 1) / CONV_THREADS));
    if (vec_ok && p.chans % VEC == 0 && p.len >= 2 * CONV_CL_WALK_STRIP * CONV_CL_WALK) {
      const int spans = (p.len + CONV_CL_WALK_STRIP * CONV_CL_WALK - 1) / (CONV_CL_WALK_STRIP * CONV_CL_WALK);
      const size_t walkers = (size_t)p.batch * spans * (p.chans / VECF);
      const dim3 wgrid((unsigned)((walkers + CONV_CL_WALK_THREADS - 1) / CONV_CL_WALK_THREADS));
      CONV_LAUNCH(conv_fwd_cl_walk_kernel, T, wgrid, dim3(CONV_CL_WALK_THREADS));
    } else if (vec_ok && p.chans % VEC == 0) CONV_LAUNCH(conv_fwd_cl_kernel, CONV_T_AL(true), grid, dim3(CONV_THREADS));
    else CONV_LAUNCH(conv_fwd_cl_kernel, CONV_T_AL(false), grid, dim3(CONV_THREADS));
  } else {
    const unsigned grid = (unsigned)min((size_t)65535 * 16, (total + CONV_THREADS - 1) / CONV_THREADS);
    hipLaunchKernelGGL(conv_fwd_generic_kernel<T>, dim3(grid), dim3(CONV_THREADS), 0, s, p, channels_last);
  }
  SSM_CHECK_LAUNCH("ssm_conv1d_fwd");
  return SSM_OK;
}

template <typename T>
static int conv_bwd_typed(const ConvParams &p, int layout, bool vec_ok, float *dw, float *dbias,
                          hipStream_t s) {
  constexpr int VEC = 16 / sizeof(T);
  int fold_count = p.batch;
  const int channels_last = layout == SSM_LAYOUT_BLC;
  if (layout == SSM_LAYOUT_ROWS_TO_BCL) {
    const int ttiles = (p.len + CONV_TR_BWD_STEPS - 1) / CONV_TR_BWD_STEPS, seg_tiles = conv_tr_seg_tiles(p.len);
    const int nseg = (ttiles + seg_tiles - 1) / seg_tiles;
    const size_t blocks = (size_t)p.batch * ((p.chans + CONV_TR_CH - 1) / CONV_TR_CH) * nseg;
    if (p.len % VEC == 0) CONV_LAUNCH(conv_bwd_tr_kernel, CONV_T_AL(true), dim3((unsigned)blocks), dim3(CONV_TR_THREADS));
    else CONV_LAUNCH(conv_bwd_tr_kernel, CONV_T_AL(false), dim3((unsigned)blocks), dim3(CONV_TR_THREADS));
    fold_count = p.batch * nseg;
  } else if (p.K <= CONV_TAPS && !channels_last) {
    // enough channels to fill the GPU with one workgroup each: a workgroup sums over the batch itself and the
    // fold of partials (a second launch of ~4 us) falls away
    ConvParams q = p;
    q.whole_batch = p.chans >= CONV_WHOLE_BATCH_MIN_CHANNELS && p.batch > 1;
    q.dw = dw; q.dbias = dbias;
    const dim3 grid(q.whole_batch ? p.chans : p.batch * p.chans);
    {
      const ConvParams &p = q;
      if (vec_ok && p.len % VEC == 0) CONV_LAUNCH(conv_bwd_cf_kernel, CONV_T_AL(true), grid, dim3(CONV_THREADS));
      else CONV_LAUNCH(conv_bwd_cf_kernel, CONV_T_AL(false), grid, dim3(CONV_THREADS));
    }
    if (q.whole_batch) {
      SSM_CHECK_LAUNCH("ssm_conv1d_bwd");
      return SSM_OK;
    }
  } else if (p.K <= CONV_TAPS && channels_last) {
    const int seg_len = conv_cl_seg_len(p.len);
    const int nseg = (p.len + seg_len - 1) / seg_len;
    constexpr int VECB = CONV_CL_BWD_BYTES / sizeof(T);
    const size_t threads = (size_t)p.batch * nseg * ((p.chans + VECB - 1) / VECB);
    const dim3 grid((unsigned)((threads + CONV_THREADS - 1) / CONV_THREADS));
    if (vec_ok && p.chans % VEC == 0) CONV_LAUNCH(conv_bwd_cl_kernel, CONV_T_AL(true), grid, dim3(CONV_THREADS));
    else CONV_LAUNCH(conv_bwd_cl_kernel, CONV_T_AL(false), grid, dim3(CONV_THREADS));
    fold_count = p.batch * nseg;
  } else {
    const int rows = p.batch * p.chans;
    hipLaunchKernelGGL(conv_bwd_generic_kernel<T>, dim3((rows + CONV_THREADS - 1) / CONV_THREADS),
                       dim3(CONV_THREADS), 0, s, p, channels_last);
  }
  SSM_CHECK_LAUNCH("ssm_conv1d_bwd");
  const int n = p.chans * (p.K + 1);
  hipLaunchKernelGGL(conv_bwd_fold_kernel, dim3((n + CONV_FOLD_COLS - 1) / CONV_FOLD_COLS), dim3(CONV_THREADS), 0, s,
                     p.partial, dw, dbias, fold_count, p.chans, p.K);
  SSM_CHECK_LAUNCH("ssm_conv1d_bwd(fold)");
  return SSM_OK;
}
#undef CONV_LAUNCH
#undef CONV_T_AL

static int conv_check(const char *who, const void *x, const void *w, const void *y, int batch, int chans, int len,
                      int K, int dtype, int layout, int act) {
  SSM_REQUIRE(x && w && y, SSM_ERR_NULL_POINTER, "%s: x, weight and output are required", who);
  SSM_REQUIRE(batch > 0 && chans > 0 && len > 0 && K > 0, SSM_ERR_BAD_SHAPE,
              "%s: batch=%d channels=%d seqlen=%d width=%d must all be positive", who, batch, chans, len, K);
  SSM_REQUIRE(valid_dtype(dtype), SSM_ERR_BAD_DTYPE, "%s: dtype=%d", who, dtype);
  SSM_REQUIRE(layout == SSM_LAYOUT_BCL || layout == SSM_LAYOUT_BLC || layout == SSM_LAYOUT_ROWS_TO_BCL, SSM_ERR_BAD_KIND,
              "%s: layout=%d", who, layout);
  SSM_REQUIRE(act == SSM_ACT_IDENTITY || act == SSM_ACT_SILU, SSM_ERR_BAD_KIND, "%s: activation=%d", who, act);
  SSM_REQUIRE((size_t)batch * chans < ((size_t)1 << 31) && (size_t)batch * chans * len < ((size_t)1 << 40),
              SSM_ERR_TOO_LARGE, "%s: tensor too large", who);
  const int es = dtype_size(dtype);
  SSM_REQUIRE(aligned_to(x, es) && aligned_to(y, es) && aligned_to(w, 4), SSM_ERR_ALIGNMENT,
              "%s: a pointer is not aligned to its element size", who);
  return SSM_OK;
}

// SSM_LAYOUT_ROWS_TO_BCL: what the rows-in kernels assume of x and of the tensors written or read as (B,C,L).
static int conv_rows_check(const char *who, const void *x, long long x_bs, long long x_rs, const void *bcl_a,
                           const void *bcl_b, const void *rows_out, int batch, int chans, int len, int K, int dtype) {
  const int es = dtype_size(dtype);
  SSM_REQUIRE(K <= CONV_TAPS && chans % CONV_TR_ALIGN == 0, SSM_ERR_BAD_SHAPE,
              "%s: rows of (B,L,C) in, (B,C,L) out takes width <= %d and a multiple of %d channels (got width=%d "
              "channels=%d): hand over a (B,C,L) copy", who, CONV_TAPS, CONV_TR_ALIGN, K, chans);
  SSM_REQUIRE(x_rs >= chans && x_rs % CONV_TR_ALIGN == 0 && x_bs % CONV_TR_ALIGN == 0 &&
              (batch == 1 || x_bs >= (long long)(len - 1) * x_rs + chans), SSM_ERR_BAD_SHAPE,
              "%s: x_row_stride=%lld, x_batch_stride=%lld must be multiples of %d, rows must not overlap", who,
              x_rs, x_bs, CONV_TR_ALIGN);
  SSM_REQUIRE((size_t)batch * ((chans + CONV_TR_CH - 1) / CONV_TR_CH) * ((len + CONV_TR_BWD_STEPS - 1) / CONV_TR_BWD_STEPS) <
                  ((size_t)1 << 31), SSM_ERR_TOO_LARGE, "%s: too many tiles", who);
  SSM_REQUIRE(aligned_to(x, CONV_TR_ALIGN * es) && aligned_to(bcl_a, 16) && (!bcl_b || aligned_to(bcl_b, 16)) &&
              (!rows_out || aligned_to(rows_out, 16)), SSM_ERR_ALIGNMENT,
              "%s: x must start on a %d-byte boundary, the dense tensors on 16-byte ones", who, CONV_TR_ALIGN * es);
  return SSM_OK;
}

}  // namespace ssm

extern "C" int ssm_conv1d_fwd(const ssm_conv1d_fwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_conv1d_fwd: args is NULL");
  int rc = conv_check("ssm_conv1d_fwd", a->x, a->weight, a->y, a->batch, a->channels, a->seqlen, a->width,
                      a->io_dtype, a->layout, a->activation);
  if (rc != SSM_OK) return rc;
  ConvParams p{};
  p.x = a->x; p.w = a->weight; p.bias = a->bias; p.y = a->y;
  p.batch = a->batch; p.chans = a->channels; p.len = a->seqlen; p.K = a->width;
  p.silu = a->activation == SSM_ACT_SILU;
  p.wide_taps = a->width == 4 && aligned_to(a->weight, 16) && (!a->bias || aligned_to(a->bias, 16));
  const bool vec_ok = aligned_to(a->x, 16) && aligned_to(a->y, 16);
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  if (a->layout == SSM_LAYOUT_ROWS_TO_BCL) {
    p.x_bs = a->x_batch_stride; p.x_rs = a->x_row_stride;
    rc = conv_rows_check("ssm_conv1d_fwd", a->x, p.x_bs, p.x_rs, a->y, nullptr, nullptr, a->batch, a->channels,
                         a->seqlen, a->width, a->io_dtype);
    if (rc != SSM_OK) return rc;
  } else {
    SSM_REQUIRE(a->x_batch_stride == 0 && a->x_row_stride == 0, SSM_ERR_BAD_KIND,
                "ssm_conv1d_fwd: strides of x go with SSM_LAYOUT_ROWS_TO_BCL only");
  }
  switch (a->io_dtype) {
    case SSM_F32: return conv_fwd_typed<float>(p, a->layout, vec_ok, s);
    case SSM_BF16: return conv_fwd_typed<bf16_t>(p, a->layout, vec_ok, s);
    default: return conv_fwd_typed<f16_t>(p, a->layout, vec_ok, s);
  }
}

extern "C" size_t ssm_conv1d_bwd_workspace_bytes(int batch, int channels, int width) {
  if (batch <= 0 || channels <= 0 || width <= 0) return 0;
  // one partial per batch row, or per (batch row, time segment) in the channels-last kernel
  return (size_t)batch * ssm::CONV_CL_SEGS * channels * (width + 1) * sizeof(float);
}

extern "C" int ssm_conv1d_bwd(const ssm_conv1d_bwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_conv1d_bwd: args is NULL");
  int rc = conv_check("ssm_conv1d_bwd", a->x, a->weight, a->dx, a->batch, a->channels, a->seqlen, a->width,
                      a->io_dtype, a->layout, a->activation);
  if (rc != SSM_OK) return rc;
  SSM_REQUIRE(a->dout && a->dweight, SSM_ERR_NULL_POINTER, "ssm_conv1d_bwd: dout and dweight are required");
  SSM_REQUIRE(a->workspace && a->workspace_bytes >= ssm_conv1d_bwd_workspace_bytes(a->batch, a->channels, a->width),
              SSM_ERR_WORKSPACE, "ssm_conv1d_bwd: workspace of %zu bytes required",
              ssm_conv1d_bwd_workspace_bytes(a->batch, a->channels, a->width));
  SSM_REQUIRE(aligned_to(a->dout, dtype_size(a->io_dtype)) && aligned_to(a->dweight, 4) && aligned_to(a->workspace, 4),
              SSM_ERR_ALIGNMENT, "ssm_conv1d_bwd: a pointer is not aligned to its element size");
  ConvParams p{};
  p.x = a->x; p.dout = a->dout; p.w = a->weight; p.bias = a->bias; p.y = a->dx;
  p.partial = reinterpret_cast<float *>(a->workspace);
  p.batch = a->batch; p.chans = a->channels; p.len = a->seqlen; p.K = a->width;
  p.silu = a->activation == SSM_ACT_SILU;
  p.wide_taps = a->width == 4 && aligned_to(a->weight, 16) && (!a->bias || aligned_to(a->bias, 16));
  const bool vec_ok = aligned_to(a->x, 16) && aligned_to(a->dx, 16) && aligned_to(a->dout, 16);
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  if (a->layout == SSM_LAYOUT_ROWS_TO_BCL) {
    p.x_bs = a->x_batch_stride; p.x_rs = a->x_row_stride;
    rc = conv_rows_check("ssm_conv1d_bwd", a->x, p.x_bs, p.x_rs, a->dout, nullptr, a->dx, a->batch, a->channels,
                         a->seqlen, a->width, a->io_dtype);
    if (rc != SSM_OK) return rc;
  } else {
    SSM_REQUIRE(a->x_batch_stride == 0 && a->x_row_stride == 0, SSM_ERR_BAD_KIND,
                "ssm_conv1d_bwd: strides of x go with SSM_LAYOUT_ROWS_TO_BCL only");
  }
  switch (a->io_dtype) {
    case SSM_F32: return conv_bwd_typed<float>(p, a->layout, vec_ok, a->dweight, a->dbias, s);
    case SSM_BF16: return conv_bwd_typed<bf16_t>(p, a->layout, vec_ok, a->dweight, a->dbias, s);
    default: return conv_bwd_typed<f16_t>(p, a->layout, vec_ok, a->dweight, a->dbias, s);
  }
}
