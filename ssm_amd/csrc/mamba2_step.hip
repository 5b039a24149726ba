// One decoding step of a Mamba-2 (SSD) block on cached states, in two launches.
//
// The block's input projection yields one row per sequence, z | xBC | dt (d_inner, d_inner + 2 G N, H
// columns).  Kernel 1 takes the xBC columns through the depthwise causal convolution on the cached window
// of the last K inputs (rolled in place) and SiLU.  Kernel 2 is the state update per (sequence, head):
//   dt = softplus(dt_raw + bias_h) (opt.),  a = exp(dt A_h)
//   S[p][n] <- a S[p][n] + dt x_p B_n ,   y_p = sum_n S[p][n] C_n + D x_p ,   y_p *= silu(z_p)
// with the state (B, H, P, N) in float32, updated in place.  The same arithmetic as the single-token
// selective_state_step with per-head parameters spread over the head's channels, minus the tensor
// operations that spreading, slicing and window rolling cost when the step is composed from the
// general operators.
#include "common.hpp"

#include <type_traits>

namespace ssm {

constexpr int M2_THREADS = 256;
constexpr int M2_MAX_K = 8;

struct Mamba2StepParams {
  const void *zxbcdt;        // (B, proj) io dtype, proj = 2 d_inner + 2 G N + H
  void *conv_state;          // (B, conv_dim, K) io dtype: the last K inputs of every conv channel, oldest first
  const float *conv_w;       // (conv_dim, K)
  const float *conv_b;       // (conv_dim,) or null
  float *xbc;                // (B, conv_dim) float32: activated conv output (workspace and by-product)
  float *state;              // (B, H, P, N) float32, in place
  const float *A, *Dk, *bias;  // (H,), (H,) or (H, P) or null, (H,) or null
  void *y;                   // (B, d_inner) io dtype
  int batch, heads, hdim, groups, nstate, width;
  int d_per_p, softplus, gate;
};

template <typename io_t>
__global__ __launch_bounds__(M2_THREADS) void mamba2_conv_kernel(const Mamba2StepParams p) {
  const int di = p.heads * p.hdim, conv_dim = di + 2 * p.groups * p.nstate, proj = 2 * di + 2 * p.groups * p.nstate + p.heads;
  const size_t e = (size_t)blockIdx.x * M2_THREADS + threadIdx.x;
  if (e >= (size_t)p.batch * conv_dim) return;
  const int c = (int)(e % conv_dim), b = (int)(e / conv_dim);
  const int K = p.width;
  io_t *win = reinterpret_cast<io_t *>(p.conv_state) + e * K;
  const float xin = to_f32(reinterpret_cast<const io_t *>(p.zxbcdt)[(size_t)b * proj + di + c]);
  // every read is unconditional (indices clamped to the window): all of them are in flight together
  float w[M2_MAX_K], tap[M2_MAX_K];
#pragma unroll
  for (int k = 0; k < M2_MAX_K; ++k) {
    w[k] = to_f32(win[min(k, K - 1)]);
    tap[k] = p.conv_w[(size_t)c * K + min(k, K - 1)];
  }
  float acc = (p.conv_b ? p.conv_b : p.conv_w)[c];
  if (!p.conv_b) acc = 0.0f;
#pragma unroll
  for (int k = 0; k < M2_MAX_K; ++k) {
    const float v = k + 1 < K ? w[min(k + 1, M2_MAX_K - 1)] : xin;          // the window after the roll
    if (k < K) {
      acc = __builtin_fmaf(tap[k], v, acc);
      win[k] = from_f32<io_t>(v);
    }
  }
  p.xbc[e] = silu_f32(acc);
}

// The convolution step on its own: x (B, C) enters the window (B, C, K), out = act(bias + taps . window).
struct ConvUpdateParams {
  const void *x;
  size_t x_stride;           // elements between the rows of x
  void *conv_state;
  const float *w, *b;
  void *out;                 // (B, C) io dtype
  int batch, chans, width, silu;
};

template <typename io_t>
__global__ __launch_bounds__(M2_THREADS) void conv_update_kernel(const ConvUpdateParams p) {
  const size_t e = (size_t)blockIdx.x * M2_THREADS + threadIdx.x;
  if (e >= (size_t)p.batch * p.chans) return;
  const int c = (int)(e % p.chans), b = (int)(e / p.chans);
  const int K = p.width;
  io_t *win = reinterpret_cast<io_t *>(p.conv_state) + e * K;
  const float xin = to_f32(reinterpret_cast<const io_t *>(p.x)[(size_t)b * p.x_stride + c]);
  float w[M2_MAX_K], tap[M2_MAX_K];
#pragma unroll
  for (int k = 0; k < M2_MAX_K; ++k) {
    w[k] = to_f32(win[min(k, K - 1)]);
    tap[k] = p.w[(size_t)c * K + min(k, K - 1)];
  }
  float acc = (p.b ? p.b : p.w)[c];
  if (!p.b) acc = 0.0f;
#pragma unroll
  for (int k = 0; k < M2_MAX_K; ++k) {
    const float v = k + 1 < K ? w[min(k + 1, M2_MAX_K - 1)] : xin;
    if (k < K) {
      acc = __builtin_fmaf(tap[k], v, acc);
      win[k] = from_f32<io_t>(v);
    }
  }
  reinterpret_cast<io_t *>(p.out)[e] = from_f32<io_t>(p.silu ? silu_f32(acc) : acc);
}

template <typename io_t>
static int launch_conv_update(const ConvUpdateParams &p, hipStream_t s) {
  const size_t total = (size_t)p.batch * p.chans;
  hipLaunchKernelGGL(conv_update_kernel<io_t>, dim3((unsigned)((total + M2_THREADS - 1) / M2_THREADS)), dim3(M2_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_conv1d_update");
  return SSM_OK;
}

// One workgroup per (sequence, head); thread = (channel p, quarter of the states).
template <typename io_t>
__global__ __launch_bounds__(M2_THREADS) void mamba2_state_kernel(const Mamba2StepParams p) {
  extern __shared__ __align__(16) float bc[];              // B[N] then C[N] of the head's group
  const int H = p.heads, P = p.hdim, N = p.nstate, G = p.groups;
  const int di = H * P, conv_dim = di + 2 * G * N, proj = 2 * di + 2 * G * N + H;
  const int h = blockIdx.x % H, b = blockIdx.x / H;
  const int g = h / (H / G);
  const io_t *row = reinterpret_cast<const io_t *>(p.zxbcdt) + (size_t)b * proj;
  const float *xb = p.xbc + (size_t)b * conv_dim;
  for (int n = threadIdx.x; n < 2 * N; n += blockDim.x)
    bc[n] = n < N ? xb[di + g * N + n] : xb[di + G * N + g * N + (n - N)];
  float dt = to_f32(row[di + conv_dim + h]) + (p.bias ? p.bias[h] : 0.0f);
  if (p.softplus) dt = softplus_f32(dt);
  const float a = exp2_hw(dt * p.A[h] * LOG2E);
  __syncthreads();
  const int nq = N / 4;                                    // states per thread
  for (int pp = threadIdx.x >> 2; pp < P; pp += blockDim.x >> 2) {
    const int q = threadIdx.x & 3;
    const float x = xb[h * P + pp];
    const float dtx = dt * x;
    float *S = p.state + (((size_t)b * H + h) * P + pp) * N + q * nq;
    const float *Bq = bc + q * nq, *Cq = bc + N + q * nq;
    float y = 0.0f;
    for (int n = 0; n < nq; n += 4) {
      float4 s = *reinterpret_cast<float4 *>(S + n);
      const float4 bv = *reinterpret_cast<const float4 *>(Bq + n), cv = *reinterpret_cast<const float4 *>(Cq + n);
      s.x = __builtin_fmaf(a, s.x, dtx * bv.x);
      s.y = __builtin_fmaf(a, s.y, dtx * bv.y);
      s.z = __builtin_fmaf(a, s.z, dtx * bv.z);
      s.w = __builtin_fmaf(a, s.w, dtx * bv.w);
      y = __builtin_fmaf(s.x, cv.x, y);
      y = __builtin_fmaf(s.y, cv.y, y);
      y = __builtin_fmaf(s.z, cv.z, y);
      y = __builtin_fmaf(s.w, cv.w, y);
      *reinterpret_cast<float4 *>(S + n) = s;
    }
    // the four quarters sit in neighbouring lanes
    y += __shfl_xor(y, 1, WAVE);
    y += __shfl_xor(y, 2, WAVE);
    if (q == 0) {
      if (p.Dk) y = __builtin_fmaf(p.Dk[p.d_per_p ? (size_t)h * P + pp : (size_t)h], x, y);
      if (p.gate) y *= silu_f32(to_f32(row[h * P + pp]));
      reinterpret_cast<io_t *>(p.y)[(size_t)b * di + h * P + pp] = from_f32<io_t>(y);
    }
  }
}

// The same update with eight states per lane (N / 8 a power of two up to 64 lanes per channel): every lane
// issues its reads - two 16-byte pieces each of the state, B and C - at once and unconditionally, the sum over
// the states is a butterfly inside the wave, and there are B*H*P*N/8 lanes to fill the device (one workgroup
// per (sequence, head) leaves most of it idle at decoding batch sizes).
template <typename io_t>
__global__ __launch_bounds__(M2_THREADS) void mamba2_state8_kernel(const Mamba2StepParams p, const int lg) {
  const int H = p.heads, P = p.hdim, N = p.nstate, G = p.groups;
  const int di = H * P, conv_dim = di + 2 * G * N, proj = 2 * di + 2 * G * N + H;
  const size_t total = ((size_t)p.batch * di) << lg;
  const size_t gid = (size_t)blockIdx.x * M2_THREADS + threadIdx.x;
  const bool live = gid < total;
  const size_t g_ = live ? gid : 0;
  const int j = (int)(g_ & (size_t)((1 << lg) - 1));
  const unsigned ch = (unsigned)(g_ >> lg);                  // b * di + h * P + p
  const int b = (int)(ch / (unsigned)di), hp = (int)(ch % (unsigned)di);
  const int h = hp / P, grp = h / (H / G);
  const io_t *row = reinterpret_cast<const io_t *>(p.zxbcdt) + (size_t)b * proj;
  const float *xb = p.xbc + (size_t)b * conv_dim;
  float *S = p.state + ((size_t)ch << lg) * 8 + (size_t)j * 8;
  const float4 s0 = *reinterpret_cast<const float4 *>(S), s1 = *reinterpret_cast<const float4 *>(S + 4);
  const float *Bq = xb + di + grp * N + j * 8, *Cq = xb + di + G * N + grp * N + j * 8;
  const float4 b0 = *reinterpret_cast<const float4 *>(Bq), b1 = *reinterpret_cast<const float4 *>(Bq + 4);
  const float4 c0 = *reinterpret_cast<const float4 *>(Cq), c1 = *reinterpret_cast<const float4 *>(Cq + 4);
  const float x = xb[hp];
  const float zraw = to_f32(row[hp]);
  float dt = to_f32(row[di + conv_dim + h]);
  const float biasv = (p.bias ? p.bias : p.A)[h];
  const float Av = p.A[h];
  const float Dv = p.Dk ? p.Dk[p.d_per_p ? (size_t)hp : (size_t)h] : 0.0f;
  if (p.bias) dt += biasv;
  if (p.softplus) dt = softplus_f32(dt);
  const float a = exp2_hw(dt * Av * LOG2E), dtx = dt * x;
  float4 n0, n1;
  n0.x = __builtin_fmaf(a, s0.x, dtx * b0.x); n0.y = __builtin_fmaf(a, s0.y, dtx * b0.y);
  n0.z = __builtin_fmaf(a, s0.z, dtx * b0.z); n0.w = __builtin_fmaf(a, s0.w, dtx * b0.w);
  n1.x = __builtin_fmaf(a, s1.x, dtx * b1.x); n1.y = __builtin_fmaf(a, s1.y, dtx * b1.y);
  n1.z = __builtin_fmaf(a, s1.z, dtx * b1.z); n1.w = __builtin_fmaf(a, s1.w, dtx * b1.w);
  float y = n0.x * c0.x;
  y = __builtin_fmaf(n0.y, c0.y, y); y = __builtin_fmaf(n0.z, c0.z, y); y = __builtin_fmaf(n0.w, c0.w, y);
  y = __builtin_fmaf(n1.x, c1.x, y); y = __builtin_fmaf(n1.y, c1.y, y);
  y = __builtin_fmaf(n1.z, c1.z, y); y = __builtin_fmaf(n1.w, c1.w, y);
  for (int m = (1 << lg) >> 1; m >= 1; m >>= 1) y += __shfl_xor(y, m, WAVE);
  if (!live) return;
  *reinterpret_cast<float4 *>(S) = n0;
  *reinterpret_cast<float4 *>(S + 4) = n1;
  if (j == 0) {
    y = __builtin_fmaf(Dv, x, y);
    if (p.gate) y *= silu_f32(zraw);
    reinterpret_cast<io_t *>(p.y)[ch] = from_f32<io_t>(y);
  }
}

template <typename io_t>
static int launch_mamba2(const Mamba2StepParams &p, hipStream_t s) {
  const int conv_dim = p.heads * p.hdim + 2 * p.groups * p.nstate;
  const size_t total = (size_t)p.batch * conv_dim;
  hipLaunchKernelGGL(mamba2_conv_kernel<io_t>, dim3((unsigned)((total + M2_THREADS - 1) / M2_THREADS)), dim3(M2_THREADS), 0, s, p);
  int lg = 0;
  while ((8 << lg) < p.nstate) ++lg;
  if ((8 << lg) == p.nstate && lg <= 6 && (p.heads * p.hdim) % 4 == 0) {       // float4 reads of B and C out of xbc
    const size_t lanes = ((size_t)p.batch * p.heads * p.hdim) << lg;
    hipLaunchKernelGGL(mamba2_state8_kernel<io_t>, dim3((unsigned)((lanes + M2_THREADS - 1) / M2_THREADS)), dim3(M2_THREADS), 0, s, p, lg);
    SSM_CHECK_LAUNCH("ssm_mamba2_decode_step");
    return SSM_OK;
  }
  const int threads = p.hdim * 4 < M2_THREADS ? ((p.hdim * 4 + WAVE - 1) / WAVE) * WAVE : M2_THREADS;
  hipLaunchKernelGGL(mamba2_state_kernel<io_t>, dim3((unsigned)(p.batch * p.heads)), dim3(threads),
                     (size_t)2 * p.nstate * sizeof(float), s, p);
  SSM_CHECK_LAUNCH("ssm_mamba2_decode_step");
  return SSM_OK;
}

}  // namespace ssm

extern "C" int ssm_mamba2_decode_step(const ssm_mamba2_decode_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_mamba2_decode_step: args is NULL");
  SSM_REQUIRE(a->zxbcdt && a->conv_state && a->conv_weight && a->xbc && a->ssm_state && a->A && a->y,
              SSM_ERR_NULL_POINTER,
              "ssm_mamba2_decode_step: zxbcdt, conv_state, conv_weight, xbc, ssm_state, A and y are required");
  SSM_REQUIRE(a->batch > 0 && a->heads > 0 && a->headdim > 0 && a->groups > 0 && a->nstate > 0 && a->conv_width > 0,
              SSM_ERR_BAD_SHAPE, "ssm_mamba2_decode_step: batch, heads, headdim, groups, nstate and conv_width must be positive");
  SSM_REQUIRE(a->heads % a->groups == 0, SSM_ERR_BAD_SHAPE, "ssm_mamba2_decode_step: groups=%d must divide heads=%d",
              a->groups, a->heads);
  SSM_REQUIRE(a->nstate % 16 == 0 && a->nstate <= 1024, SSM_ERR_BAD_SHAPE,
              "ssm_mamba2_decode_step: nstate=%d must be a multiple of 16, at most 1024", a->nstate);
  SSM_REQUIRE(a->conv_width <= M2_MAX_K, SSM_ERR_TOO_LARGE, "ssm_mamba2_decode_step: conv_width=%d exceeds %d",
              a->conv_width, M2_MAX_K);
  SSM_REQUIRE(valid_dtype(a->io_dtype), SSM_ERR_BAD_DTYPE, "ssm_mamba2_decode_step: io_dtype=%d", a->io_dtype);
  SSM_REQUIRE((size_t)a->batch * a->heads < ((size_t)1 << 31), SSM_ERR_TOO_LARGE, "ssm_mamba2_decode_step: too many heads");
  const int es = dtype_size(a->io_dtype);
  SSM_REQUIRE(aligned_to(a->zxbcdt, es) && aligned_to(a->conv_state, es) && aligned_to(a->y, es) &&
                  aligned_to(a->ssm_state, 16) && aligned_to(a->xbc, 16),
              SSM_ERR_ALIGNMENT, "ssm_mamba2_decode_step: a pointer is not sufficiently aligned");
  Mamba2StepParams p{};
  p.zxbcdt = a->zxbcdt; p.conv_state = a->conv_state; p.conv_w = a->conv_weight; p.conv_b = a->conv_bias;
  p.xbc = a->xbc; p.state = a->ssm_state; p.A = a->A; p.Dk = a->Dskip; p.bias = a->dt_bias; p.y = a->y;
  p.batch = a->batch; p.heads = a->heads; p.hdim = a->headdim; p.groups = a->groups; p.nstate = a->nstate;
  p.width = a->conv_width; p.d_per_p = a->d_per_p ? 1 : 0; p.softplus = a->dt_softplus ? 1 : 0; p.gate = a->gate ? 1 : 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  switch (a->io_dtype) {
    case SSM_F32: return launch_mamba2<float>(p, s);
    case SSM_BF16: return launch_mamba2<bf16_t>(p, s);
    default: return launch_mamba2<f16_t>(p, s);
  }
}

extern "C" int ssm_conv1d_update(const ssm_conv1d_update_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_conv1d_update: args is NULL");
  SSM_REQUIRE(a->x && a->conv_state && a->weight && a->out, SSM_ERR_NULL_POINTER,
              "ssm_conv1d_update: x, conv_state, weight and out are required");
  SSM_REQUIRE(a->batch > 0 && a->channels > 0 && a->width > 0, SSM_ERR_BAD_SHAPE,
              "ssm_conv1d_update: batch, channels and width must be positive");
  SSM_REQUIRE(a->width <= M2_MAX_K, SSM_ERR_TOO_LARGE, "ssm_conv1d_update: width=%d exceeds %d", a->width, M2_MAX_K);
  SSM_REQUIRE(a->x_row_stride >= a->channels, SSM_ERR_BAD_SHAPE, "ssm_conv1d_update: x_row_stride=%lld is less than channels=%d",
              (long long)a->x_row_stride, a->channels);
  SSM_REQUIRE(valid_dtype(a->io_dtype), SSM_ERR_BAD_DTYPE, "ssm_conv1d_update: io_dtype=%d", a->io_dtype);
  SSM_REQUIRE(a->activation == SSM_ACT_IDENTITY || a->activation == SSM_ACT_SILU, SSM_ERR_BAD_KIND,
              "ssm_conv1d_update: activation=%d", a->activation);
  const int es = dtype_size(a->io_dtype);
  SSM_REQUIRE(aligned_to(a->x, es) && aligned_to(a->conv_state, es) && aligned_to(a->out, es), SSM_ERR_ALIGNMENT,
              "ssm_conv1d_update: a pointer is not sufficiently aligned");
  ConvUpdateParams p{};
  p.x = a->x; p.x_stride = (size_t)a->x_row_stride; p.conv_state = a->conv_state; p.w = a->weight; p.b = a->bias;
  p.out = a->out; p.batch = a->batch; p.chans = a->channels; p.width = a->width; p.silu = a->activation == SSM_ACT_SILU;
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  switch (a->io_dtype) {
    case SSM_F32: return launch_conv_update<float>(p, s);
    case SSM_BF16: return launch_conv_update<bf16_t>(p, s);
    default: return launch_conv_update<f16_t>(p, s);
  }
}
