// The five operators in double precision.
//
// The reference's Python path computes in the promoted type of its inputs (src/ssm/ops/python/reference.py:9-19,
// :135-137), and its tests run torch.autograd.gradcheck on every operator of a compiled backend with float64
// tensors on the device (tests/ops/test_backend_gradients.py:1172-1201, :1291-1321, :1416-1447, :1497-1517,
// :1578-1612).  The tuned kernels of this library accumulate in float32; these kernels serve calls whose compute
// type is float64.  They are written for exactness and plain parallelism over independent rows, not for the
// roofline: one thread walks one recurrence ((batch, channel) for the scans, a row for the norm, an output element
// for the convolution), all arithmetic is double, sums that cross threads are formed in a fixed order.
//
// Operands that the reference broadcasts (projections given per channel, per batch row or per group) arrive as
// views with element strides, 0 on a broadcast axis; their gradients are written dense and reduced by the caller.
#include "common.hpp"

#include <math.h>

namespace ssm {
namespace {

constexpr int F64_THREADS = 128;

__device__ __forceinline__ double softplus64(double x) { return x > 20.0 ? x : log1p(exp(x)); }   // F.softplus, threshold 20
__device__ __forceinline__ double sigmoid64(double x) { return 1.0 / (1.0 + exp(-x)); }
// d/dx softplus(x), with the same switch to the identity
__device__ __forceinline__ double dsoftplus64(double x) { return x > 20.0 ? 1.0 : sigmoid64(x); }

inline unsigned blocks_for(long long n) { return (unsigned)((n + F64_THREADS - 1) / F64_THREADS); }

// ------------------------------------------------------------------------------------------- selective scan
// reference.py:124-197.  One thread per (batch, channel); the state lives in `last_state`.
__global__ void f64_scan_fwd_kernel(const ssm_f64_scan_args a) {
  const long long row = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= (long long)a.batch * a.dim) return;
  const int b = (int)(row / a.dim), d = (int)(row % a.dim);
  const int L = a.seqlen, N = a.nstate;
  const double *u = a.u + row * L, *dl = a.delta + row * L;
  const double *z = a.z ? a.z + row * L : nullptr;
  const double *A = a.A + (long long)d * N;
  const double *Bp = a.Bproj + b * a.b_stride[0] + d * a.b_stride[1];
  const double *Cp = a.Cproj + b * a.c_stride[0] + d * a.c_stride[1];
  const double bias = a.dt_bias ? a.dt_bias[d] : 0.0, Dk = a.Dskip ? a.Dskip[d] : 0.0;
  double *h = a.last_state + row * N;
  for (int n = 0; n < N; ++n) h[n] = 0.0;
  for (int t = 0; t < L; ++t) {
    double dt = dl[t] + bias;
    if (a.delta_softplus) dt = softplus64(dt);
    const double ut = u[t];
    double acc = 0.0;
    for (int n = 0; n < N; ++n) {
      const double hn = exp(dt * A[n]) * h[n] + dt * Bp[n * a.b_stride[2] + t * a.b_stride[3]] * ut;
      h[n] = hn;
      acc += hn * Cp[n * a.c_stride[2] + t * a.c_stride[3]];
      if (a.states) a.states[(row * L + t) * N + n] = hn;
    }
    acc += Dk * ut;
    if (a.ypre) a.ypre[row * L + t] = acc;
    if (z) acc *= z[t] * sigmoid64(z[t]);
    if (a.out) a.out[row * L + t] = acc;
  }
}

// Adjoint of the loop above, last step first.  `states` and `ypre` come from a run of the forward kernel;
// `last_state` is reused for the adjoint of the state.
__global__ void f64_scan_bwd_kernel(const ssm_f64_scan_args a) {
  const long long row = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= (long long)a.batch * a.dim) return;
  const int b = (int)(row / a.dim), d = (int)(row % a.dim);
  const int L = a.seqlen, N = a.nstate;
  const double *u = a.u + row * L, *dl = a.delta + row * L, *dy = a.dout + row * L;
  const double *z = a.z ? a.z + row * L : nullptr;
  const double *A = a.A + (long long)d * N;
  const double *Bp = a.Bproj + b * a.b_stride[0] + d * a.b_stride[1];
  const double *Cp = a.Cproj + b * a.c_stride[0] + d * a.c_stride[1];
  const double bias = a.dt_bias ? a.dt_bias[d] : 0.0, Dk = a.Dskip ? a.Dskip[d] : 0.0;
  double *gh = a.last_state + row * N;
  double *dA = a.dA_rows + row * N;
  for (int n = 0; n < N; ++n) {
    gh[n] = a.dlast_state ? a.dlast_state[row * N + n] : 0.0;
    dA[n] = 0.0;
  }
  double dD = 0.0, dbias = 0.0;
  for (int t = L - 1; t >= 0; --t) {
    const double raw = dl[t] + bias;
    const double dt = a.delta_softplus ? softplus64(raw) : raw;
    const double ut = u[t];
    double dyp = dy[t];
    if (z) {
      const double zt = z[t], sg = sigmoid64(zt);
      a.dz[row * L + t] = dyp * a.ypre[row * L + t] * (sg * (1.0 + zt * (1.0 - sg)));
      dyp *= zt * sg;
    }
    double du = Dk * dyp, ddt = 0.0;
    dD += dyp * ut;
    const double *hs = a.states + (row * L + t) * N;
    for (int n = 0; n < N; ++n) {
      const double Bt = Bp[n * a.b_stride[2] + t * a.b_stride[3]], Ct = Cp[n * a.c_stride[2] + t * a.c_stride[3]];
      const double hprev = t > 0 ? hs[n - N] : 0.0;
      const double g = gh[n] + dyp * Ct;
      const double decay = exp(dt * A[n]);
      const long long at = ((row * N) + n) * L + t;
      a.dC[at] = dyp * hs[n];
      a.dB[at] = g * dt * ut;
      du += g * dt * Bt;
      ddt += g * (A[n] * decay * hprev + Bt * ut);
      dA[n] += g * dt * decay * hprev;
      gh[n] = g * decay;
    }
    a.du[row * L + t] = du;
    const double draw = a.delta_softplus ? ddt * dsoftplus64(raw) : ddt;
    a.ddelta[row * L + t] = draw;
    dbias += draw;
  }
  if (a.dD_rows) a.dD_rows[row] = dD;
  if (a.dbias_rows) a.dbias_rows[row] = dbias;
}

// --------------------------------------------------------------------------------------- selective state step
// reference.py:217-312.  One thread per (batch, channel).
__global__ void f64_step_fwd_kernel(const ssm_f64_step_args a) {
  const long long row = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= (long long)a.batch * a.dim) return;
  const int b = (int)(row / a.dim), d = (int)(row % a.dim);
  const int N = a.nstate;
  const double *A = a.A + (long long)d * N;
  const double *Bp = a.Bproj + b * a.b_stride[0] + d * a.b_stride[1];
  const double *Cp = a.Cproj + b * a.c_stride[0] + d * a.c_stride[1];
  double dt = a.dt[row] + (a.dt_bias ? a.dt_bias[d] : 0.0);
  if (a.dt_softplus) dt = softplus64(dt);
  const double xt = a.x[row];
  double *h = a.state + row * N;
  double acc = 0.0;
  for (int n = 0; n < N; ++n) {
    const double hn = exp(dt * A[n]) * h[n] + dt * Bp[n * a.b_stride[2]] * xt;
    h[n] = hn;
    acc += hn * Cp[n * a.c_stride[2]];
  }
  if (a.Dskip) acc += a.Dskip[d] * xt;
  if (a.z) acc *= a.z[row] * sigmoid64(a.z[row]);
  a.out[row] = acc;
}

// `state` is the state before the step.
__global__ void f64_step_bwd_kernel(const ssm_f64_step_args a) {
  const long long row = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= (long long)a.batch * a.dim) return;
  const int b = (int)(row / a.dim), d = (int)(row % a.dim);
  const int N = a.nstate;
  const double *A = a.A + (long long)d * N;
  const double *Bp = a.Bproj + b * a.b_stride[0] + d * a.b_stride[1];
  const double *Cp = a.Cproj + b * a.c_stride[0] + d * a.c_stride[1];
  const double raw = a.dt[row] + (a.dt_bias ? a.dt_bias[d] : 0.0);
  const double dt = a.dt_softplus ? softplus64(raw) : raw;
  const double xt = a.x[row], Dk = a.Dskip ? a.Dskip[d] : 0.0;
  const double *h = a.state + row * N;
  double ypre = Dk * xt;
  for (int n = 0; n < N; ++n) ypre += (exp(dt * A[n]) * h[n] + dt * Bp[n * a.b_stride[2]] * xt) * Cp[n * a.c_stride[2]];
  double dyp = a.dout ? a.dout[row] : 0.0;
  if (a.z) {
    const double zt = a.z[row], sg = sigmoid64(zt);
    a.dz[row] = dyp * ypre * (sg * (1.0 + zt * (1.0 - sg)));
    dyp *= zt * sg;
  }
  double dx = Dk * dyp, ddt = 0.0;
  for (int n = 0; n < N; ++n) {
    const double Bn = Bp[n * a.b_stride[2]], Cn = Cp[n * a.c_stride[2]];
    const double decay = exp(dt * A[n]);
    const double hn = decay * h[n] + dt * Bn * xt;
    const double g = (a.dstate_new ? a.dstate_new[row * N + n] : 0.0) + dyp * Cn;
    a.dC[row * N + n] = dyp * hn;
    a.dB[row * N + n] = g * dt * xt;
    a.dA_rows[row * N + n] = g * dt * decay * h[n];
    a.dstate[row * N + n] = g * decay;
    dx += g * dt * Bn;
    ddt += g * (A[n] * decay * h[n] + Bn * xt);
  }
  a.dx[row] = dx;
  a.ddt[row] = a.dt_softplus ? ddt * dsoftplus64(raw) : ddt;
  if (a.dD_rows) a.dD_rows[row] = dyp * xt;
}

// ----------------------------------------------------------------------------- diagonal chunk scan
// reference.py:315-480.  One thread per (batch, head, p) channel; steps at or beyond a row's length emit zeros
// and leave the state alone.
__global__ void f64_dscan_fwd_kernel(const ssm_f64_dscan_args a) {
  const long long ch = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long HP = (long long)a.heads * a.hdim;
  if (ch >= a.batch * HP) return;
  const int b = (int)(ch / HP), h = (int)((ch % HP) / a.hdim), p = (int)(ch % a.hdim);
  const int L = a.seqlen, len = a.lengths ? min(max(a.lengths[b], 0), L) : L;
  const double Ak = a.A[h * a.hdim + p], Dk = a.Dskip ? a.Dskip[h * a.hdim + p] : 0.0;
  const double *Bp = a.Bproj + b * a.b_stride[0] + h * a.b_stride[2] + p * a.b_stride[3];
  const double *Cp = a.Cproj + b * a.c_stride[0] + h * a.c_stride[2] + p * a.c_stride[3];
  const double *zp = a.z ? a.z + b * a.z_stride[0] + h * a.z_stride[2] + p * a.z_stride[3] : nullptr;
  double s = a.init ? a.init[ch] : 0.0;
  for (int t = 0; t < L; ++t) {
    const long long at = ((long long)b * L + t) * HP + (ch % HP);
    if (t >= len) {
      if (a.Y) a.Y[at] = 0.0;
      if (a.states) a.states[at] = s;
      continue;
    }
    const double dt = a.dt[((long long)b * L + t) * a.heads + h], xt = a.X[at];
    s = exp(dt * Ak) * s + dt * Bp[t * a.b_stride[1]] * xt;
    if (a.states) a.states[at] = s;
    double y = s * Cp[t * a.c_stride[1]] + Dk * xt;
    if (zp) {
      const double zt = zp[t * a.z_stride[1]];
      y *= zt * sigmoid64(zt);
    }
    if (a.Y) a.Y[at] = y;
  }
}

__global__ void f64_dscan_bwd_kernel(const ssm_f64_dscan_args a) {
  const long long ch = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long HP = (long long)a.heads * a.hdim;
  if (ch >= a.batch * HP) return;
  const int b = (int)(ch / HP), h = (int)((ch % HP) / a.hdim), p = (int)(ch % a.hdim);
  const int L = a.seqlen, len = a.lengths ? min(max(a.lengths[b], 0), L) : L;
  const double Ak = a.A[h * a.hdim + p], Dk = a.Dskip ? a.Dskip[h * a.hdim + p] : 0.0;
  const double *Bp = a.Bproj + b * a.b_stride[0] + h * a.b_stride[2] + p * a.b_stride[3];
  const double *Cp = a.Cproj + b * a.c_stride[0] + h * a.c_stride[2] + p * a.c_stride[3];
  const double *zp = a.z ? a.z + b * a.z_stride[0] + h * a.z_stride[2] + p * a.z_stride[3] : nullptr;
  const double s_init = a.init ? a.init[ch] : 0.0;
  double gs = 0.0, dA = 0.0, dD = 0.0;
  for (int t = L - 1; t >= 0; --t) {
    const long long at = ((long long)b * L + t) * HP + (ch % HP);
    if (t >= len) {
      a.dX[at] = 0.0;
      a.ddt_rows[at] = 0.0;
      a.dB[at] = 0.0;
      a.dC[at] = 0.0;
      if (a.dz) a.dz[at] = 0.0;
      continue;
    }
    const double dt = a.dt[((long long)b * L + t) * a.heads + h], xt = a.X[at];
    const double Bt = Bp[t * a.b_stride[1]], Ct = Cp[t * a.c_stride[1]];
    const double st = a.states[at], sprev = t > 0 ? a.states[at - HP] : s_init;
    double dyp = a.dY[at];
    if (zp) {
      const double zt = zp[t * a.z_stride[1]], sg = sigmoid64(zt);
      a.dz[at] = dyp * (st * Ct + Dk * xt) * (sg * (1.0 + zt * (1.0 - sg)));
      dyp *= zt * sg;
    }
    const double g = gs + dyp * Ct;
    const double decay = exp(dt * Ak);
    a.dC[at] = dyp * st;
    a.dB[at] = g * dt * xt;
    a.dX[at] = g * dt * Bt + Dk * dyp;
    a.ddt_rows[at] = g * (Ak * decay * sprev + Bt * xt);
    dA += g * dt * decay * sprev;
    dD += dyp * xt;
    gs = g * decay;
  }
  a.dA_rows[ch] = dA;
  if (a.dD_rows) a.dD_rows[ch] = dD;
  if (a.dinit) a.dinit[ch] = gs;
}

// ------------------------------------------------------------------------- depthwise causal convolution
// reference.py:483-533: y[b,c,t] = act(bias[c] + sum_k w[c,k] x[b,c,t-(K-1)+k]); x, y, dy, dx as (B, C, L) views.
__device__ __forceinline__ double conv_pre(const ssm_f64_conv_args &a, int b, int c, int t) {
  double acc = a.bias ? a.bias[c] : 0.0;
  const double *x = a.x + b * a.x_stride[0] + c * a.x_stride[1];
  for (int k = 0; k < a.width; ++k) {
    const int ts = t - (a.width - 1) + k;
    if (ts >= 0) acc += a.weight[c * a.width + k] * x[ts * a.x_stride[2]];
  }
  return acc;
}

__global__ void f64_conv_fwd_kernel(const ssm_f64_conv_args a) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long CL = (long long)a.channels * a.seqlen;
  if (i >= a.batch * CL) return;
  const int b = (int)(i / CL), c = (int)((i % CL) / a.seqlen), t = (int)(i % a.seqlen);
  double v = conv_pre(a, b, c, t);
  if (a.activation == SSM_ACT_SILU) v *= sigmoid64(v);
  a.y[b * a.y_stride[0] + c * a.y_stride[1] + t * a.y_stride[2]] = v;
}

// gradient at the pre-activation, dense (B, C, L)
__global__ void f64_conv_dpre_kernel(const ssm_f64_conv_args a) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long CL = (long long)a.channels * a.seqlen;
  if (i >= a.batch * CL) return;
  const int b = (int)(i / CL), c = (int)((i % CL) / a.seqlen), t = (int)(i % a.seqlen);
  double g = a.dy[b * a.dy_stride[0] + c * a.dy_stride[1] + t * a.dy_stride[2]];
  if (a.activation == SSM_ACT_SILU) {
    const double v = conv_pre(a, b, c, t), sg = sigmoid64(v);
    g *= sg * (1.0 + v * (1.0 - sg));
  }
  a.dpre[i] = g;
}

__global__ void f64_conv_dx_kernel(const ssm_f64_conv_args a) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long CL = (long long)a.channels * a.seqlen;
  if (i >= a.batch * CL) return;
  const int b = (int)(i / CL), c = (int)((i % CL) / a.seqlen), t = (int)(i % a.seqlen);
  double acc = 0.0;
  for (int k = 0; k < a.width; ++k) {
    const int to = t + (a.width - 1) - k;           // the output step that read x[t] through tap k
    if (to < a.seqlen) acc += a.weight[c * a.width + k] * a.dpre[(long long)(b * a.channels + c) * a.seqlen + to];
  }
  a.dx[b * a.dx_stride[0] + c * a.dx_stride[1] + t * a.dx_stride[2]] = acc;
}

// one workgroup per (channel, tap); tap == width is the bias.  Threads take (batch, step) pairs in a fixed
// stride and their sums meet in a fixed tree: the same bits on every run.
__global__ void f64_conv_dw_kernel(const ssm_f64_conv_args a) {
  __shared__ double part[F64_THREADS];
  const int c = blockIdx.x / (a.width + 1), k = blockIdx.x % (a.width + 1);
  const long long BL = (long long)a.batch * a.seqlen;
  double acc = 0.0;
  for (long long j = threadIdx.x; j < BL; j += F64_THREADS) {
    const int b = (int)(j / a.seqlen), t = (int)(j % a.seqlen);
    const double g = a.dpre[(long long)(b * a.channels + c) * a.seqlen + t];
    if (k == a.width) {
      acc += g;
    } else {
      const int ts = t - (a.width - 1) + k;
      if (ts >= 0) acc += g * a.x[b * a.x_stride[0] + c * a.x_stride[1] + ts * a.x_stride[2]];
    }
  }
  part[threadIdx.x] = acc;
  __syncthreads();
  for (int s = F64_THREADS / 2; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) part[threadIdx.x] += part[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    if (k == a.width) {
      if (a.db) a.db[c] = part[0];
    } else {
      a.dw[c * a.width + k] = part[0];
    }
  }
}

// ----------------------------------------------------------------- residual add + LayerNorm / RMSNorm
// reference.py:536-609.  One thread per row (two-pass variance, as the reference forms it).
__global__ void f64_norm_fwd_kernel(const ssm_f64_norm_args a) {
  const long long r = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= a.rows) return;
  const int Hd = a.hidden;
  const double *x = a.x + r * Hd;
  const double *res = a.residual ? a.residual + r * Hd : nullptr;
  const bool pre = res && a.prenorm;
  double mean = 0.0;
  if (!a.is_rms) {
    for (int j = 0; j < Hd; ++j) mean += x[j] + (pre ? res[j] : 0.0);
    mean /= Hd;
  }
  double var = 0.0;
  for (int j = 0; j < Hd; ++j) {
    const double v = x[j] + (pre ? res[j] : 0.0) - mean;
    var += v * v;
  }
  const double rstd = 1.0 / sqrt(var / Hd + a.eps);
  a.mean[r] = mean;
  a.rstd[r] = rstd;
  for (int j = 0; j < Hd; ++j) {
    const double v = x[j] + (pre ? res[j] : 0.0);
    double y = (v - mean) * rstd * a.weight[j] + (a.bias ? a.bias[j] : 0.0);
    if (res && !a.prenorm) y += res[j];
    a.y[r * Hd + j] = y;
    if (a.residual_out) a.residual_out[r * Hd + j] = v;
  }
}

__global__ void f64_norm_bwd_rows_kernel(const ssm_f64_norm_args a) {
  const long long r = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= a.rows) return;
  const int Hd = a.hidden;
  const double *x = a.x + r * Hd, *dy = a.dy + r * Hd;
  const double *res = a.residual ? a.residual + r * Hd : nullptr;
  const bool pre = res && a.prenorm;
  const double mean = a.mean[r], rstd = a.rstd[r];
  double m1 = 0.0, m2 = 0.0;            // mean of dxhat, mean of dxhat * xhat
  for (int j = 0; j < Hd; ++j) {
    const double xhat = (x[j] + (pre ? res[j] : 0.0) - mean) * rstd, dxh = dy[j] * a.weight[j];
    m1 += dxh;
    m2 += dxh * xhat;
  }
  m1 = a.is_rms ? 0.0 : m1 / Hd;
  m2 /= Hd;
  for (int j = 0; j < Hd; ++j) {
    const double xhat = (x[j] + (pre ? res[j] : 0.0) - mean) * rstd, dxh = dy[j] * a.weight[j];
    const double dv = rstd * (dxh - m1 - xhat * m2);
    a.dx[r * Hd + j] = dv;
    if (a.dresidual) a.dresidual[r * Hd + j] = a.prenorm ? dv : dy[j];
  }
}

// one thread per column, rows in order
__global__ void f64_norm_bwd_cols_kernel(const ssm_f64_norm_args a) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= a.hidden) return;
  const bool pre = a.residual && a.prenorm;
  double dw = 0.0, db = 0.0;
  for (long long r = 0; r < a.rows; ++r) {
    const double v = a.x[r * a.hidden + j] + (pre ? a.residual[r * a.hidden + j] : 0.0);
    const double g = a.dy[r * a.hidden + j];
    dw += g * (v - a.mean[r]) * a.rstd[r];
    db += g;
  }
  a.dw[j] = dw;
  if (a.db) a.db[j] = db;
}

int check_scan(const ssm_f64_scan_args *a, const char *who) {
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "%s: args is NULL", who);
  SSM_REQUIRE(a->batch > 0 && a->dim > 0 && a->seqlen > 0 && a->nstate > 0, SSM_ERR_BAD_SHAPE,
              "%s: batch, dim, seqlen and nstate must be positive", who);
  SSM_REQUIRE(a->u && a->delta && a->A && a->Bproj && a->Cproj && a->last_state, SSM_ERR_NULL_POINTER,
              "%s: u, delta, A, Bproj, Cproj and last_state are required", who);
  return SSM_OK;
}

}  // namespace
}  // namespace ssm

using namespace ssm;

extern "C" int ssm_f64_scan_fwd(const ssm_f64_scan_args *a, void *stream) {
  if (int rc = check_scan(a, "ssm_f64_scan_fwd")) return rc;
  SSM_REQUIRE(a->out != nullptr, SSM_ERR_NULL_POINTER, "ssm_f64_scan_fwd: out is required");
  ssm_f64_scan_args k = *a;
  k.states = nullptr;
  k.ypre = nullptr;
  hipLaunchKernelGGL(f64_scan_fwd_kernel, dim3(blocks_for((long long)a->batch * a->dim)), dim3(F64_THREADS), 0,
                     (hipStream_t)stream, k);
  SSM_CHECK_LAUNCH("ssm_f64_scan_fwd");
  return SSM_OK;
}

extern "C" int ssm_f64_scan_bwd(const ssm_f64_scan_args *a, void *stream) {
  if (int rc = check_scan(a, "ssm_f64_scan_bwd")) return rc;
  SSM_REQUIRE(a->dout && a->states && a->ypre && a->du && a->ddelta && a->dA_rows && a->dB && a->dC,
              SSM_ERR_NULL_POINTER, "ssm_f64_scan_bwd: dout, states, ypre, du, ddelta, dA_rows, dB and dC are required");
  SSM_REQUIRE(!a->z || a->dz, SSM_ERR_NULL_POINTER, "ssm_f64_scan_bwd: dz is required with z");
  const dim3 grid(blocks_for((long long)a->batch * a->dim));
  ssm_f64_scan_args k = *a;
  k.out = nullptr;                       // the recomputing pass writes the states and the ungated output only
  hipLaunchKernelGGL(f64_scan_fwd_kernel, grid, dim3(F64_THREADS), 0, (hipStream_t)stream, k);
  hipLaunchKernelGGL(f64_scan_bwd_kernel, grid, dim3(F64_THREADS), 0, (hipStream_t)stream, *a);
  SSM_CHECK_LAUNCH("ssm_f64_scan_bwd");
  return SSM_OK;
}

extern "C" int ssm_f64_state_step(const ssm_f64_step_args *a, void *stream) {
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_f64_state_step: args is NULL");
  SSM_REQUIRE(a->batch > 0 && a->dim > 0 && a->nstate > 0, SSM_ERR_BAD_SHAPE, "ssm_f64_state_step: sizes must be positive");
  SSM_REQUIRE(a->state && a->x && a->dt && a->A && a->Bproj && a->Cproj && a->out, SSM_ERR_NULL_POINTER,
              "ssm_f64_state_step: state, x, dt, A, Bproj, Cproj and out are required");
  hipLaunchKernelGGL(f64_step_fwd_kernel, dim3(blocks_for((long long)a->batch * a->dim)), dim3(F64_THREADS), 0,
                     (hipStream_t)stream, *a);
  SSM_CHECK_LAUNCH("ssm_f64_state_step");
  return SSM_OK;
}

extern "C" int ssm_f64_state_step_bwd(const ssm_f64_step_args *a, void *stream) {
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_f64_state_step_bwd: args is NULL");
  SSM_REQUIRE(a->batch > 0 && a->dim > 0 && a->nstate > 0, SSM_ERR_BAD_SHAPE, "ssm_f64_state_step_bwd: sizes must be positive");
  SSM_REQUIRE(a->state && a->x && a->dt && a->A && a->Bproj && a->Cproj && a->dstate && a->dx && a->ddt && a->dA_rows &&
                  a->dB && a->dC, SSM_ERR_NULL_POINTER,
              "ssm_f64_state_step_bwd: inputs, dstate, dx, ddt, dA_rows, dB and dC are required");
  SSM_REQUIRE(!a->z || a->dz, SSM_ERR_NULL_POINTER, "ssm_f64_state_step_bwd: dz is required with z");
  hipLaunchKernelGGL(f64_step_bwd_kernel, dim3(blocks_for((long long)a->batch * a->dim)), dim3(F64_THREADS), 0,
                     (hipStream_t)stream, *a);
  SSM_CHECK_LAUNCH("ssm_f64_state_step_bwd");
  return SSM_OK;
}

static int check_dscan(const ssm_f64_dscan_args *a, const char *who) {
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "%s: args is NULL", who);
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->hdim > 0, SSM_ERR_BAD_SHAPE, "%s: sizes must be positive", who);
  SSM_REQUIRE(a->X && a->dt && a->A && a->Bproj && a->Cproj, SSM_ERR_NULL_POINTER, "%s: X, dt, A, Bproj and Cproj are required", who);
  return SSM_OK;
}

extern "C" int ssm_f64_dscan_fwd(const ssm_f64_dscan_args *a, void *stream) {
  if (int rc = check_dscan(a, "ssm_f64_dscan_fwd")) return rc;
  SSM_REQUIRE(a->Y != nullptr, SSM_ERR_NULL_POINTER, "ssm_f64_dscan_fwd: Y is required");
  ssm_f64_dscan_args k = *a;
  k.states = nullptr;
  hipLaunchKernelGGL(f64_dscan_fwd_kernel, dim3(blocks_for((long long)a->batch * a->heads * a->hdim)), dim3(F64_THREADS), 0,
                     (hipStream_t)stream, k);
  SSM_CHECK_LAUNCH("ssm_f64_dscan_fwd");
  return SSM_OK;
}

extern "C" int ssm_f64_dscan_bwd(const ssm_f64_dscan_args *a, void *stream) {
  if (int rc = check_dscan(a, "ssm_f64_dscan_bwd")) return rc;
  SSM_REQUIRE(a->dY && a->states && a->dX && a->ddt_rows && a->dA_rows && a->dB && a->dC, SSM_ERR_NULL_POINTER,
              "ssm_f64_dscan_bwd: dY, states, dX, ddt_rows, dA_rows, dB and dC are required");
  SSM_REQUIRE(!a->z || a->dz, SSM_ERR_NULL_POINTER, "ssm_f64_dscan_bwd: dz is required with z");
  const dim3 grid(blocks_for((long long)a->batch * a->heads * a->hdim));
  ssm_f64_dscan_args k = *a;
  k.Y = nullptr;
  hipLaunchKernelGGL(f64_dscan_fwd_kernel, grid, dim3(F64_THREADS), 0, (hipStream_t)stream, k);
  hipLaunchKernelGGL(f64_dscan_bwd_kernel, grid, dim3(F64_THREADS), 0, (hipStream_t)stream, *a);
  SSM_CHECK_LAUNCH("ssm_f64_dscan_bwd");
  return SSM_OK;
}

static int check_conv(const ssm_f64_conv_args *a, const char *who) {
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "%s: args is NULL", who);
  SSM_REQUIRE(a->batch > 0 && a->channels > 0 && a->seqlen > 0 && a->width > 0, SSM_ERR_BAD_SHAPE, "%s: sizes must be positive", who);
  SSM_REQUIRE(a->activation == SSM_ACT_IDENTITY || a->activation == SSM_ACT_SILU, SSM_ERR_BAD_KIND, "%s: unknown activation", who);
  SSM_REQUIRE(a->x && a->weight, SSM_ERR_NULL_POINTER, "%s: x and weight are required", who);
  return SSM_OK;
}

extern "C" int ssm_f64_conv_fwd(const ssm_f64_conv_args *a, void *stream) {
  if (int rc = check_conv(a, "ssm_f64_conv_fwd")) return rc;
  SSM_REQUIRE(a->y != nullptr, SSM_ERR_NULL_POINTER, "ssm_f64_conv_fwd: y is required");
  hipLaunchKernelGGL(f64_conv_fwd_kernel, dim3(blocks_for((long long)a->batch * a->channels * a->seqlen)), dim3(F64_THREADS), 0,
                     (hipStream_t)stream, *a);
  SSM_CHECK_LAUNCH("ssm_f64_conv_fwd");
  return SSM_OK;
}

extern "C" int ssm_f64_conv_bwd(const ssm_f64_conv_args *a, void *stream) {
  if (int rc = check_conv(a, "ssm_f64_conv_bwd")) return rc;
  SSM_REQUIRE(a->dy && a->dpre && a->dx && a->dw, SSM_ERR_NULL_POINTER, "ssm_f64_conv_bwd: dy, dpre, dx and dw are required");
  const dim3 grid(blocks_for((long long)a->batch * a->channels * a->seqlen));
  hipLaunchKernelGGL(f64_conv_dpre_kernel, grid, dim3(F64_THREADS), 0, (hipStream_t)stream, *a);
  hipLaunchKernelGGL(f64_conv_dx_kernel, grid, dim3(F64_THREADS), 0, (hipStream_t)stream, *a);
  hipLaunchKernelGGL(f64_conv_dw_kernel, dim3((unsigned)(a->channels * (a->width + 1))), dim3(F64_THREADS), 0,
                     (hipStream_t)stream, *a);
  SSM_CHECK_LAUNCH("ssm_f64_conv_bwd");
  return SSM_OK;
}

static int check_norm(const ssm_f64_norm_args *a, const char *who) {
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "%s: args is NULL", who);
  SSM_REQUIRE(a->rows > 0 && a->hidden > 0, SSM_ERR_BAD_SHAPE, "%s: rows and hidden must be positive", who);
  SSM_REQUIRE(a->x && a->weight && a->mean && a->rstd, SSM_ERR_NULL_POINTER, "%s: x, weight, mean and rstd are required", who);
  return SSM_OK;
}

extern "C" int ssm_f64_norm_fwd(const ssm_f64_norm_args *a, void *stream) {
  if (int rc = check_norm(a, "ssm_f64_norm_fwd")) return rc;
  SSM_REQUIRE(a->y != nullptr, SSM_ERR_NULL_POINTER, "ssm_f64_norm_fwd: y is required");
  hipLaunchKernelGGL(f64_norm_fwd_kernel, dim3(blocks_for(a->rows)), dim3(F64_THREADS), 0, (hipStream_t)stream, *a);
  SSM_CHECK_LAUNCH("ssm_f64_norm_fwd");
  return SSM_OK;
}

extern "C" int ssm_f64_norm_bwd(const ssm_f64_norm_args *a, void *stream) {
  if (int rc = check_norm(a, "ssm_f64_norm_bwd")) return rc;
  SSM_REQUIRE(a->dy && a->dx && a->dw, SSM_ERR_NULL_POINTER, "ssm_f64_norm_bwd: dy, dx and dw are required");
  hipLaunchKernelGGL(f64_norm_bwd_rows_kernel, dim3(blocks_for(a->rows)), dim3(F64_THREADS), 0, (hipStream_t)stream, *a);
  hipLaunchKernelGGL(f64_norm_bwd_cols_kernel, dim3(blocks_for(a->hidden)), dim3(F64_THREADS), 0, (hipStream_t)stream, *a);
  SSM_CHECK_LAUNCH("ssm_f64_norm_bwd");
  return SSM_OK;
}
