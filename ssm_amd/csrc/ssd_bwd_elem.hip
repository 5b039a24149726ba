// Element-wise stages between the passes of the state-space-duality backward, one read of every tensor each:
//
//   gate   dy = dout silu(z);  dz = dout (ypre + D x) silu'(z);  s2 = <round(dy), ypre>;  dyx = <dy, x>
//          (dy is written in the passes' operand type, in time order and reversed)
//   dx     dx = dt u + D dy;  xu = <x, u>;  s1 = <round(dt x), u>      (u arrives reversed in time)
//   db     dB[l][g][n] = sum_{h in g} dt[l][h] v[L-1-l][h][n]          (v arrives reversed in time)
//
// Rows are the (batch, step, head) vectors of P channels; a row is shared by P/4 lanes (a power of two up to
// 64) that take four neighbouring channels each, row sums are butterflies inside the wave.  All reads are
// unconditional (an absent gate reads dout in its place).
#include "common.hpp"

#include <type_traits>

namespace ssm {
namespace {

constexpr int EB_THREADS = 256;

struct ElemParams {
  const void *dout, *z, *x;
  const float *ypre, *u_rev, *dt, *Dk;
  void *dy, *dy_rev;
  void *dz, *dx;                // float32, or the type of dout / x with grads_io
  float *s1, *s2, *dyx, *xu;
  int grads_io;
  const float *w_dy, *w_x;      // (B, L, H) weights of the extra row-scaled copies, or null
  void *dy_w, *x_w;             // (B, L, H, P) dy as stored times w_dy, x times w_x, in dy's type; or null
  int batch, len, heads, hdim;
  int d_per_p, round_bf16;
  int lg;                       // lanes per row = 1 << lg
};

template <typename T>
__device__ __forceinline__ void ld4(const void *p, size_t i, float (&v)[4]) {
  const Pack<T, 4> raw = *reinterpret_cast<const Pack<T, 4> *>(reinterpret_cast<const T *>(p) + i);
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = to_f32(raw.v[j]);
}
template <typename T>
__device__ __forceinline__ void st4(void *p, size_t i, const float (&v)[4]) {
  Pack<T, 4> raw;
#pragma unroll
  for (int j = 0; j < 4; ++j) raw.v[j] = from_f32<T>(v[j]);
  *reinterpret_cast<Pack<T, 4> *>(reinterpret_cast<T *>(p) + i) = raw;
}

__device__ __forceinline__ float row_sum(float v, int lg) {
  for (int m = (1 << lg) >> 1; m >= 1; m >>= 1) v += __shfl_xor(v, m, WAVE);
  return v;
}

struct RowAt {
  bool live;
  size_t row, rev;     // (b, l, h) and (b, L-1-l, h)
  int h, c0;           // head, first of the lane's four channels
};

__device__ __forceinline__ RowAt locate(const ElemParams &p) {
  const size_t rows = (size_t)p.batch * p.len * p.heads;
  const size_t gid = (size_t)blockIdx.x * EB_THREADS + threadIdx.x;
  RowAt a;
  a.live = gid < (rows << p.lg);
  const size_t g = a.live ? gid : 0;
  a.row = g >> p.lg;
  a.c0 = (int)(g & (size_t)((1 << p.lg) - 1)) * 4;
  a.h = (int)(a.row % (size_t)p.heads);
  const size_t bl = a.row / (size_t)p.heads;
  const size_t b = bl / (size_t)p.len, l = bl % (size_t)p.len;
  a.rev = (b * p.len + (p.len - 1 - l)) * p.heads + a.h;
  return a;
}

// IO: type of dout, z, x.  OT: type of dy (the passes' operand type).
template <typename IO, typename OT>
__global__ __launch_bounds__(EB_THREADS) void ssd_bwd_gate_kernel(const ElemParams p) {
  const RowAt a = locate(p);
  const size_t at = a.row * p.hdim + a.c0;
  float go[4], zv[4], xv[4], yp[4], Dv[4];
  ld4<IO>(p.dout, at, go);
  ld4<IO>(p.z ? p.z : p.dout, at, zv);
  ld4<IO>(p.x, at, xv);
  ld4<float>(p.ypre, at, yp);
#pragma unroll
  for (int j = 0; j < 4; ++j) Dv[j] = p.Dk ? p.Dk[p.d_per_p ? a.h * p.hdim + a.c0 + j : a.h] : 0.0f;
  float dy[4], dz[4], s2 = 0.0f, dyx = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (p.z) {
      const float sg = sigmoid_f32(zv[j]);
      dy[j] = go[j] * zv[j] * sg;
      dz[j] = go[j] * __builtin_fmaf(Dv[j], xv[j], yp[j]) * (sg * __builtin_fmaf(zv[j], 1.0f - sg, 1.0f));
    } else {
      dy[j] = go[j];
      dz[j] = 0.0f;
    }
    dyx = __builtin_fmaf(dy[j], xv[j], dyx);
    s2 = __builtin_fmaf(to_f32(from_f32<OT>(dy[j])), yp[j], s2);
  }
  s2 = row_sum(s2, p.lg);
  dyx = row_sum(dyx, p.lg);
  if (!a.live) return;
  st4<OT>(p.dy, at, dy);
  if (p.dy_rev) st4<OT>(p.dy_rev, a.rev * p.hdim + a.c0, dy);
  if (p.dz) {
    if (p.grads_io) st4<IO>(p.dz, at, dz);
    else st4<float>(p.dz, at, dz);
  }
  if (p.dy_w) {
    const float w = p.w_dy[a.row];
    float t[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) t[j] = to_f32(from_f32<OT>(dy[j])) * w;
    st4<OT>(p.dy_w, at, t);
  }
  if (p.x_w) {
    const float w = p.w_x[a.row];
    float t[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) t[j] = xv[j] * w;
    st4<OT>(p.x_w, at, t);
  }
  if (a.c0 == 0) {
    p.s2[a.row] = s2;
    p.dyx[a.row] = dyx;
  }
}

template <typename IO>
__global__ __launch_bounds__(EB_THREADS) void ssd_bwd_dx_kernel(const ElemParams p) {
  const RowAt a = locate(p);
  const size_t at = a.row * p.hdim + a.c0;
  float go[4], zv[4], xv[4], uv[4], Dv[4];
  ld4<IO>(p.dout, at, go);
  ld4<IO>(p.z ? p.z : p.dout, at, zv);
  ld4<IO>(p.x, at, xv);
  ld4<float>(p.u_rev, a.rev * p.hdim + a.c0, uv);
  const float dt = p.dt[a.row];
#pragma unroll
  for (int j = 0; j < 4; ++j) Dv[j] = p.Dk ? p.Dk[p.d_per_p ? a.h * p.hdim + a.c0 + j : a.h] : 0.0f;
  float dx[4], xu = 0.0f, s1 = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float dy = p.z ? go[j] * zv[j] * sigmoid_f32(zv[j]) : go[j];
    dx[j] = __builtin_fmaf(dt, uv[j], Dv[j] * dy);
    xu = __builtin_fmaf(xv[j], uv[j], xu);
    const float xt = dt * xv[j];
    s1 = __builtin_fmaf(p.round_bf16 ? to_f32(from_f32<bf16_t>(xt)) : xt, uv[j], s1);
  }
  xu = row_sum(xu, p.lg);
  s1 = row_sum(s1, p.lg);
  if (!a.live) return;
  if (p.grads_io) st4<IO>(p.dx, at, dx);
  else st4<float>(p.dx, at, dx);
  if (a.c0 == 0) {
    p.xu[a.row] = xu;
    p.s1[a.row] = s1;
  }
}

struct DbParams {
  const float *v_rev, *dt;
  float *dB;
  int batch, len, heads, groups, nstate;
};

// One thread per four neighbouring states of a (batch, step, group); the heads of the group are added in order.
__global__ __launch_bounds__(EB_THREADS) void ssd_bwd_db_kernel(const DbParams p) {
  const int n4 = p.nstate / 4, per = p.heads / p.groups;
  const size_t total = (size_t)p.batch * p.len * p.groups * n4;
  const size_t gid = (size_t)blockIdx.x * EB_THREADS + threadIdx.x;
  if (gid >= total) return;
  const int n0 = (int)(gid % n4) * 4;
  const int g = (int)((gid / n4) % p.groups);
  const size_t bl = gid / ((size_t)n4 * p.groups);
  const size_t b = bl / (size_t)p.len, l = bl % (size_t)p.len;
  const size_t rev = b * p.len + (p.len - 1 - l);
  float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  int h = 0;
  for (; h + 4 <= per; h += 4) {
    float4 v[4];
    float w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int hh = g * per + h + k;
      v[k] = *reinterpret_cast<const float4 *>(p.v_rev + (rev * p.heads + hh) * p.nstate + n0);
      w[k] = p.dt[bl * p.heads + hh];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      s.x = __builtin_fmaf(w[k], v[k].x, s.x); s.y = __builtin_fmaf(w[k], v[k].y, s.y);
      s.z = __builtin_fmaf(w[k], v[k].z, s.z); s.w = __builtin_fmaf(w[k], v[k].w, s.w);
    }
  }
  for (; h < per; ++h) {
    const int hh = g * per + h;
    const float4 v = *reinterpret_cast<const float4 *>(p.v_rev + (rev * p.heads + hh) * p.nstate + n0);
    const float w = p.dt[bl * p.heads + hh];
    s.x = __builtin_fmaf(w, v.x, s.x); s.y = __builtin_fmaf(w, v.y, s.y);
    s.z = __builtin_fmaf(w, v.z, s.z); s.w = __builtin_fmaf(w, v.w, s.w);
  }
  *reinterpret_cast<float4 *>(p.dB + (bl * p.groups + g) * p.nstate + n0) = s;
}

bool row_lanes(int hdim, int &lg) {
  if (hdim % 4 != 0) return false;
  lg = 0;
  while ((4 << lg) < hdim) ++lg;
  return (4 << lg) == hdim && lg <= 6;
}

unsigned elem_grid(const ElemParams &p) {
  const size_t lanes = ((size_t)p.batch * p.len * p.heads) << p.lg;
  return (unsigned)((lanes + EB_THREADS - 1) / EB_THREADS);
}

// Chunk-boundary states of the two passes for the products that give dB and dC, and the anchors of the running
// sum behind ddt and dA.  One workgroup per (batch, chunk c, head): the forward state entering chunk c and the
// adjoint state entering reversed chunk nc - c (the one that sits in front of chunk c - 1 in time order) are read
// once, written as bfloat16 in time order, and their inner product is the anchor of chunk c.
struct StatesParams {
  const float *ent_f, *ent_r;     // (B, nc, H, dim)
  bf16_t *f16, *r16;              // (B, nc, H, dim)
  float *anchor;                  // (B, nc - 1, H)
  int batch, nchunks, heads, dim;
};

__global__ __launch_bounds__(EB_THREADS) void ssd_bwd_states_kernel(const StatesParams p) {
  __shared__ float part[EB_THREADS / WAVE];
  const int h = blockIdx.x % p.heads;
  const int c = (blockIdx.x / p.heads) % p.nchunks;
  const int b = blockIdx.x / (p.heads * p.nchunks);
  const int nc = p.nchunks;
  const size_t at = (((size_t)b * nc + c) * p.heads + h) * (size_t)p.dim;
  const float *F = p.ent_f + at;
  bf16_t *F16 = p.f16 + at;
  // c >= 1: the adjoint state whose place in time order is c - 1; c == 0: the one whose place is nc - 1 (no anchor)
  const int rsrc = c >= 1 ? nc - c : 0, rdst = c >= 1 ? c - 1 : nc - 1;
  const float *R = p.ent_r + (((size_t)b * nc + rsrc) * p.heads + h) * (size_t)p.dim;
  bf16_t *R16 = p.r16 + (((size_t)b * nc + rdst) * p.heads + h) * (size_t)p.dim;
  float acc = 0.0f;
  for (int i = threadIdx.x * 4; i < p.dim; i += EB_THREADS * 4) {
    const float4 f = *reinterpret_cast<const float4 *>(F + i), r = *reinterpret_cast<const float4 *>(R + i);
    acc = __builtin_fmaf(f.x, r.x, acc);
    acc = __builtin_fmaf(f.y, r.y, acc);
    acc = __builtin_fmaf(f.z, r.z, acc);
    acc = __builtin_fmaf(f.w, r.w, acc);
    const float fv[4] = {f.x, f.y, f.z, f.w}, rv[4] = {r.x, r.y, r.z, r.w};
    st4<bf16_t>(F16, i, fv);
    st4<bf16_t>(R16, i, rv);
  }
  acc = wave_sum(acc);
  if (lane_id() == 0) part[wave_id_uniform()] = acc;
  __syncthreads();
  if (threadIdx.x == 0 && c >= 1) {
    float t = 0.0f;
    for (int w = 0; w < EB_THREADS / WAVE; ++w) t += part[w];
    p.anchor[((size_t)b * (nc - 1) + (c - 1)) * p.heads + h] = t;
  }
}

// out[row][:] = x[row][:] * w[row], formed in float32 and rounded once: the step-weighted operand of the first pass.
struct ScaleParams {
  const void *x;
  const float *w;
  void *out;
  size_t rows;
  int cols;
};

template <typename IO, typename OT>
__global__ __launch_bounds__(EB_THREADS) void ssd_scale_rows_kernel(const ScaleParams p) {
  const size_t quads = p.rows * (size_t)(p.cols / 4);
  const size_t gid = (size_t)blockIdx.x * EB_THREADS + threadIdx.x;
  if (gid >= quads) return;
  const size_t row = gid / (size_t)(p.cols / 4);
  const float w = p.w[row];
  float v[4];
  ld4<IO>(p.x, gid * 4, v);
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] *= w;
  st4<OT>(p.out, gid * 4, v);
}

// The per-step scalars of the backward, one thread per (batch, chunk, head) walking its chunk:
//   q_l    = anchor + sum_{j<l} (s1_j - s2_j),  anchor = W0 for the first chunk, a_first <G, H> at a later boundary
//   ddt_l  = (A q_l + xu_l) * d(step)/d(raw dt)      (softplus' = sigmoid, and 0 outside the clamp)
//   dA    += dt_l q_l,   dbias += ddt_l              (one partial per thread, summed afterwards in a fixed order)
struct DtParams {
  const float *s1, *s2, *xu, *dte, *A, *bias, *W0, *anchor;
  const void *dt_raw;
  const unsigned char *first;     // (B, L) 1 at the first step of a packed sequence, or null
  float *ddt, *dA_part, *db_part;
  int batch, len, heads, chunk, nchunks, dt_dtype, softplus;
  float lo, hi;
};

// A workgroup takes 16 neighbouring heads of one (batch, chunk) and cuts the chunk into 16 segments: thread
// (head, segment) first adds up its segment's differences s1 - s2, the segments' sums meet in LDS, and from the
// running sum at its segment's start the thread walks its steps.  (One thread per chunk walked 256 dependent steps
// while 20 workgroups were all the launch had.)
constexpr int DT_HEADS = 16, DT_SEGS = EB_THREADS / DT_HEADS;

__global__ __launch_bounds__(EB_THREADS) void ssd_bwd_dt_kernel(const DtParams p) {
  __shared__ float seg_sum[DT_SEGS][DT_HEADS], seg_dA[DT_SEGS][DT_HEADS], seg_db[DT_SEGS][DT_HEADS];
  const int hh = threadIdx.x % DT_HEADS, sg = threadIdx.x / DT_HEADS;
  const int hblocks = (p.heads + DT_HEADS - 1) / DT_HEADS;
  const int hb = blockIdx.x % hblocks;
  const int c = (blockIdx.x / hblocks) % p.nchunks;
  const int b = blockIdx.x / (hblocks * p.nchunks);
  const int h = hb * DT_HEADS + hh;
  const bool live = h < p.heads;
  const int hc = live ? h : p.heads - 1;                       // (a lane past the last head reads the last head's values)
  const int seg_len = (p.chunk + DT_SEGS - 1) / DT_SEGS;
  const int l_begin = min(sg * seg_len, p.chunk), l_end = min(l_begin + seg_len, p.chunk);
  const float Ah = p.A[hc], bias = p.bias ? p.bias[hc] : 0.0f;
  const size_t row0 = ((size_t)b * p.len + (size_t)c * p.chunk) * p.heads + hc;
  float mine = 0.0f;
  for (int l = l_begin; l < l_end; ++l) {
    const size_t at = row0 + (size_t)l * p.heads;
    mine += p.s1[at] - p.s2[at];
  }
  seg_sum[sg][hh] = mine;
  float q;
  if (c == 0) {
    q = p.W0 ? p.W0[(size_t)b * p.heads + hc] : 0.0f;
  } else {
    float a_first = exp2_hw(p.dte[row0] * Ah * LOG2E);
    if (p.first && p.first[(size_t)b * p.len + (size_t)c * p.chunk]) a_first = 0.0f;
    q = a_first * p.anchor[((size_t)b * (p.nchunks - 1) + (c - 1)) * p.heads + hc];
  }
  __syncthreads();
  for (int k = 0; k < sg; ++k) q += seg_sum[k][hh];
  float dA = 0.0f, db = 0.0f;
  constexpr int G = 4;
  for (int l0 = l_begin; l0 < l_end; l0 += G) {
    float d[G], xu[G], dte[G], raw[G];
#pragma unroll
    for (int k = 0; k < G; ++k) {
      const size_t at = row0 + (size_t)min(l0 + k, l_end - 1) * p.heads;
      d[k] = p.s1[at] - p.s2[at];
      xu[k] = p.xu[at];
      dte[k] = p.dte[at];
      raw[k] = load_as_f32(p.dt_raw, p.dt_dtype, at) + bias;
    }
#pragma unroll
    for (int k = 0; k < G; ++k) {
      if (l0 + k < l_end) {
        const float ddte = __builtin_fmaf(Ah, q, xu[k]);
        dA = __builtin_fmaf(dte[k], q, dA);
        q += d[k];
        float v = raw[k], slope = 1.0f;
        if (p.softplus) {
          v = raw[k] > 20.0f ? raw[k] : log2_hw(1.0f + exp2_hw(raw[k] * LOG2E)) * LN2;
          slope = sigmoid_f32(raw[k]);
        }
        const float g = (v >= p.lo && v <= p.hi) ? ddte * slope : 0.0f;
        if (live) p.ddt[row0 + (size_t)(l0 + k) * p.heads] = g;
        db += g;
      }
    }
  }
  seg_dA[sg][hh] = dA;
  seg_db[sg][hh] = db;
  __syncthreads();
  if (sg == 0 && live) {
    float sa = 0.0f, sb = 0.0f;
#pragma unroll
    for (int k = 0; k < DT_SEGS; ++k) {
      sa += seg_dA[k][hh];
      sb += seg_db[k][hh];
    }
    const size_t gid = ((size_t)b * p.nchunks + c) * p.heads + h;
    p.dA_part[gid] = sa;
    p.db_part[gid] = sb;
  }
}

// Everything the backward derives from the raw steps alone, one wavefront per (b, h, chunk): the effective step
// (bias, softplus, clamp) in both layouts, its running sum times A inside the chunk, the same for the time-reversed
// sequence whose decay at a step is that of the step that follows it, and the two per-row weights
// exp(running sum) and step * exp(reversed running sum).  Whole chunks only.
struct PrepParams {
  const void *dt;
  const float *A, *bias;
  float *dA_cs, *dt_c, *dA_rev;     // (B, H, nc, Q)
  float *dte, *w_dy, *w_x;          // (B, L, H)
  int batch, len, heads, chunk, nchunks;
  int dt_dtype, softplus;
  float lo, hi;
};

__global__ __launch_bounds__(EB_THREADS) void ssd_bwd_prep_kernel(const PrepParams p) {
  const size_t gw = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int lane = lane_id();
  if (gw >= (size_t)p.batch * p.heads * p.nchunks) return;      // whole wavefronts
  const int c = (int)(gw % p.nchunks);
  const int h = (int)((gw / p.nchunks) % p.heads);
  const int b = (int)(gw / ((size_t)p.nchunks * p.heads));
  const float A = p.A[h];
  const float bias = p.bias ? p.bias[h] : 0.0f;
  const int Q = p.chunk;
  auto step_at = [&](int t) {              // the effective step; 0 past the end of the sequence
    if (t >= p.len) return 0.0f;
    float v = load_as_f32(p.dt, p.dt_dtype, ((size_t)b * p.len + t) * p.heads + h) + bias;
    if (p.softplus) v = softplus_f32(v);
    return fminf(fmaxf(v, p.lo), p.hi);
  };
  const size_t out = (((size_t)b * p.heads + h) * p.nchunks + c) * Q;
  float carry = 0.0f;
  for (int l0 = 0; l0 < Q; l0 += WAVE) {
    const int l = l0 + lane;
    const bool in = l < Q;
    const int t = c * Q + l;
    const float v = in ? step_at(t) : 0.0f;
    const float run = carry + wave_inclusive_sum(v * A);
    if (in) {
      const size_t row = ((size_t)b * p.len + t) * p.heads + h;
      p.dt_c[out + l] = v;
      p.dA_cs[out + l] = run;
      p.dte[row] = v;
      p.w_dy[row] = expf(run);
    }
    carry = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(run), WAVE - 1));
  }
  // reversed time: position i of reversed chunk nc-1-c is step t = cQ + Q-1-i, decaying by the step after it
  const size_t out_r = (((size_t)b * p.heads + h) * p.nchunks + (p.nchunks - 1 - c)) * Q;
  carry = 0.0f;
  for (int i0 = 0; i0 < Q; i0 += WAVE) {
    const int i = i0 + lane;
    const bool in = i < Q;
    const int t = c * Q + Q - 1 - i;
    const float next = in ? step_at(t + 1) : 0.0f;
    const float run = carry + wave_inclusive_sum(next * A);
    if (in) {
      p.dA_rev[out_r + i] = run;
      p.w_x[((size_t)b * p.len + t) * p.heads + h] = step_at(t) * expf(run);
    }
    carry = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(run), WAVE - 1));
  }
}


}  // namespace
}  // namespace ssm

extern "C" int ssm_ssd_bwd_gate(const ssm_ssd_bwd_gate_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_gate: args is NULL");
  SSM_REQUIRE(a->dout && a->x && a->ypre && a->dy && a->s2 && a->dyx, SSM_ERR_NULL_POINTER,
              "ssm_ssd_bwd_gate: dout, x, ypre, dy, s2 and dyx are required");
  SSM_REQUIRE((a->z != nullptr) == (a->dz != nullptr), SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_gate: dz must be given exactly when z is");
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->headdim > 0, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_bwd_gate: batch, seqlen, heads and headdim must be positive");
  ElemParams p{};
  SSM_REQUIRE(row_lanes(a->headdim, p.lg), SSM_ERR_BAD_SHAPE,
              "ssm_ssd_bwd_gate: headdim=%d must be 4 * 2^k, at most 256", a->headdim);
  SSM_REQUIRE(valid_dtype(a->io_dtype) && (a->dy_dtype == SSM_F32 || a->dy_dtype == SSM_BF16), SSM_ERR_BAD_DTYPE,
              "ssm_ssd_bwd_gate: io_dtype=%d dy_dtype=%d (dy is float32 or bfloat16)", a->io_dtype, a->dy_dtype);
  SSM_REQUIRE((size_t)a->batch * a->seqlen * a->heads < ((size_t)1 << 31), SSM_ERR_TOO_LARGE, "ssm_ssd_bwd_gate: too many rows");
  SSM_REQUIRE(aligned_to(a->dout, 8) && aligned_to(a->x, 8) && (!a->z || aligned_to(a->z, 8)) && aligned_to(a->ypre, 16) &&
                  aligned_to(a->dy, 8) && (!a->dy_rev || aligned_to(a->dy_rev, 8)) && (!a->dz || aligned_to(a->dz, 16)),
              SSM_ERR_ALIGNMENT, "ssm_ssd_bwd_gate: a pointer is not sufficiently aligned");
  p.dout = a->dout; p.z = a->z; p.x = a->x; p.ypre = a->ypre; p.Dk = a->Dskip; p.dy = a->dy; p.dy_rev = a->dy_rev;
  p.dz = a->dz; p.s2 = a->s2; p.dyx = a->dyx;
  SSM_REQUIRE((a->dy_w == nullptr || a->w_dy != nullptr) && (a->x_w == nullptr || a->w_x != nullptr), SSM_ERR_NULL_POINTER,
              "ssm_ssd_bwd_gate: dy_w needs w_dy and x_w needs w_x");
  SSM_REQUIRE((!a->dy_w || aligned_to(a->dy_w, 8)) && (!a->x_w || aligned_to(a->x_w, 8)), SSM_ERR_ALIGNMENT,
              "ssm_ssd_bwd_gate: dy_w and x_w must be 8-byte aligned");
  p.w_dy = a->w_dy; p.w_x = a->w_x; p.dy_w = a->dy_w; p.x_w = a->x_w;
  p.grads_io = a->dz_in_io_dtype ? 1 : 0;
  p.batch = a->batch; p.len = a->seqlen; p.heads = a->heads; p.hdim = a->headdim; p.d_per_p = a->d_per_p ? 1 : 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  const dim3 grid(elem_grid(p)), block(EB_THREADS);
  const bool of = a->dy_dtype == SSM_F32;
  switch (a->io_dtype) {
    case SSM_F32:
      if (of) hipLaunchKernelGGL((ssd_bwd_gate_kernel<float, float>), grid, block, 0, s, p);
      else hipLaunchKernelGGL((ssd_bwd_gate_kernel<float, bf16_t>), grid, block, 0, s, p);
      break;
    case SSM_BF16:
      if (of) hipLaunchKernelGGL((ssd_bwd_gate_kernel<bf16_t, float>), grid, block, 0, s, p);
      else hipLaunchKernelGGL((ssd_bwd_gate_kernel<bf16_t, bf16_t>), grid, block, 0, s, p);
      break;
    default:
      if (of) hipLaunchKernelGGL((ssd_bwd_gate_kernel<f16_t, float>), grid, block, 0, s, p);
      else hipLaunchKernelGGL((ssd_bwd_gate_kernel<f16_t, bf16_t>), grid, block, 0, s, p);
  }
  SSM_CHECK_LAUNCH("ssm_ssd_bwd_gate");
  return SSM_OK;
}

extern "C" int ssm_ssd_bwd_dx(const ssm_ssd_bwd_dx_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_dx: args is NULL");
  SSM_REQUIRE(a->dout && a->x && a->u_rev && a->dt && a->dx && a->xu && a->s1, SSM_ERR_NULL_POINTER,
              "ssm_ssd_bwd_dx: dout, x, u_rev, dt, dx, xu and s1 are required");
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->headdim > 0, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_bwd_dx: batch, seqlen, heads and headdim must be positive");
  ElemParams p{};
  SSM_REQUIRE(row_lanes(a->headdim, p.lg), SSM_ERR_BAD_SHAPE, "ssm_ssd_bwd_dx: headdim=%d must be 4 * 2^k, at most 256",
              a->headdim);
  SSM_REQUIRE(valid_dtype(a->io_dtype), SSM_ERR_BAD_DTYPE, "ssm_ssd_bwd_dx: io_dtype=%d", a->io_dtype);
  SSM_REQUIRE((size_t)a->batch * a->seqlen * a->heads < ((size_t)1 << 31), SSM_ERR_TOO_LARGE, "ssm_ssd_bwd_dx: too many rows");
  SSM_REQUIRE(aligned_to(a->dout, 8) && aligned_to(a->x, 8) && (!a->z || aligned_to(a->z, 8)) && aligned_to(a->u_rev, 16) &&
                  aligned_to(a->dx, 16),
              SSM_ERR_ALIGNMENT, "ssm_ssd_bwd_dx: a pointer is not sufficiently aligned");
  p.dout = a->dout; p.z = a->z; p.x = a->x; p.u_rev = a->u_rev; p.dt = a->dt; p.Dk = a->Dskip;
  p.dx = a->dx; p.xu = a->xu; p.s1 = a->s1;
  p.batch = a->batch; p.len = a->seqlen; p.heads = a->heads; p.hdim = a->headdim; p.d_per_p = a->d_per_p ? 1 : 0;
  p.round_bf16 = a->round_bf16 ? 1 : 0;
  p.grads_io = a->dx_in_io_dtype ? 1 : 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  const dim3 grid(elem_grid(p)), block(EB_THREADS);
  switch (a->io_dtype) {
    case SSM_F32: hipLaunchKernelGGL(ssd_bwd_dx_kernel<float>, grid, block, 0, s, p); break;
    case SSM_BF16: hipLaunchKernelGGL(ssd_bwd_dx_kernel<bf16_t>, grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL(ssd_bwd_dx_kernel<f16_t>, grid, block, 0, s, p);
  }
  SSM_CHECK_LAUNCH("ssm_ssd_bwd_dx");
  return SSM_OK;
}

extern "C" int ssm_ssd_bwd_db(const ssm_ssd_bwd_db_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_db: args is NULL");
  SSM_REQUIRE(a->v_rev && a->dt && a->dB, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_db: v_rev, dt and dB are required");
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->groups > 0 && a->nstate > 0 && a->heads % a->groups == 0,
              SSM_ERR_BAD_SHAPE, "ssm_ssd_bwd_db: sizes must be positive and groups must divide heads");
  SSM_REQUIRE(a->nstate % 4 == 0, SSM_ERR_BAD_SHAPE, "ssm_ssd_bwd_db: nstate=%d must be a multiple of 4", a->nstate);
  SSM_REQUIRE(aligned_to(a->v_rev, 16) && aligned_to(a->dB, 16), SSM_ERR_ALIGNMENT, "ssm_ssd_bwd_db: v_rev and dB must be 16-byte aligned");
  DbParams p{};
  p.v_rev = a->v_rev; p.dt = a->dt; p.dB = a->dB;
  p.batch = a->batch; p.len = a->seqlen; p.heads = a->heads; p.groups = a->groups; p.nstate = a->nstate;
  const size_t total = (size_t)p.batch * p.len * p.groups * (p.nstate / 4);
  SSM_REQUIRE(total < ((size_t)1 << 40), SSM_ERR_TOO_LARGE, "ssm_ssd_bwd_db: tensor too large");
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  hipLaunchKernelGGL(ssd_bwd_db_kernel, dim3((unsigned)((total + EB_THREADS - 1) / EB_THREADS)), dim3(EB_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_bwd_db");
  return SSM_OK;
}

extern "C" int ssm_ssd_bwd_states(const ssm_ssd_bwd_states_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_states: args is NULL");
  SSM_REQUIRE(a->entering_fwd && a->entering_rev && a->fwd_bf16 && a->rev_bf16, SSM_ERR_NULL_POINTER,
              "ssm_ssd_bwd_states: the two state tensors and their bfloat16 copies are required");
  SSM_REQUIRE(a->batch > 0 && a->nchunks > 0 && a->heads > 0 && a->dim > 0 && a->dim % 4 == 0, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_bwd_states: sizes must be positive and dim=%d a multiple of 4", a->dim);
  SSM_REQUIRE(a->anchor || a->nchunks == 1, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_states: anchor is required with more than one chunk");
  SSM_REQUIRE(aligned_to(a->entering_fwd, 16) && aligned_to(a->entering_rev, 16) && aligned_to(a->fwd_bf16, 8) &&
                  aligned_to(a->rev_bf16, 8),
              SSM_ERR_ALIGNMENT, "ssm_ssd_bwd_states: state tensors must be 16-byte aligned, their copies 8-byte");
  const size_t grid = (size_t)a->batch * a->nchunks * a->heads;
  SSM_REQUIRE(grid < ((size_t)1 << 31), SSM_ERR_TOO_LARGE, "ssm_ssd_bwd_states: too many (batch, chunk, head) triples");
  StatesParams p{};
  p.ent_f = a->entering_fwd; p.ent_r = a->entering_rev;
  p.f16 = reinterpret_cast<bf16_t *>(a->fwd_bf16); p.r16 = reinterpret_cast<bf16_t *>(a->rev_bf16);
  p.anchor = a->anchor;
  p.batch = a->batch; p.nchunks = a->nchunks; p.heads = a->heads; p.dim = a->dim;
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  hipLaunchKernelGGL(ssd_bwd_states_kernel, dim3((unsigned)grid), dim3(EB_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_bwd_states");
  return SSM_OK;
}

extern "C" int ssm_ssd_scale_rows(const ssm_ssd_scale_rows_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_ssd_scale_rows: args is NULL");
  SSM_REQUIRE(a->x && a->w && a->out, SSM_ERR_NULL_POINTER, "ssm_ssd_scale_rows: x, w and out are required");
  SSM_REQUIRE(a->rows > 0 && a->cols > 0 && a->cols % 4 == 0, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_scale_rows: rows must be positive and cols=%d a positive multiple of 4", a->cols);
  SSM_REQUIRE(valid_dtype(a->x_dtype) && (a->out_dtype == SSM_F32 || a->out_dtype == SSM_BF16), SSM_ERR_BAD_DTYPE,
              "ssm_ssd_scale_rows: x_dtype=%d, out_dtype=%d (float32 or bfloat16)", a->x_dtype, a->out_dtype);
  SSM_REQUIRE(aligned_to(a->x, 4 * dtype_size(a->x_dtype)) && aligned_to(a->out, 4 * dtype_size(a->out_dtype)),
              SSM_ERR_ALIGNMENT, "ssm_ssd_scale_rows: x and out must be aligned to four elements");
  ScaleParams p{};
  p.x = a->x; p.w = a->w; p.out = a->out; p.rows = (size_t)a->rows; p.cols = a->cols;
  const size_t quads = p.rows * (size_t)(p.cols / 4);
  SSM_REQUIRE(quads < ((size_t)1 << 39), SSM_ERR_TOO_LARGE, "ssm_ssd_scale_rows: tensor too large");
  const dim3 grid((unsigned)((quads + EB_THREADS - 1) / EB_THREADS)), block(EB_THREADS);
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
#define SSM_SCALE(IO)                                                                                          \
  {                                                                                                            \
    if (a->out_dtype == SSM_F32) hipLaunchKernelGGL((ssd_scale_rows_kernel<IO, float>), grid, block, 0, s, p);  \
    else hipLaunchKernelGGL((ssd_scale_rows_kernel<IO, bf16_t>), grid, block, 0, s, p);                         \
  }
  if (a->x_dtype == SSM_F32) SSM_SCALE(float) else if (a->x_dtype == SSM_BF16) SSM_SCALE(bf16_t) else SSM_SCALE(f16_t)
#undef SSM_SCALE
  SSM_CHECK_LAUNCH("ssm_ssd_scale_rows");
  return SSM_OK;
}

extern "C" int ssm_ssd_bwd_dt(const ssm_ssd_bwd_dt_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_dt: args is NULL");
  SSM_REQUIRE(a->s1 && a->s2 && a->xu && a->dt && a->dt_raw && a->A && a->ddt && a->dA_part && a->dbias_part,
              SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_dt: s1, s2, xu, dt, dt_raw, A, ddt, dA_part and dbias_part are required");
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->chunk > 0 && a->seqlen % a->chunk == 0, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_bwd_dt: sizes must be positive and chunk=%d must divide seqlen=%d", a->chunk, a->seqlen);
  SSM_REQUIRE(a->anchor || a->seqlen == a->chunk, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_dt: anchor is required with more than one chunk");
  SSM_REQUIRE(valid_dtype(a->dt_dtype), SSM_ERR_BAD_DTYPE, "ssm_ssd_bwd_dt: dt_dtype=%d", a->dt_dtype);
  DtParams p{};
  p.s1 = a->s1; p.s2 = a->s2; p.xu = a->xu; p.dte = a->dt; p.A = a->A; p.bias = a->dt_bias; p.W0 = a->q0; p.anchor = a->anchor;
  p.dt_raw = a->dt_raw; p.first = a->first_step; p.ddt = a->ddt; p.dA_part = a->dA_part; p.db_part = a->dbias_part;
  p.batch = a->batch; p.len = a->seqlen; p.heads = a->heads; p.chunk = a->chunk; p.nchunks = a->seqlen / a->chunk;
  p.dt_dtype = a->dt_dtype; p.softplus = a->dt_softplus ? 1 : 0; p.lo = a->dt_min; p.hi = a->dt_max;
  const size_t total = (size_t)p.batch * p.nchunks * ((p.heads + DT_HEADS - 1) / DT_HEADS);
  SSM_REQUIRE(total < ((size_t)1 << 31), SSM_ERR_TOO_LARGE, "ssm_ssd_bwd_dt: too many (batch, chunk, head) triples");
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  hipLaunchKernelGGL(ssd_bwd_dt_kernel, dim3((unsigned)total), dim3(EB_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_bwd_dt");
  return SSM_OK;
}

extern "C" int ssm_ssd_bwd_prep(const ssm_ssd_bwd_prep_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_prep: args is NULL");
  SSM_REQUIRE(a->dt && a->A && a->dA_cumsum && a->dt_out && a->dA_cumsum_rev && a->dt_rows && a->w_dy && a->w_x,
              SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_prep: dt, A and the six outputs are required");
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->chunk > 0 && a->seqlen % a->chunk == 0, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_bwd_prep: sizes must be positive and chunk=%d must divide seqlen=%d", a->chunk, a->seqlen);
  SSM_REQUIRE(valid_dtype(a->dt_dtype), SSM_ERR_BAD_DTYPE, "ssm_ssd_bwd_prep: dt_dtype=%d", a->dt_dtype);
  PrepParams p{};
  p.dt = a->dt; p.A = a->A; p.bias = a->dt_bias; p.dA_cs = a->dA_cumsum; p.dt_c = a->dt_out; p.dA_rev = a->dA_cumsum_rev;
  p.dte = a->dt_rows; p.w_dy = a->w_dy; p.w_x = a->w_x;
  p.batch = a->batch; p.len = a->seqlen; p.heads = a->heads; p.chunk = a->chunk; p.nchunks = a->seqlen / a->chunk;
  p.dt_dtype = a->dt_dtype; p.softplus = a->dt_softplus ? 1 : 0; p.lo = a->dt_min; p.hi = a->dt_max;
  const size_t waves = (size_t)p.batch * p.heads * p.nchunks;
  SSM_REQUIRE(waves < ((size_t)1 << 31) / WAVE, SSM_ERR_TOO_LARGE, "ssm_ssd_bwd_prep: too many (batch, head, chunk) triples");
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  hipLaunchKernelGGL(ssd_bwd_prep_kernel, dim3((unsigned)((waves * WAVE + EB_THREADS - 1) / EB_THREADS)), dim3(EB_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_bwd_prep");
  return SSM_OK;
}
