// State-space-duality (Mamba-2) operator family: C-ABI entry points and the
// shape-generic kernels.
//
//   chunk_cumsum   dt' = clamp(softplus(dt + bias)); dA_cs[c,l] = sum_{j<=l} dt'_j A_h
//   bmm_chunk      CB[c,l,s] = <a_l, b_s>                       (C B^T per chunk and group)
//   chunk_state    S_c[p,n]  = sum_l B_l[n] exp(dA_cs[last]-dA_cs[l]) dt'_l x_l[p]
//   state_passing  H_{c+1}   = exp(dA_cs[c,last]) H_c + S_c      (H_0 = initial state)
//   chunk_scan     y_l = exp(dA_cs[l]) C_l.H_c + sum_{s<=l} CB[l,s] exp(dA_cs[l]-dA_cs[s]) dt'_s x_s
//                        + D x_l ;  y_l *= silu(z_l)
//
// The three contractions have bf16 MFMA implementations (ssd_mfma.hip) that are
// taken whenever the shape allows; the kernels here accept every shape and
// dtype, accumulate in fp32 and serve as their fallback.
#include "ssd_common.hpp"

namespace ssm {

constexpr int SSD_THREADS = 256;

#ifdef SSM_TEST_HOOKS
static thread_local int g_mfma_launches = 0;   // bit0 bmm_chunk, bit1 chunk_state, bit2 chunk_scan, bit3 one-pass forward
void note_mfma_launch(int bits) { g_mfma_launches |= bits; }
#else
void note_mfma_launch(int) {}
#endif

static unsigned grid_for(size_t n) {
  const size_t g = (n + SSD_THREADS - 1) / SSD_THREADS;
  return (unsigned)(g < 1 ? 1 : g);
}

// One wavefront per (b, h, c): 64 steps at a time, running sum by a DPP scan across the lanes plus the
// carry of the blocks before; reads and writes are contiguous runs.
__global__ __launch_bounds__(SSD_THREADS) void ssd_cumsum_kernel(const SsdCumsumParams p) {
  const SsdDims &d = p.d;
  const size_t gw = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int lane = lane_id();
  const size_t total = (size_t)d.batch * d.heads * d.nchunks;
  if (gw >= total) return;                          // whole wavefronts
  const int c = (int)(gw % d.nchunks);
  const int h = (int)((gw / d.nchunks) % d.heads);
  const int b = (int)(gw / ((size_t)d.nchunks * d.heads));
  const float A = p.A[h];
  const float bias = p.bias ? p.bias[h] : 0.0f;
  float carry = 0.0f;
  const size_t out = (((size_t)b * d.heads + h) * d.nchunks + c) * d.chunk;
  for (int l0 = 0; l0 < d.chunk; l0 += WAVE) {
    const int l = l0 + lane;
    const int t = c * d.chunk + l;
    float v = 0.0f;
    if (l < d.chunk && t < d.len) {
      v = load_as_f32(p.dt, p.dt_dtype, ((size_t)b * d.len + t) * d.heads + h) + bias;
      if (p.softplus) v = softplus_f32(v);
      v = fminf(fmaxf(v, p.dt_min), p.dt_max);
    }
    const float run = carry + wave_inclusive_sum(v * A);
    if (l < d.chunk) {
      p.dt_out[out + l] = v;
      p.dA_cs[out + l] = run;
    }
    carry = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(run), WAVE - 1));
  }
}

// One thread per output element.
__global__ __launch_bounds__(SSD_THREADS) void ssd_bmm_kernel(const SsdBmmParams p) {
  const int Q = p.chunk;
  const size_t total = (size_t)p.batch * p.nchunks * p.groups * Q * Q;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int s = (int)(gid % Q), l = (int)((gid / Q) % Q);
  const int g = (int)((gid / ((size_t)Q * Q)) % p.groups);
  const int c = (int)((gid / ((size_t)Q * Q * p.groups)) % p.nchunks);
  const int b = (int)(gid / ((size_t)Q * Q * p.groups * p.nchunks));
  const int tl = c * Q + l, ts = c * Q + s;
  float acc = 0.0f;
  if (tl < p.len && ts < p.len && !(p.causal && s > l)) {
    const size_t ra = (((size_t)b * p.len + tl) * p.groups + g) * p.kdim;
    const size_t rb = (((size_t)b * p.len + ts) * p.groups + g) * p.kdim;
    for (int k = 0; k < p.kdim; ++k)
      acc = __builtin_fmaf(load_as_f32(p.a, p.in_dtype, ra + k), load_as_f32(p.b, p.in_dtype, rb + k), acc);
    if (p.seq_idx && p.seq_idx[(size_t)b * p.len + tl] != p.seq_idx[(size_t)b * p.len + ts]) acc = 0.0f;
  }
  store_any(p.out, p.out_dtype, gid, acc);
}

// One thread per (b, c, h, p, n).
__global__ __launch_bounds__(SSD_THREADS) void ssd_chunk_state_kernel(const SsdStateParams p) {
  const SsdDims &d = p.d;
  const size_t total = (size_t)d.batch * d.nchunks * d.heads * d.hdim * d.nstate;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int n = (int)(gid % d.nstate);
  const int pp = (int)((gid / d.nstate) % d.hdim);
  const int h = (int)((gid / ((size_t)d.nstate * d.hdim)) % d.heads);
  const int c = (int)((gid / ((size_t)d.nstate * d.hdim * d.heads)) % d.nchunks);
  const int b = (int)(gid / ((size_t)d.nstate * d.hdim * d.heads * d.nchunks));
  const int g = h / (d.heads / d.groups);
  const size_t cs = (((size_t)b * d.heads + h) * d.nchunks + c) * d.chunk;
  const float last = p.dA_cs[cs + d.chunk - 1];
  const int *sid = p.seq_idx ? p.seq_idx + (size_t)b * d.len : nullptr;
  const int sid_last = sid ? sid[min((c + 1) * d.chunk, d.len) - 1] : 0;
  float acc = 0.0f;
  for (int l = 0; l < d.chunk; ++l) {
    const int t = c * d.chunk + l;
    if (t >= d.len) break;
    if (sid && sid[t] != sid_last) continue;
    const float w = decay_exp(last - p.dA_cs[cs + l]) * p.dt[cs + l];
    const float bv = load_as_f32(p.Bm, p.b_dtype, (((size_t)b * d.len + t) * d.groups + g) * d.nstate + n);
    const float xv = load_as_f32(p.x, p.x_dtype, (((size_t)b * d.len + t) * d.heads + h) * d.hdim + pp);
    acc = __builtin_fmaf(bv * w, xv, acc);
  }
  store_any(p.states, p.states_dtype, gid, acc);
}

// One thread per (b, h, i): sequential over chunks.
__global__ __launch_bounds__(SSD_THREADS) void ssd_state_passing_kernel(const SsdPassParams p) {
  const size_t total = (size_t)p.batch * p.heads * p.dim;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int i = (int)(gid % p.dim);
  const int h = (int)((gid / p.dim) % p.heads);
  const int b = (int)(gid / ((size_t)p.dim * p.heads));
  float cur = p.init ? p.init[gid] : 0.0f;
  int sid_prev = 0;
  for (int c = 0; c < p.nchunks; ++c) {
    const size_t at = (((size_t)b * p.nchunks + c) * p.heads + h) * p.dim + i;
    const float contrib = load_as_f32(p.states, p.states_dtype, at);
    store_any(p.out, p.states_dtype, at, cur);
    float scale = exp2_hw(p.dA_last[((size_t)b * p.heads + h) * p.nchunks + c] * LOG2E);
    if (p.seq_idx) {
      const int sid_new = p.seq_idx[(size_t)b * p.len + min((c + 1) * p.chunk, p.len) - 1];
      if (sid_new != sid_prev) scale = 0.0f;
      sid_prev = sid_new;
    }
    cur = __builtin_fmaf(scale, cur, contrib);
  }
  p.final_states[gid] = cur;
}

// The same with float32 states in 16-byte pieces: four neighbouring elements per thread, and the reads of eight
// chunks requested before the first is used (they do not depend on the running state).
__global__ __launch_bounds__(SSD_THREADS) void ssd_state_passing_f32x4_kernel(const SsdPassParams p) {
  constexpr int GROUP = 8;
  const size_t quads = (size_t)p.batch * p.heads * (p.dim / 4);
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= quads) return;
  const int i = (int)(gid % (p.dim / 4)) * 4;
  const int h = (int)((gid / (p.dim / 4)) % p.heads);
  const int b = (int)(gid / ((size_t)(p.dim / 4) * p.heads));
  const size_t el = ((size_t)b * p.heads + h) * p.dim + i;
  float4 cur = p.init ? *reinterpret_cast<const float4 *>(p.init + el) : make_float4(0.f, 0.f, 0.f, 0.f);
  const float *src = reinterpret_cast<const float *>(p.states);
  float *dst = reinterpret_cast<float *>(p.out);
  const size_t cstride = (size_t)p.heads * p.dim;
  const size_t at0 = ((size_t)b * p.nchunks * p.heads + h) * p.dim + i;
  const float *dal = p.dA_last + ((size_t)b * p.heads + h) * p.nchunks;
  int sid_prev = 0;
  for (int c0 = 0; c0 < p.nchunks; c0 += GROUP) {
    float4 contrib[GROUP];
    float scale[GROUP];
#pragma unroll
    for (int k = 0; k < GROUP; ++k) {
      const int c = min(c0 + k, p.nchunks - 1);
      contrib[k] = *reinterpret_cast<const float4 *>(src + at0 + (size_t)c * cstride);
      scale[k] = exp2_hw(dal[c] * LOG2E);
      if (p.seq_idx) {
        const int sid_new = p.seq_idx[(size_t)b * p.len + min((c + 1) * p.chunk, p.len) - 1];
        if (sid_new != sid_prev) scale[k] = 0.0f;
        sid_prev = sid_new;
      }
    }
#pragma unroll
    for (int k = 0; k < GROUP; ++k) {
      if (c0 + k < p.nchunks) {
        *reinterpret_cast<float4 *>(dst + at0 + (size_t)(c0 + k) * cstride) = cur;
        cur.x = __builtin_fmaf(scale[k], cur.x, contrib[k].x);
        cur.y = __builtin_fmaf(scale[k], cur.y, contrib[k].y);
        cur.z = __builtin_fmaf(scale[k], cur.z, contrib[k].z);
        cur.w = __builtin_fmaf(scale[k], cur.w, contrib[k].w);
      }
    }
  }
  *reinterpret_cast<float4 *>(p.final_states + el) = cur;
}

// One thread per (b, t, h, p).
__global__ __launch_bounds__(SSD_THREADS) void ssd_chunk_scan_kernel(const SsdScanParams p) {
  const SsdDims &d = p.d;
  const size_t total = (size_t)d.batch * d.len * d.heads * d.hdim;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int pp = (int)(gid % d.hdim);
  const int h = (int)((gid / d.hdim) % d.heads);
  const int t = (int)((gid / ((size_t)d.hdim * d.heads)) % d.len);
  const int b = (int)(gid / ((size_t)d.hdim * d.heads * d.len));
  const int c = t / d.chunk, l = t % d.chunk;
  const int g = h / (d.heads / d.groups);
  const size_t cs = (((size_t)b * d.heads + h) * d.nchunks + c) * d.chunk;
  const float dal = p.dA_cs[cs + l];
  // carried-in state
  float acc = 0.0f;
  const size_t crow = (((size_t)b * d.len + t) * d.groups + g) * d.nstate;
  const size_t srow = ((((size_t)b * d.nchunks + c) * d.heads + h) * d.hdim + pp) * d.nstate;
  for (int n = 0; n < d.nstate; ++n)
    acc = __builtin_fmaf(load_as_f32(p.Cm, p.c_dtype, crow + n), load_as_f32(p.prev, p.states_dtype, srow + n), acc);
  acc *= exp2_hw(dal * LOG2E);
  if (p.seq_idx) {
    const int *sid = p.seq_idx + (size_t)b * d.len;
    const int sid_prev = c > 0 ? sid[c * d.chunk - 1] : 0;
    if (sid[t] != sid_prev) acc = 0.0f;
  }
  // within the chunk
  const size_t cbrow = ((((size_t)b * d.nchunks + c) * d.groups + g) * d.chunk + l) * d.chunk;
  for (int s = 0; s <= l; ++s) {
    const float m = load_as_f32(p.CB, p.cb_dtype, cbrow + s) * decay_exp(dal - p.dA_cs[cs + s]) * p.dt[cs + s];
    const float xv = load_as_f32(p.x, p.x_dtype, (((size_t)b * d.len + c * d.chunk + s) * d.heads + h) * d.hdim + pp);
    acc = __builtin_fmaf(m, xv, acc);
  }
  const float xl = load_as_f32(p.x, p.x_dtype, gid);
  if (p.Dk) acc = __builtin_fmaf(p.Dk[p.d_per_p ? (size_t)h * d.hdim + pp : (size_t)h], xl, acc);
  if (p.z) acc *= silu_f32(load_as_f32(p.z, p.z_dtype, gid));
  store_any(p.y, p.y_dtype, gid, acc);
}

struct SsdVarlenParams {
  const void *Bm, *x, *chunk_states;
  const float *dt, *dA_cs;
  const int *cu_seqlens;
  float *states;
  SsdDims d;
  int nseq;
  int x_dtype, b_dtype, states_dtype;
};

// One thread per (sequence, h, p, n): the state at the sequence's last step is the state entering the
// chunk of that step, decayed, if the sequence began before that chunk (or at step 0), plus the steps of
// the chunk that belong to the sequence.
__global__ __launch_bounds__(SSD_THREADS) void ssd_chunk_state_varlen_kernel(const SsdVarlenParams p) {
  const SsdDims &d = p.d;
  const size_t total = (size_t)p.nseq * d.heads * d.hdim * d.nstate;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int n = (int)(gid % d.nstate);
  const int pp = (int)((gid / d.nstate) % d.hdim);
  const int h = (int)((gid / ((size_t)d.nstate * d.hdim)) % d.heads);
  const int q = (int)(gid / ((size_t)d.nstate * d.hdim * d.heads));
  const int g = h / (d.heads / d.groups);
  const int start = p.cu_seqlens[q], end = min(p.cu_seqlens[q + 1], d.len);
  float acc = 0.0f;
  if (end > start && start >= 0) {
    const int c = (end - 1) / d.chunk;
    const size_t cs = ((size_t)h * d.nchunks + c) * d.chunk;
    const float last = p.dA_cs[cs + (end - 1 - c * d.chunk)];
    if (start < c * d.chunk || start == 0) {   // start == 0: the row's initial state belongs to the first sequence
      const size_t at = (((size_t)c * d.heads + h) * d.hdim + pp) * d.nstate + n;
      acc = load_as_f32(p.chunk_states, p.states_dtype, at) * exp2_hw(last * LOG2E);
    }
    for (int t = max(start, c * d.chunk); t < end; ++t) {
      const int l = t - c * d.chunk;
      const float w = decay_exp(last - p.dA_cs[cs + l]) * p.dt[cs + l];
      const float bv = load_as_f32(p.Bm, p.b_dtype, ((size_t)t * d.groups + g) * d.nstate + n);
      const float xv = load_as_f32(p.x, p.x_dtype, ((size_t)t * d.heads + h) * d.hdim + pp);
      acc = __builtin_fmaf(bv * w, xv, acc);
    }
  }
  p.states[gid] = acc;
}

static int dims_check(const char *who, const ssm_ssd_dims &s, SsdDims &d) {
  SSM_REQUIRE(s.batch > 0 && s.seqlen > 0 && s.heads > 0 && s.headdim > 0 && s.groups > 0 && s.nstate > 0 &&
                  s.chunk > 0,
              SSM_ERR_BAD_SHAPE, "%s: all of batch, seqlen, heads, headdim, groups, nstate, chunk must be positive", who);
  SSM_REQUIRE(s.heads % s.groups == 0, SSM_ERR_BAD_SHAPE, "%s: groups=%d must divide heads=%d", who, s.groups, s.heads);
  d.batch = s.batch; d.len = s.seqlen; d.heads = s.heads; d.hdim = s.headdim; d.groups = s.groups;
  d.nstate = s.nstate; d.chunk = s.chunk; d.nchunks = (s.seqlen + s.chunk - 1) / s.chunk;
  SSM_REQUIRE((size_t)d.batch * d.nchunks * d.heads * d.hdim * d.nstate < ((size_t)1 << 40) &&
                  (size_t)d.batch * d.len * d.heads * d.hdim < ((size_t)1 << 40),
              SSM_ERR_TOO_LARGE, "%s: tensor too large", who);
  return SSM_OK;
}

}  // namespace ssm

#ifdef SSM_TEST_HOOKS
extern "C" int ssm_ssd_mfma_launches(void) {   // include/ssm_amd_testing.h
  const int v = ssm::g_mfma_launches;
  ssm::g_mfma_launches = 0;
  return v;
}
#endif

extern "C" int ssm_ssd_chunk_cumsum(const ssm_ssd_cumsum_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a && a->dt && a->A && a->dA_cumsum && a->dt_out, SSM_ERR_NULL_POINTER,
              "ssm_ssd_chunk_cumsum: dt, A, dA_cumsum and dt_out are required");
  SsdCumsumParams p{};
  ssm_ssd_dims dd = a->dims;
  if (dd.headdim <= 0) dd.headdim = 1;
  if (dd.groups <= 0) dd.groups = 1;
  if (dd.nstate <= 0) dd.nstate = 1;
  int rc = dims_check("ssm_ssd_chunk_cumsum", dd, p.d);
  if (rc != SSM_OK) return rc;
  SSM_REQUIRE(valid_dtype(a->dt_dtype), SSM_ERR_BAD_DTYPE, "ssm_ssd_chunk_cumsum: dt_dtype=%d", a->dt_dtype);
  p.dt = a->dt; p.A = a->A; p.bias = a->dt_bias; p.dA_cs = a->dA_cumsum; p.dt_out = a->dt_out;
  p.dt_dtype = a->dt_dtype; p.softplus = a->dt_softplus ? 1 : 0; p.dt_min = a->dt_min; p.dt_max = a->dt_max;
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  hipLaunchKernelGGL(ssd_cumsum_kernel, dim3(grid_for((size_t)p.d.batch * p.d.heads * p.d.nchunks * WAVE)),
                     dim3(SSD_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_chunk_cumsum");
  return SSM_OK;
}

extern "C" int ssm_ssd_bmm_chunk(const ssm_ssd_bmm_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a && a->a && a->b && a->out, SSM_ERR_NULL_POINTER, "ssm_ssd_bmm_chunk: a, b and out are required");
  SSM_CHECK_RESERVED("ssm_ssd_bmm_chunk", a);
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->groups > 0 && a->kdim > 0 && a->chunk > 0, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_bmm_chunk: batch, seqlen, groups, kdim and chunk must be positive");
  SSM_REQUIRE(valid_dtype(a->in_dtype) && valid_dtype(a->out_dtype), SSM_ERR_BAD_DTYPE,
              "ssm_ssd_bmm_chunk: in_dtype=%d out_dtype=%d", a->in_dtype, a->out_dtype);
  SsdBmmParams p{};
  p.a = a->a; p.b = a->b; p.seq_idx = a->seq_idx; p.out = a->out;
  p.batch = a->batch; p.len = a->seqlen; p.groups = a->groups; p.kdim = a->kdim; p.chunk = a->chunk;
  p.nchunks = (a->seqlen + a->chunk - 1) / a->chunk;
  p.in_dtype = a->in_dtype; p.out_dtype = a->out_dtype; p.causal = a->causal ? 1 : 0;
  const size_t total = (size_t)p.batch * p.nchunks * p.groups * p.chunk * p.chunk;
  SSM_REQUIRE(total < ((size_t)1 << 40), SSM_ERR_TOO_LARGE, "ssm_ssd_bmm_chunk: tensor too large");
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  if (!SSM_RESERVED(a) && ssd_bmm_mfma(p, s)) {
    note_mfma_launch(1);
    SSM_CHECK_LAUNCH("ssm_ssd_bmm_chunk(mfma)");
    return SSM_OK;
  }
  if (!SSM_RESERVED(a) && ssd_bmm_tiled(p, s)) {
    SSM_CHECK_LAUNCH("ssm_ssd_bmm_chunk(tiled)");
    return SSM_OK;
  }
  hipLaunchKernelGGL(ssd_bmm_kernel, dim3(grid_for(total)), dim3(SSD_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_bmm_chunk");
  return SSM_OK;
}

extern "C" size_t ssm_ssd_chunk_state_workspace_bytes(const ssm_ssd_dims *dims) {
  using namespace ssm;
  SsdDims d;
  if (!dims || dims_check("ssm_ssd_chunk_state_workspace_bytes", *dims, d) != SSM_OK) return 0;
  return ssd_chunk_state_scratch_bytes(d);
}

extern "C" int ssm_ssd_chunk_state(const ssm_ssd_chunk_state_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a && a->Bm && a->x && a->dt && a->dA_cumsum && a->states, SSM_ERR_NULL_POINTER,
              "ssm_ssd_chunk_state: Bm, x, dt, dA_cumsum and states are required");
  SSM_CHECK_RESERVED("ssm_ssd_chunk_state", a);
  SsdStateParams p{};
  int rc = dims_check("ssm_ssd_chunk_state", a->dims, p.d);
  if (rc != SSM_OK) return rc;
  SSM_REQUIRE(valid_dtype(a->x_dtype) && valid_dtype(a->b_dtype) && valid_dtype(a->states_dtype), SSM_ERR_BAD_DTYPE,
              "ssm_ssd_chunk_state: unsupported dtype");
  p.Bm = a->Bm; p.x = a->x; p.dt = a->dt; p.dA_cs = a->dA_cumsum; p.states = a->states;
  p.scratch = a->workspace; p.scratch_bytes = a->workspace_bytes;
  p.x_dtype = a->x_dtype; p.b_dtype = a->b_dtype; p.states_dtype = a->states_dtype;
  p.seq_idx = a->seq_idx;
  p.x_scale = a->x_row_scale;
  p.x_reversed = a->x_time_reversed ? 1 : 0;
  // (float16 is left out: the conversion that rounds the product does not keep float16 subnormals, which a tensor
  // written beforehand would hold)
  SSM_REQUIRE(a->x_row_scale == nullptr || a->x_dtype == SSM_BF16, SSM_ERR_BAD_DTYPE,
              "ssm_ssd_chunk_state: x_row_scale needs bfloat16 x (x_dtype=%d)", a->x_dtype);
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  if (!SSM_RESERVED(a) && ssd_chunk_state_mfma(p, s)) {
    note_mfma_launch(2);
    SSM_CHECK_LAUNCH("ssm_ssd_chunk_state(mfma)");
    return SSM_OK;
  }
  SSM_REQUIRE(!a->x_time_reversed, SSM_ERR_BAD_SHAPE, "ssm_ssd_chunk_state: x_time_reversed is taken by the matrix-core kernel only");
  SSM_REQUIRE(a->x_row_scale == nullptr, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_chunk_state: x_row_scale is taken by the matrix-core kernel only (bfloat16 x and B, whole "
              "chunks of a multiple of 32 up to 256 steps, nstate a multiple of 16, headdim 32 or 64, a workspace)");
  if (!SSM_RESERVED(a) && ssd_chunk_state_tiled(p, s)) {
    SSM_CHECK_LAUNCH("ssm_ssd_chunk_state(tiled)");
    return SSM_OK;
  }
  const size_t total = (size_t)p.d.batch * p.d.nchunks * p.d.heads * p.d.hdim * p.d.nstate;
  hipLaunchKernelGGL(ssd_chunk_state_kernel, dim3(grid_for(total)), dim3(SSD_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_chunk_state");
  return SSM_OK;
}

extern "C" int ssm_ssd_state_passing(const ssm_ssd_state_passing_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a && a->states && a->dA_chunk_last && a->states_out && a->final_states, SSM_ERR_NULL_POINTER,
              "ssm_ssd_state_passing: states, dA_chunk_last, states_out and final_states are required");
  SSM_REQUIRE(a->batch > 0 && a->nchunks > 0 && a->heads > 0 && a->dim > 0, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_state_passing: batch, nchunks, heads and dim must be positive");
  SSM_REQUIRE(valid_dtype(a->states_dtype), SSM_ERR_BAD_DTYPE, "ssm_ssd_state_passing: states_dtype=%d",
              a->states_dtype);
  SsdPassParams p{};
  p.states = a->states; p.dA_last = a->dA_chunk_last; p.init = a->initial_states; p.out = a->states_out;
  p.final_states = a->final_states;
  p.batch = a->batch; p.nchunks = a->nchunks; p.heads = a->heads; p.dim = a->dim; p.states_dtype = a->states_dtype;
  p.seq_idx = a->seq_idx; p.len = a->seqlen; p.chunk = a->chunk;
  if (a->seq_idx)
    SSM_REQUIRE(a->chunk > 0 && a->seqlen > 0 && (a->seqlen + a->chunk - 1) / a->chunk == a->nchunks, SSM_ERR_BAD_SHAPE,
                "ssm_ssd_state_passing: with seq_idx, seqlen=%d and chunk=%d must give nchunks=%d", a->seqlen, a->chunk,
                a->nchunks);
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  if (p.states_dtype == SSM_F32 && p.dim % 4 == 0 && aligned_to(p.states, 16) && aligned_to(p.out, 16) &&
      aligned_to(p.final_states, 16) && (!p.init || aligned_to(p.init, 16)))
    hipLaunchKernelGGL(ssd_state_passing_f32x4_kernel, dim3(grid_for((size_t)p.batch * p.heads * (p.dim / 4))),
                       dim3(SSD_THREADS), 0, s, p);
  else
    hipLaunchKernelGGL(ssd_state_passing_kernel, dim3(grid_for((size_t)p.batch * p.heads * p.dim)), dim3(SSD_THREADS),
                       0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_state_passing");
  return SSM_OK;
}

extern "C" int ssm_ssd_chunk_scan(const ssm_ssd_chunk_scan_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a && a->CB && a->Cm && a->x && a->dt && a->dA_cumsum && a->prev_states && (a->y || a->dx_out),
              SSM_ERR_NULL_POINTER, "ssm_ssd_chunk_scan: CB, Cm, x, dt, dA_cumsum, prev_states and y (or dx_out) are required");
  SSM_CHECK_RESERVED("ssm_ssd_chunk_scan", a);
  SsdScanParams p{};
  int rc = dims_check("ssm_ssd_chunk_scan", a->dims, p.d);
  if (rc != SSM_OK) return rc;
  SSM_REQUIRE(valid_dtype(a->x_dtype) && valid_dtype(a->c_dtype) && valid_dtype(a->cb_dtype) &&
                  valid_dtype(a->states_dtype) && (!a->z || valid_dtype(a->z_dtype)),
              SSM_ERR_BAD_DTYPE, "ssm_ssd_chunk_scan: unsupported dtype");
  p.CB = a->CB; p.Cm = a->Cm; p.x = a->x; p.z = a->z; p.prev = a->prev_states; p.dt = a->dt; p.dA_cs = a->dA_cumsum;
  p.Dk = a->Dskip; p.y = a->y;
  p.x_dtype = a->x_dtype; p.c_dtype = a->c_dtype; p.cb_dtype = a->cb_dtype; p.states_dtype = a->states_dtype;
  p.z_dtype = a->z_dtype; p.d_per_p = a->d_per_p ? 1 : 0;
  p.seq_idx = a->seq_idx;
  p.y_dtype = a->y_f32 ? SSM_F32 : a->x_dtype;
  p.x_scale = a->x_row_scale;
  p.x_reversed = a->x_time_reversed ? 1 : 0;
  SSM_REQUIRE(a->x_row_scale == nullptr || a->x_dtype == SSM_BF16, SSM_ERR_BAD_DTYPE,
              "ssm_ssd_chunk_scan: x_row_scale needs bfloat16 x (x_dtype=%d)", a->x_dtype);
  if (a->dx_out) {
    SSM_REQUIRE(a->dx_x && a->dx_dt && a->dx_xu && a->dx_s1, SSM_ERR_NULL_POINTER,
                "ssm_ssd_chunk_scan: dx_out needs dx_x, dx_dt, dx_xu and dx_s1");
    SSM_REQUIRE(aligned_to(a->dx_x, 2) && aligned_to(a->dx_out, a->dx_out_f32 ? 4 : 2) && aligned_to(a->dx_dt, 4) &&
                    aligned_to(a->dx_xu, 4) && aligned_to(a->dx_s1, 4),
                SSM_ERR_ALIGNMENT, "ssm_ssd_chunk_scan: a dx_* pointer is not aligned to its element");
    p.dx.x = a->dx_x; p.dx.dt = a->dx_dt; p.dx.Dk = a->dx_Dskip; p.dx.dx = a->dx_out; p.dx.xu = a->dx_xu; p.dx.s1 = a->dx_s1;
    p.dx.d_per_p = a->dx_d_per_p ? 1 : 0; p.dx.dx_f32 = a->dx_out_f32 ? 1 : 0; p.dx.round_dtx = a->dx_round_dtx ? 1 : 0;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  if (!SSM_RESERVED(a) && ssd_chunk_scan_mfma(p, s)) {
    note_mfma_launch(4);
    SSM_CHECK_LAUNCH("ssm_ssd_chunk_scan(mfma)");
    return SSM_OK;
  }
  SSM_REQUIRE(!a->x_time_reversed, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_chunk_scan: x_time_reversed is taken by the matrix-core kernel only, and not together with Dskip");
  SSM_REQUIRE(a->dx_out == nullptr, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_chunk_scan: dx_out is written by the matrix-core kernel only (bfloat16 x, C and CB, float32 states, "
              "no z, Dskip or seq_idx, whole chunks of a multiple of 32 up to 256 steps, nstate a multiple of 16, headdim 32 or 64)");
  SSM_REQUIRE(a->x_row_scale == nullptr, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_chunk_scan: x_row_scale is taken by the matrix-core kernel only (bfloat16 x, C and CB, "
              "whole chunks of a multiple of 32 up to 256 steps, nstate a multiple of 16, headdim 32 or 64)");
  if (!SSM_RESERVED(a) && ssd_chunk_scan_tiled(p, s)) {
    SSM_CHECK_LAUNCH("ssm_ssd_chunk_scan(tiled)");
    return SSM_OK;
  }
  const size_t total = (size_t)p.d.batch * p.d.len * p.d.heads * p.d.hdim;
  hipLaunchKernelGGL(ssd_chunk_scan_kernel, dim3(grid_for(total)), dim3(SSD_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_chunk_scan");
  return SSM_OK;
}

extern "C" int ssm_ssd_chunk_state_varlen(const ssm_ssd_chunk_state_varlen_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a && a->Bm && a->x && a->dt && a->dA_cumsum && a->chunk_states && a->cu_seqlens && a->states,
              SSM_ERR_NULL_POINTER,
              "ssm_ssd_chunk_state_varlen: Bm, x, dt, dA_cumsum, chunk_states, cu_seqlens and states are required");
  SsdVarlenParams p{};
  int rc = dims_check("ssm_ssd_chunk_state_varlen", a->dims, p.d);
  if (rc != SSM_OK) return rc;
  SSM_REQUIRE(p.d.batch == 1, SSM_ERR_BAD_SHAPE, "ssm_ssd_chunk_state_varlen: packed sequences need batch=1 (got %d)",
              p.d.batch);
  SSM_REQUIRE(a->nseq > 0, SSM_ERR_BAD_SHAPE, "ssm_ssd_chunk_state_varlen: nseq=%d", a->nseq);
  SSM_REQUIRE(valid_dtype(a->x_dtype) && valid_dtype(a->b_dtype) && valid_dtype(a->states_dtype), SSM_ERR_BAD_DTYPE,
              "ssm_ssd_chunk_state_varlen: unsupported dtype");
  p.Bm = a->Bm; p.x = a->x; p.chunk_states = a->chunk_states; p.dt = a->dt; p.dA_cs = a->dA_cumsum;
  p.cu_seqlens = a->cu_seqlens; p.states = a->states; p.nseq = a->nseq;
  p.x_dtype = a->x_dtype; p.b_dtype = a->b_dtype; p.states_dtype = a->states_dtype;
  const size_t total = (size_t)p.nseq * p.d.heads * p.d.hdim * p.d.nstate;
  SSM_REQUIRE(total < ((size_t)1 << 40), SSM_ERR_TOO_LARGE, "ssm_ssd_chunk_state_varlen: tensor too large");
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  hipLaunchKernelGGL(ssd_chunk_state_varlen_kernel, dim3(grid_for(total)), dim3(SSD_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_chunk_state_varlen");
  return SSM_OK;
}
