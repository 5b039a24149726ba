// chunk_state and chunk_scan of the state-space-duality forward for every call the bf16 kernels do not
// take (float32 or float16 tensors, mixed dtypes, head and state sizes of any value, ragged ends):
// 64x64 output tiles per workgroup, operands staged through LDS as float32 with zero fill, products on
// the float32 matrix cores (v_mfma_f32_32x32x2_f32), so results keep float32 accuracy.
//
//   chunk_state:  states[p][n] = sum_l x[l][p] * (exp(cs_last - cs_l) dt_l) B[l][n]
//   chunk_scan:   y[l][p] = exp(cs_l) sum_n C[l][n] prev[p][n]
//                         + sum_{s<=l} CB[l][s] exp(cs_l - cs_s) dt_s x[s][p]  + D x[l][p],  times silu(z)
#include "ssd_common.hpp"

#include <type_traits>

namespace ssm {
namespace {

// Element reads while staging.  T = void: the element type is looked up at run time (calls that mix
// types); otherwise every streamed tensor of the call has type T.  Indices are clamped into the tensor
// and the value dropped afterwards where a tile hangs over an edge, so that no read sits behind a
// lane-dependent branch and a thread's reads of one slab are in flight together.
template <typename T>
__device__ __forceinline__ float tl_ld(const void *p, int dtype, size_t i) {
  if constexpr (std::is_void<T>::value) return load_as_f32(p, dtype, i);
  else return to_f32(reinterpret_cast<const T *>(p)[i]);
}

constexpr int TL_THREADS = 256;   // 4 waves, 2 x 2 blocks of 32 x 32
constexpr int TL_MN = 64;         // tile edge of the output
constexpr int TL_K = 32;          // depth of one staged slab
constexpr int TL_S = TL_MN + 1;   // row stride in LDS (odd: transposed writes spread over the banks)

struct Slabs {
  float a[TL_K][TL_S];            // a[k][m]
  float b[TL_K][TL_S];            // b[k][n]
};

// acc(32x32 block (wr, wc)) += a^T b over the slab.  Operand layout of the instruction: lane i supplies
// A[i % 32][i / 32] and B[i / 32][i % 32].
__device__ __forceinline__ void slab_mma(const Slabs &t, int wr, int wc, int lane, f32x16_t &acc) {
  const int half = lane >> 5, col = lane & 31;
#pragma unroll
  for (int kk = 0; kk < TL_K; kk += 2)
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(t.a[kk + half][wr * 32 + col], t.b[kk + half][wc * 32 + col], acc, 0, 0, 0);
}

// Slab element e = tid + 256 j of a source whose tile index m is contiguous in memory / whose depth k is.
__device__ __forceinline__ void along_m(int e, int &k, int &m) { m = e & (TL_MN - 1); k = e >> 6; }
__device__ __forceinline__ void along_k(int e, int &k, int &m) { k = e & (TL_K - 1); m = e >> 5; }

template <typename T>
__global__ __launch_bounds__(TL_THREADS) void ssd_chunk_state_tiled_kernel(const SsdStateParams p) {
  __shared__ Slabs t;
  extern __shared__ float wq[];                            // weight of every step of the chunk
  const SsdDims &d = p.d;
  const int Q = d.chunk;
  const int ptiles = (d.hdim + TL_MN - 1) / TL_MN, ntiles = (d.nstate + TL_MN - 1) / TL_MN;
  int blk = blockIdx.x;
  const int n0 = (blk % ntiles) * TL_MN; blk /= ntiles;
  const int p0 = (blk % ptiles) * TL_MN; blk /= ptiles;
  const int h = blk % d.heads; blk /= d.heads;
  const int c = blk % d.nchunks, b = blk / d.nchunks;
  const int g = h / (d.heads / d.groups);
  const int qlen = min(Q, d.len - c * Q);
  const size_t cs = (((size_t)b * d.heads + h) * d.nchunks + c) * Q;
  const int tid = threadIdx.x, lane = tid & (WAVE - 1), w = tid >> 6, wr = w >> 1, wc = w & 1;
  {
    const float last = p.dA_cs[cs + Q - 1];
    const int *sid = p.seq_idx ? p.seq_idx + (size_t)b * d.len : nullptr;
    const int sid_last = sid ? sid[c * Q + qlen - 1] : 0;
    for (int l = tid; l < Q; l += TL_THREADS) {
      float wv = 0.0f;
      if (l < qlen && !(sid && sid[c * Q + l] != sid_last)) wv = decay_exp(last - p.dA_cs[cs + l]) * p.dt[cs + l];
      wq[l] = wv;
    }
  }
  f32x16_t acc = {0};
  for (int k0 = 0; k0 < qlen; k0 += TL_K) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TL_K * TL_MN / TL_THREADS; ++j) {
      int k, m;
      along_m(tid + TL_THREADS * j, k, m);
      const int l = min(k0 + k, qlen - 1);
      const size_t row = (size_t)b * d.len + c * Q + l;
      float xv = tl_ld<T>(p.x, p.x_dtype, (row * d.heads + h) * d.hdim + min(p0 + m, d.hdim - 1));
      float bv = tl_ld<T>(p.Bm, p.b_dtype, (row * d.groups + g) * d.nstate + min(n0 + m, d.nstate - 1)) * wq[l];
      if (k0 + k >= qlen || p0 + m >= d.hdim) xv = 0.0f;
      if (k0 + k >= qlen || n0 + m >= d.nstate) bv = 0.0f;
      t.a[k][m] = xv;
      t.b[k][m] = bv;
    }
    __syncthreads();
    slab_mma(t, wr, wc, lane, acc);
  }
  const int col = n0 + wc * 32 + (lane & 31);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = p0 + wr * 32 + crow(r, lane >> 5);
    if (row < d.hdim && col < d.nstate)
      store_any(p.states, p.states_dtype, ((((size_t)b * d.nchunks + c) * d.heads + h) * d.hdim + row) * d.nstate + col, acc[r]);
  }
}

template <typename T>
__global__ __launch_bounds__(TL_THREADS) void ssd_chunk_scan_tiled_kernel(const SsdScanParams p) {
  __shared__ Slabs t;
  extern __shared__ float dyn[];                           // cs[Q], dt[Q] of the chunk
  const SsdDims &d = p.d;
  const int Q = d.chunk;
  float *csq = dyn, *dtq = dyn + Q;
  const int ptiles = (d.hdim + TL_MN - 1) / TL_MN, ltiles = (Q + TL_MN - 1) / TL_MN;
  int blk = blockIdx.x;
  const int p0 = (blk % ptiles) * TL_MN; blk /= ptiles;
  const int l0 = (ltiles - 1 - blk % ltiles) * TL_MN; blk /= ltiles;    // longest tiles first
  const int h = blk % d.heads; blk /= d.heads;
  const int c = blk % d.nchunks, b = blk / d.nchunks;
  const int qlen = min(Q, d.len - c * Q);
  if (l0 >= qlen) return;
  const int g = h / (d.heads / d.groups);
  const size_t cs = (((size_t)b * d.heads + h) * d.nchunks + c) * Q;
  const int tid = threadIdx.x, lane = tid & (WAVE - 1), w = tid >> 6, wr = w >> 1, wc = w & 1;
  for (int l = tid; l < Q; l += TL_THREADS) {
    csq[l] = p.dA_cs[cs + l];
    dtq[l] = l < qlen ? p.dt[cs + l] : 0.0f;
  }
  f32x16_t acc = {0};
  // the state entering the chunk, read out by C
  for (int k0 = 0; k0 < d.nstate; k0 += TL_K) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TL_K * TL_MN / TL_THREADS; ++j) {
      int k, m;
      along_k(tid + TL_THREADS * j, k, m);
      const int n = min(k0 + k, d.nstate - 1);
      float cv = tl_ld<T>(p.Cm, p.c_dtype, (((size_t)b * d.len + c * Q + min(l0 + m, qlen - 1)) * d.groups + g) * d.nstate + n);
      float sv = tl_ld<T>(p.prev, p.states_dtype,
                          ((((size_t)b * d.nchunks + c) * d.heads + h) * d.hdim + min(p0 + m, d.hdim - 1)) * d.nstate + n);
      if (k0 + k >= d.nstate || l0 + m >= qlen) cv = 0.0f;
      if (k0 + k >= d.nstate || p0 + m >= d.hdim) sv = 0.0f;
      t.a[k][m] = cv;
      t.b[k][m] = sv;
    }
    __syncthreads();
    slab_mma(t, wr, wc, lane, acc);
  }
  {
    const int *sid = p.seq_idx ? p.seq_idx + (size_t)b * d.len : nullptr;
    const int sid_prev = sid && c > 0 ? sid[c * Q - 1] : 0;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int l = min(l0 + wr * 32 + crow(r, lane >> 5), Q - 1);
      float f = exp2_hw(csq[l] * LOG2E);
      if (sid && l < qlen && sid[c * Q + l] != sid_prev) f = 0.0f;
      acc[r] *= f;
    }
  }
  // steps of the chunk up to the tile's last row
  const int send = min(l0 + TL_MN, qlen);
  for (int k0 = 0; k0 < send; k0 += TL_K) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TL_K * TL_MN / TL_THREADS; ++j) {
      int k, m;
      along_k(tid + TL_THREADS * j, k, m);
      const int s = min(k0 + k, Q - 1), l = min(l0 + m, Q - 1);
      float v = tl_ld<T>(p.CB, p.cb_dtype, ((((size_t)b * d.nchunks + c) * d.groups + g) * Q + l) * Q + s) *
                decay_exp(csq[l] - csq[s]) * dtq[s];
      if (k0 + k > l0 + m || l0 + m >= qlen) v = 0.0f;
      t.a[k][m] = v;
    }
#pragma unroll
    for (int j = 0; j < TL_K * TL_MN / TL_THREADS; ++j) {
      int k, m;
      along_m(tid + TL_THREADS * j, k, m);
      const int s = min(k0 + k, send - 1);
      float v = tl_ld<T>(p.x, p.x_dtype, (((size_t)b * d.len + c * Q + s) * d.heads + h) * d.hdim + min(p0 + m, d.hdim - 1));
      if (k0 + k >= send || p0 + m >= d.hdim) v = 0.0f;
      t.b[k][m] = v;
    }
    __syncthreads();
    slab_mma(t, wr, wc, lane, acc);
  }
  const int pp = p0 + wc * 32 + (lane & 31);
  if (pp >= d.hdim) return;
  const float Dv = p.Dk ? p.Dk[p.d_per_p ? (size_t)h * d.hdim + pp : (size_t)h] : 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int l = l0 + wr * 32 + crow(r, lane >> 5);
    if (l >= qlen) continue;
    const size_t at = (((size_t)b * d.len + c * Q + l) * d.heads + h) * d.hdim + pp;
    float v = acc[r];
    if (p.Dk) v = __builtin_fmaf(Dv, tl_ld<T>(p.x, p.x_dtype, at), v);
    if (p.z) v *= silu_f32(tl_ld<T>(p.z, p.z_dtype, at));
    store_any(p.y, p.y_dtype, at, v);
  }
}

// CB[l][s] = <a_l, b_s> over the K columns of both, zero above the diagonal when causal or across
// sequences of a packed batch.
template <typename T>
__global__ __launch_bounds__(TL_THREADS) void ssd_bmm_tiled_kernel(const SsdBmmParams p) {
  __shared__ Slabs t;
  const int Q = p.chunk, tiles = (Q + TL_MN - 1) / TL_MN;
  int blk = blockIdx.x;
  const int s0 = (blk % tiles) * TL_MN; blk /= tiles;
  const int l0 = (blk % tiles) * TL_MN; blk /= tiles;
  const int g = blk % p.groups; blk /= p.groups;
  const int c = blk % p.nchunks, b = blk / p.nchunks;
  const int qlen = min(Q, p.len - c * Q);
  const int tid = threadIdx.x, lane = tid & (WAVE - 1), w = tid >> 6, wr = w >> 1, wc = w & 1;
  f32x16_t acc = {0};
  const bool live = l0 < qlen && s0 < qlen && !(p.causal && s0 > l0 + TL_MN - 1);
  for (int k0 = 0; live && k0 < p.kdim; k0 += TL_K) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TL_K * TL_MN / TL_THREADS; ++j) {
      int k, m;
      along_k(tid + TL_THREADS * j, k, m);
      const int kk = min(k0 + k, p.kdim - 1);
      float av = tl_ld<T>(p.a, p.in_dtype, (((size_t)b * p.len + c * Q + min(l0 + m, qlen - 1)) * p.groups + g) * p.kdim + kk);
      float bv = tl_ld<T>(p.b, p.in_dtype, (((size_t)b * p.len + c * Q + min(s0 + m, qlen - 1)) * p.groups + g) * p.kdim + kk);
      if (k0 + k >= p.kdim || l0 + m >= qlen) av = 0.0f;
      if (k0 + k >= p.kdim || s0 + m >= qlen) bv = 0.0f;
      t.a[k][m] = av;
      t.b[k][m] = bv;
    }
    __syncthreads();
    slab_mma(t, wr, wc, lane, acc);
  }
  const int sc = s0 + wc * 32 + (lane & 31);
  if (sc >= Q) return;
  const int *sid = p.seq_idx ? p.seq_idx + (size_t)b * p.len + c * Q : nullptr;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int l = l0 + wr * 32 + crow(r, lane >> 5);
    if (l >= Q) continue;
    float v = acc[r];
    if (l >= qlen || sc >= qlen || (p.causal && sc > l) || (sid && sid[l] != sid[sc])) v = 0.0f;
    store_any(p.out, p.out_dtype, ((((size_t)b * p.nchunks + c) * p.groups + g) * Q + l) * Q + sc, v);
  }
}

constexpr int TL_MAX_CHUNK = 4096;   // chunk-long arrays in LDS beside the slabs

}  // namespace

bool ssd_bmm_tiled(const SsdBmmParams &p, hipStream_t s) {
  const size_t per = (size_t)((p.chunk + TL_MN - 1) / TL_MN);
  const size_t tiles = (size_t)p.batch * p.nchunks * p.groups * per * per;
  if (tiles >= ((size_t)1 << 31)) return false;
  const dim3 grid((unsigned)tiles), block(TL_THREADS);
  if (p.in_dtype == SSM_F32) hipLaunchKernelGGL(ssd_bmm_tiled_kernel<float>, grid, block, 0, s, p);
  else if (p.in_dtype == SSM_BF16) hipLaunchKernelGGL(ssd_bmm_tiled_kernel<bf16_t>, grid, block, 0, s, p);
  else hipLaunchKernelGGL(ssd_bmm_tiled_kernel<f16_t>, grid, block, 0, s, p);
  return true;
}

bool ssd_chunk_state_tiled(const SsdStateParams &p, hipStream_t s) {
  const SsdDims &d = p.d;
  const size_t tiles = (size_t)d.batch * d.nchunks * d.heads * ((d.hdim + TL_MN - 1) / TL_MN) * ((d.nstate + TL_MN - 1) / TL_MN);
  if (d.chunk > TL_MAX_CHUNK || tiles >= ((size_t)1 << 31)) return false;
  const dim3 grid((unsigned)tiles), block(TL_THREADS);
  const size_t lds = (size_t)d.chunk * sizeof(float);
  const bool same = p.x_dtype == p.b_dtype;
  if (same && p.x_dtype == SSM_F32) hipLaunchKernelGGL(ssd_chunk_state_tiled_kernel<float>, grid, block, lds, s, p);
  else if (same && p.x_dtype == SSM_BF16) hipLaunchKernelGGL(ssd_chunk_state_tiled_kernel<bf16_t>, grid, block, lds, s, p);
  else if (same && p.x_dtype == SSM_F16) hipLaunchKernelGGL(ssd_chunk_state_tiled_kernel<f16_t>, grid, block, lds, s, p);
  else hipLaunchKernelGGL(ssd_chunk_state_tiled_kernel<void>, grid, block, lds, s, p);
  return true;
}

bool ssd_chunk_scan_tiled(const SsdScanParams &p, hipStream_t s) {
  const SsdDims &d = p.d;
  const size_t tiles = (size_t)d.batch * d.nchunks * d.heads * ((d.hdim + TL_MN - 1) / TL_MN) * ((d.chunk + TL_MN - 1) / TL_MN);
  if (d.chunk > TL_MAX_CHUNK || tiles >= ((size_t)1 << 31)) return false;
  const dim3 grid((unsigned)tiles), block(TL_THREADS);
  const size_t lds = (size_t)2 * d.chunk * sizeof(float);
  const bool same = p.x_dtype == p.c_dtype && p.x_dtype == p.cb_dtype && p.x_dtype == p.states_dtype &&
                    (!p.z || p.z_dtype == p.x_dtype);
  if (same && p.x_dtype == SSM_F32) hipLaunchKernelGGL(ssd_chunk_scan_tiled_kernel<float>, grid, block, lds, s, p);
  else if (same && p.x_dtype == SSM_BF16) hipLaunchKernelGGL(ssd_chunk_scan_tiled_kernel<bf16_t>, grid, block, lds, s, p);
  else if (same && p.x_dtype == SSM_F16) hipLaunchKernelGGL(ssd_chunk_scan_tiled_kernel<f16_t>, grid, block, lds, s, p);
  else hipLaunchKernelGGL(ssd_chunk_scan_tiled_kernel<void>, grid, block, lds, s, p);
  return true;
}

}  // namespace ssm
