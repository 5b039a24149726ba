// bf16 MFMA kernels of the state-space-duality family for gfx950
// (v_mfma_f32_32x32x16_bf16: 32x32 fp32 tile += 32x16 (A) * 16x32 (B)).
//
// Register layout of one instruction, lane l of 64:
//   A operand  8 bf16: row  m = l % 32, k = 8 * (l / 32) + j
//   B operand  8 bf16: col  n = l % 32, k = 8 * (l / 32) + j
//   C / D     16 fp32: col  n = l % 32, row m = 8 * (r / 4) + 4 * (l / 32) + r % 4
// Both operands want the reduction index contiguous per lane.  C B^T and C.S
// have it contiguous in memory already; contractions over time (chunk_state and
// the x operand of chunk_scan) read x through an LDS tile transposed on the way
// in, and chunk_state reads B through a once-per-call transposed copy.
//
// Taken for bf16 inputs when L % Q == 0, Q % 32 == 0, Q <= 256, N % 16 == 0 and
// P is 32 or 64; every other case runs the shape-generic kernels.
#include "ssd_common.hpp"

namespace ssm {

constexpr int MF_THREADS = 256;
constexpr int MF_WAVES = 4;
constexpr int XT_PAD = 8;      // bf16 elements of padding per transposed row

// Offset (in bf16 elements) of (p, l) inside the transposed, XOR-swizzled x tile.
// The swizzle permutes 16-byte pieces inside aligned groups of (lowest set bit of Q / 8)
// pieces, at most 8, so that it never leaves the row.
__device__ __forceinline__ int xt_off(int p, int l, int stride) {
  const int pieces = (stride - XT_PAD) >> 3;
  const int mask = min(8, pieces & -pieces) - 1;
  return p * stride + ((((l >> 3) ^ ((p >> 3) & mask))) << 3) + (l & 7);
}

// Transpose the [Q][P] bf16 slab x[b, t0.., h, :] into LDS as [P][Q] (optionally
// scaling row l by w[l]).  A thread moves 8x8 blocks: eight 16-byte global reads
// along p, eight 16-byte LDS writes along l.
// PRE: row l is first multiplied by pre[l] (global memory, the chunk's Q values) and rounded to E -- the operand
// then is exactly the tensor round(x * pre) that a separate launch would have written.
template <bool WEIGHTED, bool PRE, typename E>
__device__ __forceinline__ void stage_xT(E *xT, const E *x, long row_stride, int Q, int P,
                                         const float *w_lds, int stride, const float *pre = nullptr) {
  const int pblocks = P >> 3;
  const int nblocks = (Q >> 3) * pblocks;
  for (int blk = threadIdx.x; blk < nblocks; blk += MF_THREADS) {
    const int pb = blk % pblocks, lb = blk / pblocks;
    float v[8][8];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const V8<E> raw = load_frag_e<E>(x + (long)(lb * 8 + r) * row_stride + pb * 8);
      const float w = WEIGHTED ? w_lds[lb * 8 + r] : 1.0f;
      const float pr = PRE ? pre[lb * 8 + r] : 1.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float e = (float)raw[i];
        if (PRE) e = (float)(E)(e * pr);
        v[r][i] = WEIGHTED ? e * w : e;
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      V8<E> col;
#pragma unroll
      for (int r = 0; r < 8; ++r) col[r] = (E)v[r][i];
      *reinterpret_cast<V8<E> *>(xT + xt_off(pb * 8 + i, lb * 8, stride)) = col;
    }
  }
}

// ------------------------------------------------------------------ bmm_chunk
// out[b,c,g,l,s] = <a[b,cQ+l,g,:], b[b,cQ+s,g,:]>; one workgroup per 64x64 tile.
template <typename E, typename out_t>
__global__ __launch_bounds__(MF_THREADS) void ssd_bmm_mfma_kernel(const SsdBmmParams p) {
  const int Q = p.chunk, K = p.kdim;
  const int tiles = Q / 64 + (Q % 64 ? 1 : 0);          // 64-wide tiles per side (Q % 32 == 0)
  const int wave = wave_id_uniform(), lane = lane_id();
  const int unit = blockIdx.x / (tiles * tiles);
  const int tile = blockIdx.x % (tiles * tiles);
  const int g = unit % p.groups;
  const int c = (unit / p.groups) % p.nchunks;
  const int b = unit / (p.groups * p.nchunks);
  const int l0 = (tile / tiles) * 64 + (wave >> 1) * 32;
  const int s0 = (tile % tiles) * 64 + (wave & 1) * 32;
  if (l0 >= Q || s0 >= Q) return;
  out_t *out = reinterpret_cast<out_t *>(p.out) + (((size_t)b * p.nchunks + c) * p.groups + g) * (size_t)Q * Q;
  const int g2 = lane >> 5, m = lane & 31;
  f32x16_t acc = {0};
  const bool skip = p.causal && s0 > l0 + 31;
  if (!skip) {
    const E *arow = reinterpret_cast<const E *>(p.a) + (((size_t)b * p.len + c * Q + l0 + m) * p.groups + g) * K + 8 * g2;
    const E *brow = reinterpret_cast<const E *>(p.b) + (((size_t)b * p.len + c * Q + s0 + m) * p.groups + g) * K + 8 * g2;
    for (int k0 = 0; k0 < K; k0 += 16) acc = mma(load_frag_e<E>(arow + k0), load_frag_e<E>(brow + k0), acc);
  }
  const int *sid = p.seq_idx ? p.seq_idx + (size_t)b * p.len + c * Q : nullptr;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int l = l0 + crow(r, g2), s = s0 + m;
    float v = acc[r];
    if (p.causal && s > l) v = 0.0f;
    if (sid && sid[l] != sid[s]) v = 0.0f;
    out[(size_t)l * Q + s] = from_f32<out_t>(v);
  }
}

// ------------------------------------------------------------------ backward: dCB
// dCB[b,c,g,l,s] = sum over the heads h of group g of  dt[s,h] exp(cs[l,h] - cs[s,h]) <dy[l,h,:], x[s,h,:]>  for s <= l,
// zero above the diagonal: the matrix from which both dB (= dCB^T C) and dC (= dCB B) of a chunk's own steps follow,
// so that the sum over heads is taken once, before the products with C and B.  One workgroup per 64x64 tile, a wave
// per 32x32 block; per head the block of <dy, x> is formed on the matrix cores from operands read straight from
// memory (rows of dy and x with the channel axis contiguous) and added with its per-element weight in float32.
struct SsdDcbParams {
  const __bf16 *dy, *x;        // (B, L, H, P)
  const float *dt, *dA_cs;     // (B, H, nc, Q)
  float *out;                  // (B, nc, G, Q, Q)
  int batch, len, heads, hdim, groups, chunk, nchunks;
};

template <int KS>              // P = 16 * KS
__global__ __launch_bounds__(MF_THREADS) void ssd_bwd_dcb_kernel(const SsdDcbParams p) {
  // One workgroup per 32x32 block on or below the diagonal; its four waves take every fourth head of the group
  // (a head is one round trip to memory and little arithmetic, so the heads must be spread over many waves), and
  // their sums meet in LDS.
  __shared__ float part[MF_WAVES - 1][16][WAVE];
  const int Q = p.chunk, P = 16 * KS, H = p.heads;
  const int nb = Q / 32, nblk = nb * (nb + 1) / 2;
  const int wave = wave_id_uniform(), lane = lane_id();
  // Consecutive workgroup numbers go to different XCDs (eight, each with its own L2).  All blocks of a (batch,
  // chunk, group) unit read the same rows of dy and x, so a unit's blocks are given numbers that are equal mod 8:
  // they run on one XCD and its L2 fetches the unit's operands once.
  const int units = p.batch * p.nchunks * p.groups;
  int unit, tri;
  if (units % 8 == 0) {
    const int k = (int)blockIdx.x >> 3;
    unit = (k / nblk) * 8 + ((int)blockIdx.x & 7);
    tri = k % nblk;                                       // (lb, sb) with sb <= lb, row by row
  } else {
    unit = blockIdx.x / nblk;
    tri = blockIdx.x % nblk;
  }
  int lb = 0;
  while (tri > lb) tri -= ++lb;
  const int sb = tri;
  const int g = unit % p.groups;
  const int c = (unit / p.groups) % p.nchunks;
  const int b = unit / (p.groups * p.nchunks);
  const int l0 = lb * 32, s0 = sb * 32;
  float *out = p.out + (((size_t)b * p.nchunks + c) * p.groups + g) * (size_t)Q * Q;
  const int g2 = lane >> 5, m = lane & 31;
  f32x16_t acc = {0};
  const int per = H / p.groups;
  const bool diag = s0 == l0;
  const size_t trow = (size_t)H * P;
  const size_t csb = (((size_t)b * H + (size_t)g * per) * p.nchunks + c) * Q;
  // Rows of dy and x are 10 KB apart in memory, so a fragment read straight from them (lane = row) touches 32
  // cache lines for 32 bytes each.  A wave reads its head's 2 x 32 rows with consecutive lanes on consecutive
  // 16-byte pieces instead (every line whole, once) and turns them into fragments through a tile of its own in LDS.
  constexpr int PIECES = 2 * KS;                  // 16-byte pieces per row
  constexpr int RS = 16 * KS + 8;                 // elements between rows of the tile: conflict-free 16-byte reads
  __shared__ __align__(16) __bf16 tile[MF_WAVES][2][32 * RS];
  const __bf16 *abase = p.dy + ((size_t)b * p.len + (size_t)c * Q + l0) * trow + (size_t)g * per * P;
  const __bf16 *bbase = p.x + ((size_t)b * p.len + (size_t)c * Q + s0) * trow + (size_t)g * per * P;
  bf16x8_t ra[KS], rb[KS];
  auto request = [&](int head) {
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      const int idx = j * WAVE + lane, row = idx / PIECES, piece = idx % PIECES;
      ra[j] = load_frag(abase + (size_t)row * trow + (size_t)head * P + 8 * piece);
      rb[j] = load_frag(bbase + (size_t)row * trow + (size_t)head * P + 8 * piece);
    }
  };
  if (wave < per) request(wave);
  for (int hh = wave; hh < per; hh += MF_WAVES) {
    const float *cs = p.dA_cs + csb + (size_t)hh * p.nchunks * Q;
    const float *dts = p.dt + csb + (size_t)hh * p.nchunks * Q;
    const float cs_s = cs[s0 + m], dt_s = dts[s0 + m];
    float4 cl[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) cl[j] = *reinterpret_cast<const float4 *>(cs + l0 + 8 * j + 4 * g2);
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      const int idx = j * WAVE + lane, row = idx / PIECES, piece = idx % PIECES;
      *reinterpret_cast<bf16x8_t *>(&tile[wave][0][row * RS + 8 * piece]) = ra[j];
      *reinterpret_cast<bf16x8_t *>(&tile[wave][1][row * RS + 8 * piece]) = rb[j];
    }
    bf16x8_t fa[KS], fb[KS];
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      fa[k] = load_frag(&tile[wave][0][m * RS + 16 * k + 8 * g2]);
      fb[k] = load_frag(&tile[wave][1][m * RS + 16 * k + 8 * g2]);
    }
    if (hh + MF_WAVES < per) request(hh + MF_WAVES);     // the wave's next head, requested before this head's arithmetic
    f32x16_t t = {0};
#pragma unroll
    for (int k = 0; k < KS; ++k) t = mma(fa[k], fb[k], t);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float cs_l = r % 4 == 0 ? cl[r / 4].x : r % 4 == 1 ? cl[r / 4].y : r % 4 == 2 ? cl[r / 4].z : cl[r / 4].w;
      float w = dt_s * exp2_hw(fminf(cs_l - cs_s, 0.0f) * LOG2E);
      if (diag && s0 + m > l0 + crow(r, g2)) w = 0.0f;
      acc[r] = __builtin_fmaf(w, t[r], acc[r]);
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) part[wave - 1][r][lane] = acc[r];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float v = ((acc[r] + part[0][r][lane]) + part[1][r][lane]) + part[2][r][lane];
      out[(size_t)(l0 + crow(r, g2)) * Q + s0 + m] = v;
      if (!diag) out[(size_t)(s0 + crow(r, g2)) * Q + l0 + m] = 0.0f;      // the mirrored block above the diagonal
    }
  }
}

// ---------------------------------------------------------------- transpose B
// Bt[b,g,n,t] = Bm[b,t,g,n]   (bf16), tiles of 64 x 64 through LDS.
__global__ __launch_bounds__(MF_THREADS) void ssd_transpose_kernel(const uint16_t *src, uint16_t *dst, int len, int groups,
                                                                    int nstate) {
  __shared__ uint16_t tile[64][66];
  const int tb = blockIdx.x, nb = blockIdx.y;
  const int bg = blockIdx.z;
  const int b = bg / groups, g = bg % groups;
  for (int e = threadIdx.x; e < 64 * 64; e += MF_THREADS) {
    const int tl = e / 64, nl = e % 64;
    const int t = tb * 64 + tl, n = nb * 64 + nl;
    tile[tl][nl] = (t < len && n < nstate) ? src[(((size_t)b * len + t) * groups + g) * nstate + n] : (uint16_t)0;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 64 * 64; e += MF_THREADS) {
    const int nl = e / 64, tl = e % 64;
    const int t = tb * 64 + tl, n = nb * 64 + nl;
    if (t < len && n < nstate) dst[(((size_t)b * groups + g) * nstate + n) * len + t] = tile[tl][nl];
  }
}

// ---------------------------------------------------------------- chunk_state
// states[b,c,h,p,n] = sum_l xw[l][p] * B[l][n];  one workgroup per (b, c, h).
template <typename E, typename st_t, int PT>
__global__ __launch_bounds__(MF_THREADS) void ssd_chunk_state_mfma_kernel(const SsdStateParams p, const E *Bt) {
  const SsdDims &d = p.d;
  const int Q = d.chunk, P = 32 * PT, N = d.nstate;
  const int stride = Q + XT_PAD;
  extern __shared__ __align__(16) unsigned char smem[];
  E *xT = reinterpret_cast<E *>(smem);                         // [P][Q + pad]
  float *w = reinterpret_cast<float *>(smem + (size_t)P * stride * 2);   // [Q]
  const int wave = wave_id_uniform(), lane = lane_id();
  const int h = blockIdx.x % d.heads;
  const int c = (blockIdx.x / d.heads) % d.nchunks;
  const int b = blockIdx.x / (d.heads * d.nchunks);
  const int g = h / (d.heads / d.groups);
  const size_t cs = (((size_t)b * d.heads + h) * d.nchunks + c) * Q;
  const float last = p.dA_cs[cs + Q - 1];
  // packed sequences: steps of another sequence than the chunk's last step add nothing
  const int *sid = p.seq_idx ? p.seq_idx + (size_t)b * d.len + (size_t)c * Q : nullptr;
  const int sid_last = sid ? sid[Q - 1] : 0;
  for (int l = threadIdx.x; l < Q; l += MF_THREADS)
    w[l] = (sid && sid[l] != sid_last) ? 0.0f : decay_exp(last - p.dA_cs[cs + l]) * p.dt[cs + l];
  __syncthreads();
  // the chunk's first row and the step from row to row (backwards from the mirrored row when x is in forward time
  // and the call in reversed time)
  const size_t first = p.x_reversed ? (size_t)d.len - 1 - (size_t)c * Q : (size_t)c * Q;
  const long xstep = p.x_reversed ? -(long)d.heads * P : (long)d.heads * P;
  const E *xg = reinterpret_cast<const E *>(p.x) + (((size_t)b * d.len + first) * d.heads + h) * P;
  if (p.x_scale) stage_xT<true, true, E>(xT, xg, xstep, Q, P, w, stride, p.x_scale + cs);
  else stage_xT<true, false, E>(xT, xg, xstep, Q, P, w, stride);
  __syncthreads();

  const int g2 = lane >> 5, m = lane & 31;
  st_t *out = reinterpret_cast<st_t *>(p.states) + ((((size_t)b * d.nchunks + c) * d.heads + h) * P) * (size_t)N;
  for (int n0 = wave * 32; n0 < N; n0 += MF_WAVES * 32) {
    f32x16_t acc[PT];
#pragma unroll
    for (int i = 0; i < PT; ++i) acc[i] = (f32x16_t){0};
    const bool ncol_ok = n0 + m < N;
    const E *bt = Bt + (((size_t)b * d.groups + g) * N + (ncol_ok ? n0 + m : 0)) * (size_t)d.len + (size_t)c * Q + 8 * g2;
    for (int k0 = 0; k0 < Q; k0 += 16) {
      V8<E> bf = load_frag_e<E>(bt + k0);
      if (!ncol_ok) bf = (V8<E>){0};
#pragma unroll
      for (int i = 0; i < PT; ++i) {
        const V8<E> af = load_frag_e<E>(xT + xt_off(32 * i + m, k0 + 8 * g2, stride));
        acc[i] = mma(af, bf, acc[i]);
      }
    }
    if (ncol_ok) {
#pragma unroll
      for (int i = 0; i < PT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) out[(size_t)(32 * i + crow(r, g2)) * N + n0 + m] = from_f32<st_t>(acc[i][r]);
    }
  }
}

// ----------------------------------------------------------------- chunk_scan
// One workgroup per (b, c, h); wave w owns row blocks w, nlb-1-w, w+4, ... of 32 rows.
// DX (1: dx in the element type, 2: in float32): the result is not written; it is the u of the backward's reversed
// pass and goes straight into dx and the two row sums that need it (SsdDxEpilogue).
template <typename E, typename st_t, int PT, int DX = 0>
__global__ __launch_bounds__(MF_THREADS) void ssd_chunk_scan_mfma_kernel(const SsdScanParams p) {
  const SsdDims &d = p.d;
  const int Q = d.chunk, P = 32 * PT, N = d.nstate;
  const int stride = Q + XT_PAD;
  extern __shared__ __align__(16) unsigned char smem[];
  E *xT = reinterpret_cast<E *>(smem);                          // [P][Q + pad], unweighted
  float *dAs = reinterpret_cast<float *>(smem + (size_t)P * stride * 2);  // [Q]
  float *dts = dAs + Q;                                                   // [Q]
  float *ent = dts + Q;                                                   // [Q] 1 where the entering state reaches the step
  const int wave = wave_id_uniform(), lane = lane_id();
  const int h = blockIdx.x % d.heads;
  const int c = (blockIdx.x / d.heads) % d.nchunks;
  const int b = blockIdx.x / (d.heads * d.nchunks);
  const int g = h / (d.heads / d.groups);
  const size_t cs = (((size_t)b * d.heads + h) * d.nchunks + c) * Q;
  // packed sequences: the entering state belongs to the sequence of the last step before this chunk (id 0 at the
  // start of the row); products across sequences inside the chunk are zero in CB already
  const int *sid = p.seq_idx ? p.seq_idx + (size_t)b * d.len : nullptr;
  const int sid_prev = (sid && c > 0) ? sid[(size_t)c * Q - 1] : 0;
  for (int l = threadIdx.x; l < Q; l += MF_THREADS) {
    dAs[l] = p.dA_cs[cs + l] * LOG2E;              // in units of log 2: the factors below are exp2 of differences
    dts[l] = p.dt[cs + l];
    ent[l] = (sid && sid[(size_t)c * Q + l] != sid_prev) ? 0.0f : 1.0f;
  }
  const size_t xrow = (size_t)d.heads * P;                                 // elements between time steps
  const size_t xbase = (((size_t)b * d.len + (size_t)c * Q) * d.heads + h) * P;
  const E *xg = reinterpret_cast<const E *>(p.x) + xbase;
  // The epilogue's reads (x and dt at the chunk's steps in forward time) come at the very end of the workgroup's life
  // with nothing left to hide them behind: one early read per row and half line brings them near, its value unused.
  unsigned near0 = 0, near1 = 0;
  float near2 = 0.0f;
  if constexpr (DX) {
    const int rl = threadIdx.x % Q;
    const size_t row = ((size_t)b * d.len + (d.len - 1 - (c * Q + rl))) * d.heads + h;
    const unsigned *xr = reinterpret_cast<const unsigned *>(reinterpret_cast<const E *>(p.dx.x) + row * P);
    near0 = xr[0];
    near1 = xr[P / 4];
    near2 = p.dx.dt[row];
  }
  {
    // (the rows of the mirrored chunk, backwards, when x is in forward time and the call in reversed time)
    const E *xs = p.x_reversed ? reinterpret_cast<const E *>(p.x) + (((size_t)b * d.len + (d.len - 1 - (size_t)c * Q)) * d.heads + h) * P : xg;
    const long xstep = p.x_reversed ? -(long)xrow : (long)xrow;
    if (p.x_scale) stage_xT<false, true, E>(xT, xs, xstep, Q, P, nullptr, stride, p.x_scale + cs);
    else stage_xT<false, false, E>(xT, xs, xstep, Q, P, nullptr, stride);
  }
  // The state entering the chunk, [P][N], as bfloat16 in LDS: read once by the workgroup in whole lines (a fragment
  // read straight from memory, lane = row, touches 32 lines for 32 bytes each, and every row block would read it again).
  E *Sb = reinterpret_cast<E *>(ent + Q);                       // [P][N + 8]
  const int SR = N + 8;
  {
    const st_t *Sg0 = reinterpret_cast<const st_t *>(p.prev) + ((((size_t)b * d.nchunks + c) * d.heads + h) * P) * (size_t)N;
    const int pieces = N / 8;
    for (int e = threadIdx.x; e < P * pieces; e += MF_THREADS) {
      const int row = e / pieces, piece = e % pieces;
      const st_t *sp = Sg0 + (size_t)row * N + 8 * piece;
      V8<E> v;
      if constexpr (sizeof(st_t) == 2) {
        v = load_frag_e<E>(sp);
      } else {
        const float4 lo = *reinterpret_cast<const float4 *>(sp), hi = *reinterpret_cast<const float4 *>(sp + 4);
        const float t8[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        v = pack8_e<E>(t8);
      }
      *reinterpret_cast<V8<E> *>(Sb + row * SR + 8 * piece) = v;
    }
  }
  __syncthreads();

  const int g2 = lane >> 5, m = lane & 31;
  const int nlb = Q / 32;
  const E *Cg = reinterpret_cast<const E *>(p.Cm) + (((size_t)b * d.len + (size_t)c * Q) * d.groups + g) * N;
  const size_t c_stride = (size_t)d.groups * N;
  const E *CBg = reinterpret_cast<const E *>(p.CB) + (((size_t)b * d.nchunks + c) * d.groups + g) * (size_t)Q * Q;
  const E *zg = p.z ? reinterpret_cast<const E *>(p.z) + xbase : nullptr;
  E *yg = reinterpret_cast<E *>(p.y) + xbase;
  float *yf = reinterpret_cast<float *>(p.y) + xbase;
  const bool y_f32 = p.y_dtype == SSM_F32;

  // The products are formed transposed (the x / state fragment as the first operand): a lane then holds, for its row
  // l0 + m of the chunk, channels 32 i + 8 q + 4 g2 + (0..3) in acc[i][4 q + (0..3)], and a row's factors are one
  // value per lane.  A wave owns at most two row blocks (Q <= 256): it forms both, and once every wave is through
  // (the staged tiles are free then) turns each into rows through a tile of its own in LDS, so that the epilogue's
  // reads and writes are whole runs of a row's channels on neighbouring lanes.
  auto block_of = [&](int lb, f32x16_t (&acc)[PT]) {
    const int l0 = 32 * lb;
    const int lrow = l0 + m;                        // this lane's row: as an operand and in the result
#pragma unroll
    for (int i = 0; i < PT; ++i) acc[i] = (f32x16_t){0};
    // carried-in state: S[p][:] . C[l][:]
    const E *crow_p = Cg + (size_t)lrow * c_stride + 8 * g2;
    for (int n0 = 0; n0 < N; n0 += 16) {
      const V8<E> af = load_frag_e<E>(crow_p + n0);
#pragma unroll
      for (int i = 0; i < PT; ++i) acc[i] = mma(load_frag_e<E>(Sb + (32 * i + m) * SR + n0 + 8 * g2), af, acc[i]);
    }
    const float dal = dAs[lrow];
    {
      const float sc = exp2_hw(dal) * ent[lrow];
#pragma unroll
      for (int i = 0; i < PT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] *= sc;
    }
    // within the chunk: M[l][s] = CB[l][s] exp(dA_l - dA_s) dt_s for s <= l (the difference clamped at 0, as the
    // published kernels do); only the row block's own 32 columns hold any s > l
    const E *cbrow = CBg + (size_t)lrow * Q + 8 * g2;
    auto columns = [&](int s0, auto diagonal) {
      float cb[8];
      unpack8(load_frag_e<E>(cbrow + s0), cb);
      const int sbase = s0 + 8 * g2;
      const float4 a0 = *reinterpret_cast<const float4 *>(dAs + sbase), a1 = *reinterpret_cast<const float4 *>(dAs + sbase + 4);
      const float4 t0 = *reinterpret_cast<const float4 *>(dts + sbase), t1 = *reinterpret_cast<const float4 *>(dts + sbase + 4);
      const float das[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
      const float dtv[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
      float mv[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float v = cb[j] * exp2_hw(fminf(dal - das[j], 0.0f)) * dtv[j];
        mv[j] = (!decltype(diagonal)::value || sbase + j <= lrow) ? v : 0.0f;
      }
      const V8<E> af = pack8_e<E>(mv);
#pragma unroll
      for (int i = 0; i < PT; ++i) {
        const V8<E> bf = load_frag_e<E>(xT + xt_off(32 * i + m, sbase, stride));
        acc[i] = mma(bf, af, acc[i]);
      }
    };
    for (int s0 = 0; s0 < l0; s0 += 16) columns(s0, std::false_type{});
    columns(l0, std::true_type{});
    columns(l0 + 16, std::true_type{});
  };

  const int npairs = (nlb + 1) / 2;                  // <= MF_WAVES (checked by the host)
  const bool has0 = wave < npairs, has1 = has0 && (nlb - 1 - wave) != wave;
  f32x16_t acc0[PT], acc1[PT];
  if (has0) block_of(wave, acc0);
  if (has1) block_of(nlb - 1 - wave, acc1);
  __syncthreads();                                   // nobody reads the staged tiles any more

  constexpr int SCR = 32 * PT + 4;                   // floats per row of a wave's tile (the pad spreads the banks)
  constexpr int LPR = 8 * PT, RPI = WAVE / LPR;      // lanes per row, rows per instruction
  float *scr = reinterpret_cast<float *>(smem) + (size_t)wave * (32 * SCR);
  const int rsub = lane / LPR, c4 = (lane % LPR) * 4;
  // Nothing inside the loops over a tile's rows is decided at run time (the options are template arguments of the
  // lambdas below) and every address is a base the workgroup shares plus a 32-bit byte offset: the reads of all of
  // a tile's rows are then issued together.
  using Yes = std::true_type;
  using No = std::false_type;

  auto to_rows = [&](const f32x16_t (&acc)[PT]) {
#pragma unroll
    for (int i = 0; i < PT; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<float4 *>(scr + m * SCR + 32 * i + 8 * q + 4 * g2) =
            make_float4(acc[i][4 * q], acc[i][4 * q + 1], acc[i][4 * q + 2], acc[i][4 * q + 3]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the wave's own tile: written, now read by other lanes
  };
  auto tile_row = [&](int it, float (&v)[4]) {
    const float4 t4 = *reinterpret_cast<const float4 *>(scr + (it * RPI + rsub) * SCR + c4);
    v[0] = t4.x; v[1] = t4.y; v[2] = t4.z; v[3] = t4.w;
  };

  if constexpr (DX) {
    // dx = dt u + D dy and the two row sums, at the forward-time step of every row.  Row l of the chunk is forward
    // step t0 + (Q-1-l), t0 the chunk's earliest.
    const SsdDxEpilogue &e = p.dx;
    const size_t row0 = ((size_t)b * d.len + (d.len - (size_t)(c + 1) * Q)) * d.heads + h;
    const E *xf = reinterpret_cast<const E *>(e.x) + row0 * P;
    const E *dyg = p.x_reversed ? reinterpret_cast<const E *>(p.x) + row0 * P : xg;      // dy in forward time: x's rows
    const float *dtf = e.dt + row0;
    float *xuf = e.xu + row0, *s1f = e.s1 + row0;
    float4 Dp = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (e.Dk) {
      if (e.d_per_p) Dp = *reinterpret_cast<const float4 *>(e.Dk + (size_t)h * P + c4);
      else Dp.x = Dp.y = Dp.z = Dp.w = e.Dk[h];
    }
    const float Dv4[4] = {Dp.x, Dp.y, Dp.z, Dp.w};
    const bool rnd = e.round_dtx != 0;
    auto rows_dx = [&](int lb, const f32x16_t (&acc)[PT]) {
      to_rows(acc);
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int l = 32 * lb + it * RPI + rsub;
        const unsigned rowoff = (unsigned)(Q - 1 - l) * (unsigned)d.heads;                    // rows of (B, L, H)
        const unsigned at = rowoff * (unsigned)P + (unsigned)c4;                             // elements of (B, L, H, P)
        float v[4], xv[4], dyv[4], dxv[4];
        tile_row(it, v);
        const float dtv = *at_bytes<const float>(dtf, rowoff * 4u);
        load4_e<E>(at_bytes<const E>(xf, at * (unsigned)sizeof(E)), xv);
        // the pass's own operand is dy (read even without a skip term, whose factor is zero then)
        load4_e<E>(at_bytes<const E>(dyg, (p.x_reversed ? at : (unsigned)l * (unsigned)xrow + (unsigned)c4) * (unsigned)sizeof(E)), dyv);
        float xu = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          dxv[j] = __builtin_fmaf(Dv4[j], dyv[j], dtv * v[j]);
          xu = __builtin_fmaf(xv[j], v[j], xu);
          const float xt = dtv * xv[j];
          s1 = __builtin_fmaf(rnd ? (float)(E)xt : xt, v[j], s1);
        }
        if constexpr (DX == 2)
          *at_bytes<float4>(reinterpret_cast<float *>(e.dx) + row0 * P, at * 4u) = make_float4(dxv[0], dxv[1], dxv[2], dxv[3]);
        else
          store4_e<E>(at_bytes<E>(reinterpret_cast<E *>(e.dx) + row0 * P, at * (unsigned)sizeof(E)), dxv);
        xu = lane_run_sum_last<LPR>(xu);
        s1 = lane_run_sum_last<LPR>(s1);
        if (lane % LPR == LPR - 1) {
          *at_bytes<float>(xuf, rowoff * 4u) = xu;
          *at_bytes<float>(s1f, rowoff * 4u) = s1;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // read before the next tile is written over it
    };
    if (has0) rows_dx(wave, acc0);
    if (has1) rows_dx(nlb - 1 - wave, acc1);
    asm volatile("" ::"v"(near0), "v"(near1), "v"(near2));      // (the early reads end here)
  } else {
    // + D x, gate, store
    float4 Dp = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (p.Dk) {
      if (p.d_per_p) Dp = *reinterpret_cast<const float4 *>(p.Dk + (size_t)h * P + c4);
      else Dp.x = Dp.y = Dp.z = Dp.w = p.Dk[h];
    }
    const float Dv4[4] = {Dp.x, Dp.y, Dp.z, Dp.w};
    auto rows_y = [&](int lb, const f32x16_t (&acc)[PT], auto has_d, auto has_z, auto out_f32) {
      to_rows(acc);
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int l = 32 * lb + it * RPI + rsub;
        const unsigned at = (unsigned)l * (unsigned)xrow + (unsigned)c4;
        float v[4];
        tile_row(it, v);
        if constexpr (decltype(has_d)::value) {
          float xv[4];
          load4_e<E>(at_bytes<const E>(xg, at * (unsigned)sizeof(E)), xv);
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = __builtin_fmaf(Dv4[j], xv[j], v[j]);
        }
        if constexpr (decltype(has_z)::value) {
          float zv[4];
          load4_e<E>(at_bytes<const E>(zg, at * (unsigned)sizeof(E)), zv);
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] *= silu_f32(zv[j]);
        }
        if constexpr (decltype(out_f32)::value) *at_bytes<float4>(yf, at * 4u) = make_float4(v[0], v[1], v[2], v[3]);
        else store4_e<E>(at_bytes<E>(yg, at * (unsigned)sizeof(E)), v);
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // read before the next tile is written over it
    };
    auto both = [&](auto has_d, auto has_z, auto out_f32) {
      if (has0) rows_y(wave, acc0, has_d, has_z, out_f32);
      if (has1) rows_y(nlb - 1 - wave, acc1, has_d, has_z, out_f32);
    };
    const int opts = (p.Dk ? 4 : 0) | (zg ? 2 : 0) | (y_f32 ? 1 : 0);
    switch (opts) {
      case 0: both(No{}, No{}, No{}); break;
      case 1: both(No{}, No{}, Yes{}); break;
      case 2: both(No{}, Yes{}, No{}); break;
      case 3: both(No{}, Yes{}, Yes{}); break;
      case 4: both(Yes{}, No{}, No{}); break;
      case 5: both(Yes{}, No{}, Yes{}); break;
      case 6: both(Yes{}, Yes{}, No{}); break;
      default: both(Yes{}, Yes{}, Yes{}); break;
    }
  }
}

static bool mfma_shape_ok(const SsdDims &d) {
  return d.len % d.chunk == 0 && d.chunk % 32 == 0 && d.chunk <= 256 && d.nstate % 16 == 0 &&
         (d.hdim == 32 || d.hdim == 64);
}

bool ssd_bmm_mfma(const SsdBmmParams &p, hipStream_t s) {
  // 16-bit operands of one type; the product in float32 or in the operands' type
  if (p.in_dtype != SSM_BF16 && p.in_dtype != SSM_F16) return false;
  if (p.out_dtype != SSM_F32 && p.out_dtype != p.in_dtype) return false;
  if (p.len % p.chunk != 0 || p.chunk % 32 != 0 || p.kdim % 16 != 0) return false;
  if (!aligned_to(p.a, 16) || !aligned_to(p.b, 16)) return false;
  const int tiles = (p.chunk + 63) / 64;
  const dim3 grid((unsigned)((size_t)p.batch * p.nchunks * p.groups * tiles * tiles)), block(MF_THREADS);
  if (p.in_dtype == SSM_BF16) {
    if (p.out_dtype == SSM_F32) hipLaunchKernelGGL((ssd_bmm_mfma_kernel<__bf16, float>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((ssd_bmm_mfma_kernel<__bf16, bf16_t>), grid, block, 0, s, p);
  } else {
    if (p.out_dtype == SSM_F32) hipLaunchKernelGGL((ssd_bmm_mfma_kernel<_Float16, float>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((ssd_bmm_mfma_kernel<_Float16, f16_t>), grid, block, 0, s, p);
  }
  return true;
}

size_t ssd_chunk_state_scratch_bytes(const SsdDims &d) {
  return (size_t)d.batch * d.groups * d.nstate * d.len * 2;
}

bool ssd_chunk_state_mfma(const SsdStateParams &p, hipStream_t s) {
  const SsdDims &d = p.d;
  const bool half = p.x_dtype == SSM_BF16 || p.x_dtype == SSM_F16;
  if (!mfma_shape_ok(d) || !half || p.b_dtype != p.x_dtype) return false;
  if (p.states_dtype != SSM_F32 && p.states_dtype != p.x_dtype) return false;
  if (!p.scratch || p.scratch_bytes < ssd_chunk_state_scratch_bytes(d)) return false;
  if (!aligned_to(p.x, 16) || !aligned_to(p.scratch, 16) || d.len % 8 != 0) return false;
  hipLaunchKernelGGL(ssd_transpose_kernel, dim3((d.len + 63) / 64, (d.nstate + 63) / 64, d.batch * d.groups),
                     dim3(MF_THREADS), 0, s, reinterpret_cast<const uint16_t *>(p.Bm), reinterpret_cast<uint16_t *>(p.scratch),
                     d.len, d.groups, d.nstate);
  const size_t lds = (size_t)d.hdim * (d.chunk + XT_PAD) * 2 + (size_t)d.chunk * 4;
  const unsigned grid = (unsigned)((size_t)d.batch * d.nchunks * d.heads);
#define SSM_LAUNCH_CS(E, ST, PT)                                                                           \
  {                                                                                                        \
    auto kernel = ssd_chunk_state_mfma_kernel<E, ST, PT>;                                                  \
    if (allow_dynamic_lds(kernel, lds) != hipSuccess) { (void)hipGetLastError(); return false; }           \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(MF_THREADS), lds, s, p, reinterpret_cast<const E *>(p.scratch)); \
  }
#define SSM_LAUNCH_CS_E(E, ST16)                                                                           \
  {                                                                                                        \
    if (p.states_dtype == SSM_F32) {                                                                       \
      if (d.hdim == 64) SSM_LAUNCH_CS(E, float, 2) else SSM_LAUNCH_CS(E, float, 1)                         \
    } else {                                                                                               \
      if (d.hdim == 64) SSM_LAUNCH_CS(E, ST16, 2) else SSM_LAUNCH_CS(E, ST16, 1)                           \
    }                                                                                                      \
  }
  if (p.x_dtype == SSM_BF16) SSM_LAUNCH_CS_E(__bf16, bf16_t)
  else SSM_LAUNCH_CS_E(_Float16, f16_t)
#undef SSM_LAUNCH_CS_E
#undef SSM_LAUNCH_CS
  return true;
}

bool ssd_chunk_scan_mfma(const SsdScanParams &p, hipStream_t s) {
  const SsdDims &d = p.d;
  const bool half = p.x_dtype == SSM_BF16 || p.x_dtype == SSM_F16;
  if (!mfma_shape_ok(d) || !half || p.c_dtype != p.x_dtype || p.cb_dtype != p.x_dtype) return false;
  if ((p.states_dtype != SSM_F32 && p.states_dtype != p.x_dtype) || (p.z && p.z_dtype != p.x_dtype)) return false;
  if (p.y_dtype != SSM_F32 && p.y_dtype != p.x_dtype) return false;
  if (!aligned_to(p.x, 16) || !aligned_to(p.Cm, 16) || !aligned_to(p.CB, 16) || !aligned_to(p.prev, 16)) return false;
  // the epilogue moves four channels at a time
  if ((p.y && !aligned_to(p.y, 16)) || (p.z && !aligned_to(p.z, 8))) return false;
  if (p.dx.dx && (!aligned_to(p.dx.dx, 16) || !aligned_to(p.dx.x, 8))) return false;
  if ((p.Dk && p.d_per_p && !aligned_to(p.Dk, 16)) || (p.dx.dx && p.dx.Dk && p.dx.d_per_p && !aligned_to(p.dx.Dk, 16))) return false;
  size_t lds = (size_t)d.hdim * (d.chunk + XT_PAD) * 2 + (size_t)d.chunk * 12 + (size_t)d.hdim * (d.nstate + 8) * 2;
  // afterwards the same memory holds a tile of 32 rows per wave that has row blocks (two each: chunk <= 256)
  const size_t tiles = (size_t)((d.chunk / 32 + 1) / 2) * 32 * (d.hdim + 4) * 4;
  if ((d.chunk / 32 + 1) / 2 > MF_WAVES) return false;
  if (p.x_reversed && p.Dk) return false;            // the skip term reads x at the call's own rows
  if ((size_t)d.chunk * d.heads * d.hdim * 4 >= ((size_t)1 << 31)) return false;     // a chunk's rows in 32-bit byte offsets
  if (lds < tiles) lds = tiles;
  const unsigned grid = (unsigned)((size_t)d.batch * d.nchunks * d.heads);
  if (p.dx.dx) {
    // the backward's own call: bfloat16 operands, float32 states, nothing of the forward's epilogue
    if (p.x_dtype != SSM_BF16 || p.states_dtype != SSM_F32 || p.z || p.Dk || p.seq_idx) return false;
#define SSM_LAUNCH_DX(PT, MODE)                                                                            \
  {                                                                                                        \
    auto kernel = ssd_chunk_scan_mfma_kernel<__bf16, float, PT, MODE>;                                     \
    if (allow_dynamic_lds(kernel, lds) != hipSuccess) { (void)hipGetLastError(); return false; }           \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(MF_THREADS), lds, s, p);                                   \
  }
    if (d.hdim == 64) { if (p.dx.dx_f32) SSM_LAUNCH_DX(2, 2) else SSM_LAUNCH_DX(2, 1) }
    else { if (p.dx.dx_f32) SSM_LAUNCH_DX(1, 2) else SSM_LAUNCH_DX(1, 1) }
#undef SSM_LAUNCH_DX
    return true;
  }
#define SSM_LAUNCH_SC(E, ST, PT)                                                                           \
  {                                                                                                        \
    auto kernel = ssd_chunk_scan_mfma_kernel<E, ST, PT>;                                                   \
    if (allow_dynamic_lds(kernel, lds) != hipSuccess) { (void)hipGetLastError(); return false; }           \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(MF_THREADS), lds, s, p);                                   \
  }
#define SSM_LAUNCH_SC_E(E, ST16)                                                                           \
  {                                                                                                        \
    if (p.states_dtype == SSM_F32) {                                                                       \
      if (d.hdim == 64) SSM_LAUNCH_SC(E, float, 2) else SSM_LAUNCH_SC(E, float, 1)                         \
    } else {                                                                                               \
      if (d.hdim == 64) SSM_LAUNCH_SC(E, ST16, 2) else SSM_LAUNCH_SC(E, ST16, 1)                           \
    }                                                                                                      \
  }
  if (p.x_dtype == SSM_BF16) SSM_LAUNCH_SC_E(__bf16, bf16_t)
  else SSM_LAUNCH_SC_E(_Float16, f16_t)
#undef SSM_LAUNCH_SC_E
#undef SSM_LAUNCH_SC
  return true;
}

}  // namespace ssm

extern "C" int ssm_ssd_bwd_dcb(const ssm_ssd_bwd_dcb_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_ssd_bwd_dcb: args is NULL");
  SSM_REQUIRE(a->dy && a->x && a->dt && a->dA_cumsum && a->dCB, SSM_ERR_NULL_POINTER,
              "ssm_ssd_bwd_dcb: dy, x, dt, dA_cumsum and dCB are required");
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->groups > 0 && a->chunk > 0 && a->heads % a->groups == 0,
              SSM_ERR_BAD_SHAPE, "ssm_ssd_bwd_dcb: sizes must be positive and groups must divide heads");
  SSM_REQUIRE(a->headdim == 32 || a->headdim == 64, SSM_ERR_BAD_SHAPE, "ssm_ssd_bwd_dcb: headdim=%d, supported: 32, 64",
              a->headdim);
  SSM_REQUIRE(a->chunk % 32 == 0 && a->seqlen % a->chunk == 0, SSM_ERR_BAD_SHAPE,
              "ssm_ssd_bwd_dcb: chunk=%d must be a multiple of 32 and divide seqlen=%d", a->chunk, a->seqlen);
  SSM_REQUIRE(aligned_to(a->dy, 16) && aligned_to(a->x, 16) && aligned_to(a->dA_cumsum, 16) && aligned_to(a->dt, 4) &&
                  aligned_to(a->dCB, 4),
              SSM_ERR_ALIGNMENT, "ssm_ssd_bwd_dcb: dy, x and dA_cumsum must be 16-byte aligned");
  SsdDcbParams p{};
  p.dy = reinterpret_cast<const __bf16 *>(a->dy);
  p.x = reinterpret_cast<const __bf16 *>(a->x);
  p.dt = a->dt; p.dA_cs = a->dA_cumsum; p.out = a->dCB;
  p.batch = a->batch; p.len = a->seqlen; p.heads = a->heads; p.hdim = a->headdim; p.groups = a->groups;
  p.chunk = a->chunk; p.nchunks = a->seqlen / a->chunk;
  const int nb = p.chunk / 32;
  const size_t grid = (size_t)p.batch * p.nchunks * p.groups * (nb * (nb + 1) / 2);
  SSM_REQUIRE(grid < ((size_t)1 << 31), SSM_ERR_TOO_LARGE, "ssm_ssd_bwd_dcb: too many blocks");
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  if (p.hdim == 64) hipLaunchKernelGGL(ssd_bwd_dcb_kernel<4>, dim3((unsigned)grid), dim3(MF_THREADS), 0, s, p);
  else hipLaunchKernelGGL(ssd_bwd_dcb_kernel<2>, dim3((unsigned)grid), dim3(MF_THREADS), 0, s, p);
  SSM_CHECK_LAUNCH("ssm_ssd_bwd_dcb");
  return SSM_OK;
}
