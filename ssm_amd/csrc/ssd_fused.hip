// Mamba-2 SSD forward as one pass over the sequence: a workgroup owns 32 channels
// (half a head) of one (batch, head), walks its chunks in order and keeps the running
// state S (32 x N, fp32) in MFMA accumulators, so neither the per-chunk states nor
// the state entering each chunk ever travel through HBM.
//
// Per chunk (Q steps, 32-step blocks lb = 0 .. Q/32-1, e_k = last step of block k,
// cs[l] = running sum of dt A inside the chunk, cs[e_-1] := 0):
//
//   y_l = exp(cs_l) C_l.S  +  sum_{s<=l} CB[l,s] exp(cs_l - cs_s) dt_s x_s  (+ D x_l, gate)
//
// Only the 32x32 blocks on the diagonal need a decay factor per element.  For a
// block of earlier steps the factor splits into three pieces that are all <= 1,
//   exp(cs_l - cs_s) = exp(cs_l - cs[e_{lb-1}]) . exp(cs[e_{lb-1}] - cs[e_sb]) . exp(cs[e_sb] - cs_s),
// a per-row factor applied once to the accumulator, a per-block scalar applied
// as the accumulator moves from one block of s to the next (acc = acc * g_sb + CB_blk x~_blk
// with g_k = exp(cs[e_k] - cs[e_{k-1}])), and a per-step weight folded with dt
// into the staged operand x~_s = x_s dt_s exp(cs[e_sb] - cs_s).  The carried state
// enters the same recurrence as its first term.  The state update
//   S <- S * g_k + x~_blk^T B_blk          for k = 0 .. Q/32-1
// uses the same x~ tile and ends each chunk with S decayed by exp(cs[Q-1]).
//
// B, C and CB are re-laid once per call so that every MFMA operand fragment is
// one contiguous KiB (64 lanes x 8 bf16).
//
// Requires bf16 or fp16 tensors (the kernels are compiled per element type), P = 64, Q in {64, 128, 256}, N in {64, 128} and L % Q == 0.
//
// A head with A > 0 (a growing state): the published kernels evaluate the decays inside a chunk as
// exp(min(x, 0)) - chunk_state's weights and chunk_scan's in-chunk factors - and leave the two factors on the
// carried state alone (exp(cs_l) on C_l.S, exp(cs[Q-1]) in state passing).  Steps are not negative, so all
// running-sum differences of such a head are >= 0 and every factor of the split above, bounded by 1 one by
// one, is exactly 1, as the clamp wants; what remains is to apply the unclamped growth to the carried state,
// once per chunk in front of the state update and once per row on the carried term.  The sign of A is read
// per head inside the kernel: no call depends on the host having looked at the values of A.
#include "ssd_common.hpp"

namespace ssm {

constexpr int FU_P = 64;
constexpr int FRAG = 512;                                  // bf16 elements per operand fragment

struct SsdFusedParams {                 // x, z, y and the fragment copies hold the call's 16-bit element type
  const void *x, *z;
  void *y;
  const float *dA2, *dtv;               // (B,H,nc,Q): log2-scaled running sum, step
  const void *Cblk, *Btblk, *CBblk;     // fragment-blocked copies
  const float *Dk, *init, *A;
  float *final_states;
  int batch, len, heads, groups, nstate, chunk, nchunks, d_per_p;
};

template <typename E> struct Vec4;
template <> struct Vec4<__bf16> { typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 type; };
template <> struct Vec4<_Float16> { typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 type; };
template <typename E> using V4 = typename Vec4<E>::type;

__device__ __forceinline__ void wave_lds_sync() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// ---------------------------------------------------------------------- prep
// One launch prepares everything the fused kernel reads besides x and z; the
// workgroups (256 threads) take one of three roles by their index:
//
//  dt:   one workgroup per (b, c, 4 heads).  The (Q x 4) slab of dt is read row by
//        row (16 contiguous bytes per step) into LDS transposed to [head][step];
//        then one wave per head forms dt' = clamp(softplus(dt + bias)) and the
//        running sum of dt' A (stored scaled by log2 e, the unit of the fused
//        kernel's exponentials).
//  pack: one wave per operand fragment of C and B^T.  Fragment (lane, j) of a
//        32 x 16 block: row 32 rb + lane % 32, column 16 kb + 8 (lane / 32) + j.
//          Cblk [(b,c,g)][lb][kn]  from C  (rows = time, columns = state)
//          Btblk[(b,c,g)][ks][nt]  from B  (rows = state, columns = time)
//  CB:   one wave per 32 x 32 block on or below the diagonal of C B^T of a chunk:
//        MFMA over the state dimension, then through a wave-private LDS tile into
//          CBblk[(b,c,g)][lb][ks]  (rows = l, columns = s),
//        with zeros above the diagonal inside the diagonal blocks.
constexpr int PD_HEADS = 4;
struct SsdPrepParams {
  SsdCumsumParams cs;
  float *dA2;
  const void *Cm, *Bm;                   // element type of the call
  void *Cblk, *Btblk, *CBblk;
  unsigned n_dt, n_pack;                 // workgroups of the first two roles
  const int *seq_idx;                    // (B, L) sequence ids of a packed batch, or null
  size_t b_row, c_row;                   // elements between the (G, N) blocks of consecutive steps in Bm / Cm
};

// Packed sequences: the first step of a sequence gets an extra decay of 2^-64 (a jump in the running sum),
// so that nothing of the sequences before it - state or in-chunk terms - reaches it or the steps after it:
// exp2(cs_l - cs_s) then carries that factor whenever a boundary lies in (s, l].  The steps of one sequence
// see the same jumps on both sides of the difference; with every step of a 256-step chunk a boundary the sum
// reaches 2^14, where float32 still resolves 1e-3 of the exponent.
constexpr float SEQ_JUMP_LN = -64.0f * 0.69314718056f;

__device__ __forceinline__ void prep_dt_role(const SsdCumsumParams &p, float *dA2, const int *seq_idx, int wg, float *lds) {
  float (*tile)[256 + 1] = reinterpret_cast<float (*)[256 + 1]>(lds);
  const SsdDims &d = p.d;
  const int Q = d.chunk;
  const int hgroups = (d.heads + PD_HEADS - 1) / PD_HEADS;
  const int hg = wg % hgroups;
  const int c = (wg / hgroups) % d.nchunks;
  const int b = wg / (hgroups * d.nchunks);
  const int h0 = hg * PD_HEADS;
  for (int e = threadIdx.x; e < Q * PD_HEADS; e += 256) {
    const int l = e / PD_HEADS, hh = e % PD_HEADS;
    float v = 0.0f;
    if (h0 + hh < d.heads) v = load_as_f32(p.dt, p.dt_dtype, ((size_t)b * d.len + (size_t)c * Q + l) * d.heads + h0 + hh);
    tile[hh][l] = v;
  }
  __syncthreads();
  const int wave = wave_id_uniform(), lane = lane_id();
  const int per = (Q + 63) >> 6;
  for (int hh = wave; hh < PD_HEADS; hh += 4) {
    const int h = h0 + hh;
    if (h >= d.heads) break;
    const float A = p.A[h];
    const float bias = p.bias ? p.bias[h] : 0.0f;
    float v[4], run[4];
    float tot = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int l = lane * per + i;
      v[i] = 0.0f;
      if (i < per && l < Q) {
        float x = tile[hh][l] + bias;
        if (p.softplus) x = softplus_f32(x);
        v[i] = fminf(fmaxf(x, p.dt_min), p.dt_max);
      }
      tot = __builtin_fmaf(v[i], A, tot);
      if (seq_idx && i < per && l < Q) {
        const size_t t = (size_t)c * Q + l;
        const int *sid = seq_idx + (size_t)b * d.len;
        if (t == 0 ? sid[0] != 0 : sid[t] != sid[t - 1]) tot += SEQ_JUMP_LN;
      }
      run[i] = tot;
    }
    float incl = tot;
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) {
      const float t = __shfl_up(incl, off, WAVE);
      if (lane >= off) incl += t;
    }
    const float excl = incl - tot;
    const size_t out = (((size_t)b * d.heads + h) * d.nchunks + c) * (size_t)Q;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int l = lane * per + i;
      if (i < per && l < Q) {
        p.dt_out[out + l] = v[i];
        dA2[out + l] = (excl + run[i]) * LOG2E;
      }
    }
  }
}

template <typename E>
__device__ __forceinline__ void prep_pack_role(const SsdPrepParams &pp, unsigned wg) {
  const E *Cm = reinterpret_cast<const E *>(pp.Cm), *Bm = reinterpret_cast<const E *>(pp.Bm);
  const SsdDims &d = pp.cs.d;
  const int wave = wave_id_uniform(), lane = lane_id();
  const int Q = d.chunk, N = d.nstate, nc = d.nchunks, groups = d.groups, len = d.len;
  const int NLB = Q >> 5, KS = Q >> 4, KN = N >> 4, NT = N >> 5;
  const size_t units = (size_t)d.batch * nc * groups;
  const size_t nC = units * NLB * KN, nB = units * KS * NT;
  size_t f = (size_t)wg * 4 + wave;
  if (f >= nC + nB) return;
  const bool is_c = f < nC;
  if (!is_c) f -= nC;
  const int per_unit = is_c ? NLB * KN : KS * NT;
  const int inner = (int)(f % per_unit);
  const size_t unit = f / per_unit;
  const int g = (int)(unit % groups);
  const int c = (int)((unit / groups) % nc);
  const int b = (int)(unit / ((size_t)groups * nc));
  const int m = lane & 31, g2 = lane >> 5;
  V8<E> v;
  if (is_c) {
    const int lb = inner / KN, kn = inner % KN;
    v = load_frag_e<E>(Cm + ((size_t)b * len + (size_t)c * Q + 32 * lb + m) * pp.c_row + (size_t)g * N + 16 * kn + 8 * g2);
  } else {
    const int ks = inner / NT, nt = inner % NT;
    const E *col = Bm + ((size_t)b * len + (size_t)c * Q + 16 * ks + 8 * g2) * pp.b_row + (size_t)g * N + 32 * nt + m;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = col[(size_t)j * pp.b_row];
  }
  *reinterpret_cast<V8<E> *>(reinterpret_cast<E *>(is_c ? pp.Cblk : pp.Btblk) + f * FRAG + lane * 8) = v;
}

template <typename E>
__device__ __forceinline__ void prep_cb_role(const SsdPrepParams &pp, unsigned wg, float *lds) {
  const SsdDims &d = pp.cs.d;
  const int wave = wave_id_uniform(), lane = lane_id();
  const int Q = d.chunk, N = d.nstate, groups = d.groups;
  const int NLB = Q >> 5, KS = Q >> 4;
  const int per_unit = NLB * (NLB + 1) / 2;
  const size_t units = (size_t)d.batch * d.nchunks * groups;
  const size_t blk = (size_t)wg * 4 + wave;
  if (blk >= units * per_unit) return;
  const size_t unit = blk / per_unit;
  const int idx = (int)(blk % per_unit);
  int lb = 0;
  while ((lb + 1) * (lb + 2) / 2 <= idx) ++lb;
  const int sb = idx - lb * (lb + 1) / 2;
  const int g = (int)(unit % groups);
  const size_t bc = unit / groups;                        // b * nchunks + c: the chunk's first row is bc * Q
  const int m = lane & 31, g2 = lane >> 5;
  const E *crow_p = reinterpret_cast<const E *>(pp.Cm) + (bc * Q + 32 * lb + m) * pp.c_row + (size_t)g * N + 8 * g2;
  const E *brow_p = reinterpret_cast<const E *>(pp.Bm) + (bc * Q + 32 * sb + m) * pp.b_row + (size_t)g * N + 8 * g2;
  f32x16_t acc = {0};
  for (int k0 = 0; k0 < N; k0 += 16) acc = mma(load_frag_e<E>(crow_p + k0), load_frag_e<E>(brow_p + k0), acc);
  float (*tile)[33] = reinterpret_cast<float (*)[33]>(lds + wave * 32 * 33);
#pragma unroll
  for (int r = 0; r < 16; ++r) tile[crow(r, g2)][m] = acc[r];
  wave_lds_sync();
  E *out = reinterpret_cast<E *>(pp.CBblk) + ((unit * NLB + lb) * KS + 2 * sb) * FRAG + lane * 8;
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int sl = 16 * kk + 8 * g2 + j;
      v[j] = (sb < lb || sl <= m) ? tile[m][sl] : 0.0f;
    }
    *reinterpret_cast<V8<E> *>(out + kk * FRAG) = pack8_e<E>(v);
  }
}

template <typename E>
__global__ __launch_bounds__(256) void ssd_fused_prep_kernel(const SsdPrepParams pp) {
  __shared__ float lds[4 * 32 * 33];
  const unsigned wg = blockIdx.x;
  if (wg < pp.n_dt) prep_dt_role(pp.cs, pp.dA2, pp.seq_idx, (int)wg, lds);
  else if (wg < pp.n_dt + pp.n_pack) prep_pack_role<E>(pp, wg - pp.n_dt);
  else prep_cb_role<E>(pp, wg - pp.n_dt - pp.n_pack, lds);
}

// ------------------------------------------------- fused kernel, half a head
// One workgroup of 4 waves walks the chunks of 32 channels (half a head): blockIdx ->
// (b, h, half).  Per chunk:
//   barrier; the carried state S goes to LDS as bf16 and the chunk's x, already in
//     registers, is staged twice, plain and weighted, transposed to [p][s];
//   barrier; Y = C S (carried state), then the blocks of (CB o decay) X below and on the
//     diagonal for this wave's two row blocks;
//   barrier; requests for z, and for the next chunk's x, dt and running sums, go out (the
//     only reads that come from HBM: they are grouped so that the wave meets their
//     latency once); S <- S g + B^T X~; skip term, gate and the store of Y.
// Wave w owns the row blocks NLB - 1 - w and w (every wave the same number of blocks
// below the diagonal) and the n-tile w of S^T.  Its fragments of C, CB and B^T form one
// stream (C for both row blocks, CB of the first row block, CB of the second, B^T) that
// runs through a ring of four registers; a register is refilled right after its use with
// the fragment four places on, across the phases and into the next chunk.
// All global accesses are buffer accesses: the lane's part of the address is a 32-bit
// offset that does not change, the rest is scalar.
constexpr int FH_THREADS = 256;
constexpr int FH_TILE_BYTES = 16384;                       // [32][256] bf16
constexpr int FH_LDS_BYTES = 3 * FH_TILE_BYTES + 4 * 256 * 4;

typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2_t;

// 2 GiB window from p on; accesses carry byte offsets below that.
__device__ __forceinline__ rsrc_t make_rsrc(const void *p) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, 0x7fffffff, 0x00020000);
}
template <typename E>
__device__ __forceinline__ V8<E> buf_load16(rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(V8<E>, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
template <typename E>
__device__ __forceinline__ V4<E> buf_load8(rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(V4<E>, __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0));
}
__device__ __forceinline__ float4 buf_load_f4(rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
__device__ __forceinline__ float buf_load_f1(rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}

// Where the part of a wave's fragment stream after the fragments of C lies: byte offsets from Cblk.
struct HalfStream {
  rsrc_t r;
  int vf;                    // lane * 16
  int n_first, n_both;       // fragments of CB of the first row block, of both
  int off_first, off_second, off_bt, bt_step;
};
// Places i (even) and i + 1 of the stream; both lie in the same part of it.
template <typename E>
__device__ __forceinline__ void stream_pair(const HalfStream &st, int i, V8<E> &fa, V8<E> &fb) {
  const int o1 = st.off_first + (i << 10);
  const int o2 = st.off_second + ((i - st.n_first) << 10);
  const int o3 = st.off_bt + (i - st.n_both) * st.bt_step;
  const bool in1 = i < st.n_first, in2 = i < st.n_both;
  const int o12 = in1 ? o1 : o2;
  const int off = in2 ? o12 : o3;
  const int step = in2 ? 1024 : st.bt_step;
  fa = buf_load16<E>(st.r, st.vf, off);
  fb = buf_load16<E>(st.r, st.vf, off + step);
}

// Blocks below the diagonal and the diagonal block of row block `lb` into `acc` (one 32 x 32
// tile: lane = column l, registers = rows p).  The fragments of block sb are the stream's places
// pos0 + 2 sb, + 1; (a0, a1) is the register pair that holds those of the diagonal block and of
// every second block before it, (b0, b1) the other pair.
// With SKIP, the per-head skip factor dskip joins the diagonal of the last operand (CB dt + D at
// s = l, rounded to bf16 as one number), so that the product with the plain x adds D x.
template <typename E, bool SKIP>
__device__ __forceinline__ void half_row_block(f32x16_t &acc, V8<E> &a0, V8<E> &a1, V8<E> &b0, V8<E> &b1,
                                               int lb, int pos0, const HalfStream &st, const E *xw, const E *xr,
                                               const float *dAs, const float *dqs, const float *l2s, int Q, int qmask,
                                               int m, int g2, float dskip) {
  float prev_end = 0.0f;
  const int lrow = 32 * lb + m;
  const float dal = dAs[lrow];
#define FH_BLOCK(FA, FB, SB)                                                                    \
  {                                                                                             \
    const float endv = dAs[32 * (SB) + 31];                                                     \
    const float gs = exp2_hw(fminf(endv - prev_end, 0.0f));                                     \
    prev_end = endv;                                                                            \
    _Pragma("unroll") for (int r = 0; r < 16; ++r) acc[r] *= gs;                                \
    const V8<E> x0 = load_frag_e<E>(xw + m * Q + (((4 * (SB) + g2) ^ (m & qmask)) << 3));       \
    const V8<E> x1 = load_frag_e<E>(xw + m * Q + (((4 * (SB) + 2 + g2) ^ (m & qmask)) << 3));   \
    acc = mma(x0, FA, acc);                                                                     \
    acc = mma(x1, FB, acc);                                                                     \
    stream_pair<E>(st, pos0 + 2 * (SB) + 4, FA, FB);                                            \
  }
  const int odd = lb & 1;
  if (odd) FH_BLOCK(b0, b1, 0)
  for (int sb0 = odd; sb0 < lb; sb0 += 2) {
    FH_BLOCK(a0, a1, sb0)
    FH_BLOCK(b0, b1, sb0 + 1)
  }
#undef FH_BLOCK
  const float rf = exp2_hw(fminf(dal - prev_end, 0.0f));
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] *= rf;
  // the diagonal block: its fragments of CB hold zeros above the diagonal, so that the decay
  // only needs a bound there
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    const V8<E> f = kk == 0 ? a0 : a1;
    const int sbase = 32 * lb + 16 * kk + 8 * g2;
    const float4 q0 = *reinterpret_cast<const float4 *>(dqs + sbase), q1 = *reinterpret_cast<const float4 *>(dqs + sbase + 4);
    const float4 c0 = *reinterpret_cast<const float4 *>(l2s + sbase), c1 = *reinterpret_cast<const float4 *>(l2s + sbase + 4);
    const float dq[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    const float cap[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    float mv[8];
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
      // dt_s exp(min(cs_l - cs_s, 0)) as one exponential: min(a, 0) + b = min(a + b, b) with b = log2 dt_s.  The
      // bound is inactive on and below the diagonal of a decaying head, is the clamp of a growing one, and keeps
      // the (zeroed) places above the diagonal finite.
      const float e = exp2_hw(fminf(dal + dq[jj], cap[jj]));
      if (SKIP) {
        // (CB dt + D at s = l, rounded to the element type as one number)
        // element jj of fragment kk lies on the diagonal in lane 16 kk + jj (g2 = 0) and lane 32 + 16 kk + 8 + jj (g2 = 1)
        const unsigned long long on_diag = (1ull << (16 * kk + jj)) | (1ull << (40 + 16 * kk + jj));
        float sel;
        asm volatile("v_cndmask_b32_e64 %0, 0, %1, %2" : "=v"(sel) : "v"(dskip), "s"(on_diag));   // volatile: rebuilt at each use, not kept
        mv[jj] = __builtin_fmaf((float)f[jj], e, sel);
      } else {
        mv[jj] = (float)f[jj] * e;
      }
    }
    const V8<E> a = load_frag_e<E>(xr + m * Q + (((4 * lb + 2 * kk + g2) ^ (m & qmask)) << 3));
    acc = mma(a, pack8_e<E>(mv), acc);
  }
  stream_pair<E>(st, pos0 + 2 * lb + 4, a0, a1);
}

// acc[p][l] += D[p] x[l][p] for row block lb, x read from the plain tile (per-channel skip factors).
template <typename E>
__device__ __forceinline__ void half_skip_term(f32x16_t &acc, int lb, const E *xr, int Q, int qmask, int m, int g2,
                                               const float *Dp) {
  const int lrow = 32 * lb + m;
  const int xcol = lrow & 7, xchunk = lrow >> 3;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 d4 = *reinterpret_cast<const float4 *>(Dp + 8 * q + 4 * g2);
    const float dv[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int prow = 8 * q + 4 * g2 + j;
      const float xv = (float)xr[prow * Q + ((xchunk ^ (prow & qmask)) << 3) + xcol];
      acc[4 * q + j] = __builtin_fmaf(dv[j], xv, acc[4 * q + j]);
    }
  }
}

template <typename E, int Q, int N, int DMODE, bool HAS_Z>
__global__ __launch_bounds__(FH_THREADS) __attribute__((amdgpu_waves_per_eu(3, 3)))
void ssd_fused_half_kernel(const SsdFusedParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  E *xw = reinterpret_cast<E *>(smem);                                  // x~ [32][Q]
  E *xr = reinterpret_cast<E *>(smem + FH_TILE_BYTES);                  // x  [32][Q]
  E *sbf = reinterpret_cast<E *>(smem + 2 * FH_TILE_BYTES);             // S in 16 bits [32][N]; later the output staging
  float *dAs = reinterpret_cast<float *>(smem + 3 * FH_TILE_BYTES);     // [Q] log2-scaled running sum
  float *dqs = dAs + 256;                                               // [Q] log2(dt) - running sum: exponent offset of a step as a source
  float *wss = dqs + 256;                                               // [Q] staging weight dt exp(cs[l | 31] - cs[l])
  float *l2s = wss + 256;                                               // [Q] log2(dt): the bound of a source step's exponent

  const int H = p.heads, G = p.groups, nc = p.nchunks;
  constexpr int NLB = Q >> 5, NT = N >> 5, KS = Q >> 4, KN = N >> 4;
  constexpr int qmask = Q >= 128 ? 15 : (Q >> 3) - 1, nmask = N >= 128 ? 15 : (N >> 3) - 1;
  const int wave = wave_id_uniform(), lane = lane_id();
  const int g2 = lane >> 5, m = lane & 31;
  // Workgroups go to the 8 XCDs round-robin by blockIdx: renumber them so that each XCD (own L2)
  // works on neighbouring heads of one batch row, which stream the same fragments of C, B and CB.
  int vid = (int)blockIdx.x;
  if ((gridDim.x & 7) == 0) vid = (vid & 7) * (int)(gridDim.x >> 3) + (vid >> 3);
  const int half = vid & 1;
  const int h = (vid >> 1) % H, b = (vid >> 1) / H;
  const int g = h / (H / G);
  const int p0 = 32 * half;
  // with four or more pairs of row blocks (state tiles) every wave has some: say so at compile time, the
  // waits for loads are exact only on straight-line code
  const bool yact = (NLB >> 1) >= 4 ? true : wave < (NLB >> 1);
  const int lbF = NLB - 1 - wave, lbS = wave;          // first: many blocks below the diagonal, second: few
  const int nt_s = wave;
  const bool sact = NT >= 4 ? true : nt_s < NT;
  const bool has_init = p.init != nullptr;
  const int xrow_b = H * FU_P * 2;                     // bytes between rows of x, z and y
  const float dhead = DMODE == 1 ? p.Dk[h] : 0.0f;
  const bool grow = p.A[h] > 0.0f;                     // a growing state: see the head of this file
  const int tid = wave * WAVE + lane;

  // ---- buffers and the lanes' constant offsets
  const size_t xbase = ((size_t)b * p.len * H + h) * FU_P + p0;
  const E *px = reinterpret_cast<const E *>(p.x);
  const rsrc_t rx = make_rsrc(px + xbase), ry = make_rsrc(reinterpret_cast<E *>(p.y) + xbase);
  const rsrc_t rz = make_rsrc(HAS_Z ? reinterpret_cast<const E *>(p.z) + xbase : px + xbase);
  const size_t tbase = ((size_t)b * H + h) * nc * Q;   // dA2 and dtv are laid out alike
  const rsrc_t rt = make_rsrc(p.dtv + tbase);
  const int t_dA = (int)((const char *)p.dA2 - (const char *)p.dtv);
  const rsrc_t rf = make_rsrc(p.Cblk);
  const int f_cb = (int)((const char *)p.CBblk - (const char *)p.Cblk), f_bt = (int)((const char *)p.Btblk - (const char *)p.Cblk);
  const int srow = min(tid >> 3, (Q >> 3) - 1) * 8, spb = tid & 7;
  const int v_raw = srow * xrow_b + spb * 8;                       // x for staging: rows srow.., 4 channels
  const int v_row = (lane >> 2) * xrow_b + (lane & 3) * 16;        // row-major passes: row lane / 4, 8 channels
  const int v_t = min(tid, Q - 1) * 4;
  HalfStream st;
  st.r = rf;
  st.vf = lane * 16;
  st.bt_step = NT << 10;
  // waves without row blocks start two places on, so that the state update finds the ring alike
  st.n_first = yact ? 2 * lbF + 2 : 0;
  st.n_both = yact ? 2 * NLB + 2 : 2;

  f32x16_t S = {0};
  if (sact && has_init) {
    const float *ip = p.init + (((size_t)b * H + h) * FU_P + p0 + m) * N + 32 * nt_s;
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = ip[crow(r, g2)];
  }
  f32x16_t accF, accS;
  V8<E> f0, f1, f2, f3;
  // what a chunk reads from HBM, requested one chunk ahead: x, dt and the running sums
  V4<E> raw[8];
  float dA_t, dt_t;
#define FH_REQUEST_CHUNK(CC)                                                                              \
  {                                                                                                       \
    const int xo_ = (CC) * Q * xrow_b, to_ = (CC) * Q * 4;                                                \
    _Pragma("unroll") for (int r = 0; r < 8; ++r) raw[r] = buf_load8<E>(rx, v_raw, xo_ + r * xrow_b);        \
    dA_t = buf_load_f1(rt, v_t, t_dA + to_);                                                              \
    dt_t = buf_load_f1(rt, v_t, to_);                                                                     \
  }
  // fragments of C of chunk CC: (f0, f1) = (first, second row block) at kn = 0, (f2, f3) at kn = 1
#define FH_C_OFF(CC, LB, KNI) ((((((b * nc + (CC)) * G + g) * NLB + (LB)) * KN + (KNI))) << 10)
  FH_REQUEST_CHUNK(0)
  if (yact && has_init) {
    f0 = buf_load16<E>(rf, st.vf, FH_C_OFF(0, lbF, 0));
    f1 = buf_load16<E>(rf, st.vf, FH_C_OFF(0, lbS, 0));
    f2 = buf_load16<E>(rf, st.vf, FH_C_OFF(0, lbF, 1));
    f3 = buf_load16<E>(rf, st.vf, FH_C_OFF(0, lbS, 1));
  }

  for (int c = 0; c < nc; ++c) {
    // LDS addresses are rebuilt from the lane number in every chunk: kept across chunks they would
    // occupy more registers than they cost to recompute
    // The SIMD serves its oldest wave first: left alone, the workgroup that came to a CU last would run
    // at the lowest rate throughout and finish long after the others.  Rotating the priority with the
    // chunk number shares the CU evenly (slot = presumably the n-th workgroup on its CU).
    {
      const int pr = (c + ((int)blockIdx.x >> 3) / 32) % 3;
      if (pr == 0) __builtin_amdgcn_s_setprio(0);
      else if (pr == 1) __builtin_amdgcn_s_setprio(1);
      else __builtin_amdgcn_s_setprio(2);
    }
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int lane = ln, g2 = ln >> 5, m = ln & 31, tid = wave * WAVE + ln;
    const int spb = tid & 7, slb8 = tid >> 3;
    const int unit = (b * nc + c) * G + g;
    const bool carry = c > 0 || has_init;
    st.off_first = f_cb + (((unit * NLB + lbF) * KS) << 10);
    st.off_second = yact ? f_cb + (((unit * NLB + lbS) * KS) << 10) : f_bt + (((unit * KS) * NT + min(nt_s, NT - 1)) << 10);
    st.off_bt = f_bt + (((unit * KS) * NT + min(nt_s, NT - 1)) << 10);

    __syncthreads();                       // previous chunk: every read of the tiles and the output staging are over
    if (sact && carry) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        V4<E> v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = (E)S[4 * q + j];
        const int chunk16 = 4 * nt_s + q;
        *reinterpret_cast<V4<E> *>(sbf + m * N + ((chunk16 ^ (m & nmask)) << 3) + 4 * g2) = v;
      }
    }
    if (tid < Q) {                         // whole waves: Q is a multiple of 64
      // weight of a step towards the end of its block of 32: the running sum there is in lane | 31
      const float w_t = dt_t * exp2_hw(fminf(__shfl(dA_t, lane | 31, WAVE) - dA_t, 0.0f));
      const float l2_t = log2_hw(dt_t);    // dt = 0: -inf, a weight of zero
      dAs[tid] = dA_t;
      dqs[tid] = l2_t - dA_t;
      l2s[tid] = l2_t;
      wss[tid] = w_t;
      wave_lds_sync();                     // the eight weights this thread needs come from its own wave
      const float4 wa = *reinterpret_cast<const float4 *>(wss + slb8 * 8), wb = *reinterpret_cast<const float4 *>(wss + slb8 * 8 + 4);
      const float w8[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
      // ---- stage x~ and x, transposed to [p][s]
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        V8<E> colw, colr;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          colr[r] = raw[r][i];
          colw[r] = (E)((float)raw[r][i] * w8[r]);
        }
        const int prow = spb * 4 + i;
        const int at = prow * Q + ((slb8 ^ (prow & qmask)) << 3);
        *reinterpret_cast<V8<E> *>(xw + at) = colw;
        *reinterpret_cast<V8<E> *>(xr + at) = colr;
      }
    }
    __syncthreads();

    // ---- carried state: acc[p][l] = sum_n S[p][n] C[l][n] for both row blocks
    if (yact && carry) {
      const int cF = FH_C_OFF(c, lbF, 0), cS = FH_C_OFF(c, lbS, 0);
#define FH_STEP_A(FF, FS, KK)                                                                     \
      {                                                                                           \
        const V8<E> a = load_frag_e<E>(sbf + m * N + (((2 * (KK) + g2) ^ (m & nmask)) << 3));     \
        accF = mma(a, FF, accF);                                                                  \
        accS = mma(a, FS, accS);                                                                  \
      }
      {                                    // the first step starts the accumulators
        const V8<E> a = load_frag_e<E>(sbf + m * N + ((g2 ^ (m & nmask)) << 3));
        accF = mma(a, f0, (f32x16_t){0});
        accS = mma(a, f1, (f32x16_t){0});
        f0 = buf_load16<E>(rf, st.vf, cF + (2 << 10));
        f1 = buf_load16<E>(rf, st.vf, cS + (2 << 10));
        FH_STEP_A(f2, f3, 1)
        f2 = buf_load16<E>(rf, st.vf, cF + (3 << 10));
        f3 = buf_load16<E>(rf, st.vf, cS + (3 << 10));
      }
      for (int kn0 = 2; kn0 < KN - 2; kn0 += 2) {
        FH_STEP_A(f0, f1, kn0)
        f0 = buf_load16<E>(rf, st.vf, cF + ((kn0 + 2) << 10));
        f1 = buf_load16<E>(rf, st.vf, cS + ((kn0 + 2) << 10));
        FH_STEP_A(f2, f3, kn0 + 1)
        f2 = buf_load16<E>(rf, st.vf, cF + ((kn0 + 3) << 10));
        f3 = buf_load16<E>(rf, st.vf, cS + ((kn0 + 3) << 10));
      }
      FH_STEP_A(f0, f1, KN - 2)
      stream_pair<E>(st, 0, f0, f1);
      FH_STEP_A(f2, f3, KN - 1)
      stream_pair<E>(st, 2, f2, f3);
#undef FH_STEP_A
      if (grow) {                          // the carried term of a growing head takes exp(cs_l), unclamped
        const float gF = exp2_hw(fmaxf(dAs[32 * lbF + m], 0.0f)), gS = exp2_hw(fmaxf(dAs[32 * lbS + m], 0.0f));
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          accF[r] *= gF;
          accS[r] *= gS;
        }
      }
    } else if (yact) {                     // first chunk without an initial state
      accF = (f32x16_t){0};
      accS = (f32x16_t){0};
      stream_pair<E>(st, 0, f0, f1);
      stream_pair<E>(st, 2, f2, f3);
    } else {                               // no row blocks: straight to where the state update expects the ring
      stream_pair<E>(st, 2, f2, f3);
      stream_pair<E>(st, 4, f0, f1);
    }

    // ---- the two row blocks.  Pair q of the stream lives in (f0, f1) if q is even, in (f2, f3) if odd:
    // the diagonal block of the first row block is pair lbF, that of the second pair NLB.
    if (yact) {
      if (lbF & 1) half_row_block<E, DMODE == 1>(accF, f2, f3, f0, f1, lbF, 0, st, xw, xr, dAs, dqs, l2s, Q, qmask, m, g2, dhead);
      else half_row_block<E, DMODE == 1>(accF, f0, f1, f2, f3, lbF, 0, st, xw, xr, dAs, dqs, l2s, Q, qmask, m, g2, dhead);
      half_row_block<E, DMODE == 1>(accS, f0, f1, f2, f3, lbS, st.n_first, st, xw, xr, dAs, dqs, l2s, Q, qmask, m, g2, dhead);
      if constexpr (DMODE == 2) {
        half_skip_term<E>(accF, lbF, xr, Q, qmask, m, g2, p.Dk + h * FU_P + p0);
        half_skip_term<E>(accS, lbS, xr, Q, qmask, m, g2, p.Dk + h * FU_P + p0);
      }
    }
    __syncthreads();                       // every wave is past the carried state: its tile becomes the output staging

    // ---- state: S^T[n][p] <- S^T g_k + sum_{s in block k} B[s][n] x~[s][p], and the chunk's reads from
    // HBM: the gate operands of this wave's rows (in the row-major order of the output pass) and the next
    // chunk's inputs.  Vector memory reads of a wave return in order, so whatever is requested after a
    // read from HBM waits for it: the requests go out after the first four steps, behind the ring's first
    // refills.  The ring stands one pair on; its last refills are the next chunk's first fragments of C.
    const int cn = min(c + 1, nc - 1);
    V8<E> zF[2], zS[2];
    const int row_o = c * Q * xrow_b;
    float prev_end = 0.0f;
#define FH_STEP_C(F, KK)                                                                        \
      {                                                                                         \
        const V8<E> xf = load_frag_e<E>(xw + m * Q + (((2 * (KK) + g2) ^ (m & qmask)) << 3));   \
        S = mma(F, xf, S);                                                                      \
      }
#define FH_SCALE_C(KK)                                                                          \
      {                                                                                         \
        const float endv = dAs[16 * (KK) + 31];                                                 \
        const float gs = exp2_hw(fminf(endv - prev_end, 0.0f));                                 \
        prev_end = endv;                                                                        \
        _Pragma("unroll") for (int r = 0; r < 16; ++r) S[r] *= gs;                              \
      }
#define FH_REQUEST_HBM                                                                          \
      {                                                                                         \
        if (yact && HAS_Z) {                                                                    \
          _Pragma("unroll") for (int pass = 0; pass < 2; ++pass) {                              \
            zF[pass] = buf_load16<E>(rz, v_row, row_o + (32 * lbF + 16 * pass) * xrow_b);          \
            zS[pass] = buf_load16<E>(rz, v_row, row_o + (32 * lbS + 16 * pass) * xrow_b);          \
          }                                                                                     \
        }                                                                                       \
        FH_REQUEST_CHUNK(cn)                                                                    \
        /* the requests go out here: the scheduler must not sink them into the update */        \
        asm volatile("" ::: "memory");                                                          \
      }
    if (sact && grow) {                    // the carried state of a growing head takes exp(cs[Q-1]), unclamped
      const float gt = exp2_hw(fmaxf(dAs[Q - 1], 0.0f));
#pragma unroll
      for (int r = 0; r < 16; ++r) S[r] *= gt;
    }
    if (sact) {
#pragma unroll
      for (int k0 = 0; k0 < KS; k0 += 4) {
        const bool more = k0 + 4 < KS;
        FH_SCALE_C(k0)
        FH_STEP_C(f2, k0)
        if (more) f2 = buf_load16<E>(rf, st.vf, st.off_bt + (k0 + 4) * st.bt_step);
        else if (yact) f2 = buf_load16<E>(rf, st.vf, FH_C_OFF(cn, lbF, 1));
        FH_STEP_C(f3, k0 + 1)
        if (more) f3 = buf_load16<E>(rf, st.vf, st.off_bt + (k0 + 5) * st.bt_step);
        else if (yact) f3 = buf_load16<E>(rf, st.vf, FH_C_OFF(cn, lbS, 1));
        FH_SCALE_C(k0 + 2)
        FH_STEP_C(f0, k0 + 2)
        if (more) f0 = buf_load16<E>(rf, st.vf, st.off_bt + (k0 + 6) * st.bt_step);
        else if (yact) f0 = buf_load16<E>(rf, st.vf, FH_C_OFF(cn, lbF, 0));
        FH_STEP_C(f1, k0 + 3)
        if (more) f1 = buf_load16<E>(rf, st.vf, st.off_bt + (k0 + 7) * st.bt_step);
        else if (yact) f1 = buf_load16<E>(rf, st.vf, FH_C_OFF(cn, lbS, 0));
        if (k0 == 0) FH_REQUEST_HBM
      }
    } else {
      FH_REQUEST_HBM
      if (yact) {
        f0 = buf_load16<E>(rf, st.vf, FH_C_OFF(cn, lbF, 0));
        f1 = buf_load16<E>(rf, st.vf, FH_C_OFF(cn, lbS, 0));
        f2 = buf_load16<E>(rf, st.vf, FH_C_OFF(cn, lbF, 1));
        f3 = buf_load16<E>(rf, st.vf, FH_C_OFF(cn, lbS, 1));
      }
    }
#undef FH_REQUEST_HBM
#undef FH_STEP_C
#undef FH_SCALE_C
    // the gate operands are first looked at here: without this the scheduler starts converting them in
    // the middle of the state update, which then waits for the reads from HBM after all
    if (HAS_Z) asm volatile("" : "+v"(zF[0]), "+v"(zF[1]), "+v"(zS[0]), "+v"(zS[1]) : : "memory");
    // ---- the output through a wave-private 32 x 32 fp32 tile to row-major 16-byte accesses: gate, store
    if (yact) {
      float *stg = reinterpret_cast<float *>(smem + 2 * FH_TILE_BYTES) + wave * 1024;
#pragma unroll
      for (int which = 0; which < 2; ++which) {
        const int lb = which == 0 ? lbF : lbS;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 v = which == 0 ? make_float4(accF[4 * q], accF[4 * q + 1], accF[4 * q + 2], accF[4 * q + 3])
                                      : make_float4(accS[4 * q], accS[4 * q + 1], accS[4 * q + 2], accS[4 * q + 3]);
          *reinterpret_cast<float4 *>(stg + m * 32 + (((2 * q + g2) ^ (m & 7)) << 2)) = v;
        }
        wave_lds_sync();
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
          const int l = (lane >> 2) + 16 * pass, c4 = lane & 3;
          const float4 v0 = *reinterpret_cast<const float4 *>(stg + l * 32 + (((2 * c4) ^ (l & 7)) << 2));
          const float4 v1 = *reinterpret_cast<const float4 *>(stg + l * 32 + (((2 * c4 + 1) ^ (l & 7)) << 2));
          float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
          if (HAS_Z) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] *= silu_f32((float)(which == 0 ? zF[pass][j] : zS[pass][j]));
          }
          // A 16-byte buffer store reads its data registers a few cycles after it issues.  The compiler's
          // hazard model holds that a scalar-register offset covers that delay; on this chip an arithmetic
          // instruction that rewrites the registers in the next two slots has been seen to get ahead of the
          // read under load (wrong dwords in the last quarter of each 16 lanes).  So the data stays live, and
          // idle slots follow the store.
          const u32x4_t packed = __builtin_bit_cast(u32x4_t, pack8_e<E>(v));
          __builtin_amdgcn_raw_buffer_store_b128(packed, ry, v_row, row_o + (32 * lb + 16 * pass) * xrow_b, 0);
          asm volatile("s_nop 3" : : "v"(packed) : "memory");
        }
        wave_lds_sync();
      }
    }
  }
#undef FH_REQUEST_CHUNK
#undef FH_C_OFF

  if (p.final_states && sact) {
    float *fp = p.final_states + (((size_t)b * H + h) * FU_P + p0 + m) * N + 32 * nt_s;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<float4 *>(fp + 8 * q + 4 * g2) = make_float4(S[4 * q], S[4 * q + 1], S[4 * q + 2], S[4 * q + 3]);
  }
}

static size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

struct FusedLayout {
  size_t dt_out, dA2, Cblk, Btblk, CBblk, total;
};

static FusedLayout fused_layout(const SsdDims &d) {
  FusedLayout f;
  const size_t per_step = align_up((size_t)d.batch * d.heads * d.len * sizeof(float));
  const size_t bc = align_up((size_t)d.batch * d.len * d.groups * d.nstate * 2);
  const size_t cb = align_up((size_t)d.batch * d.nchunks * d.groups * d.chunk * d.chunk * 2);
  size_t at = 0;
  f.dt_out = at; at += per_step;
  f.dA2 = at; at += per_step;
  f.Cblk = at; at += bc;
  f.Btblk = at; at += bc;
  f.CBblk = at; at += cb;
  f.total = at;
  return f;
}

static bool fused_shape_ok(const SsdDims &d) {
  const bool q_ok = d.chunk == 64 || d.chunk == 128 || d.chunk == 256;
  const bool n_ok = d.nstate == 64 || d.nstate == 128;
  if (!(q_ok && n_ok && d.hdim == FU_P && d.len % d.chunk == 0 && d.heads % d.groups == 0)) return false;
  // the kernel addresses with 32-bit byte offsets: inside one batch row of x, z and y, inside the
  // per-step arrays and inside the fragment copies
  const size_t lim = (size_t)1 << 31;
  const FusedLayout f = fused_layout(d);
  return (size_t)d.len * d.heads * FU_P * 2 < lim && f.Cblk - f.dt_out + (size_t)d.len * 4 < lim && f.total - f.Cblk < lim;
}

}  // namespace ssm

static int fused_dims(const char *who, const ssm_ssd_dims *s, ssm::SsdDims &d) {
  using namespace ssm;
  SSM_REQUIRE(s, SSM_ERR_NULL_POINTER, "%s: dims is required", who);
  SSM_REQUIRE(s->batch > 0 && s->seqlen > 0 && s->heads > 0 && s->headdim > 0 && s->groups > 0 && s->nstate > 0 &&
                  s->chunk > 0,
              SSM_ERR_BAD_SHAPE, "%s: all of batch, seqlen, heads, headdim, groups, nstate, chunk must be positive", who);
  SSM_REQUIRE(s->heads % s->groups == 0, SSM_ERR_BAD_SHAPE, "%s: groups=%d must divide heads=%d", who, s->groups,
              s->heads);
  d.batch = s->batch; d.len = s->seqlen; d.heads = s->heads; d.hdim = s->headdim; d.groups = s->groups;
  d.nstate = s->nstate; d.chunk = s->chunk; d.nchunks = (s->seqlen + s->chunk - 1) / s->chunk;
  SSM_REQUIRE((size_t)d.batch * d.len * d.heads * d.hdim < ((size_t)1 << 40), SSM_ERR_TOO_LARGE, "%s: tensor too large",
              who);
  return SSM_OK;
}

extern "C" int ssm_ssd_combined_supported(const ssm_ssd_dims *dims, int io_dtype) {
  ssm::SsdDims d;
  if (fused_dims("ssm_ssd_combined_supported", dims, d) != SSM_OK) return 0;
  return (io_dtype == SSM_BF16 || io_dtype == SSM_F16) && ssm::fused_shape_ok(d) ? 1 : 0;
}

extern "C" size_t ssm_ssd_combined_workspace_bytes(const ssm_ssd_dims *dims) {
  ssm::SsdDims d;
  if (fused_dims("ssm_ssd_combined_workspace_bytes", dims, d) != SSM_OK) return 0;
  return ssm::fused_layout(d).total;
}

extern "C" int ssm_ssd_combined_fwd(const ssm_ssd_combined_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a && a->x && a->dt && a->A && a->Bm && a->Cm && a->y, SSM_ERR_NULL_POINTER,
              "ssm_ssd_combined_fwd: x, dt, A, Bm, Cm and y are required");
  SsdDims d;
  int rc = fused_dims("ssm_ssd_combined_fwd", &a->dims, d);
  if (rc != SSM_OK) return rc;
  SSM_REQUIRE(a->io_dtype == SSM_BF16 || a->io_dtype == SSM_F16, SSM_ERR_BAD_DTYPE,
              "ssm_ssd_combined_fwd: x, z, y, Bm and Cm must be bf16 or fp16 (one type for all)");
  SSM_REQUIRE(valid_dtype(a->dt_dtype), SSM_ERR_BAD_DTYPE, "ssm_ssd_combined_fwd: dt_dtype=%d", a->dt_dtype);
  SSM_REQUIRE(fused_shape_ok(d), SSM_ERR_BAD_SHAPE,
              "ssm_ssd_combined_fwd: needs headdim 64, chunk in {64,128,256}, nstate in {64,128} and "
              "seqlen %% chunk == 0 (got headdim=%d chunk=%d nstate=%d seqlen=%d)",
              d.hdim, d.chunk, d.nstate, d.len);
  const FusedLayout lay = fused_layout(d);
  SSM_REQUIRE(a->workspace && a->workspace_bytes >= lay.total, SSM_ERR_WORKSPACE,
              "ssm_ssd_combined_fwd: workspace of %zu bytes required", lay.total);
  SSM_REQUIRE(aligned_to(a->x, 16) && aligned_to(a->y, 16) && (!a->z || aligned_to(a->z, 16)) && aligned_to(a->Bm, 16) &&
                  aligned_to(a->Cm, 16) && aligned_to(a->workspace, 256) &&
                  (!a->Dskip || aligned_to(a->Dskip, a->d_per_p ? 16 : 4)) && (!a->final_states || aligned_to(a->final_states, 16)) &&
                  (!a->initial_states || aligned_to(a->initial_states, 4)),
              SSM_ERR_ALIGNMENT, "ssm_ssd_combined_fwd: tensors must be 16-byte aligned (workspace 256; a per-head Dskip 4)");
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  unsigned char *ws = reinterpret_cast<unsigned char *>(a->workspace);

  const size_t bcg = (size_t)d.batch * d.nchunks * d.groups;
  const int NLB = d.chunk >> 5, KS = d.chunk >> 4, KN = d.nstate >> 4, NT = d.nstate >> 5;
  SsdPrepParams pp{};
  SsdCumsumParams &cp = pp.cs;
  cp.dt = a->dt; cp.A = a->A; cp.bias = a->dt_bias;
  cp.dA_cs = nullptr;
  cp.dt_out = reinterpret_cast<float *>(ws + lay.dt_out);
  cp.d = d; cp.dt_dtype = a->dt_dtype; cp.softplus = a->dt_softplus ? 1 : 0; cp.dt_min = a->dt_min; cp.dt_max = a->dt_max;
  pp.dA2 = reinterpret_cast<float *>(ws + lay.dA2);
  pp.Cm = a->Cm; pp.Bm = a->Bm;
  const size_t dense_row = (size_t)d.groups * d.nstate;
  SSM_REQUIRE(a->b_row_stride >= 0 && a->c_row_stride >= 0 && (a->b_row_stride == 0 || (size_t)a->b_row_stride >= dense_row) &&
                  (a->c_row_stride == 0 || (size_t)a->c_row_stride >= dense_row) && a->b_row_stride % 8 == 0 && a->c_row_stride % 8 == 0,
              SSM_ERR_BAD_SHAPE, "ssm_ssd_combined_fwd: b_row_stride=%lld c_row_stride=%lld must be 0 or at least groups * nstate=%zu, in multiples of 8",
              (long long)a->b_row_stride, (long long)a->c_row_stride, dense_row);
  pp.b_row = a->b_row_stride ? (size_t)a->b_row_stride : dense_row;
  pp.c_row = a->c_row_stride ? (size_t)a->c_row_stride : dense_row;
  void *Cblk = ws + lay.Cblk, *Btblk = ws + lay.Btblk;
  pp.Cblk = Cblk; pp.Btblk = Btblk; pp.CBblk = ws + lay.CBblk;
  const size_t n_dt = (size_t)d.batch * d.nchunks * ((d.heads + PD_HEADS - 1) / PD_HEADS);
  const size_t n_pack = (bcg * NLB * KN + bcg * KS * NT + 3) / 4;
  const size_t n_cb = (bcg * (NLB * (NLB + 1) / 2) + 3) / 4;
  SSM_REQUIRE(n_dt + n_pack + n_cb < ((size_t)1 << 31), SSM_ERR_TOO_LARGE, "ssm_ssd_combined_fwd: too many workgroups");
  pp.n_dt = (unsigned)n_dt; pp.n_pack = (unsigned)n_pack;
  pp.seq_idx = a->seq_idx;
  const bool f16 = a->io_dtype == SSM_F16;
  if (f16) hipLaunchKernelGGL(ssd_fused_prep_kernel<_Float16>, dim3((unsigned)(n_dt + n_pack + n_cb)), dim3(256), 0, s, pp);
  else hipLaunchKernelGGL(ssd_fused_prep_kernel<__bf16>, dim3((unsigned)(n_dt + n_pack + n_cb)), dim3(256), 0, s, pp);
  SSM_CHECK_LAUNCH("ssm_ssd_combined_fwd(prep)");

  SsdFusedParams fp{};
  fp.x = a->x; fp.z = a->z;
  fp.y = a->y;
  fp.dA2 = reinterpret_cast<const float *>(ws + lay.dA2); fp.dtv = cp.dt_out;
  fp.Cblk = Cblk; fp.CBblk = ws + lay.CBblk; fp.Btblk = Btblk;
  fp.Dk = a->Dskip; fp.init = a->initial_states; fp.A = a->A; fp.final_states = a->final_states;
  fp.batch = d.batch; fp.len = d.len; fp.heads = d.heads; fp.groups = d.groups; fp.nstate = d.nstate; fp.chunk = d.chunk;
  fp.nchunks = d.nchunks; fp.d_per_p = a->d_per_p ? 1 : 0;
  const int dmode = !a->Dskip ? 0 : (a->d_per_p ? 2 : 1);
  const unsigned grid = (unsigned)(d.batch * d.heads) * 2;
#define SSM_LAUNCH_FUSED(QQ, NN, DM, HZ)                                                           \
  {                                                                                                \
    auto kernel = f16 ? ssd_fused_half_kernel<_Float16, QQ, NN, DM, HZ> : ssd_fused_half_kernel<__bf16, QQ, NN, DM, HZ>; \
    if (allow_dynamic_lds(kernel, FH_LDS_BYTES) != hipSuccess) {                                   \
      set_error("ssm_ssd_combined_fwd: cannot reserve %d bytes of LDS", FH_LDS_BYTES);             \
      return SSM_ERR_LAUNCH;                                                                       \
    }                                                                                              \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(FH_THREADS), FH_LDS_BYTES, s, fp);                 \
  }
#define SSM_LAUNCH_FUSED_DZ(QQ, NN)                                                                \
  {                                                                                                \
    if (a->z) {                                                                                    \
      if (dmode == 0) SSM_LAUNCH_FUSED(QQ, NN, 0, true)                                            \
      else if (dmode == 1) SSM_LAUNCH_FUSED(QQ, NN, 1, true)                                       \
      else SSM_LAUNCH_FUSED(QQ, NN, 2, true)                                                       \
    } else {                                                                                       \
      if (dmode == 0) SSM_LAUNCH_FUSED(QQ, NN, 0, false)                                           \
      else if (dmode == 1) SSM_LAUNCH_FUSED(QQ, NN, 1, false)                                      \
      else SSM_LAUNCH_FUSED(QQ, NN, 2, false)                                                      \
    }                                                                                              \
  }
  if (d.nstate == 128) {
    if (d.chunk == 256) SSM_LAUNCH_FUSED_DZ(256, 128)
    else if (d.chunk == 128) SSM_LAUNCH_FUSED_DZ(128, 128)
    else SSM_LAUNCH_FUSED_DZ(64, 128)
  } else {
    if (d.chunk == 256) SSM_LAUNCH_FUSED_DZ(256, 64)
    else if (d.chunk == 128) SSM_LAUNCH_FUSED_DZ(128, 64)
    else SSM_LAUNCH_FUSED_DZ(64, 64)
  }
#undef SSM_LAUNCH_FUSED_DZ
#undef SSM_LAUNCH_FUSED
  SSM_CHECK_LAUNCH("ssm_ssd_combined_fwd");
  note_mfma_launch(8);
  return SSM_OK;
}
