// Mamba-2 SSD forward as one pass over the sequence: a workgroup owns one
// (batch, head), walks its chunks in order and keeps the running state
// S (P x N, fp32) in MFMA accumulators, so neither the per-chunk states nor
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
// Requires bf16 tensors, P = 64, Q in {64, 128, 256}, N in {64, 128},
// L % Q == 0 and A <= 0 (the factors above are clamped to 1 individually).
#include "ssd_common.hpp"

namespace ssm {

constexpr int FU_THREADS = 512;
constexpr int FU_P = 64;
constexpr int FU_TILE_BYTES = 32768;                       // [64][256] bf16
constexpr int FU_LDS_BYTES = 2 * FU_TILE_BYTES + 3 * 256 * 4;
constexpr int FRAG = 512;                                  // bf16 elements per operand fragment

struct SsdFusedParams {
  const __bf16 *x, *z;
  __bf16 *y;
  const float *dA2, *dtv, *ws;          // (B,H,nc,Q): log2-scaled running sum, step, staged weight
  const __bf16 *Cblk, *Btblk, *CBblk;   // fragment-blocked copies
  const float *Dk, *init;
  float *final_states;
  int batch, len, heads, groups, nstate, chunk, nchunks, d_per_p;
};

typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;

__device__ __forceinline__ void wave_lds_sync() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// ------------------------------------------------------------------ prep: dt
// One workgroup per (b, c, 4 heads): the (Q x 4) slab of dt is read row by row
// (16 contiguous bytes per step) into LDS transposed to [head][step]; then one
// wave per head forms dt' = clamp(softplus(dt + bias)), the running sum of dt' A
// and the staged weight  ws[l] = dt'_l exp(cs[l | 31] - cs[l]).
constexpr int PD_HEADS = 4;
__global__ __launch_bounds__(256) void ssd_fused_prep_dt_kernel(const SsdCumsumParams p, float *dA2, float *ws) {
  __shared__ float tile[PD_HEADS][256 + 1];
  const SsdDims &d = p.d;
  const int Q = d.chunk;
  const int hgroups = (d.heads + PD_HEADS - 1) / PD_HEADS;
  const int hg = (int)blockIdx.x % hgroups;
  const int c = ((int)blockIdx.x / hgroups) % d.nchunks;
  const int b = (int)blockIdx.x / (hgroups * d.nchunks);
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
    wave_lds_sync();                       // the row is re-used for the running sums
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int l = lane * per + i;
      if (i < per && l < Q) {
        const float a = excl + run[i];
        tile[hh][l] = a;
        p.dA_cs[out + l] = a;
        p.dt_out[out + l] = v[i];
        dA2[out + l] = a * LOG2E;
      }
    }
    wave_lds_sync();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int l = lane * per + i;
      if (i < per && l < Q) ws[out + l] = v[i] * decay_exp(tile[hh][l | 31] - tile[hh][l]);
    }
  }
}

// ---------------------------------------------------------------- prep: pack
// Fragment (lane, j) of a 32 x 16 operand block: row 32 rb + lane % 32,
// column 16 kb + 8 (lane / 32) + j.  One wave per fragment; the first
// B nc G (NLB KN) fragments are those of C, the rest those of B^T:
//   Cblk [(b,c,g)][lb][kn]  from C  (rows = time, columns = state)
//   Btblk[(b,c,g)][ks][nt]  from B  (rows = state, columns = time)
// (CBblk[(b,c,g)][lb][ks], rows = l, columns = s, is written by the C B^T kernel.)
__global__ __launch_bounds__(256) void ssd_fused_pack_kernel(const __bf16 *Cm, const __bf16 *Bm, __bf16 *Cblk, __bf16 *Btblk,
                                                             int batch, int len, int groups, int nstate, int chunk) {
  const int wave = wave_id_uniform(), lane = lane_id();
  const int Q = chunk, N = nstate, nc = len / Q;
  const int NLB = Q >> 5, KS = Q >> 4, KN = N >> 4, NT = N >> 5;
  const size_t units = (size_t)batch * nc * groups;
  const size_t nC = units * NLB * KN, nB = units * KS * NT;
  size_t f = (size_t)blockIdx.x * 4 + wave;
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
  bf16x8_t v;
  if (is_c) {
    const int lb = inner / KN, kn = inner % KN;
    v = load_frag(Cm + (((size_t)b * len + (size_t)c * Q + 32 * lb + m) * groups + g) * N + 16 * kn + 8 * g2);
  } else {
    const int ks = inner / NT, nt = inner % NT;
    const __bf16 *col = Bm + (((size_t)b * len + (size_t)c * Q + 16 * ks + 8 * g2) * groups + g) * N + 32 * nt + m;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = col[(size_t)j * groups * N];
  }
  *reinterpret_cast<bf16x8_t *>((is_c ? Cblk : Btblk) + f * FRAG + lane * 8) = v;
}

// --------------------------------------------------------------- fused kernel
// Waves 0..7.  For the output phases wave w owns the 32 rows of block
// lb = w (w < 4) or 11 - w, both 32-wide halves of P, so that the two waves
// sharing a SIMD carry equal numbers of blocks below the diagonal.  For the state
// phases wave w owns the 32 x 32 tile (n-tile w / 2, p-tile w % 2) of S^T.
// Accumulators hold transposed tiles: lane = column (l for y, p for S^T),
// registers = rows (p for y, n for S^T).
// DMODE: 0 no skip term, 1 D per head, 2 D per (head, channel).
template <int DMODE, bool HAS_Z>
__global__ __launch_bounds__(FU_THREADS)
void ssd_fused_kernel(const SsdFusedParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  __bf16 *xw = reinterpret_cast<__bf16 *>(smem);                       // x~ [64][Q]; between chunks S as bf16 [64][N]
  __bf16 *xr = reinterpret_cast<__bf16 *>(smem + FU_TILE_BYTES);       // x  [64][Q]; later the output staging
  float *dAs = reinterpret_cast<float *>(smem + 2 * FU_TILE_BYTES);    // [Q] log2-scaled running sum
  float *dts = dAs + 256;                                              // [Q]
  float *wss = dts + 256;                                              // [Q] staged weight

  const int Q = p.chunk, N = p.nstate, H = p.heads, G = p.groups, nc = p.nchunks;
  const int NLB = Q >> 5, NT = N >> 5, KS = Q >> 4, KN = N >> 4;
  const int qmask = min(15, (Q >> 3) - 1), nmask = min(15, (N >> 3) - 1);
  const int tid = (int)threadIdx.x;
  const int wave = wave_id_uniform(), lane = lane_id();
  const int g2 = lane >> 5, m = lane & 31;
  const int h = (int)blockIdx.x % H, b = (int)blockIdx.x / H;
  const int g = h / (H / G);
  const int lb = wave < 4 ? wave : 11 - wave;
  const bool yact = lb < NLB;
  const int pt_s = wave & 1, nt_s = wave >> 1;
  const bool sact = nt_s < NT;
  const bool has_init = p.init != nullptr;
  const size_t xrow = (size_t)H * FU_P;                                // elements between time steps

  f32x16_t S = {0};
  if (sact && has_init) {
    const float *ip = p.init + (((size_t)b * H + h) * FU_P + 32 * pt_s + m) * N + 32 * nt_s;
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = ip[crow(r, g2)];
  }
  f32x16_t acc[2];

  // staging role: a thread transposes 8 time steps x 4 head channels into both tiles

  for (int c = 0; c < nc; ++c) {
    // Lane-derived addresses are recomputed per chunk (the opaque copy keeps them from
    // being hoisted out of the loop and held in registers across all of it).
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int lane = ln, g2 = ln >> 5, m = ln & 31, tid = wave * WAVE + ln;
    const bool s_on = tid < 2 * Q;
    const int spb = tid & 15, slb8 = tid >> 4;
    const size_t cs = (((size_t)b * H + h) * nc + c) * Q;
    const size_t unit = ((size_t)b * nc + c) * G + g;
    const __bf16 *xg = p.x + (((size_t)b * p.len + (size_t)c * Q) * H + h) * FU_P;
    const bool carry = c > 0 || has_init;
    // Operand fragments stream through four registers sets: f0 is consumed, f1..f3 are in
    // flight, a new read (clamped to the last fragment) enters at f3.
    bf16x8_t f0, f1, f2, f3;

    // fragments of C for the carried-state product: in flight across the barriers below
    const __bf16 *cf = p.Cblk + ((unit * NLB + lb) * KN) * FRAG + lane * 8;
    if (yact && carry) {
      f0 = load_frag(cf);
      f1 = load_frag(cf + (size_t)min(1, KN - 1) * FRAG);
      f2 = load_frag(cf + (size_t)min(2, KN - 1) * FRAG);
      f3 = load_frag(cf + (size_t)min(3, KN - 1) * FRAG);
    }

    __syncthreads();                       // previous chunk: output staging and x~ reads are over
    if (sact && carry) {
      const int prow = 32 * pt_s + m;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        bf16x4_t v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = (__bf16)S[4 * q + j];
        const int chunk16 = 4 * nt_s + q;
        *reinterpret_cast<bf16x4_t *>(xw + prow * N + ((chunk16 ^ (prow & nmask)) << 3) + 4 * g2) = v;
      }
    }
    if (tid < Q) {
      dAs[tid] = p.dA2[cs + tid];
      dts[tid] = p.dtv[cs + tid];
      wss[tid] = p.ws[cs + tid];
    }
    // global reads for the staging that follows the carried-state product
    bf16x4_t raw[8];                       // read by every thread (clamped rows) so that the values
    {                                      // are not defined under a divergent branch
      const int srow = min(slb8, (Q >> 3) - 1) * 8;
#pragma unroll
      for (int r = 0; r < 8; ++r)
        raw[r] = *reinterpret_cast<const bf16x4_t *>(xg + (size_t)(srow + r) * xrow + spb * 4);
    }
    __syncthreads();

    // ---- carried state: acc[p][l] = sum_n S[p][n] C[l][n]
    acc[0] = (f32x16_t){0};
    acc[1] = (f32x16_t){0};
    if (yact && carry) {
      // four steps per trip, one register set each: a set is refilled as soon as it is consumed
      // (no copies between sets: a copy would wait for the read it moves)
#define FU_STEP_A(F, KK)                                                                        \
      {                                                                                         \
        const bf16x8_t f = F;                                                                   \
        F = load_frag(cf + (size_t)min((KK) + 4, KN - 1) * FRAG);                               \
        _Pragma("unroll") for (int pt = 0; pt < 2; ++pt) {                                      \
          const int prow = 32 * pt + m;                                                         \
          const bf16x8_t a = load_frag(xw + prow * N + (((2 * (KK) + g2) ^ (prow & nmask)) << 3)); \
          acc[pt] = mma(a, f, acc[pt]);                                                         \
        }                                                                                       \
      }
      for (int k0 = 0; k0 < KN; k0 += 4) {
        FU_STEP_A(f0, k0)
        FU_STEP_A(f1, k0 + 1)
        FU_STEP_A(f2, k0 + 2)
        FU_STEP_A(f3, k0 + 3)
      }
#undef FU_STEP_A
    }
    // fragments of CB for this wave's rows: in flight while the tiles are staged
    const __bf16 *cbf = p.CBblk + ((unit * NLB + lb) * KS) * FRAG + lane * 8;
    const int nkb = 2 * lb + 2;            // 16-step fragments up to and including the diagonal block
    if (yact) {
      f0 = load_frag(cbf);
      f1 = load_frag(cbf + (size_t)FRAG);
      f2 = load_frag(cbf + (size_t)min(2, nkb - 1) * FRAG);
      f3 = load_frag(cbf + (size_t)min(3, nkb - 1) * FRAG);
    }
    __syncthreads();                       // S (bf16) consumed: the x~ tile may be written

    // ---- stage x~ and x, transposed to [p][s]
    if (s_on) {
      const float4 a0 = *reinterpret_cast<const float4 *>(wss + slb8 * 8), a1 = *reinterpret_cast<const float4 *>(wss + slb8 * 8 + 4);
      const float w8[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bf16x8_t colw, colr;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          colr[r] = raw[r][i];
          colw[r] = (__bf16)((float)raw[r][i] * w8[r]);
        }
        const int prow = spb * 4 + i;
        const int at = prow * Q + ((slb8 ^ (prow & qmask)) << 3);
        *reinterpret_cast<bf16x8_t *>(xw + at) = colw;
        *reinterpret_cast<bf16x8_t *>(xr + at) = colr;
      }
    }
    __syncthreads();
    // ---- blocks below the diagonal, then the diagonal block
    if (yact) {
      float prev_end = 0.0f;
      const int lrow = 32 * lb + m;
      const float dal = dAs[lrow];
      // two 32-step blocks per trip: block sb0 streams through (f0, f1), block sb0 + 1 through (f2, f3)
#define FU_BLOCK_B(FA, FB, SB)                                                                  \
      {                                                                                         \
        const float endv = dAs[32 * (SB) + 31];                                                 \
        const float gs = exp2_hw(fminf(endv - prev_end, 0.0f));                                 \
        prev_end = endv;                                                                        \
        _Pragma("unroll") for (int r = 0; r < 16; ++r) {                                        \
          acc[0][r] *= gs;                                                                      \
          acc[1][r] *= gs;                                                                      \
        }                                                                                       \
        const bf16x8_t fa = FA, fb = FB;                                                        \
        FA = load_frag(cbf + (size_t)min(2 * (SB) + 4, nkb - 1) * FRAG);                        \
        FB = load_frag(cbf + (size_t)min(2 * (SB) + 5, nkb - 1) * FRAG);                        \
        _Pragma("unroll") for (int kk = 0; kk < 2; ++kk) {                                      \
          _Pragma("unroll") for (int pt = 0; pt < 2; ++pt) {                                    \
            const int prow = 32 * pt + m;                                                       \
            const bf16x8_t a = load_frag(xw + prow * Q + (((4 * (SB) + 2 * kk + g2) ^ (prow & qmask)) << 3)); \
            acc[pt] = mma(a, kk == 0 ? fa : fb, acc[pt]);                                       \
          }                                                                                     \
        }                                                                                       \
      }
      // Block sb streams through (f0, f1) when sb is even and (f2, f3) when it is odd; the loop
      // takes two blocks per trip without a guard between them, so an odd count starts with
      // block 0 on its own.
      if (lb & 1) {
        FU_BLOCK_B(f0, f1, 0)
        for (int sb0 = 1; sb0 < lb; sb0 += 2) {
          FU_BLOCK_B(f2, f3, sb0)
          FU_BLOCK_B(f0, f1, sb0 + 1)
        }
        f0 = f2;                            // the diagonal block's fragments
        f1 = f3;
      } else {
        for (int sb0 = 0; sb0 < lb; sb0 += 2) {
          FU_BLOCK_B(f0, f1, sb0)
          FU_BLOCK_B(f2, f3, sb0 + 1)
        }
      }
#undef FU_BLOCK_B
      // diagonal block: the per-row factor once, then the factor of every element
      const float rf = exp2_hw(fminf(dal - prev_end, 0.0f));
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[0][r] *= rf;
        acc[1][r] *= rf;
      }
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const int ks = 2 * lb + kk;
        const bf16x8_t f = kk == 0 ? f0 : f1;
        const int sbase = 16 * ks + 8 * g2;
        const float4 a0 = *reinterpret_cast<const float4 *>(dAs + sbase), a1 = *reinterpret_cast<const float4 *>(dAs + sbase + 4);
        const float4 t0 = *reinterpret_cast<const float4 *>(dts + sbase), t1 = *reinterpret_cast<const float4 *>(dts + sbase + 4);
        const float das[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        const float dtv[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
        float mv[8];
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
          const float v = (float)f[jj] * exp2_hw(dal - das[jj]) * dtv[jj];
          mv[jj] = (sbase + jj <= lrow) ? v : 0.0f;
        }
        const bf16x8_t bf = pack8(mv);
#pragma unroll
        for (int pt = 0; pt < 2; ++pt) {
          const int prow = 32 * pt + m;
          const bf16x8_t a = load_frag(xr + prow * Q + (((2 * ks + g2) ^ (prow & qmask)) << 3));
          acc[pt] = mma(a, bf, acc[pt]);
        }
      }
      // skip term D x_l from the plain tile (this lane's column l, the 16 rows p of each half)
      if constexpr (DMODE != 0) {
        const int xcol = lrow & 7, xchunk = lrow >> 3;
        const float dh = DMODE == 1 ? p.Dk[h] : 0.0f;
#pragma unroll
        for (int pt = 0; pt < 2; ++pt)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float dv[4] = {dh, dh, dh, dh};
            if constexpr (DMODE == 2) {
              const float4 d4 = *reinterpret_cast<const float4 *>(p.Dk + (size_t)h * FU_P + 32 * pt + 8 * q + 4 * g2);
              dv[0] = d4.x; dv[1] = d4.y; dv[2] = d4.z; dv[3] = d4.w;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int prow = 32 * pt + 8 * q + 4 * g2 + j;
              const float xv = (float)xr[prow * Q + ((xchunk ^ (prow & qmask)) << 3) + xcol];
              acc[pt][4 * q + j] = __builtin_fmaf(dv[j], xv, acc[pt][4 * q + j]);
            }
          }
      }
    }

    // gate operands of this wave's rows, in the row-major order of the output pass
    bf16x8_t zreg[2], znext[2];
    const __bf16 *zg = p.z + (xg - p.x) + (size_t)(32 * lb + (lane >> 2)) * xrow + 8 * (lane & 3);
    if (yact && HAS_Z) {                   // requested now, used after the state update
#pragma unroll
      for (int pass = 0; pass < 2; ++pass) {
        zreg[pass] = load_frag(zg + (size_t)(16 * pass) * xrow);
        znext[pass] = load_frag(zg + (size_t)(16 * pass) * xrow + 32);
      }
    }
    // ---- state: S^T[n][p] <- S^T g_k + sum_{s in block k} B[s][n] x~[s][p]
    if (sact) {
      const __bf16 *btf = p.Btblk + ((unit * KS) * NT + nt_s) * FRAG + lane * 8;
      const size_t kstep = (size_t)NT * FRAG;
      f0 = load_frag(btf);
      f1 = load_frag(btf + kstep);
      f2 = load_frag(btf + (size_t)min(2, KS - 1) * kstep);
      f3 = load_frag(btf + (size_t)min(3, KS - 1) * kstep);
      float prev_end = 0.0f;
      const int prow = 32 * pt_s + m;
#define FU_STEP_C(F, KK)                                                                        \
      {                                                                                         \
        const bf16x8_t f = F;                                                                   \
        F = load_frag(btf + (size_t)min((KK) + 4, KS - 1) * kstep);                             \
        const bf16x8_t xf = load_frag(xw + prow * Q + (((2 * (KK) + g2) ^ (prow & qmask)) << 3)); \
        S = mma(f, xf, S);                                                                      \
      }
      for (int k0 = 0; k0 < KS; k0 += 4) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          {
            const float endv = dAs[16 * (k0 + 2 * half) + 31];
            const float gs = exp2_hw(fminf(endv - prev_end, 0.0f));
            prev_end = endv;
#pragma unroll
            for (int r = 0; r < 16; ++r) S[r] *= gs;
          }
          if (half == 0) {
            FU_STEP_C(f0, k0)
            FU_STEP_C(f1, k0 + 1)
          } else {
            FU_STEP_C(f2, k0 + 2)
            FU_STEP_C(f3, k0 + 3)
          }
        }
      }
#undef FU_STEP_C
    }
    __syncthreads();                       // the plain tile is free: it becomes the output staging
    // ---- output: through a wave-private 32 x 32 fp32 tile to row-major 16-byte accesses
    if (yact) {
      float *stg = reinterpret_cast<float *>(smem + FU_TILE_BYTES) + wave * 1024;
      __bf16 *yg = p.y + (xg - p.x);
#pragma unroll
      for (int pt = 0; pt < 2; ++pt) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 v = make_float4(acc[pt][4 * q], acc[pt][4 * q + 1], acc[pt][4 * q + 2], acc[pt][4 * q + 3]);
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
            for (int j = 0; j < 8; ++j) v[j] *= silu_f32((float)(pt == 0 ? zreg[pass][j] : znext[pass][j]));
          }
          *reinterpret_cast<bf16x8_t *>(yg + (size_t)(32 * lb + l) * xrow + 32 * pt + 8 * c4) = pack8(v);
        }
        wave_lds_sync();
      }
    }
  }

  if (p.final_states && sact) {
    float *fp = p.final_states + (((size_t)b * H + h) * FU_P + 32 * pt_s + m) * N + 32 * nt_s;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<float4 *>(fp + 8 * q + 4 * g2) = make_float4(S[4 * q], S[4 * q + 1], S[4 * q + 2], S[4 * q + 3]);
  }
}

static size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

struct FusedLayout {
  size_t dA_cs, dt_out, dA2, ws, Cblk, Btblk, CBblk, total;
};

static FusedLayout fused_layout(const SsdDims &d) {
  FusedLayout f;
  const size_t per_step = align_up((size_t)d.batch * d.heads * d.len * sizeof(float));
  const size_t bc = align_up((size_t)d.batch * d.len * d.groups * d.nstate * 2);
  const size_t cb = align_up((size_t)d.batch * d.nchunks * d.groups * d.chunk * d.chunk * 2);
  size_t at = 0;
  f.dA_cs = at; at += per_step;
  f.dt_out = at; at += per_step;
  f.dA2 = at; at += per_step;
  f.ws = at; at += per_step;
  f.Cblk = at; at += bc;
  f.Btblk = at; at += bc;
  f.CBblk = at; at += cb;
  f.total = at;
  return f;
}

static bool fused_shape_ok(const SsdDims &d) {
  const bool q_ok = d.chunk == 64 || d.chunk == 128 || d.chunk == 256;
  const bool n_ok = d.nstate == 64 || d.nstate == 128;
  return q_ok && n_ok && d.hdim == FU_P && d.len % d.chunk == 0 && d.heads % d.groups == 0;
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
  return io_dtype == SSM_BF16 && ssm::fused_shape_ok(d) ? 1 : 0;
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
  SSM_REQUIRE(a->io_dtype == SSM_BF16, SSM_ERR_BAD_DTYPE, "ssm_ssd_combined_fwd: x, z, y, Bm and Cm must be bf16");
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
                  (!a->Dskip || aligned_to(a->Dskip, 16)) && (!a->final_states || aligned_to(a->final_states, 16)) &&
                  (!a->initial_states || aligned_to(a->initial_states, 4)),
              SSM_ERR_ALIGNMENT, "ssm_ssd_combined_fwd: tensors must be 16-byte aligned (workspace 256)");
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  unsigned char *ws = reinterpret_cast<unsigned char *>(a->workspace);

  SsdCumsumParams cp{};
  cp.dt = a->dt; cp.A = a->A; cp.bias = a->dt_bias;
  cp.dA_cs = reinterpret_cast<float *>(ws + lay.dA_cs);
  cp.dt_out = reinterpret_cast<float *>(ws + lay.dt_out);
  cp.d = d; cp.dt_dtype = a->dt_dtype; cp.softplus = a->dt_softplus ? 1 : 0; cp.dt_min = a->dt_min; cp.dt_max = a->dt_max;
  const size_t units = (size_t)d.batch * d.nchunks * ((d.heads + PD_HEADS - 1) / PD_HEADS);
  hipLaunchKernelGGL(ssd_fused_prep_dt_kernel, dim3((unsigned)units), dim3(256), 0, s, cp,
                     reinterpret_cast<float *>(ws + lay.dA2), reinterpret_cast<float *>(ws + lay.ws));
  SSM_CHECK_LAUNCH("ssm_ssd_combined_fwd(prep dt)");

  SsdBmmParams bp{};
  bp.a = a->Cm; bp.b = a->Bm; bp.seq_idx = nullptr; bp.out = ws + lay.CBblk;
  bp.batch = d.batch; bp.len = d.len; bp.groups = d.groups; bp.kdim = d.nstate; bp.chunk = d.chunk; bp.nchunks = d.nchunks;
  bp.in_dtype = SSM_BF16; bp.out_dtype = SSM_BF16; bp.causal = 1; bp.blocked = 1;
  SSM_REQUIRE(ssd_bmm_mfma(bp, s), SSM_ERR_BAD_SHAPE, "ssm_ssd_combined_fwd: C B^T kernel rejected the shape");
  SSM_CHECK_LAUNCH("ssm_ssd_combined_fwd(bmm)");

  const size_t bcg = (size_t)d.batch * d.nchunks * d.groups;
  const int NLB = d.chunk >> 5, KS = d.chunk >> 4, KN = d.nstate >> 4, NT = d.nstate >> 5;
  __bf16 *Cblk = reinterpret_cast<__bf16 *>(ws + lay.Cblk), *Btblk = reinterpret_cast<__bf16 *>(ws + lay.Btblk);
  const size_t frags = bcg * NLB * KN + bcg * KS * NT;
  hipLaunchKernelGGL(ssd_fused_pack_kernel, dim3((unsigned)((frags + 3) / 4)), dim3(256), 0, s,
                     reinterpret_cast<const __bf16 *>(a->Cm), reinterpret_cast<const __bf16 *>(a->Bm), Cblk, Btblk,
                     d.batch, d.len, d.groups, d.nstate, d.chunk);
  SSM_CHECK_LAUNCH("ssm_ssd_combined_fwd(pack)");

  SsdFusedParams fp{};
  fp.x = reinterpret_cast<const __bf16 *>(a->x); fp.z = reinterpret_cast<const __bf16 *>(a->z);
  fp.y = reinterpret_cast<__bf16 *>(a->y);
  fp.dA2 = reinterpret_cast<const float *>(ws + lay.dA2); fp.dtv = cp.dt_out; fp.ws = reinterpret_cast<const float *>(ws + lay.ws);
  fp.Cblk = Cblk; fp.CBblk = reinterpret_cast<const __bf16 *>(ws + lay.CBblk); fp.Btblk = Btblk;
  fp.Dk = a->Dskip; fp.init = a->initial_states; fp.final_states = a->final_states;
  fp.batch = d.batch; fp.len = d.len; fp.heads = d.heads; fp.groups = d.groups; fp.nstate = d.nstate; fp.chunk = d.chunk;
  fp.nchunks = d.nchunks; fp.d_per_p = a->d_per_p ? 1 : 0;
  const int dmode = !a->Dskip ? 0 : (a->d_per_p ? 2 : 1);
  const unsigned grid = (unsigned)(d.batch * d.heads);
#define SSM_LAUNCH_FUSED(DM, HZ)                                                                   \
  {                                                                                                \
    auto kernel = ssd_fused_kernel<DM, HZ>;                                                        \
    if (allow_dynamic_lds(kernel, FU_LDS_BYTES) != hipSuccess) {                                   \
      (void)hipGetLastError();                                                                     \
      set_error("ssm_ssd_combined_fwd: cannot reserve %d bytes of LDS", FU_LDS_BYTES);             \
      return SSM_ERR_LAUNCH;                                                                       \
    }                                                                                              \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(FU_THREADS), FU_LDS_BYTES, s, fp);                 \
  }
  if (a->z) {
    if (dmode == 0) SSM_LAUNCH_FUSED(0, true) else if (dmode == 1) SSM_LAUNCH_FUSED(1, true) else SSM_LAUNCH_FUSED(2, true)
  } else {
    if (dmode == 0) SSM_LAUNCH_FUSED(0, false) else if (dmode == 1) SSM_LAUNCH_FUSED(1, false) else SSM_LAUNCH_FUSED(2, false)
  }
#undef SSM_LAUNCH_FUSED
  SSM_CHECK_LAUNCH("ssm_ssd_combined_fwd");
  note_mfma_launch(8);
  return SSM_OK;
}
