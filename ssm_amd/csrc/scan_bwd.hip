// Selective scan, backward, for gfx950.
//
// Per (batch, channel) row, with a_t = exp(delta_t A), b_t = delta_t u_t B_t:
//   forward    h_t  = a_t h_{t-1} + b_t ,   pre_t = <h_t, C_t> + D u_t ,  y_t = pre_t silu(z_t)
//   adjoint    gh_t = g_t C_t + q_{t+1} ,   q_t = a_t gh_t                (g_t = dout_t silu(z_t))
//   dC_t += g_t h_t             dB_t += gh_t delta_t u_t      du_t = delta_t <gh_t, B_t> + g_t D
//   ddelta_t = u_t <gh_t, B_t> + sum_n q_t h_{t-1} A_n        dA_n += q_t h_{t-1} delta_t
// Nothing but the inputs and the state entering each 512-step chunk (written by
// the forward kernel) is saved: h is recomputed chunk by chunk, chunks being
// visited last to first so that q can be carried backwards.
//
// Work split.  A workgroup of 8 wavefronts walks a block of channels that share
// one B/C group.  For one (row, chunk) the 8 wavefronts split the STATE axis
// (wave w owns states 2w and 2w+1), lanes split time (8 consecutive steps per
// lane) and both directions are DPP scans (the reverse one on lane-reversed
// operands).  That way dB/dC - which sum over all channels of a group - simply
// accumulate in registers while the workgroup moves from channel to channel,
// and are written once per chunk as one partial per workgroup; a fold kernel
// adds the partials in a fixed order.  Quantities that sum over states (pre,
// <gh,B>, the A-term of ddelta) are exchanged through LDS once per row.
// There are no atomics: results are bit-reproducible.
#include "common.hpp"

#include <type_traits>
#include <utility>

namespace ssm {

constexpr int BW_K = 8;                  // steps per lane
constexpr int BW_T = WAVE * BW_K;        // 512 steps per chunk
constexpr int BW_WAVES = 8;
constexpr int BW_THREADS = WAVE * BW_WAVES;
constexpr int BW_MAX_N = 2 * BW_WAVES;   // 16 states per pass

struct ScanBwdParams {
  const void *u, *delta, *z, *dout, *Bp, *Cp;
  const float *A, *Dk, *bias, *dlast, *chunk_states;
  void *du, *ddelta, *dz;
  float *dA_rows;        // (B, D, N)  per-row sums, folded over batch afterwards
  float *dD_rows;        // (B, D)
  float *dbias_rows;     // (B, D)
  float *dB_part;        // BVARY: (B, nblk, N, L) partials ; else (B, D, N) per-row sums
  float *dC_part;
  int batch, dim, len, nstate;
  int bc_dtype;
  int b_kind, c_kind, b_groups, c_groups;
  int softplus;
  int rows_per_wg;       // channels walked by one workgroup (all in one B group and one C group)
  int nblk;              // workgroups per batch row = dim / rows_per_wg
  int bc_vec_ok;
  int spin_limit;        // wave-per-row kernel: looks at a neighbour's slot count before a wave gives up (scan_bwd_fast.hpp)
};

// Stage one [BW_MAX_N][BW_T] slab of a time-varying projection (fp32, transposed
// so that lane l finds steps 8l..8l+7 of state n at n*T + {l*4, 256 + l*4}).
__device__ __forceinline__ float4 bw_tile_quad_slow(const void *src, int dtype, size_t off, int t, int len) {
  float4 v;
  v.x = (t + 0 < len) ? load_as_f32(src, dtype, off + 0) : 0.0f;
  v.y = (t + 1 < len) ? load_as_f32(src, dtype, off + 1) : 0.0f;
  v.z = (t + 2 < len) ? load_as_f32(src, dtype, off + 2) : 0.0f;
  v.w = (t + 3 < len) ? load_as_f32(src, dtype, off + 3) : 0.0f;
  return v;
}

__device__ __forceinline__ float4 bw_quad_from16(uint2 raw, int dtype) {
  float4 v;
  if (dtype == SSM_BF16) {
    v.x = __uint_as_float(raw.x << 16);
    v.y = __uint_as_float(raw.x & 0xffff0000u);
    v.z = __uint_as_float(raw.y << 16);
    v.w = __uint_as_float(raw.y & 0xffff0000u);
  } else {
    union { uint32_t u; _Float16 h[2]; } a, b;
    a.u = raw.x;
    b.u = raw.y;
    v.x = (float)a.h[0];
    v.y = (float)a.h[1];
    v.z = (float)b.h[0];
    v.w = (float)b.h[1];
  }
  return v;
}

__device__ __forceinline__ void bw_stage_tile(float *dst, const void *src, int dtype, size_t src_off, int len,
                                              int t0, int nn, bool vec_ok) {
  constexpr int QT = BW_T / 4;
  constexpr int PER = BW_MAX_N * QT / BW_THREADS;          // quads per thread: 4
  auto place = [&](int e) { const int nl = e / QT, tl = (e % QT) * 4; return dst + nl * BW_T + ((tl % BW_K) >> 2) * (WAVE * 4) + (tl / BW_K) * 4; };
  if (vec_ok && t0 + BW_T <= len && nn == BW_MAX_N) {
    // whole slab inside the sequence: every read of the thread is requested before the first is used
    static_assert(PER == 4, "four quads per thread");
    const int e0 = threadIdx.x, e1 = e0 + BW_THREADS, e2 = e1 + BW_THREADS, e3 = e2 + BW_THREADS;
    auto at = [&](int e) { return src_off + (size_t)(e / QT) * len + t0 + (e % QT) * 4; };
    if (dtype == SSM_F32) {
      const float *f = reinterpret_cast<const float *>(src);
      const float4 v0 = *reinterpret_cast<const float4 *>(f + at(e0)), v1 = *reinterpret_cast<const float4 *>(f + at(e1));
      const float4 v2 = *reinterpret_cast<const float4 *>(f + at(e2)), v3 = *reinterpret_cast<const float4 *>(f + at(e3));
      *reinterpret_cast<float4 *>(place(e0)) = v0;
      *reinterpret_cast<float4 *>(place(e1)) = v1;
      *reinterpret_cast<float4 *>(place(e2)) = v2;
      *reinterpret_cast<float4 *>(place(e3)) = v3;
    } else {
      const uint16_t *h = reinterpret_cast<const uint16_t *>(src);
      const uint2 r0 = *reinterpret_cast<const uint2 *>(h + at(e0)), r1 = *reinterpret_cast<const uint2 *>(h + at(e1));
      const uint2 r2 = *reinterpret_cast<const uint2 *>(h + at(e2)), r3 = *reinterpret_cast<const uint2 *>(h + at(e3));
      *reinterpret_cast<float4 *>(place(e0)) = bw_quad_from16(r0, dtype);
      *reinterpret_cast<float4 *>(place(e1)) = bw_quad_from16(r1, dtype);
      *reinterpret_cast<float4 *>(place(e2)) = bw_quad_from16(r2, dtype);
      *reinterpret_cast<float4 *>(place(e3)) = bw_quad_from16(r3, dtype);
    }
    return;
  }
  for (int e = threadIdx.x; e < BW_MAX_N * QT; e += BW_THREADS) {
    const int nl = e / QT;
    const int tl = (e % QT) * 4;
    const int t = t0 + tl;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (nl < nn) {
      const size_t off = src_off + (size_t)nl * len + t;
      if (vec_ok && t + 4 <= len) {
        if (dtype == SSM_F32) v = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(src) + off);
        else v = bw_quad_from16(*reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(src) + off), dtype);
      } else {
        v = bw_tile_quad_slow(src, dtype, off, t, len);
      }
    }
    *reinterpret_cast<float4 *>(place(e)) = v;
  }
}

#define SSM_BW_STEP2(CTRL)                                \
  "v_fmac_f32_dpp %1, %1, %0 " CTRL "\n\t"                \
  "v_fmac_f32_dpp %3, %3, %2 " CTRL "\n\t"                \
  "v_mul_f32_dpp %0, %0, %0 " CTRL "\n\t"                 \
  "v_mul_f32_dpp %2, %2, %2 " CTRL "\n\t"

// Two independent inclusive scans of affine maps (see wave_scan_affine); only the
// offsets b0/b1 are complete in every lane afterwards.
__device__ __forceinline__ void bw_scan_x2(float &a0, float &b0, float &a1, float &b1) {
  asm volatile(
      "s_nop 4\n\t"
      SSM_BW_STEP2("row_shr:1 row_mask:0xf bank_mask:0xf")
      SSM_BW_STEP2("row_shr:2 row_mask:0xf bank_mask:0xf")
      SSM_BW_STEP2("row_shr:4 row_mask:0xf bank_mask:0xf")
      SSM_BW_STEP2("row_shr:8 row_mask:0xf bank_mask:0xf")
      SSM_BW_STEP2("row_bcast:15 row_mask:0xa bank_mask:0xf")
      "v_fmac_f32_dpp %1, %1, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %3, %3, %2 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1));
}

// The 24 partial sums of one step (8 waves x {pre, <gh,B>, A-term}), all requested before the first
// is used.  Written out because the compiler, short of registers at this point, otherwise reads them
// one by one and waits for each (24 LDS latencies per row).
template <int OFF>
__device__ __forceinline__ float bw_lds_read(unsigned addr) {
  float v;
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
template <int... J>
__device__ __forceinline__ void bw_read_parts(const float *p, float (&pv)[3 * BW_WAVES], std::integer_sequence<int, J...>) {
  const unsigned addr = (unsigned)(uintptr_t)p;            // low half of a generic LDS address = LDS offset
  ((pv[J] = bw_lds_read<((J / 3) * 3 * BW_T + (J % 3) * BW_T) * 4>(addr)), ...);
  // the values exist only after this wait: it takes them as operands so that no use can move above it
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(pv[0]), "+v"(pv[1]), "+v"(pv[2]), "+v"(pv[3]), "+v"(pv[4]), "+v"(pv[5]), "+v"(pv[6]), "+v"(pv[7]),
                 "+v"(pv[8]), "+v"(pv[9]), "+v"(pv[10]), "+v"(pv[11]), "+v"(pv[12]), "+v"(pv[13]), "+v"(pv[14]),
                 "+v"(pv[15]), "+v"(pv[16]), "+v"(pv[17]), "+v"(pv[18]), "+v"(pv[19]), "+v"(pv[20]), "+v"(pv[21]),
                 "+v"(pv[22]), "+v"(pv[23]));
}

__device__ __forceinline__ float lane_gather(float v, int src_lane) {
  return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane << 2, __float_as_int(v)));
}

// LDS admits one workgroup per CU, i.e. two waves per SIMD: telling the compiler so lets its scheduler spend
// registers on keeping several LDS reads in flight instead of waiting for each in turn.
template <typename io_t, bool BVARY, bool CVARY, bool HAS_Z>
__global__ __launch_bounds__(BW_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void scan_bwd_kernel(const ScanBwdParams p) {
  constexpr int K = BW_K, T = BW_T;
  extern __shared__ __align__(16) float lds[];
  // layout: [B tile][C tile][elem: delta,u,g][partials: 8 x 3 x T][red 2 x 8 x 2], then per (row, state):
  // qcarry, A log2(e), chunk-entering state, constant B and C, sums for dA / dB / dC; per row: D, bias, sums
  float *Bs = lds;
  float *Cs = Bs + (BVARY ? BW_MAX_N * T : 0);
  float *e_dl = Cs + (CVARY ? BW_MAX_N * T : 0);
  float *e_u = e_dl + T;
  float *e_g = e_u + T;
  float *part = e_g + T;                          // [wave][3][T]
  float *red = part + BW_WAVES * 3 * T;           // [2][BW_WAVES][2]
  const int RN = p.rows_per_wg * BW_MAX_N;
  float *qcarry = red + 2 * BW_WAVES * 2;         // [rows_per_wg][16] each from here on
  float *A2s = qcarry + RN, *Hins = A2s + RN, *Bcs = Hins + RN, *Ccs = Bcs + RN;
  float *sumA = Ccs + RN, *sumB = sumA + RN, *sumC = sumB + RN;
  float *Dks = sumC + RN;                         // [rows_per_wg] each
  float *biass = Dks + p.rows_per_wg, *sumD = biass + p.rows_per_wg, *sumb = sumD + p.rows_per_wg;

  const int wave = wave_id_uniform();
  const int lane = lane_id();
  const int tid = threadIdx.x;
  const int b = (int)blockIdx.x / p.nblk;
  const int blk = (int)blockIdx.x % p.nblk;
  const int d_first = blk * p.rows_per_wg;
  const int L = p.len, N = p.nstate;
  const int nchunks = (L + T - 1) / T;
  const int n0 = 2 * wave, n1 = 2 * wave + 1;
  const bool v0 = n0 < N, v1 = n1 < N;

  size_t b_tile_off = 0, c_tile_off = 0;
  if (BVARY) b_tile_off = ((size_t)b * p.b_groups + d_first / (p.dim / p.b_groups)) * (size_t)N * L;
  if (CVARY) c_tile_off = ((size_t)b * p.c_groups + d_first / (p.dim / p.c_groups)) * (size_t)N * L;

  // Everything a row needs besides its four streams is fetched here, once: inside the row loop a read
  // from global memory that the next instruction depends on costs more than the row's arithmetic.
  // Per-row sums are kept in LDS and written at the end.
  for (int e = tid; e < RN; e += BW_THREADS) {
    const int r = e / BW_MAX_N, n = e % BW_MAX_N;
    const int d = d_first + r;
    const size_t row = (size_t)b * p.dim + d;
    const bool valid = n < N;
    qcarry[e] = (p.dlast && valid) ? p.dlast[row * N + n] : 0.0f;      // adjoint from beyond the end
    A2s[e] = valid ? p.A[(size_t)d * N + n] * LOG2E : 0.0f;
    float bc = 0.0f, cc = 0.0f;
    if (!BVARY && valid) bc = load_as_f32(p.Bp, p.bc_dtype, ((p.b_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N + n);
    if (!CVARY && valid) cc = load_as_f32(p.Cp, p.bc_dtype, ((p.c_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N + n);
    Bcs[e] = bc;
    Ccs[e] = cc;
    sumA[e] = sumB[e] = sumC[e] = 0.0f;
  }
  for (int r = tid; r < p.rows_per_wg; r += BW_THREADS) {
    Dks[r] = p.Dk ? p.Dk[d_first + r] : 0.0f;
    biass[r] = p.bias ? p.bias[d_first + r] : 0.0f;
    sumD[r] = sumb[r] = 0.0f;
  }
  const io_t *zsrc = reinterpret_cast<const io_t *>(HAS_Z ? p.z : p.u);

  const int rev_lane = WAVE - 1 - lane;
#define BT(i)

  for (int c = nchunks - 1; c >= 0; --c) {
    const int t0 = c * T;
    BT(0)
    __syncthreads();     // tiles and qcarry free / visible
    BT(1)
    if (BVARY) bw_stage_tile(Bs, p.Bp, p.bc_dtype, b_tile_off, L, t0, N, p.bc_vec_ok != 0);
    if (CVARY) bw_stage_tile(Cs, p.Cp, p.bc_dtype, c_tile_off, L, t0, N, p.bc_vec_ok != 0);
    for (int e = tid; e < RN; e += BW_THREADS) {           // the rows' states entering this chunk
      const int r = e / BW_MAX_N, n = e % BW_MAX_N;
      const size_t row = (size_t)b * p.dim + d_first + r;
      Hins[e] = n < N ? p.chunk_states[(row * nchunks + c) * (size_t)N + n] : 0.0f;
    }

    float accB[2][K], accC[2][K];
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int i = 0; i < K; ++i) accB[w][i] = accC[w][i] = 0.0f;

    // The four inputs of element (row, t0 + tid) are requested one row ahead: the reads of
    // row r + 1 are in flight while the wave works on the states of row r.
    const int te = t0 + tid;
    const int te_c = min(te, L - 1);
    io_t nx_u, nx_dl, nx_go, nx_z;
    {
      const size_t idx = ((size_t)b * p.dim + d_first) * L + te_c;
      nx_u = reinterpret_cast<const io_t *>(p.u)[idx];
      nx_dl = reinterpret_cast<const io_t *>(p.delta)[idx];
      nx_go = reinterpret_cast<const io_t *>(p.dout)[idx];
      nx_z = zsrc[idx];
    }

    // per-row sums of dD and dbias: the waves' partial sums of row r lie in red[r & 1]
    auto fold_red = [&](int r) {
      const float *rr = red + (size_t)(r & 1) * BW_WAVES * 2;
      float sD = 0.0f, sb = 0.0f;
      for (int wv = 0; wv < BW_WAVES; ++wv) {
        sD += rr[wv * 2];
        sb += rr[wv * 2 + 1];
      }
      sumD[r] += sD;
      sumb[r] += sb;
    };

    BT(2)
    // One row.  FULL: the chunk lies wholly inside the sequence, so nothing in the row is conditional on
    // the step index; the compiler then knows exactly how many memory operations are in flight at each
    // wait and the reads requested a row ahead are not held up by the previous row's stores.
    auto do_row = [&](auto full_tag, int r) {
      constexpr bool FULL = decltype(full_tag)::value;
      const int d = d_first + r;
      const size_t row = (size_t)b * p.dim + d;
      const float Dk = Dks[r];

      // ---- element-wise stage: thread tid owns step t0 + tid of this row
      float el_u = 0.0f, el_dl = 0.0f, el_g = 0.0f, el_sig = 1.0f, el_dz = 0.0f;
      const io_t cur_u = nx_u, cur_dl = nx_dl, cur_go = nx_go, cur_z = nx_z;
      {
        const int rn = min(r + 1, p.rows_per_wg - 1);
        const size_t idx = ((size_t)b * p.dim + d_first + rn) * L + te_c;
        nx_u = reinterpret_cast<const io_t *>(p.u)[idx];
        nx_dl = reinterpret_cast<const io_t *>(p.delta)[idx];
        nx_go = reinterpret_cast<const io_t *>(p.dout)[idx];
        nx_z = zsrc[idx];
      }
      if (FULL || te < L) {
        el_u = to_f32(cur_u);
        float draw = to_f32(cur_dl);
        draw += biass[r];
        if (p.softplus) {
          el_dl = softplus_f32(draw);
          el_sig = draw > 20.0f ? 1.0f : sigmoid_f32(draw);
        } else {
          el_dl = draw;
        }
        const float go = to_f32(cur_go);
        if (HAS_Z) {
          const float zv = to_f32(cur_z);
          const float sg = sigmoid_f32(zv);
          el_g = go * zv * sg;
          el_dz = go * sg * __builtin_fmaf(zv, 1.0f - sg, 1.0f);      // dout * silu'(z)
        } else {
          el_g = go;
        }
      }
      e_dl[tid] = el_dl;
      e_u[tid] = el_u;
      e_g[tid] = el_g;
      BT(3)
      __syncthreads();                                                  // (1) staged row visible
      BT(4)
      if (tid == 0 && r > 0) fold_red(r - 1);

      // ---- per-state work: this wave owns states n0, n1
      float dl[K], uu[K], g[K];
      {
        const float4 a0 = *reinterpret_cast<const float4 *>(e_dl + lane * K);
        const float4 a1 = *reinterpret_cast<const float4 *>(e_dl + lane * K + 4);
        const float4 b0 = *reinterpret_cast<const float4 *>(e_u + lane * K);
        const float4 b1 = *reinterpret_cast<const float4 *>(e_u + lane * K + 4);
        const float4 c0 = *reinterpret_cast<const float4 *>(e_g + lane * K);
        const float4 c1 = *reinterpret_cast<const float4 *>(e_g + lane * K + 4);
        dl[0] = a0.x; dl[1] = a0.y; dl[2] = a0.z; dl[3] = a0.w; dl[4] = a1.x; dl[5] = a1.y; dl[6] = a1.z; dl[7] = a1.w;
        uu[0] = b0.x; uu[1] = b0.y; uu[2] = b0.z; uu[3] = b0.w; uu[4] = b1.x; uu[5] = b1.y; uu[6] = b1.z; uu[7] = b1.w;
        g[0] = c0.x; g[1] = c0.y; g[2] = c0.z; g[3] = c0.w; g[4] = c1.x; g[5] = c1.y; g[6] = c1.z; g[7] = c1.w;
      }
      float dsum = 0.0f;
#pragma unroll
      for (int i = 0; i < K; ++i) dsum += dl[i];

      float a[2][K], hp[2][K], cc[2][K], bq[2][K];   // decay, state before step, g*C, B values
      float P[2], h[2], Hin[2], A2[2], Qa[2], Pr[2], qin_carry[2];
      float pre[K], sgb[K], dda[K];                   // partial sums over this wave's states
#pragma unroll
      for (int i = 0; i < K; ++i) pre[i] = sgb[i] = dda[i] = 0.0f;

#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const int n = w == 0 ? n0 : n1;
        const bool valid = w == 0 ? v0 : v1;
        const int rn_ = r * BW_MAX_N + n;              // n < 16 always: invalid states hold zeros
        A2[w] = A2s[rn_];
        Hin[w] = Hins[rn_];
        qin_carry[w] = qcarry[rn_];
        const float bconst = Bcs[rn_], cconst = Ccs[rn_];
        const int nrow = valid ? n : 0;
#pragma unroll
        for (int q4 = 0; q4 < K / 4; ++q4) {
          float4 bv, cv;
          if (BVARY) bv = *reinterpret_cast<const float4 *>(Bs + nrow * T + q4 * (WAVE * 4) + lane * 4);
          else bv = make_float4(bconst, bconst, bconst, bconst);
          if (CVARY) cv = *reinterpret_cast<const float4 *>(Cs + nrow * T + q4 * (WAVE * 4) + lane * 4);
          else cv = make_float4(cconst, cconst, cconst, cconst);
          if (!valid) { bv = make_float4(0.f, 0.f, 0.f, 0.f); cv = bv; }
          bq[w][q4 * 4 + 0] = bv.x; bq[w][q4 * 4 + 1] = bv.y; bq[w][q4 * 4 + 2] = bv.z; bq[w][q4 * 4 + 3] = bv.w;
          cc[w][q4 * 4 + 0] = cv.x; cc[w][q4 * 4 + 1] = cv.y; cc[w][q4 * 4 + 2] = cv.z; cc[w][q4 * 4 + 3] = cv.w;
        }
        // forward fold of the lane's 8 steps
        float hh = 0.0f;
#pragma unroll
        for (int i = 0; i < K; ++i) {
          a[w][i] = exp2_hw(dl[i] * A2[w]);
          hh = __builtin_fmaf(a[w][i], hh, dl[i] * uu[i] * bq[w][i]);
        }
        P[w] = exp2_hw(dsum * A2[w]);
        Pr[w] = P[w];
        h[w] = __builtin_fmaf(P[w], lane == 0 ? Hin[w] : 0.0f, hh);
      }
      BT(5)
      bw_scan_x2(P[0], h[0], P[1], h[1]);
      BT(6)
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        // replay forward: hp[i] = state before step i, hcur = state after it
        float hcur = wave_prev(h[w], Hin[w]);
        float Q = 0.0f;
#pragma unroll
        for (int i = 0; i < K; ++i) {
          hp[w][i] = hcur;
          hcur = __builtin_fmaf(a[w][i], hcur, dl[i] * uu[i] * bq[w][i]);
          pre[i] = __builtin_fmaf(hcur, cc[w][i], pre[i]);
          const float gc = g[i] * cc[w][i];
          accC[w][i] = __builtin_fmaf(g[i], hcur, accC[w][i]);
          cc[w][i] = gc;                        // from here on cc holds g_t * C_t
        }
        // reverse fold: q_first = Pr * q_in + Qa
#pragma unroll
        for (int i = K - 1; i >= 0; --i) Q = a[w][i] * (cc[w][i] + Q);
        Qa[w] = Q;
      }
      // reverse scan: run the forward scan on lane-reversed operands
      float rP0 = lane_gather(Pr[0], rev_lane), rQ0 = lane_gather(Qa[0], rev_lane);
      float rP1 = lane_gather(Pr[1], rev_lane), rQ1 = lane_gather(Qa[1], rev_lane);
      rQ0 = __builtin_fmaf(rP0, lane == 0 ? qin_carry[0] : 0.0f, rQ0);
      rQ1 = __builtin_fmaf(rP1, lane == 0 ? qin_carry[1] : 0.0f, rQ1);
      bw_scan_x2(rP0, rQ0, rP1, rQ1);
      // reversed lane j now holds q at the first step of original lane 63-j
      const float qn0 = wave_read_lane(rQ0, WAVE - 1), qn1 = wave_read_lane(rQ1, WAVE - 1);
      float qin[2];
      {
        const int src = (WAVE - 2 - lane) & (WAVE - 1);        // original lane + 1, in the reversed domain
        const float t0v = lane_gather(rQ0, src), t1v = lane_gather(rQ1, src);
        qin[0] = lane == WAVE - 1 ? qin_carry[0] : t0v;
        qin[1] = lane == WAVE - 1 ? qin_carry[1] : t1v;
      }
      BT(8)
      float dA_acc[2] = {0.0f, 0.0f}, dBc_acc[2] = {0.0f, 0.0f};
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        float q = qin[w];
#pragma unroll
        for (int i = K - 1; i >= 0; --i) {
          const float gh = cc[w][i] + q;
          const float du_i = dl[i] * uu[i];
          if (BVARY) accB[w][i] = __builtin_fmaf(gh, du_i, accB[w][i]);
          else dBc_acc[w] = __builtin_fmaf(gh, du_i, dBc_acc[w]);
          sgb[i] = __builtin_fmaf(gh, bq[w][i], sgb[i]);
          q = a[w][i] * gh;
          const float wv = q * hp[w][i];
          dda[i] = __builtin_fmaf(wv, A2[w], dda[i]);
          dA_acc[w] = __builtin_fmaf(wv, dl[i], dA_acc[w]);
        }
      }
      // partial sums over this wave's two states -> LDS
      {
        float *pw = part + (size_t)wave * 3 * T + lane * K;
        *reinterpret_cast<float4 *>(pw) = make_float4(pre[0], pre[1], pre[2], pre[3]);
        *reinterpret_cast<float4 *>(pw + 4) = make_float4(pre[4], pre[5], pre[6], pre[7]);
        *reinterpret_cast<float4 *>(pw + T) = make_float4(sgb[0], sgb[1], sgb[2], sgb[3]);
        *reinterpret_cast<float4 *>(pw + T + 4) = make_float4(sgb[4], sgb[5], sgb[6], sgb[7]);
        *reinterpret_cast<float4 *>(pw + 2 * T) = make_float4(dda[0], dda[1], dda[2], dda[3]);
        *reinterpret_cast<float4 *>(pw + 2 * T + 4) = make_float4(dda[4], dda[5], dda[6], dda[7]);
      }
      // per-row, per-state sums (this wave is the only writer of these addresses)
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const int n = w == 0 ? n0 : n1;
        const bool valid = w == 0 ? v0 : v1;
        const float sA = wave_sum(dA_acc[w]);
        float sB = 0.0f, sC = 0.0f;
        if (!BVARY) sB = wave_sum(dBc_acc[w]);
        if (!CVARY) {
          float t = 0.0f;
#pragma unroll
          for (int i = 0; i < K; ++i) t += accC[w][i];
          sC = wave_sum(t);
#pragma unroll
          for (int i = 0; i < K; ++i) accC[w][i] = 0.0f;
        }
        if (valid && lane == 0) {
          const int o = r * BW_MAX_N + n;
          sumA[o] += sA;
          if (!BVARY) sumB[o] += sB;
          if (!CVARY) sumC[o] += sC;
          qcarry[o] = w == 0 ? qn0 : qn1;
        }
      }
      BT(10)
      __syncthreads();                                                  // (2) partials visible
      BT(11)

      // ---- finish element tid of this row
      float pv[3 * BW_WAVES];
      bw_read_parts(part + tid, pv, std::make_integer_sequence<int, 3 * BW_WAVES>{});
      float s_pre = 0.0f, s_gb = 0.0f, s_da = 0.0f;
#pragma unroll
      for (int wv = 0; wv < BW_WAVES; ++wv) {
        s_pre += pv[3 * wv];
        s_gb += pv[3 * wv + 1];
        s_da += pv[3 * wv + 2];
      }
      BT(7)
      float dD_c = 0.0f, dbias_c = 0.0f;
      if (FULL || te < L) {
        const size_t idx = row * L + te;
        const float du = __builtin_fmaf(s_gb, el_dl, el_g * Dk);
        const float ddl = __builtin_fmaf(s_gb, el_u, s_da * LN2) * el_sig;
        reinterpret_cast<io_t *>(p.du)[idx] = from_f32<io_t>(du);
        reinterpret_cast<io_t *>(p.ddelta)[idx] = from_f32<io_t>(ddl);
        if (HAS_Z) reinterpret_cast<io_t *>(p.dz)[idx] = from_f32<io_t>(el_dz * __builtin_fmaf(Dk, el_u, s_pre));
        dD_c = el_g * el_u;
        dbias_c = ddl;
      }
      BT(9)
      {
        const float sD = wave_sum(dD_c), sb = wave_sum(dbias_c);
        float *rr = red + (size_t)(r & 1) * BW_WAVES * 2;
        if (lane == 0) {
          rr[wave * 2] = sD;
          rr[wave * 2 + 1] = sb;
        }
      }
      BT(2)
      // No barrier here: the next row's element-wise stage writes e_* (last read before barrier 2),
      // its per-state work writes `part` only after barrier 1 of that row, which every wave reaches
      // after it has finished the sums above; `red` alternates between two buffers and is folded
      // after that same barrier.
    };
    if (t0 + T <= L)
      for (int r = 0; r < p.rows_per_wg; ++r) do_row(std::true_type{}, r);
    else
      for (int r = 0; r < p.rows_per_wg; ++r) do_row(std::false_type{}, r);
    __syncthreads();
    if (tid == 0) fold_red(p.rows_per_wg - 1);

    // ---- flush this chunk's dB / dC partials (sum over the workgroup's channels)
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const int n = w == 0 ? n0 : n1;
      const bool valid = w == 0 ? v0 : v1;
      if (!valid) continue;
      const size_t base = (((size_t)b * p.nblk + blk) * N + n) * (size_t)L + t0 + lane * K;
      const bool full = t0 + lane * K + K <= L && L % 4 == 0;
      if (BVARY) {
        if (full) {
          *reinterpret_cast<float4 *>(p.dB_part + base) = make_float4(accB[w][0], accB[w][1], accB[w][2], accB[w][3]);
          *reinterpret_cast<float4 *>(p.dB_part + base + 4) = make_float4(accB[w][4], accB[w][5], accB[w][6], accB[w][7]);
        } else {
#pragma unroll
          for (int i = 0; i < K; ++i)
            if (t0 + lane * K + i < L) p.dB_part[base + i] = accB[w][i];
        }
      }
      if (CVARY) {
        if (full) {
          *reinterpret_cast<float4 *>(p.dC_part + base) = make_float4(accC[w][0], accC[w][1], accC[w][2], accC[w][3]);
          *reinterpret_cast<float4 *>(p.dC_part + base + 4) = make_float4(accC[w][4], accC[w][5], accC[w][6], accC[w][7]);
        } else {
#pragma unroll
          for (int i = 0; i < K; ++i)
            if (t0 + lane * K + i < L) p.dC_part[base + i] = accC[w][i];
        }
      }
    }
  }
  // ---- the per-row sums
  __syncthreads();
  for (int e = tid; e < RN; e += BW_THREADS) {
    const int r = e / BW_MAX_N, n = e % BW_MAX_N;
    if (n < N) {
      const size_t o = ((size_t)b * p.dim + d_first + r) * N + n;
      p.dA_rows[o] = sumA[e];
      if (!BVARY) p.dB_part[o] = sumB[e];
      if (!CVARY) p.dC_part[o] = sumC[e];
    }
  }
  for (int r = tid; r < p.rows_per_wg; r += BW_THREADS) {
    const size_t row = (size_t)b * p.dim + d_first + r;
    p.dD_rows[row] = sumD[r];
    p.dbias_rows[row] = sumb[r];
  }
#undef BT
}

// out[o][i] = sum_{j < count} in[(o * count + j) * inner + i], fixed order.  The terms of an output are read
// eight at a time (independent reads in flight together) and added in order.
__global__ __launch_bounds__(256) void fold_sum_kernel(const float *in, float *out, size_t outer, int count,
                                                       size_t inner) {
  const size_t total = outer * inner;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
    const size_t o = e / inner, i = e % inner;
    const float *src = in + o * count * inner + i;
    float s = 0.0f;
    int j = 0;
    for (; j + 8 <= count; j += 8) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = src[(size_t)(j + k) * inner];
#pragma unroll
      for (int k = 0; k < 8; ++k) s += v[k];
    }
    for (; j < count; ++j) s += src[(size_t)j * inner];
    out[e] = s;
  }
}

// The same for four neighbouring outputs per thread (inner a multiple of four, 16-byte aligned tensors).
__global__ __launch_bounds__(256) void fold_sum_vec4_kernel(const float *in, float *out, size_t outer, int count,
                                                            size_t inner) {
  const size_t inner4 = inner / 4, total = outer * inner4;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
    const size_t o = e / inner4, i = (e % inner4) * 4;
    const float *src = in + o * count * inner + i;
    float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    int j = 0;
    for (; j + 4 <= count; j += 4) {
      float4 v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = *reinterpret_cast<const float4 *>(src + (size_t)(j + k) * inner);
#pragma unroll
      for (int k = 0; k < 4; ++k) { s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w; }
    }
    for (; j < count; ++j) {
      const float4 v = *reinterpret_cast<const float4 *>(src + (size_t)j * inner);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    *reinterpret_cast<float4 *>(out + o * inner + i) = s;
  }
}

// out[i] = sum_{j < count} in[j * inner + i]
__global__ __launch_bounds__(256) void fold_rows_kernel(const float *in, float *out, int count, size_t inner) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < inner; i += (size_t)gridDim.x * blockDim.x) {
    float s = 0.0f;
    int j = 0;
    for (; j + 8 <= count; j += 8) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = in[(size_t)(j + k) * inner + i];
#pragma unroll
      for (int k = 0; k < 8; ++k) s += v[k];
    }
    for (; j < count; ++j) s += in[(size_t)j * inner + i];
    out[i] = s;
  }
}

// Up to five such sums in one launch (dA, dD, the bias and, for projections constant in time, dB and dC: launches
// of a few microseconds each, of which the gaps between them were as long as the work): workgroup ranges per job.
constexpr int FOLD_JOBS = 5;
struct FoldJobs {
  const float *in[FOLD_JOBS];
  float *out[FOLD_JOBS];
  size_t inner[FOLD_JOBS];
  int count[FOLD_JOBS];
  unsigned first_block[FOLD_JOBS + 1];
  int n;
};

__global__ __launch_bounds__(256) void fold_rows_multi_kernel(const FoldJobs jobs) {
  int j = 0;
  while (j + 1 < jobs.n && blockIdx.x >= jobs.first_block[j + 1]) ++j;
  const float *in = jobs.in[j];
  float *out = jobs.out[j];
  const size_t inner = jobs.inner[j];
  const int count = jobs.count[j];
  const size_t blocks = jobs.first_block[j + 1] - jobs.first_block[j];
  for (size_t i = (size_t)(blockIdx.x - jobs.first_block[j]) * blockDim.x + threadIdx.x; i < inner; i += blocks * blockDim.x) {
    float s = 0.0f;
    int k0 = 0;
    for (; k0 + 8 <= count; k0 += 8) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = in[(size_t)(k0 + k) * inner + i];
#pragma unroll
      for (int k = 0; k < 8; ++k) s += v[k];
    }
    for (; k0 < count; ++k0) s += in[(size_t)k0 * inner + i];
    out[i] = s;
  }
}

static unsigned fold_grid(size_t n) {
  const size_t g = (n + 255) / 256;
  return (unsigned)(g < 1 ? 1 : (g > 65535 ? 65535 : g));
}

void launch_fold_rows(const float *in, float *out, int count, size_t inner, hipStream_t s) {
  hipLaunchKernelGGL(fold_rows_kernel, dim3(fold_grid(inner)), dim3(256), 0, s, in, out, count, inner);
}

// The same sum when there are few outputs and many terms each: a workgroup takes up to 16 neighbouring
// outputs of one `o`; its 256 threads are those outputs x slices of the terms, added in a fixed order
// (slice by slice, then over the slices).
__global__ __launch_bounds__(256) void fold_sum_wide_kernel(const float *in, float *out, int count, size_t inner,
                                                            int cols, int blocks_per_outer) {
  __shared__ float part[256];
  const int slices = 256 / cols;
  const int cl = threadIdx.x % cols, sl = threadIdx.x / cols;
  const size_t o = blockIdx.x / blocks_per_outer;
  const size_t i = (size_t)(blockIdx.x % blocks_per_outer) * cols + cl;
  float sum = 0.0f;
  if (i < inner && sl < slices) {
    // eight terms at a time: their reads are in flight together, the additions keep their order
    int j = sl;
    for (; j + 7 * slices < count; j += 8 * slices) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = in[(o * count + j + k * slices) * inner + i];
#pragma unroll
      for (int k = 0; k < 8; ++k) sum += v[k];
    }
    for (; j < count; j += slices) sum += in[(o * count + j) * inner + i];
  }
  part[threadIdx.x] = sum;
  __syncthreads();
  if (sl == 0 && i < inner) {
    float t = 0.0f;
    for (int k = 0; k < slices; ++k) t += part[k * cols + cl];
    out[o * inner + i] = t;
  }
}

void launch_fold_sum(const float *in, float *out, size_t outer, int count, size_t inner, hipStream_t s) {
  if (outer * inner < 65536 && count >= 64) {
    const int cols = inner >= 16 ? 16 : (inner >= 8 ? 8 : (inner >= 4 ? 4 : (inner >= 2 ? 2 : 1)));
    const int bpo = (int)((inner + cols - 1) / cols);
    hipLaunchKernelGGL(fold_sum_wide_kernel, dim3((unsigned)(outer * bpo)), dim3(256), 0, s, in, out, count, inner, cols,
                       bpo);
    return;
  }
  if (inner % 4 == 0 && aligned_to(in, 16) && aligned_to(out, 16)) {
    hipLaunchKernelGGL(fold_sum_vec4_kernel, dim3(fold_grid(outer * inner / 4)), dim3(256), 0, s, in, out, outer, count, inner);
    return;
  }
  hipLaunchKernelGGL(fold_sum_kernel, dim3(fold_grid(outer * inner)), dim3(256), 0, s, in, out, outer, count, inner);
}

struct BwdPlan {
  int rows_per_wg, nblk;
  size_t off_dA, off_dD, off_dbias, off_dB, off_dC, total;   // byte offsets into the workspace
};

static BwdPlan plan_bwd(int batch, int dim, int len, int nstate, int b_kind, int c_kind, int b_groups,
                        int c_groups) {
  const bool bv = b_kind == SSM_PROJ_BGNL, cv = c_kind == SSM_PROJ_BGNL;
  const int per_b = bv ? dim / b_groups : dim, per_c = cv ? dim / c_groups : dim;
  // Block of channels (<= 32) that stays inside one B group and one C group; among
  // the divisors >= 8 prefer one whose grid is a whole number of 256-CU rounds.
  int rows = 1;
  for (int r = 32; r >= 1; --r)
    if (per_b % r == 0 && per_c % r == 0) { rows = r; break; }
  for (int r = 32; r >= 8; --r)
    if (per_b % r == 0 && per_c % r == 0 && ((size_t)batch * (dim / r)) % 256 == 0) { rows = r; break; }
  BwdPlan pl;
  pl.rows_per_wg = rows;
  pl.nblk = dim / rows;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += (bytes + 255) / 256 * 256; return o; };
  pl.off_dA = take((size_t)batch * dim * nstate * 4);
  pl.off_dD = take((size_t)batch * dim * 4);
  pl.off_dbias = take((size_t)batch * dim * 4);
  pl.off_dB = take(bv ? (size_t)batch * pl.nblk * nstate * len * 4 : (size_t)batch * dim * nstate * 4);
  pl.off_dC = take(cv ? (size_t)batch * pl.nblk * nstate * len * 4 : (size_t)batch * dim * nstate * 4);
  pl.total = off;
  return pl;
}

template <typename io_t>
static int launch_bwd(const ScanBwdParams &p, hipStream_t s) {
  const bool bv = p.b_kind == SSM_PROJ_BGNL, cv = p.c_kind == SSM_PROJ_BGNL;
  const size_t lds = ((size_t)((int)bv + (int)cv) * BW_MAX_N * BW_T + 3 * BW_T + BW_WAVES * 3 * BW_T +
                      2 * BW_WAVES * 2 + (size_t)p.rows_per_wg * (8 * BW_MAX_N + 4)) * sizeof(float);
  const unsigned grid = (unsigned)((size_t)p.batch * p.nblk);
#define SSM_BW_LAUNCH(BV, CV)                                                              \
  {                                                                                        \
    auto kernel = p.z ? scan_bwd_kernel<io_t, BV, CV, true> : scan_bwd_kernel<io_t, BV, CV, false>; \
    if (allow_dynamic_lds(kernel, lds) != hipSuccess) {                                    \
      (void)hipGetLastError();                                                             \
      set_error("ssm_scan_bwd: cannot reserve %zu bytes of LDS", lds);                     \
      return SSM_ERR_LAUNCH;                                                               \
    }                                                                                      \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(BW_THREADS), lds, s, p);                   \
  }
  if (bv && cv) SSM_BW_LAUNCH(true, true)
  else if (bv) SSM_BW_LAUNCH(true, false)
  else if (cv) SSM_BW_LAUNCH(false, true)
  else SSM_BW_LAUNCH(false, false)
#undef SSM_BW_LAUNCH
  SSM_CHECK_LAUNCH("ssm_scan_bwd");
  return SSM_OK;
}

}  // namespace ssm

#include "scan_bwd_fast.hpp"
#include "scan_bwd_rowbc.hpp"

extern "C" size_t ssm_scan_bwd_workspace_bytes(int batch, int dim, int seqlen, int nstate, int b_kind, int c_kind,
                                               int b_groups, int c_groups) {
  using namespace ssm;
  if (batch <= 0 || dim <= 0 || seqlen <= 0 || nstate <= 0) return 0;
  if (b_kind == SSM_PROJ_BGNL && (b_groups <= 0 || dim % b_groups)) return 0;
  if (c_kind == SSM_PROJ_BGNL && (c_groups <= 0 || dim % c_groups)) return 0;
  return plan_bwd(batch, dim, seqlen, nstate, b_kind, c_kind, b_groups, c_groups).total;
}

// Whether a call takes the kernel for projections of their own per channel (scan_bwd_rowbc.hpp): B and C of shape
// (B, D, N, L), activations in aligned rows of whole 8-step runs.  A selector of 1 (test-hooks build) keeps the
// general kernel.
static bool scan_bwd_is_per_row(const ssm_scan_bwd_args *a) {
  using namespace ssm;
  if (!a || SSM_RESERVED(a) == 1) return false;
  if (a->b_kind != SSM_PROJ_BGNL || a->c_kind != SSM_PROJ_BGNL || a->b_groups != a->dim || a->c_groups != a->dim) return false;
  if (a->seqlen <= 0 || a->seqlen % 8 != 0 || a->nstate <= 0 || a->nstate > BW_MAX_N) return false;
  if (!valid_dtype(a->io_dtype) || !(a->bc_dtype == a->io_dtype || a->bc_dtype == SSM_F32)) return false;
  const int bs = dtype_size(a->bc_dtype);
  return aligned_to(a->u, 16) && aligned_to(a->delta, 16) && aligned_to(a->dout, 16) && aligned_to(a->du, 16) &&
         aligned_to(a->ddelta, 16) && (!a->z || (aligned_to(a->z, 16) && aligned_to(a->dz, 16))) &&
         aligned_to(a->Bproj, 8 * bs) && aligned_to(a->Cproj, 8 * bs) && aligned_to(a->dB, 16) && aligned_to(a->dC, 16);
}

// Whether a call takes the wave-per-row kernel for projections that are constant in time, (D, N) or (B, D, N).
static bool scan_bwd_is_const_row(const ssm_scan_bwd_args *a) {
  using namespace ssm;
  if (!a || SSM_RESERVED(a) == 1) return false;
  if (a->b_kind == SSM_PROJ_BGNL || a->c_kind == SSM_PROJ_BGNL) return false;
  if (a->seqlen <= 0 || a->seqlen % 8 != 0 || a->nstate <= 0 || a->nstate > BW_MAX_N) return false;
  if (!valid_dtype(a->io_dtype) || !valid_dtype(a->bc_dtype)) return false;
  return aligned_to(a->u, 16) && aligned_to(a->delta, 16) && aligned_to(a->dout, 16) && aligned_to(a->du, 16) &&
         aligned_to(a->ddelta, 16) && (!a->z || (aligned_to(a->z, 16) && aligned_to(a->dz, 16)));
}

extern "C" size_t ssm_scan_bwd_per_row_workspace_bytes(const ssm_scan_bwd_args *a) {
  if (!scan_bwd_is_per_row(a)) return 0;
  return ssm::plan_bwd(a->batch, a->dim, a->seqlen, a->nstate, a->b_kind, a->c_kind, a->b_groups, a->c_groups).off_dB;
}

extern "C" int ssm_scan_bwd(const ssm_scan_bwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_scan_bwd: args is NULL");
  SSM_CHECK_RESERVED("ssm_scan_bwd", a);
  SSM_REQUIRE(a->u && a->delta && a->A && a->Bproj && a->Cproj && a->dout && a->chunk_states &&
                  a->du && a->ddelta && a->dA && a->dB && a->dC,
              SSM_ERR_NULL_POINTER,
              "ssm_scan_bwd: u, delta, A, Bproj, Cproj, dout, chunk_states, du, ddelta, dA, dB and dC are required");
  SSM_REQUIRE(!a->z == !a->dz, SSM_ERR_NULL_POINTER, "ssm_scan_bwd: z and dz must be given together");
  SSM_REQUIRE(!a->Dskip || a->dD, SSM_ERR_NULL_POINTER, "ssm_scan_bwd: dD is required when Dskip is given");
  SSM_REQUIRE(a->batch > 0 && a->dim > 0 && a->seqlen > 0 && a->nstate > 0, SSM_ERR_BAD_SHAPE,
              "ssm_scan_bwd: batch=%d dim=%d seqlen=%d nstate=%d must all be positive", a->batch, a->dim, a->seqlen,
              a->nstate);
  SSM_REQUIRE(a->nstate <= BW_MAX_N, SSM_ERR_TOO_LARGE,
              "ssm_scan_bwd: nstate=%d exceeds %d per call (split the state axis)", a->nstate, BW_MAX_N);
  SSM_REQUIRE(valid_dtype(a->io_dtype) && valid_dtype(a->bc_dtype), SSM_ERR_BAD_DTYPE,
              "ssm_scan_bwd: io_dtype=%d bc_dtype=%d", a->io_dtype, a->bc_dtype);
  auto kind_ok = [](int k) { return k == SSM_PROJ_DN || k == SSM_PROJ_BDN || k == SSM_PROJ_BGNL; };
  SSM_REQUIRE(kind_ok(a->b_kind) && kind_ok(a->c_kind), SSM_ERR_BAD_KIND, "ssm_scan_bwd: b_kind=%d c_kind=%d",
              a->b_kind, a->c_kind);
  const bool bv = a->b_kind == SSM_PROJ_BGNL, cv = a->c_kind == SSM_PROJ_BGNL;
  if (bv) SSM_REQUIRE(a->b_groups > 0 && a->dim % a->b_groups == 0, SSM_ERR_BAD_SHAPE,
                      "ssm_scan_bwd: b_groups=%d must divide dim=%d", a->b_groups, a->dim);
  if (cv) SSM_REQUIRE(a->c_groups > 0 && a->dim % a->c_groups == 0, SSM_ERR_BAD_SHAPE,
                      "ssm_scan_bwd: c_groups=%d must divide dim=%d", a->c_groups, a->dim);
  SSM_REQUIRE((size_t)a->batch * a->dim < ((size_t)1 << 31) &&
                  (size_t)a->batch * a->dim * a->seqlen < ((size_t)1 << 40),
              SSM_ERR_TOO_LARGE, "ssm_scan_bwd: tensor too large");
  const BwdPlan pl = plan_bwd(a->batch, a->dim, a->seqlen, a->nstate, a->b_kind, a->c_kind,
                              bv ? a->b_groups : 1, cv ? a->c_groups : 1);
  const bool per_row = scan_bwd_is_per_row(a);
  SSM_REQUIRE(a->dbc_dtype == SSM_F32 || (per_row && a->dbc_dtype == a->bc_dtype), SSM_ERR_BAD_DTYPE,
              "ssm_scan_bwd: dbc_dtype=%d: dB and dC are float32, or of the projections' type in a call for which "
              "ssm_scan_bwd_per_row_workspace_bytes() is not 0", a->dbc_dtype);
  const size_t ws_need = per_row ? pl.off_dB : pl.total;     // per row: no partial sums of dB and dC
  SSM_REQUIRE(a->workspace && a->workspace_bytes >= ws_need && aligned_to(a->workspace, 256), SSM_ERR_WORKSPACE,
              "ssm_scan_bwd: a 256-byte aligned workspace of %zu bytes is required", ws_need);
  const int es = dtype_size(a->io_dtype), bs = dtype_size(a->bc_dtype);
  SSM_REQUIRE(aligned_to(a->u, es) && aligned_to(a->delta, es) && aligned_to(a->dout, es) && aligned_to(a->du, es) &&
                  aligned_to(a->ddelta, es) && (!a->z || (aligned_to(a->z, es) && aligned_to(a->dz, es))) &&
                  aligned_to(a->Bproj, bs) && aligned_to(a->Cproj, bs) && aligned_to(a->dB, 16) &&
                  aligned_to(a->dC, 16),
              SSM_ERR_ALIGNMENT, "ssm_scan_bwd: a pointer is not sufficiently aligned");

  char *ws = reinterpret_cast<char *>(a->workspace);
  ScanBwdParams p{};
  p.u = a->u; p.delta = a->delta; p.z = a->z; p.dout = a->dout; p.Bp = a->Bproj; p.Cp = a->Cproj;
  p.A = a->A; p.Dk = a->Dskip; p.bias = a->dt_bias; p.dlast = a->dlast_state; p.chunk_states = a->chunk_states;
  p.du = a->du; p.ddelta = a->ddelta; p.dz = a->dz;
  p.dA_rows = reinterpret_cast<float *>(ws + pl.off_dA);
  p.dD_rows = reinterpret_cast<float *>(ws + pl.off_dD);
  p.dbias_rows = reinterpret_cast<float *>(ws + pl.off_dbias);
  p.dB_part = reinterpret_cast<float *>(ws + pl.off_dB);
  p.dC_part = reinterpret_cast<float *>(ws + pl.off_dC);
  p.batch = a->batch; p.dim = a->dim; p.len = a->seqlen; p.nstate = a->nstate;
  p.bc_dtype = a->bc_dtype; p.b_kind = a->b_kind; p.c_kind = a->c_kind;
  p.b_groups = bv ? a->b_groups : 1; p.c_groups = cv ? a->c_groups : 1;
  p.softplus = a->delta_softplus ? 1 : 0;
  p.rows_per_wg = pl.rows_per_wg; p.nblk = pl.nblk;
  p.bc_vec_ok = a->seqlen % 4 == 0 && aligned_to(a->Bproj, 4 * bs) && aligned_to(a->Cproj, 4 * bs);
  // A selector of 2 (test-hooks build) lets no wave wait for its neighbour at all, so that the give-up path of
  // the wave-per-row kernel runs: every wave goes on at once and poisons dB and dC.
  p.spin_limit = SSM_RESERVED(a) == 2 ? 0 : (1 << 16);

  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  int rc;
  // The specialised kernel: activations in aligned rows of whole 8-step runs, time-varying B and C of the
  // activations' type or float32, groups that workgroups of 16, 32 or 48 channels tile, and no more partial
  // sums than the workspace was sized for.  A selector of 1 keeps the general kernel.
  int fast_rpw = 0;
  if (bv && cv && SSM_RESERVED(a) != 1 && a->seqlen % 8 == 0 &&
      (a->bc_dtype == a->io_dtype || a->bc_dtype == SSM_F32) && aligned_to(a->u, 16) && aligned_to(a->delta, 16) &&
      aligned_to(a->dout, 16) && aligned_to(a->du, 16) && aligned_to(a->ddelta, 16) &&
      (!a->z || (aligned_to(a->z, 16) && aligned_to(a->dz, 16))) && aligned_to(a->Bproj, 4 * bs) &&
      aligned_to(a->Cproj, 4 * bs)) {
    fast_rpw = scan_bwd_fast_rpw(a->batch, a->dim, a->dim / p.b_groups, a->dim / p.c_groups);
    if (fast_rpw && a->dim / (BF_WAVES * fast_rpw) > pl.nblk) fast_rpw = 0;
  }
  if (scan_bwd_is_const_row(a)) {
    switch (a->io_dtype) {
      case SSM_F32: rc = launch_bwd_row_const<float>(p, s); break;
      case SSM_BF16: rc = launch_bwd_row_const<bf16_t>(p, s); break;
      default: rc = launch_bwd_row_const<f16_t>(p, s); break;
    }
  } else if (per_row) {
    const bool bc32 = a->bc_dtype == SSM_F32, o32 = a->dbc_dtype == SSM_F32;
    if (a->io_dtype == SSM_F32) rc = launch_bwd_rowbc<float, float, float>(p, a->dB, a->dC, s);
    else if (a->io_dtype == SSM_BF16)
      rc = bc32 ? launch_bwd_rowbc<bf16_t, float, float>(p, a->dB, a->dC, s)
                : (o32 ? launch_bwd_rowbc<bf16_t, bf16_t, float>(p, a->dB, a->dC, s) : launch_bwd_rowbc<bf16_t, bf16_t, bf16_t>(p, a->dB, a->dC, s));
    else
      rc = bc32 ? launch_bwd_rowbc<f16_t, float, float>(p, a->dB, a->dC, s)
                : (o32 ? launch_bwd_rowbc<f16_t, f16_t, float>(p, a->dB, a->dC, s) : launch_bwd_rowbc<f16_t, f16_t, f16_t>(p, a->dB, a->dC, s));
  } else if (fast_rpw) {
    p.rows_per_wg = BF_WAVES * fast_rpw;
    p.nblk = a->dim / p.rows_per_wg;
    const bool bc32 = a->bc_dtype == SSM_F32;
    if (a->io_dtype == SSM_F32) rc = launch_bwd_fast<float, float>(p, fast_rpw, s);
    else if (a->io_dtype == SSM_BF16) rc = bc32 ? launch_bwd_fast<bf16_t, float>(p, fast_rpw, s) : launch_bwd_fast<bf16_t, bf16_t>(p, fast_rpw, s);
    else rc = bc32 ? launch_bwd_fast<f16_t, float>(p, fast_rpw, s) : launch_bwd_fast<f16_t, f16_t>(p, fast_rpw, s);
  } else {
    switch (a->io_dtype) {
      case SSM_F32: rc = launch_bwd<float>(p, s); break;
      case SSM_BF16: rc = launch_bwd<bf16_t>(p, s); break;
      default: rc = launch_bwd<f16_t>(p, s); break;
    }
  }
  if (rc != SSM_OK) return rc;

  const int Bn = a->batch, D = a->dim, N = a->nstate, L = a->seqlen;
  // dA (D,N), dD (D,), dbias (D,): sums over the batch; dB / dC in the shape of the given projection.  The sums
  // over rows share one launch.
  FoldJobs jobs{};
  auto add_job = [&](const float *in, float *out, int count, size_t inner) {
    const int j = jobs.n++;
    jobs.in[j] = in; jobs.out[j] = out; jobs.count[j] = count; jobs.inner[j] = inner;
    jobs.first_block[j + 1] = jobs.first_block[j] + fold_grid(inner);
  };
  add_job(p.dA_rows, a->dA, Bn, (size_t)D * N);
  if (a->dD) add_job(p.dD_rows, a->dD, Bn, (size_t)D);
  if (a->ddt_bias) add_job(p.dbias_rows, a->ddt_bias, Bn, (size_t)D);
  auto fold_proj = [&](int kind, int groups, const float *partial, float *out) {
    if (kind == SSM_PROJ_BGNL) {
      // (B, G, nblk/G, N*L) -> (B, G, N*L)
      const int per_group = p.nblk / groups;
      launch_fold_sum(partial, out, (size_t)Bn * groups, per_group, (size_t)N * L, s);
    } else if (kind == SSM_PROJ_BDN) {
      add_job(partial, out, 1, (size_t)Bn * D * N);
    } else {
      add_job(partial, out, Bn, (size_t)D * N);
    }
  };
  if (!per_row) {
    fold_proj(a->b_kind, p.b_groups, p.dB_part, reinterpret_cast<float *>(a->dB));
    fold_proj(a->c_kind, p.c_groups, p.dC_part, reinterpret_cast<float *>(a->dC));
  }
  hipLaunchKernelGGL(fold_rows_multi_kernel, dim3(jobs.first_block[jobs.n]), dim3(256), 0, s, jobs);
  SSM_CHECK_LAUNCH("ssm_scan_bwd(fold)");
  return SSM_OK;
}
