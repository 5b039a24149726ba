// Selective scan, forward, for gfx950.
//
// One wavefront owns one (batch, channel) row.  Time is cut into chunks of
// T = 64*K steps; inside a chunk lane l owns the K consecutive steps
// [l*K, l*K+K).  For every state index n the lane folds its K steps into one
// affine map h -> P h + S, the 64 maps are composed with a DPP scan
// (row_shr 1/2/4/8, row_bcast 15/31), the state entering the lane is read from
// the previous lane, and the K steps are replayed from that state to emit
// y += h * C.  The running state of the row (one float per n) is carried from
// chunk to chunk in a VGPR (lane n holds state n; LDS beyond 64 states) and,
// after the last chunk, is the op's last_state.
//
// Time-varying B/C of one (batch, group) are shared by all channels of the
// group: the workgroup (up to 8 wavefronts = 8 channels of one group) stages
// them once per chunk in LDS as fp32, transposed so that a lane fetches the
// values of four consecutive steps with one conflict-free 128-bit read.
// Two state indices are processed together so that the DPP steps of one hide
// the register-read hazards of the other.
#pragma once
#include "common.hpp"

#include <type_traits>

namespace ssm {

constexpr int SCAN_MAX_WAVES = 8;    // channels per workgroup
constexpr int SCAN_MAX_N = 256;      // state size limit
constexpr int SCAN_LANE_STATES = 64; // states whose carry lives in a VGPR

struct ScanFwdParams {
  const void *u, *delta, *z, *Bp, *Cp;
  const float *A, *Dk, *bias;
  void *out, *last;
  float *chunk_states;   // optional (B, D, nchunks, N): row state entering each chunk
  int batch, dim, len, nstate;
  int bc_dtype;
  int b_kind, c_kind, b_groups, c_groups;
  int softplus;
  int vec_ok;     // rows of u/delta/z/out are 16-byte aligned
  int bc_vec_ok;  // rows of B/C allow 4-element vector loads
};

// Copy the [nn][T] slab of one time-varying projection into LDS as fp32.
// src_off is the element offset of (b, g, nb, 0); rows are `len` apart.
template <int K>
__device__ __forceinline__ void stage_tile(float *dst, const void *src, int dtype, size_t src_off,
                                           int len, int t0, int nn, bool vec_ok) {
  constexpr int T = WAVE * K;
  constexpr int QT = T / 4;
  for (int e = threadIdx.x; e < nn * QT; e += blockDim.x) {
    const int nl = e / QT;
    const int tl = (e % QT) * 4;
    const int t = t0 + tl;
    const size_t off = src_off + (size_t)nl * len + t;
    float4 v;
    if (vec_ok && t + 4 <= len) {
      if (dtype == SSM_F32) {
        v = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(src) + off);
      } else {
        const uint2 raw = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(src) + off);
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
      }
    } else {
      v.x = (t + 0 < len) ? load_as_f32(src, dtype, off + 0) : 0.0f;
      v.y = (t + 1 < len) ? load_as_f32(src, dtype, off + 1) : 0.0f;
      v.z = (t + 2 < len) ? load_as_f32(src, dtype, off + 2) : 0.0f;
      v.w = (t + 3 < len) ? load_as_f32(src, dtype, off + 3) : 0.0f;
    }
    const int owner = tl / K;        // lane that owns these four steps
    const int item = tl % K;         // first of the four within the lane's run
    *reinterpret_cast<float4 *>(dst + nl * T + (item >> 2) * (WAVE * 4) + owner * 4) = v;
  }
}

// DPP scan steps written out by hand.  Lanes whose DPP source does not exist
// (or whose row is masked off) are disabled for that instruction, so they keep
// their value: exactly the identity element.  A VGPR written by a VALU
// instruction must not be read through DPP within the next two issue slots;
// the two-stream version interleaves independent work, the one-stream version
// pads with s_nop.
#define SSM_DPP_STEP2(CTRL)                               \
  "v_fmac_f32_dpp %1, %1, %0 " CTRL "\n\t"                \
  "v_fmac_f32_dpp %3, %3, %2 " CTRL "\n\t"                \
  "v_mul_f32_dpp %0, %0, %0 " CTRL "\n\t"                 \
  "v_mul_f32_dpp %2, %2, %2 " CTRL "\n\t"
#define SSM_DPP_STEP1(CTRL)                               \
  "v_fmac_f32_dpp %1, %1, %0 " CTRL "\n\t"                \
  "v_mul_f32_dpp %0, %0, %0 " CTRL "\n\t"                 \
  "s_nop 1\n\t"

__device__ __forceinline__ void wave_scan_affine_x2(float &a0, float &b0, float &a1, float &b1) {
  asm volatile(
      "s_nop 4\n\t"
      SSM_DPP_STEP2("row_shr:1 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP2("row_shr:2 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP2("row_shr:4 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP2("row_shr:8 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP2("row_bcast:15 row_mask:0xa bank_mask:0xf")
      "v_fmac_f32_dpp %1, %1, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %3, %3, %2 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1));
}

__device__ __forceinline__ void wave_scan_affine_x1(float &a0, float &b0) {
  asm volatile(
      "s_nop 4\n\t"
      SSM_DPP_STEP1("row_shr:1 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP1("row_shr:2 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP1("row_shr:4 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP1("row_shr:8 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP1("row_bcast:15 row_mask:0xa bank_mask:0xf")
      "v_fmac_f32_dpp %1, %1, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      : "+v"(a0), "+v"(b0));
}

// Note: after the last step only b (the composed offset) is complete in every
// lane; a is complete in rows 0-1 only and is not used afterwards.

// RPW rows per wave share one staged B/C slab (only used when all N states fit one
// slab, so that nothing has to persist per row across slabs).
template <typename io_t, int K, int NB, bool BVARY, bool CVARY, bool SMALLN, int RPW>
__global__ __launch_bounds__(WAVE *SCAN_MAX_WAVES) void scan_fwd_kernel(const ScanFwdParams p) {
  constexpr int T = WAVE * K;
  extern __shared__ __align__(16) float tiles[];           // B tile [NB][T] then C tile [NB][T]
  __shared__ float carry_hi[SMALLN ? 1 : SCAN_MAX_WAVES][SMALLN ? 1 : SCAN_MAX_N - SCAN_LANE_STATES];

  const int waves = (int)(blockDim.x >> 6);
  const int rows = waves * RPW;                            // channels per workgroup
  const int wave = wave_id_uniform();
  const int lane = lane_id();
  const int blocks_per_batch = p.dim / rows;
  const int b = (int)blockIdx.x / blocks_per_batch;
  const int d0 = ((int)blockIdx.x % blocks_per_batch) * rows;
  const int L = p.len, N = p.nstate;
  const bool vec_ok = p.vec_ok != 0;
  const bool fast_rows = vec_ok && p.len % K == 0;       // aligned rows of whole runs

  constexpr bool bvary = BVARY, cvary = CVARY;
  float *Bs = tiles;
  float *Cs = tiles + (bvary ? NB * T : 0);
  size_t b_tile = 0, c_tile = 0;     // element offset of the group's projection at n = 0, t = 0
  if (bvary) b_tile = ((size_t)b * p.b_groups + d0 / (p.dim / p.b_groups)) * (size_t)N * L;
  if (cvary) c_tile = ((size_t)b * p.c_groups + d0 / (p.dim / p.c_groups)) * (size_t)N * L;

  // per-row constants spread over lanes: lane n holds the value for state n (n < 64)
  float A2_lanes[RPW], Bc_lanes[RPW], Cc_lanes[RPW], carry_lanes[RPW];
#pragma unroll
  for (int rr = 0; rr < RPW; ++rr) {
    const int d = d0 + wave * RPW + rr;
    A2_lanes[rr] = lane < N ? p.A[(size_t)d * N + lane] * LOG2E : 0.0f;
    const size_t bo = ((p.b_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
    const size_t co = ((p.c_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
    Bc_lanes[rr] = (!bvary && lane < N) ? load_as_f32(p.Bp, p.bc_dtype, bo + lane) : 0.0f;
    Cc_lanes[rr] = (!cvary && lane < N) ? load_as_f32(p.Cp, p.bc_dtype, co + lane) : 0.0f;
    carry_lanes[rr] = 0.0f;
  }
  if (!SMALLN)
    for (int n = SCAN_LANE_STATES + lane; n < N; n += WAVE) carry_hi[wave][n - SCAN_LANE_STATES] = 0.0f;

  const int nchunks = (L + T - 1) / T;
  for (int c = 0; c < nchunks; ++c) {
    const int t0 = c * T;
    const int t = t0 + lane * K;
    float dl[K], du[K], y[K];
    float dsum = 0.0f;

    for (int nb = 0; nb < N; nb += NB) {
      const int nn = min(NB, N - nb);
      if constexpr (bvary || cvary) {
        __syncthreads();   // every wave is done with the previous slab
        if constexpr (bvary) stage_tile<K>(Bs, p.Bp, p.bc_dtype, b_tile + (size_t)nb * L, L, t0, nn, p.bc_vec_ok != 0);
        if constexpr (cvary) stage_tile<K>(Cs, p.Cp, p.bc_dtype, c_tile + (size_t)nb * L, L, t0, nn, p.bc_vec_ok != 0);
        __syncthreads();
      }

#pragma unroll
      for (int rr = 0; rr < RPW; ++rr) {
        const int d = d0 + wave * RPW + rr;
        const size_t row = (size_t)b * p.dim + d;
        const float *A_row = p.A + (size_t)d * N;
        const size_t b_off = ((p.b_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;
        const size_t c_off = ((p.c_kind == SSM_PROJ_BDN ? (size_t)b * p.dim : 0) + d) * (size_t)N;

        if (nb == 0) {
          // load this row's K steps per lane: delta' and delta' * u, y starts at D * u
          const float Dk = p.Dk ? p.Dk[d] : 0.0f;
          const float bias = p.bias ? p.bias[d] : 0.0f;
          float uu[K];
          if (fast_rows) {
            // whole runs, read unconditionally and together (a lane past the end re-reads the last run; its
            // steps become the identity below and nothing of it is stored)
            const size_t at = row * L + min(t, L - K);
            const Pack<io_t, K> ur = *reinterpret_cast<const Pack<io_t, K> *>(reinterpret_cast<const io_t *>(p.u) + at);
            const Pack<io_t, K> dr = *reinterpret_cast<const Pack<io_t, K> *>(reinterpret_cast<const io_t *>(p.delta) + at);
#pragma unroll
            for (int i = 0; i < K; ++i) {
              uu[i] = to_f32(ur.v[i]);
              dl[i] = to_f32(dr.v[i]);
            }
          } else {
            load_run<io_t, K>(reinterpret_cast<const io_t *>(p.u) + row * L, t, L, vec_ok, uu);
            load_run<io_t, K>(reinterpret_cast<const io_t *>(p.delta) + row * L, t, L, vec_ok, dl);
          }
          if (p.chunk_states) {
            float *cs = p.chunk_states + (row * nchunks + c) * (size_t)N;
            if (lane < N) cs[lane] = carry_lanes[rr];
            if (!SMALLN)
              for (int n = SCAN_LANE_STATES + lane; n < N; n += WAVE) cs[n] = carry_hi[wave][n - SCAN_LANE_STATES];
          }
          dsum = 0.0f;
          if (p.softplus) {
#pragma unroll
            for (int i = 0; i < K; ++i) dl[i] = softplus_f32(dl[i] + bias);
          } else {
#pragma unroll
            for (int i = 0; i < K; ++i) dl[i] += bias;
          }
          if (t + K > L) {                      // steps past the end are the identity map
#pragma unroll
            for (int i = 0; i < K; ++i) dl[i] = (t + i < L) ? dl[i] : 0.0f;
          }
#pragma unroll
          for (int i = 0; i < K; ++i) {
            du[i] = dl[i] * uu[i];
            y[i] = Dk * uu[i];
            dsum += dl[i];
          }
        }

        // One or two state indices at a time.  W is a compile-time width so that
        // the per-state arrays stay in registers.
        auto process = [&](auto width_tag, int nl) {
          constexpr int W = decltype(width_tag)::value;
          float a[W][K], bx[W][K], P[W], h[W], A2[W], H[W], cconst[W];
#pragma unroll
          for (int w = 0; w < W; ++w) {
            const int n = nb + nl + w;
            const bool in_lanes = SMALLN || n < SCAN_LANE_STATES;
            A2[w] = in_lanes ? wave_read_lane(A2_lanes[rr], n) : A_row[n] * LOG2E;
            const float bconst = bvary ? 0.0f
                                       : (in_lanes ? wave_read_lane(Bc_lanes[rr], n)
                                                   : load_as_f32(p.Bp, p.bc_dtype, b_off + n));
            cconst[w] = cvary ? 0.0f
                              : (in_lanes ? wave_read_lane(Cc_lanes[rr], n) : load_as_f32(p.Cp, p.bc_dtype, c_off + n));
            H[w] = in_lanes ? wave_read_lane(carry_lanes[rr], n) : carry_hi[wave][n - SCAN_LANE_STATES];
            // fold the lane's K steps into (P, h): state_out = P * state_in + h
#pragma unroll
            for (int q = 0; q < K / 4; ++q) {
              float4 bv;
              if constexpr (bvary) bv = *reinterpret_cast<const float4 *>(Bs + (nl + w) * T + q * (WAVE * 4) + lane * 4);
              else bv = make_float4(bconst, bconst, bconst, bconst);
              const float bq[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const int i = q * 4 + j;
                a[w][i] = exp2_hw(dl[i] * A2[w]);
                bx[w][i] = du[i] * bq[j];
                h[w] = i == 0 ? bx[w][0] : __builtin_fmaf(a[w][i], h[w], bx[w][i]);
              }
            }
            P[w] = exp2_hw(dsum * A2[w]);
            // lane 0 absorbs the state carried in from the previous chunk
            h[w] = __builtin_fmaf(P[w], lane == 0 ? H[w] : 0.0f, h[w]);
          }
          if constexpr (W == 2) wave_scan_affine_x2(P[0], h[0], P[1], h[1]);
          else wave_scan_affine_x1(P[0], h[0]);
#pragma unroll
          for (int w = 0; w < W; ++w) {
            const int n = nb + nl + w;
            // h[w] is now the row state at the END of each lane's run
            float hs = wave_prev(h[w], H[w]);                       // state entering this lane
            const float hend = wave_read_lane(h[w], WAVE - 1);      // state leaving the chunk
            if (SMALLN || n < SCAN_LANE_STATES) {
              carry_lanes[rr] = lane == n ? hend : carry_lanes[rr];
            } else if (lane == 0) {
              carry_hi[wave][n - SCAN_LANE_STATES] = hend;
            }
            // replay the K steps from the true entering state
#pragma unroll
            for (int q = 0; q < K / 4; ++q) {
              float4 cv;
              if constexpr (cvary) cv = *reinterpret_cast<const float4 *>(Cs + (nl + w) * T + q * (WAVE * 4) + lane * 4);
              else cv = make_float4(cconst[w], cconst[w], cconst[w], cconst[w]);
              const float cq[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const int i = q * 4 + j;
                hs = __builtin_fmaf(a[w][i], hs, bx[w][i]);
                y[i] = __builtin_fmaf(hs, cq[j], y[i]);
              }
            }
          }
        };

        int nl = 0;
        for (; nl + 2 <= nn; nl += 2) process(std::integral_constant<int, 2>{}, nl);
        if (nl < nn) process(std::integral_constant<int, 1>{}, nl);

        if (nb + NB >= N) {
          if (p.z) {
            float zz[K];
            load_run<io_t, K>(reinterpret_cast<const io_t *>(p.z) + row * L, t, L, vec_ok, zz);
#pragma unroll
            for (int i = 0; i < K; ++i) y[i] *= silu_f32(zz[i]);
          }
          store_run<io_t, K>(reinterpret_cast<io_t *>(p.out) + row * L, t, L, vec_ok, y);
        }
      }
    }
  }

  if (p.last) {
#pragma unroll
    for (int rr = 0; rr < RPW; ++rr) {
      const size_t row = (size_t)b * p.dim + d0 + wave * RPW + rr;
      io_t *last_row = reinterpret_cast<io_t *>(p.last) + row * N;
      if (lane < N) last_row[lane] = from_f32<io_t>(carry_lanes[rr]);
      if (!SMALLN)
        for (int n = SCAN_LANE_STATES + lane; n < N; n += WAVE)
          last_row[n] = from_f32<io_t>(carry_hi[wave][n - SCAN_LANE_STATES]);
    }
  }
}

template <typename io_t, int K, int NB, bool BV, bool CV, bool SN, int RPW>
static int launch_scan_fwd(const ScanFwdParams &p, int rows, hipStream_t stream) {
  const size_t lds = (size_t)((int)BV + (int)CV) * NB * WAVE * K * sizeof(float);
  auto kernel = scan_fwd_kernel<io_t, K, NB, BV, CV, SN, RPW>;
  if (allow_dynamic_lds(kernel, lds) != hipSuccess) {
    (void)hipGetLastError();
    set_error("ssm_scan_fwd: cannot reserve %zu bytes of LDS", lds);
    return SSM_ERR_LAUNCH;
  }
  // `rows` channels per workgroup = waves * RPW
  const unsigned grid = (unsigned)((size_t)p.batch * (p.dim / rows));
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(WAVE * (rows / RPW)), lds, stream, p);
  SSM_CHECK_LAUNCH("ssm_scan_fwd");
  return SSM_OK;
}

template <typename io_t, int K, int NB>
static int dispatch_flags(const ScanFwdParams &p, int rows, hipStream_t s) {
  const bool bv = p.b_kind == SSM_PROJ_BGNL, cv = p.c_kind == SSM_PROJ_BGNL;
  const bool sn = p.nstate <= SCAN_LANE_STATES;
  // two rows per wave when a workgroup of 16 channels fits one group and all states fit one slab
  if (bv && cv && sn && rows == 2 * SCAN_MAX_WAVES) return launch_scan_fwd<io_t, K, NB, true, true, true, 2>(p, rows, s);
  if (bv && cv && sn && rows == 3 * SCAN_MAX_WAVES) return launch_scan_fwd<io_t, K, NB, true, true, true, 3>(p, rows, s);
  if (bv && cv && sn && rows == 4 * SCAN_MAX_WAVES) return launch_scan_fwd<io_t, K, NB, true, true, true, 4>(p, rows, s);
  if (bv && cv && sn && rows == 6 * SCAN_MAX_WAVES) return launch_scan_fwd<io_t, K, NB, true, true, true, 6>(p, rows, s);
  const int key = (bv ? 4 : 0) | (cv ? 2 : 0) | (sn ? 1 : 0);
  switch (key) {
    case 0: return launch_scan_fwd<io_t, K, NB, false, false, false, 1>(p, rows, s);
    case 1: return launch_scan_fwd<io_t, K, NB, false, false, true, 1>(p, rows, s);
    case 2: return launch_scan_fwd<io_t, K, NB, false, true, false, 1>(p, rows, s);
    case 3: return launch_scan_fwd<io_t, K, NB, false, true, true, 1>(p, rows, s);
    case 4: return launch_scan_fwd<io_t, K, NB, true, false, false, 1>(p, rows, s);
    case 5: return launch_scan_fwd<io_t, K, NB, true, false, true, 1>(p, rows, s);
    case 6: return launch_scan_fwd<io_t, K, NB, true, true, false, 1>(p, rows, s);
    default: return launch_scan_fwd<io_t, K, NB, true, true, true, 1>(p, rows, s);
  }
}

// tune = K * 100 + NB
template <typename io_t>
int scan_fwd_dispatch(const ScanFwdParams &p, int tune, int rows, hipStream_t s) {
  switch (tune) {
    case 408: return dispatch_flags<io_t, 4, 8>(p, rows, s);
    case 808: return dispatch_flags<io_t, 8, 8>(p, rows, s);
    case 816: return dispatch_flags<io_t, 8, 16>(p, rows, s);
    case 1616: return dispatch_flags<io_t, 8, 16>(p, rows, s);      // 816 with two rows per wave (see entry point)
    case 2416: case 3216: case 4816: return dispatch_flags<io_t, 8, 16>(p, rows, s);   // 816 with 3, 4, 6 rows per wave
    default:
      set_error("ssm_scan_fwd: unsupported selector %d (408, 808, 816, 1616, 2416)", tune);
      return SSM_ERR_BAD_KIND;
  }
}

}  // namespace ssm
