// Selective scan, forward: the kernel for the common call shape.
//
//   time-varying grouped B and C (B, G, N, L), N <= 16, rows of u / delta / z / out
//   aligned to 16 bytes, L a multiple of 16.
//
// Same decomposition as scan_fwd_kernel.hpp (time in chunks of 512 steps, a lane
// owns a run of consecutive steps, per state a fold / lane scan / replay),
// specialised so that nothing in the row loop is decided at run time: element
// types are template parameters, the B/C slab holds all states, the slab reads
// and the transcendental instructions of a fold are issued together, and the
// number of wavefronts per workgroup and of states in flight are compile-time
// choices that set the register budget and with it how many wavefronts share a
// SIMD.  LPR lanes work on one row: with LPR = 64 a lane owns 8 steps; with
// LPR = 32 it owns 16 and a wavefront walks two rows at once, which halves the
// scan steps, carries and whole-run factors per state step.
#pragma once
#include "scan_fwd_kernel.hpp"

namespace ssm {

constexpr int FAST_T = 512;    // steps per chunk (= ssm_scan_chunk_len())
constexpr int FAST_N = 16;     // states held by the slab

// [n][T] slab of one projection into LDS as fp32; a lane's K steps end up as K/4 float4
// at [n][q][lane of the row] so that the reads of a wave are conflict-free.
template <typename bc_t, int LPR>
__device__ __forceinline__ void fast_stage(float *dst, const bc_t *src, int len, int t0, int nn, int nthreads) {
  constexpr int K = FAST_T / LPR, QT = FAST_T / 4;
  for (int e = threadIdx.x; e < nn * QT; e += nthreads) {
    const int nl = e / QT;
    const int tl = (e % QT) * 4;
    const int t = t0 + tl;
    const bool inside = t < len;                       // len % 4 == 0: a group of four is inside or outside as a whole
    const bc_t *at = src + (size_t)nl * len + (inside ? t : 0);
    const Pack<bc_t, 4> raw = *reinterpret_cast<const Pack<bc_t, 4> *>(at);
    float4 v;
    v.x = inside ? to_f32(raw.v[0]) : 0.0f;
    v.y = inside ? to_f32(raw.v[1]) : 0.0f;
    v.z = inside ? to_f32(raw.v[2]) : 0.0f;
    v.w = inside ? to_f32(raw.v[3]) : 0.0f;
    const int owner = tl / K, item = tl % K;
    *reinterpret_cast<float4 *>(dst + nl * FAST_T + (item >> 2) * (LPR * 4) + owner * 4) = v;
  }
}

// softplus(x) for the step size: log(1 + e^x) with the rounding of 1 + e^x restored, and x itself once e^x
// would overflow (softplus(x) >= x always, and the formula at min(x, 60) is below x beyond 60).
__device__ __forceinline__ float fast_softplus(float x) {
  const float e = exp2_hw(fminf(x, 60.0f) * LOG2E);
  const float w = 1.0f + e;
  const float r = __builtin_fmaf(log2_hw(w), LN2, e - (w - 1.0f));
  return fmaxf(r, x);
}

// 2^x of a lane's whole run and of one more value in consecutive instructions.  Left to the compiler they are
// spread between the multiplications, and a transcendental instruction between plain ones costs about half
// as much again as one that follows another.
__device__ __forceinline__ void exp2_run(float (&a)[8], float &P) {
  asm volatile(
      "v_exp_f32 %0, %0\n\tv_exp_f32 %1, %1\n\tv_exp_f32 %2, %2\n\tv_exp_f32 %3, %3\n\t"
      "v_exp_f32 %4, %4\n\tv_exp_f32 %5, %5\n\tv_exp_f32 %6, %6\n\tv_exp_f32 %7, %7\n\tv_exp_f32 %8, %8\n\t"
      : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]), "+v"(P));
}
__device__ __forceinline__ void exp2_run(float (&a)[16], float &P) {
  asm volatile(
      "v_exp_f32 %0, %0\n\tv_exp_f32 %1, %1\n\tv_exp_f32 %2, %2\n\tv_exp_f32 %3, %3\n\t"
      "v_exp_f32 %4, %4\n\tv_exp_f32 %5, %5\n\tv_exp_f32 %6, %6\n\tv_exp_f32 %7, %7\n\t"
      "v_exp_f32 %8, %8\n\tv_exp_f32 %9, %9\n\tv_exp_f32 %10, %10\n\tv_exp_f32 %11, %11\n\t"
      "v_exp_f32 %12, %12\n\tv_exp_f32 %13, %13\n\tv_exp_f32 %14, %14\n\tv_exp_f32 %15, %15\n\tv_exp_f32 %16, %16\n\t"
      : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]), "+v"(a[8]),
        "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]), "+v"(a[15]), "+v"(P));
}

// The scans of scan_fwd_kernel.hpp over the 32 lanes of each half of the wave: the same steps without the last.
__device__ __forceinline__ void half_scan_affine_x2(float &a0, float &b0, float &a1, float &b1) {
  asm volatile(
      "s_nop 4\n\t"
      SSM_DPP_STEP2("row_shr:1 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP2("row_shr:2 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP2("row_shr:4 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP2("row_shr:8 row_mask:0xf bank_mask:0xf")
      "v_fmac_f32_dpp %1, %1, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %3, %3, %2 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1));
}
__device__ __forceinline__ void half_scan_affine_x1(float &a0, float &b0) {
  asm volatile(
      "s_nop 4\n\t"
      SSM_DPP_STEP1("row_shr:1 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP1("row_shr:2 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP1("row_shr:4 row_mask:0xf bank_mask:0xf")
      SSM_DPP_STEP1("row_shr:8 row_mask:0xf bank_mask:0xf")
      "v_fmac_f32_dpp %1, %1, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      : "+v"(a0), "+v"(b0));
}

// Value that lane `src` of the own group of LPR lanes holds (the whole wave for LPR = 64: through a scalar
// register; a half: through the LDS crossbar, which costs no vector-ALU slot).
template <int LPR>
__device__ __forceinline__ float group_read_lane(float v, int src, int lane) {
  if constexpr (LPR == WAVE) return wave_read_lane(v, src);
  else return __int_as_float(__builtin_amdgcn_ds_bpermute(((lane & ~(LPR - 1)) + src) * 4, __float_as_int(v)));
}

// DB: two slabs in LDS (for variants of which one workgroup fills a CU): the slab of the next chunk is staged by
// each wave as soon as it is done with its rows of this one, while slower waves still work, and a chunk costs
// one barrier instead of two.
template <typename io_t, typename bc_t, int LPR, int RPW, int WAVES, int W, int OCC, bool DB>
__global__ __launch_bounds__(WAVE *WAVES) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void scan_fwd_fast_kernel(const ScanFwdParams p) {
  constexpr int T = FAST_T, K = T / LPR, SUBS = WAVE / LPR;
  extern __shared__ __align__(16) float tiles[];           // B [16][T] then C [16][T] (twice with DB)
  float *Bs = tiles, *Cs = tiles + FAST_N * T;

  constexpr int rows = WAVES * RPW * SUBS;
  const int wave = wave_id_uniform();
  const int lane = lane_id();
  const int sl = lane & (LPR - 1);            // lane within the row
  const int sub = lane / LPR;                 // which of the wave's rows
  const int blocks_per_batch = p.dim / rows;
  const int b = (int)blockIdx.x / blocks_per_batch;
  const int d0 = ((int)blockIdx.x % blocks_per_batch) * rows;
  const int L = p.len, N = p.nstate;
  const bc_t *Bg = reinterpret_cast<const bc_t *>(p.Bp) + ((size_t)b * p.b_groups + d0 / (p.dim / p.b_groups)) * (size_t)N * L;
  const bc_t *Cg = reinterpret_cast<const bc_t *>(p.Cp) + ((size_t)b * p.c_groups + d0 / (p.dim / p.c_groups)) * (size_t)N * L;
  const io_t *U = reinterpret_cast<const io_t *>(p.u), *DT = reinterpret_cast<const io_t *>(p.delta);
  const io_t *Z = reinterpret_cast<const io_t *>(p.z);
  io_t *Y = reinterpret_cast<io_t *>(p.out);

  // per-row constants: lane n of a row's lanes holds the value for state n
  float A2_lanes[RPW], carry_lanes[RPW], Dk[RPW], bias[RPW];
#pragma unroll
  for (int rr = 0; rr < RPW; ++rr) {
    const int d = d0 + (wave * RPW + rr) * SUBS + sub;
    A2_lanes[rr] = sl < N ? p.A[(size_t)d * N + sl] * LOG2E : 0.0f;
    carry_lanes[rr] = 0.0f;
    Dk[rr] = p.Dk ? p.Dk[d] : 0.0f;
    bias[rr] = p.bias ? p.bias[d] : 0.0f;
  }

  const int nchunks = (L + T - 1) / T;
  for (int c = 0; c < nchunks; ++c) {
    const int t0 = c * T;
    const int t = t0 + sl * K;
    const bool live = t < L;                 // L % K == 0: a lane's run is inside or outside as a whole
    const int tc = live ? t : 0;

    if constexpr (DB) {
      if (c == 0) {
        fast_stage<bc_t, LPR>(Bs, Bg, L, 0, N, WAVE * WAVES);
        fast_stage<bc_t, LPR>(Cs, Cg, L, 0, N, WAVE * WAVES);
      }
      __syncthreads();           // slab c is complete; every wave is done with slab c - 1 (staged over below)
      Bs = tiles + (c & 1) * 2 * FAST_N * T;
      Cs = Bs + FAST_N * T;
    } else {
      __syncthreads();
      fast_stage<bc_t, LPR>(Bs, Bg, L, t0, N, WAVE * WAVES);
      fast_stage<bc_t, LPR>(Cs, Cg, L, t0, N, WAVE * WAVES);
      __syncthreads();
    }

#pragma unroll
    for (int rr = 0; rr < RPW; ++rr) {
      const int d = d0 + (wave * RPW + rr) * SUBS + sub;
      const size_t row = (size_t)b * p.dim + d;
      const size_t at = row * L + tc;
      float dl[K], du[K], y[K];
      Pack<io_t, K> zr;
      {
        const Pack<io_t, K> ur = *reinterpret_cast<const Pack<io_t, K> *>(U + at);
        const Pack<io_t, K> dr = *reinterpret_cast<const Pack<io_t, K> *>(DT + at);
        if (p.z) zr = *reinterpret_cast<const Pack<io_t, K> *>(Z + at);
        if (p.chunk_states && sl < N) p.chunk_states[(row * nchunks + c) * (size_t)N + sl] = carry_lanes[rr];
#pragma unroll
        for (int i = 0; i < K; ++i) dl[i] = to_f32(dr.v[i]) + bias[rr];
        if (p.softplus) {
#pragma unroll
          for (int i = 0; i < K; ++i) dl[i] = fast_softplus(dl[i]);
        }
        if (t0 + T > L) {                      // only the last chunk can have lanes past the end: the identity map there
#pragma unroll
          for (int i = 0; i < K; ++i) dl[i] = live ? dl[i] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < K; ++i) {
          const float uu = to_f32(ur.v[i]);
          du[i] = dl[i] * uu;
          y[i] = Dk[rr] * uu;
        }
      }
      float dsum = 0.0f;
#pragma unroll
      for (int i = 0; i < K; ++i) dsum += dl[i];

      auto process = [&](auto width_tag, int n0) {
        constexpr int WW = decltype(width_tag)::value;
        float a[WW][K], bx[WW][K], P[WW], h[WW], H[WW], A2[WW];
        // the slab reads of these states are requested before anything else, so that they return while the
        // exponentials run
        float4 bv[WW][K / 4];
#pragma unroll
        for (int w = 0; w < WW; ++w) {
#pragma unroll
          for (int q = 0; q < K / 4; ++q)
            bv[w][q] = *reinterpret_cast<const float4 *>(Bs + (n0 + w) * T + q * (LPR * 4) + sl * 4);
          A2[w] = group_read_lane<LPR>(A2_lanes[rr], n0 + w, lane);
          H[w] = group_read_lane<LPR>(carry_lanes[rr], n0 + w, lane);
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int w = 0; w < WW; ++w) {
#pragma unroll
          for (int i = 0; i < K; ++i) a[w][i] = dl[i] * A2[w];
          P[w] = dsum * A2[w];
        }
        // all transcendentals of the fold back to back
#pragma unroll
        for (int w = 0; w < WW; ++w) exp2_run(a[w], P[w]);
#pragma unroll
        for (int w = 0; w < WW; ++w) {
#pragma unroll
          for (int q = 0; q < K / 4; ++q) {
            const float bq[4] = {bv[w][q].x, bv[w][q].y, bv[w][q].z, bv[w][q].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int i = q * 4 + j;
              bx[w][i] = du[i] * bq[j];
              h[w] = i == 0 ? bx[w][0] : __builtin_fmaf(a[w][i], h[w], bx[w][i]);
            }
          }
          // the first lane of a row absorbs the state carried in from the previous chunk
          h[w] = __builtin_fmaf(P[w], sl == 0 ? H[w] : 0.0f, h[w]);
        }
        float4 cv[WW][K / 4];
#pragma unroll
        for (int w = 0; w < WW; ++w)
#pragma unroll
          for (int q = 0; q < K / 4; ++q)
            cv[w][q] = *reinterpret_cast<const float4 *>(Cs + (n0 + w) * T + q * (LPR * 4) + sl * 4);
        if constexpr (LPR == WAVE) {
          if constexpr (WW == 2) wave_scan_affine_x2(P[0], h[0], P[1], h[1]);
          else wave_scan_affine_x1(P[0], h[0]);
        } else {
          if constexpr (WW == 2) half_scan_affine_x2(P[0], h[0], P[1], h[1]);
          else half_scan_affine_x1(P[0], h[0]);
        }
#pragma unroll
        for (int w = 0; w < WW; ++w) {
          // h[w] is the row state at the end of each lane's run; a lane starts from its predecessor's
          float hs = wave_prev(h[w], H[w]);
          if constexpr (LPR != WAVE) hs = sl == 0 ? H[w] : hs;
          const float hend = group_read_lane<LPR>(h[w], LPR - 1, lane);
          carry_lanes[rr] = sl == n0 + w ? hend : carry_lanes[rr];
#pragma unroll
          for (int q = 0; q < K / 4; ++q) {
            const float cq[4] = {cv[w][q].x, cv[w][q].y, cv[w][q].z, cv[w][q].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int i = q * 4 + j;
              hs = __builtin_fmaf(a[w][i], hs, bx[w][i]);
              y[i] = __builtin_fmaf(hs, cq[j], y[i]);
            }
          }
        }
      };

      // The SIMD serves its oldest wave first.  Turning the order of the workgroup's waves on a SIMD round from
      // state to state keeps them out of step with each other (one in its exponentials while another replays),
      // which is worth 7 % of the kernel's time with three waves per SIMD.
      auto turn = [&](int k) {
        constexpr int RANKS = WAVES / 4;
        if constexpr (RANKS >= 3) {
          const int pr = (k + (wave >> 2)) % RANKS;
          if (pr == 0) __builtin_amdgcn_s_setprio(0);
          else if (pr == 1) __builtin_amdgcn_s_setprio(1);
          else if (pr == 2) __builtin_amdgcn_s_setprio(2);
          else __builtin_amdgcn_s_setprio(3);
        }
      };
      int n0 = 0;
      if constexpr (W == 2)
        for (; n0 + 2 <= N; n0 += 2) {
          turn(n0 >> 1);
          process(std::integral_constant<int, 2>{}, n0);
        }
      for (; n0 < N; ++n0) {
        turn(n0);
        process(std::integral_constant<int, 1>{}, n0);
      }

      if (p.z) {
#pragma unroll
        for (int i = 0; i < K; ++i) {
          const float zz = to_f32(zr.v[i]);
          y[i] *= zz * rcp_hw(1.0f + exp2_hw(-LOG2E * zz));
        }
      }
      if (live) {
        Pack<io_t, K> o;
#pragma unroll
        for (int i = 0; i < K; ++i) o.v[i] = from_f32<io_t>(y[i]);
        *reinterpret_cast<Pack<io_t, K> *>(Y + at) = o;
      }
    }
    if constexpr (DB) {
      if (c + 1 < nchunks) {
        float *nb = tiles + ((c + 1) & 1) * 2 * FAST_N * T;
        fast_stage<bc_t, LPR>(nb, Bg, L, t0 + T, N, WAVE * WAVES);
        fast_stage<bc_t, LPR>(nb + FAST_N * T, Cg, L, t0 + T, N, WAVE * WAVES);
      }
    }
  }

  if (p.last) {
#pragma unroll
    for (int rr = 0; rr < RPW; ++rr) {
      const size_t row = (size_t)b * p.dim + d0 + (wave * RPW + rr) * SUBS + sub;
      if (sl < N) reinterpret_cast<io_t *>(p.last)[row * N + sl] = from_f32<io_t>(carry_lanes[rr]);
    }
  }
}

// The same scan for projections that few channels share (down to one B/C group per channel, the layout
// (B, D, N, L) a Mamba-1 block passes): nothing is staged.  A wave owns one row, a lane its 8-step run, and the
// lane reads the 16 bytes of B and of C of its run for every state straight from memory (consecutive lanes,
// consecutive bytes), one state ahead of the arithmetic.  No LDS, no barrier: the call is bound by those reads.
// CONST_BC: the same walk for projections that do not vary in time, (D, N) or (B, D, N) (the reference's other
// accepted forms, src/ssm/ops/python/reference.py:22-56): a row's N values of B and of C sit in lanes like A, nothing
// of the projections is read inside the loop.
// K: steps per lane, 8 or 16; with 16 a chunk of the walk is two chunks of FAST_T steps and the state that enters
// the second one (what lane 32 starts from) is written to chunk_states as well.
template <typename io_t, typename bc_t, int WAVES, int OCC, bool CONST_BC = false, int K = 8>
__global__ __launch_bounds__(WAVE *WAVES) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void scan_fwd_rowbc_kernel(const ScanFwdParams p) {
  constexpr int T = WAVE * K;
  static_assert(T == FAST_T || T == 2 * FAST_T, "chunks of the walk are one or two chunks of the forward's states");
  const int wave = wave_id_uniform();
  const int lane = lane_id();
  const size_t row = (size_t)blockIdx.x * WAVES + wave;
  if (row >= (size_t)p.batch * p.dim) return;                // no barrier below: a wave may leave alone
  const int b = (int)(row / p.dim), d = (int)(row % p.dim);
  const int L = p.len, N = p.nstate;
  const bc_t *Bg = reinterpret_cast<const bc_t *>(p.Bp), *Cg = reinterpret_cast<const bc_t *>(p.Cp);
  float B_lanes = 0.0f, C_lanes = 0.0f;
  if constexpr (CONST_BC) {
    if (lane < N) {
      B_lanes = load_as_f32(p.Bp, p.bc_dtype, (p.b_kind == SSM_PROJ_BDN ? row : (size_t)d) * N + lane);
      C_lanes = load_as_f32(p.Cp, p.bc_dtype, (p.c_kind == SSM_PROJ_BDN ? row : (size_t)d) * N + lane);
    }
  } else {
    Bg += ((size_t)b * p.b_groups + d / (p.dim / p.b_groups)) * (size_t)N * L;
    Cg += ((size_t)b * p.c_groups + d / (p.dim / p.c_groups)) * (size_t)N * L;
  }
  const io_t *U = reinterpret_cast<const io_t *>(p.u), *DT = reinterpret_cast<const io_t *>(p.delta);
  const io_t *Z = reinterpret_cast<const io_t *>(p.z);
  io_t *Y = reinterpret_cast<io_t *>(p.out);

  const float A2_lanes = lane < N ? p.A[(size_t)d * N + lane] * LOG2E : 0.0f;
  float carry_lanes = 0.0f;
  const float Dk = p.Dk ? p.Dk[d] : 0.0f, bias = p.bias ? p.bias[d] : 0.0f;

  const int nchunks = (L + T - 1) / T;
  const int state_chunks = (L + FAST_T - 1) / FAST_T;         // rows of chunk_states per (batch, channel)
  for (int c = 0; c < nchunks; ++c) {
    const int t = c * T + lane * K;
    const bool live = t < L;
    const int tc = live ? t : 0;
    const size_t at = row * L + tc;
    float dl[K], du[K], y[K];
    Pack<io_t, K> zr;
    Pack<bc_t, K> braw, craw;
    if constexpr (!CONST_BC) {
      braw = *reinterpret_cast<const Pack<bc_t, K> *>(Bg + tc);
      craw = *reinterpret_cast<const Pack<bc_t, K> *>(Cg + tc);
    }
    {
      const Pack<io_t, K> ur = *reinterpret_cast<const Pack<io_t, K> *>(U + at);
      const Pack<io_t, K> dr = *reinterpret_cast<const Pack<io_t, K> *>(DT + at);
      if (p.z) zr = *reinterpret_cast<const Pack<io_t, K> *>(Z + at);
      if (p.chunk_states && lane < N) p.chunk_states[(row * state_chunks + c * (T / FAST_T)) * (size_t)N + lane] = carry_lanes;
#pragma unroll
      for (int i = 0; i < K; ++i) dl[i] = to_f32(dr.v[i]) + bias;
      if (p.softplus) {
#pragma unroll
        for (int i = 0; i < K; ++i) dl[i] = fast_softplus(dl[i]);
      }
#pragma unroll
      for (int i = 0; i < K; ++i) {
        const float uu = to_f32(ur.v[i]);
        dl[i] = live ? dl[i] : 0.0f;
        du[i] = dl[i] * uu;
        y[i] = Dk * uu;
      }
    }
    float dsum = 0.0f;
#pragma unroll
    for (int i = 0; i < K; ++i) dsum += dl[i];

    for (int n = 0; n < N; ++n) {
      // the next state's projections are requested before this state's arithmetic
      const int nn = n + 1 < N ? n + 1 : n;
      Pack<bc_t, K> bnext, cnext;
      float bq[K], cq[K];
      if constexpr (!CONST_BC) {
        bnext = *reinterpret_cast<const Pack<bc_t, K> *>(Bg + (size_t)nn * L + tc);
        cnext = *reinterpret_cast<const Pack<bc_t, K> *>(Cg + (size_t)nn * L + tc);
#pragma unroll
        for (int i = 0; i < K; ++i) {
          bq[i] = to_f32(braw.v[i]);
          cq[i] = to_f32(craw.v[i]);
        }
      } else {
        const float bn = wave_read_lane(B_lanes, n), cn = wave_read_lane(C_lanes, n);
#pragma unroll
        for (int i = 0; i < K; ++i) {
          bq[i] = bn;
          cq[i] = cn;
        }
      }
      const float A2 = wave_read_lane(A2_lanes, n);
      const float H = wave_read_lane(carry_lanes, n);
      float a[K], bx[K], P = dsum * A2, h;
#pragma unroll
      for (int i = 0; i < K; ++i) a[i] = dl[i] * A2;
      exp2_run(a, P);
#pragma unroll
      for (int i = 0; i < K; ++i) {
        bx[i] = du[i] * bq[i];
        h = i == 0 ? bx[0] : __builtin_fmaf(a[i], h, bx[i]);
      }
      h = __builtin_fmaf(P, lane == 0 ? H : 0.0f, h);
      wave_scan_affine_x1(P, h);
      float hs = wave_prev(h, H);
      const float hend = wave_read_lane(h, WAVE - 1);
      carry_lanes = lane == n ? hend : carry_lanes;
      if constexpr (T == 2 * FAST_T) {
        // the state entering the second half of the chunk: what lane 32 starts from
        const float hmid = wave_read_lane(hs, WAVE / 2);
        if (p.chunk_states && lane == n && c * 2 + 1 < state_chunks)
          p.chunk_states[(row * state_chunks + c * 2 + 1) * (size_t)N + n] = hmid;
      }
#pragma unroll
      for (int i = 0; i < K; ++i) {
        hs = __builtin_fmaf(a[i], hs, bx[i]);
        y[i] = __builtin_fmaf(hs, cq[i], y[i]);
      }
      if constexpr (!CONST_BC) {
        braw = bnext;
        craw = cnext;
      }
    }

    if (p.z) {
#pragma unroll
      for (int i = 0; i < K; ++i) {
        const float zz = to_f32(zr.v[i]);
        y[i] *= zz * rcp_hw(1.0f + exp2_hw(-LOG2E * zz));
      }
    }
    if (live) {
      Pack<io_t, K> o;
#pragma unroll
      for (int i = 0; i < K; ++i) o.v[i] = from_f32<io_t>(y[i]);
      *reinterpret_cast<Pack<io_t, K> *>(Y + at) = o;
    }
  }
  if (p.last && lane < N) reinterpret_cast<io_t *>(p.last)[row * N + lane] = from_f32<io_t>(carry_lanes);
}

template <typename io_t, typename bc_t>
static int launch_scan_fwd_rowbc(const ScanFwdParams &p, hipStream_t stream) {
  constexpr int WAVES = 4;
  const size_t rows = (size_t)p.batch * p.dim;
  hipLaunchKernelGGL((scan_fwd_rowbc_kernel<io_t, bc_t, WAVES, 6>), dim3((unsigned)((rows + WAVES - 1) / WAVES)),
                     dim3(WAVE * WAVES), 0, stream, p);
  SSM_CHECK_LAUNCH("ssm_scan_fwd");
  return SSM_OK;
}

template <typename io_t, typename bc_t, int LPR, int RPW, int WAVES, int W, int OCC, bool DB = false>
static int launch_scan_fwd_fast(const ScanFwdParams &p, hipStream_t stream) {
  const size_t lds = (size_t)(DB ? 4 : 2) * FAST_N * FAST_T * sizeof(float);
  auto kernel = scan_fwd_fast_kernel<io_t, bc_t, LPR, RPW, WAVES, W, OCC, DB>;
  if (allow_dynamic_lds(kernel, lds) != hipSuccess) {
    (void)hipGetLastError();
    set_error("ssm_scan_fwd: cannot reserve %zu bytes of LDS", lds);
    return SSM_ERR_LAUNCH;
  }
  const unsigned grid = (unsigned)((size_t)p.batch * (p.dim / (WAVES * RPW * (WAVE / LPR))));
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(WAVE * WAVES), lds, stream, p);
  SSM_CHECK_LAUNCH("ssm_scan_fwd");
  return SSM_OK;
}

template <typename io_t>
static int launch_scan_fwd_row_const(const ScanFwdParams &p, hipStream_t stream) {
  constexpr int WAVES = 4;
  const size_t rows = (size_t)p.batch * p.dim;
  const dim3 grid((unsigned)((rows + WAVES - 1) / WAVES)), block(WAVE * WAVES);
  const int tail = p.len % (2 * FAST_T);
  if (p.len % 16 == 0 && p.len >= 2 * FAST_T && (tail == 0 || tail > FAST_T))
    hipLaunchKernelGGL((scan_fwd_rowbc_kernel<io_t, float, WAVES, 4, true, 16>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((scan_fwd_rowbc_kernel<io_t, float, WAVES, 6, true>), grid, block, 0, stream, p);
  SSM_CHECK_LAUNCH("ssm_scan_fwd");
  return SSM_OK;
}

// Channels per workgroup of a variant; 0 for an unknown one.
// variant = 10000 * (rows a wave walks at once) + 1000 * (rows a wave walks in turn) + 10 * waves + states in flight
inline int scan_fwd_fast_rows(int variant) {
  switch (variant) {
    case 13082: case 12121: return 24;
    case 11082: return 8;
    case 22121: case 22123: return 48;
    case 21081: return 16;
    case 31041: return 1;       // a row per wave, projections read straight from memory
    case 31042: return 1;       // a row per wave, projections constant in time
    default: return 0;
  }
}

template <typename io_t, typename bc_t>
int scan_fwd_fast_dispatch(const ScanFwdParams &p, int variant, hipStream_t s) {
  switch (variant) {
    case 13082: return launch_scan_fwd_fast<io_t, bc_t, 64, 3, 8, 2, 4>(p, s);     // 4 waves per SIMD
    case 12121: return launch_scan_fwd_fast<io_t, bc_t, 64, 2, 12, 1, 6>(p, s);    // 6 waves per SIMD
    case 11082: return launch_scan_fwd_fast<io_t, bc_t, 64, 1, 8, 2, 4>(p, s);
    case 22121: return launch_scan_fwd_fast<io_t, bc_t, 32, 2, 12, 1, 3>(p, s);    // 3 waves per SIMD, 16-step runs
    case 22123: return launch_scan_fwd_fast<io_t, bc_t, 32, 2, 12, 1, 3, true>(p, s);   // the same with two slabs
    case 21081: return launch_scan_fwd_fast<io_t, bc_t, 32, 1, 8, 1, 4>(p, s);
    case 31041: return launch_scan_fwd_rowbc<io_t, bc_t>(p, s);
    case 31042: return launch_scan_fwd_row_const<io_t>(p, s);
    default:
      set_error("ssm_scan_fwd: unknown variant %d of the specialised kernel", variant);
      return SSM_ERR_BAD_KIND;
  }
}

}  // namespace ssm
