// Selective scan, backward: the kernel for the common call shape (time-varying grouped B and C,
// at most 16 states, activations of any supported type in aligned rows of whole 8-step runs).  Included by
// scan_bwd.hip after ScanBwdParams.
//
// A wavefront owns one row at a time and walks its states one after the other, lanes split
// time as in the forward kernel (8 steps per lane, 512 per chunk, chunks last to first).  For a
// state: recompute h from the chunk's entering state (fold, lane scan, replay), fold the
// adjoint q_t = a_t (g_t C_t + q_{t+1}) backwards over the lane's run, compose the lanes' maps
// with the same scan on lane-reversed operands, replay backwards with the true adjoint.  What
// sums over states (pre-activation, <gh, B>, the A-term of d delta) never leaves the lane's
// registers; what sums over the channels of a group (dB, dC) is added into an LDS tile by the
// 16 wavefronts of the workgroup, which are kept on 16 different states by a skew: wave w works
// on state (w + slot) mod 16, so a state's part of the tile passes from wave w + 1 to wave w from
// one slot to the next.  A wave counts its finished slots in LDS and, before it touches the tile
// (a plain read, add, write at the very end of the slot), waits for the count of the wave it
// takes over from; the rest of a slot needs no agreement between waves, which may drift apart by
// most of a slot.  (A workgroup barrier per slot costs 25 % of the kernel's time here, LDS float
// atomics, which take the 64 lanes one by one on this chip, eight times the whole kernel.)
// Every element is added to by one wave at a time in a fixed order, so results are the same bits
// on every run.  The tile goes to memory once per chunk as one partial per workgroup.
// 128 KB of LDS: one workgroup of 16 waves per CU, four waves per SIMD.
#pragma once
#include "scan_fwd_fast.hpp"

namespace ssm {

constexpr int BF_WAVES = 16;
constexpr int BF_THREADS = WAVE * BF_WAVES;
constexpr int BF_K = 8;
constexpr int BF_DEP = 1;             // wave w takes a state over from wave w + BF_DEP (-1 measured 2 % slower)

__device__ __forceinline__ float lane_from(float v, int src_lane) {
  return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane << 2, __float_as_int(v)));
}

// Wait until the count at `flag` (LDS, written by one other wave of the workgroup, only ever growing) has reached
// `want`; false if it has not after `spin_limit` looks (2^16 in every call of the library: about three milliseconds).  Every wave of a workgroup is resident and the
// waves' waits form no cycle (a wave in slot k waits for slot k - 1 of its neighbour), so the wait ends; the bound
// is there so that a mistake elsewhere ends as NaN in dB and dC (the caller poisons its sums), not as waves that
// never finish or as sums that are silently wrong.
typedef __attribute__((address_space(3))) int lds_int;

__device__ __forceinline__ bool wait_for_slots(lds_int *flag, int want, int spin_limit) {
  bool reached = false;
  for (int spin = 0; spin < spin_limit; ++spin) {
    const int seen = __builtin_amdgcn_readfirstlane(*(volatile lds_int *)flag);
    if (seen >= want) {
      reached = true;
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  __asm__ volatile("" ::: "memory");
  return reached;
}

template <typename io_t, typename bc_t, int RPW, bool HAS_Z>
__global__ __launch_bounds__(BF_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4)))
void scan_bwd_fast_kernel(const ScanBwdParams p) {
  constexpr int K = BF_K, T = FAST_T, NS = FAST_N;
  extern __shared__ __align__(16) float lds[];
  float *Bs = lds, *Cs = Bs + NS * T;            // projections of the chunk, [n][q][lane][4]
  float *accB = Cs + NS * T, *accC = accB + NS * T;   // sums over the workgroup's rows, same layout
  // per row, touched by the wave that owns the row only: A log2(e), the adjoint carried between chunks and the
  // sum for dA per state; the sums for dD and the bias
  float *rowA2 = accC + NS * T, *rowq = rowA2 + BF_WAVES * RPW * NS, *rowdA = rowq + BF_WAVES * RPW * NS;
  float *rowdD = rowdA + BF_WAVES * RPW * NS, *rowdb = rowdD + BF_WAVES * RPW;
  lds_int *done = (lds_int *)reinterpret_cast<int *>(rowdb + BF_WAVES * RPW);     // per wave: slots finished since the kernel began

  constexpr int rows = BF_WAVES * RPW;
  const int wave = wave_id_uniform();
  const int lane = lane_id();
  const int tid = threadIdx.x;
  const int b = (int)blockIdx.x / p.nblk;
  const int blk = (int)blockIdx.x % p.nblk;
  const int d_first = blk * rows;
  const int L = p.len, N = p.nstate;
  const int nchunks = (L + T - 1) / T;
  const int rev_lane = WAVE - 1 - lane;
  const bc_t *Bg = reinterpret_cast<const bc_t *>(p.Bp) + ((size_t)b * p.b_groups + d_first / (p.dim / p.b_groups)) * (size_t)N * L;
  const bc_t *Cg = reinterpret_cast<const bc_t *>(p.Cp) + ((size_t)b * p.c_groups + d_first / (p.dim / p.c_groups)) * (size_t)N * L;
  const io_t *U = reinterpret_cast<const io_t *>(p.u), *DT = reinterpret_cast<const io_t *>(p.delta);
  const io_t *GO = reinterpret_cast<const io_t *>(p.dout), *Z = reinterpret_cast<const io_t *>(HAS_Z ? p.z : p.u);
  io_t *DU = reinterpret_cast<io_t *>(p.du), *DDL = reinterpret_cast<io_t *>(p.ddelta), *DZ = reinterpret_cast<io_t *>(p.dz);

  for (int rr = 0; rr < RPW; ++rr) {
    const int r = wave * RPW + rr, d = d_first + r;
    const size_t row = (size_t)b * p.dim + d;
    if (lane < NS) {
      rowA2[r * NS + lane] = lane < N ? p.A[(size_t)d * N + lane] * LOG2E : 0.0f;
      rowq[r * NS + lane] = (p.dlast && lane < N) ? p.dlast[row * N + lane] : 0.0f;      // adjoint from beyond the end
      rowdA[r * NS + lane] = 0.0f;
    }
    if (lane == 0) rowdD[r] = rowdb[r] = 0.0f;
  }
  if (lane == 0) done[wave] = 0;
  int nslots = 0;                          // the same in every wave at the same point of the walk

  for (int c = nchunks - 1; c >= 0; --c) {
    const int t0 = c * T;
    const int t = t0 + lane * K;
    const bool live = t < L;
    const int tc = live ? t : 0;

    __syncthreads();                       // the sums of the chunk before are in memory, its slabs are free
    fast_stage<bc_t, WAVE>(Bs, Bg, L, t0, N, BF_THREADS);
    fast_stage<bc_t, WAVE>(Cs, Cg, L, t0, N, BF_THREADS);
    for (int e = tid; e < 2 * NS * T / 4; e += BF_THREADS) reinterpret_cast<float4 *>(accB)[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();

#pragma nounroll
    for (int rr = 0; rr < RPW; ++rr) {
      const int r = wave * RPW + rr, d = d_first + r;
      const size_t row = (size_t)b * p.dim + d;
      const size_t at = row * L + tc;
      const float A2_lanes = rowA2[r * NS + (lane & (NS - 1))];
      float qcarry = rowq[r * NS + (lane & (NS - 1))], dA_lanes = 0.0f;
      const float Dk = p.Dk ? p.Dk[d] : 0.0f, bias = p.bias ? p.bias[d] : 0.0f;
      float dD_part = 0.0f, db_part = 0.0f;
      const Pack<io_t, K> ur = *reinterpret_cast<const Pack<io_t, K> *>(U + at);
      const Pack<io_t, K> dr = *reinterpret_cast<const Pack<io_t, K> *>(DT + at);
      const Pack<io_t, K> gr = *reinterpret_cast<const Pack<io_t, K> *>(GO + at);
      Pack<io_t, K> zr;
      if (HAS_Z) zr = *reinterpret_cast<const Pack<io_t, K> *>(Z + at);
      const float Hin_lanes = lane < N ? p.chunk_states[(row * nchunks + c) * (size_t)N + lane] : 0.0f;

      float dl[K], du[K], g[K], ghB[K], At[K], pre[K];
      float dsum = 0.0f;
#pragma unroll
      for (int i = 0; i < K; ++i) {
        float x = to_f32(dr.v[i]) + bias;
        if (p.softplus) x = fast_softplus(x);
        dl[i] = live ? x : 0.0f;                       // steps past the end: identity maps, no contributions
        du[i] = dl[i] * to_f32(ur.v[i]);
        float gg = live ? to_f32(gr.v[i]) : 0.0f;
        if (HAS_Z) {
          const float zz = to_f32(zr.v[i]);
          gg *= zz * rcp_hw(1.0f + exp2_hw(-LOG2E * zz));
        }
        g[i] = gg;
        ghB[i] = At[i] = pre[i] = 0.0f;
        dsum += dl[i];
      }

      for (int slot = 0; slot < NS; ++slot) {
        const int n = (BF_DEP * wave + slot) & (NS - 1);
        // the SIMD serves its oldest wave first; turn the order round slot by slot so that its four waves keep pace
        {
          const int pr = (slot + (wave >> 2)) & 3;
          if (pr == 0) __builtin_amdgcn_s_setprio(0);
          else if (pr == 1) __builtin_amdgcn_s_setprio(1);
          else if (pr == 2) __builtin_amdgcn_s_setprio(2);
          else __builtin_amdgcn_s_setprio(3);
        }
        if (n < N) {
          float bq[K], cq[K];
#pragma unroll
          for (int q = 0; q < K / 4; ++q) {
            const float4 bv = *reinterpret_cast<const float4 *>(Bs + n * T + q * (WAVE * 4) + lane * 4);
            const float4 cv = *reinterpret_cast<const float4 *>(Cs + n * T + q * (WAVE * 4) + lane * 4);
            bq[4 * q] = bv.x; bq[4 * q + 1] = bv.y; bq[4 * q + 2] = bv.z; bq[4 * q + 3] = bv.w;
            cq[4 * q] = cv.x; cq[4 * q + 1] = cv.y; cq[4 * q + 2] = cv.z; cq[4 * q + 3] = cv.w;
          }
          const float A2 = wave_read_lane(A2_lanes, n);
          const float Hin = wave_read_lane(Hin_lanes, n);
          const float qc = wave_read_lane(qcarry, n);
          float a[K], P = dsum * A2;
#pragma unroll
          for (int i = 0; i < K; ++i) a[i] = dl[i] * A2;
          exp2_run(a, P);
          // ---- states: fold, scan over the lanes, replay
          float h = du[0] * bq[0];
#pragma unroll
          for (int i = 1; i < K; ++i) h = __builtin_fmaf(a[i], h, du[i] * bq[i]);
          h = __builtin_fmaf(P, lane == 0 ? Hin : 0.0f, h);
          float Pf = P;
          wave_scan_affine_x1(Pf, h);
          float hv[K + 1];                               // hv[i]: the state before step i of the run
          hv[0] = wave_prev(h, Hin);
#pragma unroll
          for (int i = 0; i < K; ++i) {
            hv[i + 1] = __builtin_fmaf(a[i], hv[i], du[i] * bq[i]);
            pre[i] = __builtin_fmaf(hv[i + 1], cq[i], pre[i]);
          }
          // ---- adjoint: fold backwards from zero, scan over the reversed lanes, replay backwards
          float ql = 0.0f;
#pragma unroll
          for (int i = K - 1; i >= 0; --i) ql = a[i] * __builtin_fmaf(g[i], cq[i], ql);
          float Pr = lane_from(P, rev_lane), qr = lane_from(ql, rev_lane);
          qr = __builtin_fmaf(Pr, lane == 0 ? qc : 0.0f, qr);      // reversed lane 0 is the chunk's last run
          wave_scan_affine_x1(Pr, qr);
          const float qnew = wave_read_lane(qr, WAVE - 1);       // adjoint leaving the chunk towards earlier steps
          qcarry = lane == n ? qnew : qcarry;
          float qn = lane_from(wave_prev(qr, qc), rev_lane);     // adjoint entering this lane's run from the right
          float sA = 0.0f;
          float sb[K], sc[K];
#pragma unroll
          for (int i = K - 1; i >= 0; --i) {
            const float gh = __builtin_fmaf(g[i], cq[i], qn);
            sc[i] = g[i] * hv[i + 1];
            sb[i] = gh * du[i];
            ghB[i] = __builtin_fmaf(gh, bq[i], ghB[i]);
            qn = a[i] * gh;
            const float qh = qn * hv[i];
            At[i] = __builtin_fmaf(qh, A2, At[i]);
            sA = __builtin_fmaf(qh, dl[i], sA);
          }
          const float tot = wave_sum(sA);
          dA_lanes += lane == n ? tot : 0.0f;
          // The skew gives this wave the state's part of both tiles to itself for the slot (plain read, add,
          // write), once the wave that had it in the slot before is through with it.
          float4 *aB = reinterpret_cast<float4 *>(accB + n * T + lane * 4), *aC = reinterpret_cast<float4 *>(accC + n * T + lane * 4);
          if (!wait_for_slots(done + ((wave + BF_DEP) & (BF_WAVES - 1)), nslots, p.spin_limit)) sb[0] = sc[0] = __builtin_nanf("");
#pragma unroll
          for (int q = 0; q < K / 4; ++q) {
            float4 vb = aB[q * WAVE], vc = aC[q * WAVE];
            vb.x += sb[4 * q]; vb.y += sb[4 * q + 1]; vb.z += sb[4 * q + 2]; vb.w += sb[4 * q + 3];
            vc.x += sc[4 * q]; vc.y += sc[4 * q + 1]; vc.z += sc[4 * q + 2]; vc.w += sc[4 * q + 3];
            aB[q * WAVE] = vb;
            aC[q * WAVE] = vc;
          }
        }
        // LDS takes a wave's instructions in order: the tile writes above are in before this count is
        ++nslots;
        __asm__ volatile("" ::: "memory");
        if (lane == 0) *(volatile lds_int *)(done + wave) = nslots;
      }

      // ---- what the row's elements receive
      float du_o[K], dd_o[K], dz_o[K];
#pragma unroll
      for (int i = 0; i < K; ++i) {
        const float uu = to_f32(ur.v[i]);
        du_o[i] = __builtin_fmaf(dl[i], ghB[i], g[i] * Dk);
        float dd = __builtin_fmaf(uu, ghB[i], At[i] * LN2);
        if (p.softplus) {
          const float e = exp2_hw(fminf(to_f32(dr.v[i]) + bias, 60.0f) * LOG2E);
          dd *= e * rcp_hw(1.0f + e);                  // softplus' = sigmoid
        }
        dd = live ? dd : 0.0f;
        dd_o[i] = dd;
        db_part += dd;
        dD_part = __builtin_fmaf(g[i], uu, dD_part);
        if (HAS_Z) {
          const float zz = to_f32(zr.v[i]);
          const float s = rcp_hw(1.0f + exp2_hw(-LOG2E * zz));
          const float full = __builtin_fmaf(Dk, uu, pre[i]);
          dz_o[i] = to_f32(gr.v[i]) * full * s * __builtin_fmaf(zz, 1.0f - s, 1.0f);
        }
      }
      {
        const float sd = wave_sum(dD_part), sb = wave_sum(db_part);
        if (lane < NS) {
          rowq[r * NS + lane] = qcarry;
          rowdA[r * NS + lane] += dA_lanes;
        }
        if (lane == 0) {
          rowdD[r] += sd;
          rowdb[r] += sb;
        }
      }
      if (live) {
        Pack<io_t, K> o;
#pragma unroll
        for (int i = 0; i < K; ++i) o.v[i] = from_f32<io_t>(du_o[i]);
        *reinterpret_cast<Pack<io_t, K> *>(DU + at) = o;
#pragma unroll
        for (int i = 0; i < K; ++i) o.v[i] = from_f32<io_t>(dd_o[i]);
        *reinterpret_cast<Pack<io_t, K> *>(DDL + at) = o;
        if (HAS_Z) {
#pragma unroll
          for (int i = 0; i < K; ++i) o.v[i] = from_f32<io_t>(dz_o[i]);
          *reinterpret_cast<Pack<io_t, K> *>(DZ + at) = o;
        }
      }
    }

    __syncthreads();
    // the chunk's sums over this workgroup's rows: one partial per workgroup
    for (int e = tid; e < 2 * N * WAVE; e += BF_THREADS) {
      const int which = e / (N * WAVE), r = e % (N * WAVE);
      const int n = r / WAVE, ln = r % WAVE;
      const int tt = t0 + ln * K;
      if (tt < L) {
        const float *src = (which ? accC : accB) + n * T + ln * 4;
        const float4 v0 = *reinterpret_cast<const float4 *>(src);
        const float4 v1 = *reinterpret_cast<const float4 *>(src + WAVE * 4);
        float *dst = (which ? p.dC_part : p.dB_part) + (((size_t)b * p.nblk + blk) * N + n) * (size_t)L + tt;
        *reinterpret_cast<float4 *>(dst) = v0;
        *reinterpret_cast<float4 *>(dst + 4) = v1;
      }
    }
  }

  for (int rr = 0; rr < RPW; ++rr) {
    const int r = wave * RPW + rr;
    const size_t row = (size_t)b * p.dim + d_first + r;
    if (lane < N) p.dA_rows[row * N + lane] = rowdA[r * NS + lane];
    if (lane == 0) {
      p.dD_rows[row] = rowdD[r];
      p.dbias_rows[row] = rowdb[r];
    }
  }
}

// Rows per wave in turn for which the workgroups (16 waves) tile the groups, or 0.
inline int scan_bwd_fast_rpw(int batch, int dim, int per_b, int per_c) {
  const int cand[3] = {3, 2, 1};
  int best = 0;
  for (int i = 0; i < 3; ++i) {
    const int r = BF_WAVES * cand[i];
    if (per_b % r || per_c % r) continue;
    if (!best) best = cand[i];
    if ((size_t)batch * (dim / r) >= 256) return cand[i];       // the largest block that still gives every CU one
  }
  return best;
}

template <typename io_t, typename bc_t>
static int launch_bwd_fast(const ScanBwdParams &p, int rpw, hipStream_t s) {
  const size_t ldsb = ((size_t)4 * FAST_N * FAST_T + (size_t)BF_WAVES * rpw * (3 * FAST_N + 2) + BF_WAVES) * sizeof(float);
  const unsigned grid = (unsigned)((size_t)p.batch * p.nblk);
#define SSM_BF_LAUNCH(R, HZ)                                                                   \
  {                                                                                            \
    auto kernel = scan_bwd_fast_kernel<io_t, bc_t, R, HZ>;                                     \
    if (allow_dynamic_lds(kernel, ldsb) != hipSuccess) {                                       \
      (void)hipGetLastError();                                                                 \
      set_error("ssm_scan_bwd: cannot reserve %zu bytes of LDS", ldsb);                        \
      return SSM_ERR_LAUNCH;                                                                   \
    }                                                                                          \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(BF_THREADS), ldsb, s, p);                      \
  }
  if (p.z) {
    if (rpw == 3) SSM_BF_LAUNCH(3, true) else if (rpw == 2) SSM_BF_LAUNCH(2, true) else SSM_BF_LAUNCH(1, true)
  } else {
    if (rpw == 3) SSM_BF_LAUNCH(3, false) else if (rpw == 2) SSM_BF_LAUNCH(2, false) else SSM_BF_LAUNCH(1, false)
  }
#undef SSM_BF_LAUNCH
  SSM_CHECK_LAUNCH("ssm_scan_bwd");
  return SSM_OK;
}

}  // namespace ssm
