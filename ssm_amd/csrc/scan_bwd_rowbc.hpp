// Selective scan, backward, for projections of their own per channel: B and C of shape (B, D, N, L), the form in
// which the reference's own Mamba1 module calls the operator (src/ssm/modules/mamba1.py:229-246: per-channel
// parameters scaled by a per-token gate).  Included by scan_bwd.hip after scan_bwd_fast.hpp.
//
// Nothing sums over channels here, so a row needs no one else: a wavefront owns one row for the whole call and
// walks its chunks last to first and, inside a chunk, its states one after the other with the arithmetic of the
// wave-per-row kernel (scan_bwd_fast.hpp) -- recompute the states from the chunk's entering state, fold the adjoint
// backwards, compose the lanes' maps on lane-reversed operands, replay.  B and C are read straight from memory,
// 8 steps per lane, one state ahead of the arithmetic; dB and dC of those 8 steps go straight to their place in
// the result, in float32 or in the projections' own type.  No LDS, no barrier, no partial sums to fold for dB and
// dC: the call is bound by those four streams (2 x 16 bytes read and 2 x 16-32 bytes written per lane and state
// against 4 x 16 bytes per lane for the whole row).  Two waves per SIMD: a state's four vectors in flight and the
// row's sums take more than 128 registers, and at 168 the kernel with the gate still spills (config 1's shape in bf16:
// 0.95 ms at four waves per SIMD with 47-64 registers spilled, 0.75 ms at three, 0.70 ms at two).
//
// CONST_BC: the same walk for projections that do not vary in time, (D, N) or (B, D, N) -- the reference's other
// accepted forms (src/ssm/ops/python/reference.py:22-56), and what its Mamba1 block's per-channel projections
// reduce to once the per-token gate is taken out of the recurrence.  A row's N values of B and of C sit in lanes like
// A; dB and dC are sums over time, kept in lanes like dA and left per row for the folds over the batch.  Nothing
// of the size of the projections moves, so the kernel is bound by its arithmetic and runs four waves per SIMD.
#pragma once
#include "scan_bwd_fast.hpp"

namespace ssm {

constexpr int BR_WAVES = 4;

// K: steps per lane, 8 or 16 (a lane's run; 64 runs make a chunk of the walk).  The states that enter chunks come
// from the forward in steps of FAST_T = 512, so a walk in chunks of 1024 takes every second one.
template <typename io_t, typename bc_t, typename out_t, bool HAS_Z, bool CONST_BC = false, int K = BF_K, int OCC = (CONST_BC ? 4 : 2)>
__global__ __launch_bounds__(WAVE *BR_WAVES) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void scan_bwd_rowbc_kernel(const ScanBwdParams p, out_t *dBo, out_t *dCo) {
  constexpr int T = WAVE * K;
  static_assert(T % FAST_T == 0, "chunks of the walk are whole chunks of the forward");
  const int wave = wave_id_uniform();
  const int lane = lane_id();
  const size_t row = (size_t)blockIdx.x * BR_WAVES + wave;
  if (row >= (size_t)p.batch * p.dim) return;                // no barrier below: a wave may leave alone
  const int d = (int)(row % p.dim);
  const int L = p.len, N = p.nstate;
  const int nchunks = (L + T - 1) / T;
  const int fwd_chunks = (L + FAST_T - 1) / FAST_T;           // rows of chunk_states per (batch, channel)
  const int rev_lane = WAVE - 1 - lane;
  const size_t proj0 = CONST_BC ? 0 : row * (size_t)N * L;    // the row's own (N, L) block of B, C, dB and dC
  const bc_t *Bg = reinterpret_cast<const bc_t *>(p.Bp) + proj0, *Cg = reinterpret_cast<const bc_t *>(p.Cp) + proj0;
  out_t *dBg = dBo + proj0, *dCg = dCo + proj0;
  // CONST_BC: lane n holds B[n] and C[n] of the row ((D, N), or (B, D, N) with the batch entry's own) and their sums
  float B_lanes = 0.0f, C_lanes = 0.0f, dB_lanes = 0.0f, dC_lanes = 0.0f;
  if (CONST_BC && lane < N) {
    B_lanes = load_as_f32(p.Bp, p.bc_dtype, (p.b_kind == SSM_PROJ_BDN ? row : (size_t)d) * N + lane);
    C_lanes = load_as_f32(p.Cp, p.bc_dtype, (p.c_kind == SSM_PROJ_BDN ? row : (size_t)d) * N + lane);
  }
  const io_t *U = reinterpret_cast<const io_t *>(p.u), *DT = reinterpret_cast<const io_t *>(p.delta);
  const io_t *GO = reinterpret_cast<const io_t *>(p.dout), *Z = reinterpret_cast<const io_t *>(HAS_Z ? p.z : p.u);
  io_t *DU = reinterpret_cast<io_t *>(p.du), *DDL = reinterpret_cast<io_t *>(p.ddelta), *DZ = reinterpret_cast<io_t *>(p.dz);

  // lane n holds what belongs to state n: A log2(e), the adjoint carried between chunks, the sum for dA
  const float A2_lanes = lane < N ? p.A[(size_t)d * N + lane] * LOG2E : 0.0f;
  float qcarry = (p.dlast && lane < N) ? p.dlast[row * N + lane] : 0.0f;
  float dA_lanes = 0.0f;
  const float Dk = p.Dk ? p.Dk[d] : 0.0f, bias = p.bias ? p.bias[d] : 0.0f;
  float dD_part = 0.0f, db_part = 0.0f;

  for (int c = nchunks - 1; c >= 0; --c) {
    const int t = c * T + lane * K;
    const bool live = t < L;
    const int tc = live ? t : 0;
    const size_t at = row * L + tc;
    Pack<bc_t, K> braw, craw;
    if (!CONST_BC) {
      braw = *reinterpret_cast<const Pack<bc_t, K> *>(Bg + tc);
      craw = *reinterpret_cast<const Pack<bc_t, K> *>(Cg + tc);
    }
    const Pack<io_t, K> ur = *reinterpret_cast<const Pack<io_t, K> *>(U + at);
    const Pack<io_t, K> dr = *reinterpret_cast<const Pack<io_t, K> *>(DT + at);
    const Pack<io_t, K> gr = *reinterpret_cast<const Pack<io_t, K> *>(GO + at);
    Pack<io_t, K> zr;
    if (HAS_Z) zr = *reinterpret_cast<const Pack<io_t, K> *>(Z + at);
    const float Hin_lanes = lane < N ? p.chunk_states[(row * fwd_chunks + c * (T / FAST_T)) * (size_t)N + lane] : 0.0f;

    float dl[K], du[K], g[K], ghB[K], At[K], pre[K];
    float dsum = 0.0f;
#pragma unroll
    for (int i = 0; i < K; ++i) {
      float x = to_f32(dr.v[i]) + bias;
      if (p.softplus) x = fast_softplus(x);
      dl[i] = live ? x : 0.0f;                         // steps past the end: identity maps, no contributions
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

    for (int n = 0; n < N; ++n) {
      // the next state's projections are requested before this state's arithmetic
      const int nn = n + 1 < N ? n + 1 : n;
      Pack<bc_t, K> bnext, cnext;
      float bq[K], cq[K];
      if (!CONST_BC) {
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
      float hv[K + 1];                                 // hv[i]: the state before step i of the run
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
      qr = __builtin_fmaf(Pr, lane == 0 ? qc : 0.0f, qr);        // reversed lane 0 is the chunk's last run
      wave_scan_affine_x1(Pr, qr);
      const float qnew = wave_read_lane(qr, WAVE - 1);         // adjoint leaving the chunk towards earlier steps
      qcarry = lane == n ? qnew : qcarry;
      float qn = lane_from(wave_prev(qr, qc), rev_lane);       // adjoint entering this lane's run from the right
      float sA = 0.0f, sB = 0.0f, sC = 0.0f;
      Pack<out_t, K> ob, oc;
#pragma unroll
      for (int i = K - 1; i >= 0; --i) {
        const float gh = __builtin_fmaf(g[i], cq[i], qn);
        if (!CONST_BC) {
          oc.v[i] = from_f32<out_t>(g[i] * hv[i + 1]);
          ob.v[i] = from_f32<out_t>(gh * du[i]);
        } else {
          sC = __builtin_fmaf(g[i], hv[i + 1], sC);
          sB = __builtin_fmaf(gh, du[i], sB);
        }
        ghB[i] = __builtin_fmaf(gh, bq[i], ghB[i]);
        qn = a[i] * gh;
        const float qh = qn * hv[i];
        At[i] = __builtin_fmaf(qh, A2, At[i]);
        sA = __builtin_fmaf(qh, dl[i], sA);
      }
      const float tot = wave_sum(sA);
      dA_lanes += lane == n ? tot : 0.0f;
      if (!CONST_BC) {
        if (live) {
          *reinterpret_cast<Pack<out_t, K> *>(dBg + (size_t)n * L + tc) = ob;
          *reinterpret_cast<Pack<out_t, K> *>(dCg + (size_t)n * L + tc) = oc;
        }
        braw = bnext;
        craw = cnext;
      } else {
        const float totB = wave_sum(sB), totC = wave_sum(sC);
        dB_lanes += lane == n ? totB : 0.0f;
        dC_lanes += lane == n ? totC : 0.0f;
      }
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
        dd *= e * rcp_hw(1.0f + e);                    // softplus' = sigmoid
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

  const float sd = wave_sum(dD_part), sb = wave_sum(db_part);
  if (lane < N) p.dA_rows[row * N + lane] = dA_lanes;
  if (CONST_BC && lane < N) {
    p.dB_part[row * N + lane] = dB_lanes;
    p.dC_part[row * N + lane] = dC_lanes;
  }
  if (lane == 0) {
    p.dD_rows[row] = sd;
    p.dbias_rows[row] = sb;
  }
}

// Projections constant in time: the partial sums per row go to p.dB_part / p.dC_part, (B, D, N) float32.
template <typename io_t>
static int launch_bwd_row_const(const ScanBwdParams &p, hipStream_t s) {
  const size_t rows = (size_t)p.batch * p.dim;
  const dim3 grid((unsigned)((rows + BR_WAVES - 1) / BR_WAVES)), block(WAVE * BR_WAVES);
  // 16-step runs halve the lane scans and wave sums per step; their 243 registers leave two waves per SIMD (at three,
  // 66 spill): 303 against 323 us at 8 x 1536 x 2048.  For sequences that fill chunks of 1024 steps.
  const int tail = p.len % 1024;
  if (p.len % 16 == 0 && p.len >= 1024 && (tail == 0 || tail > 512)) {
    if (p.z) hipLaunchKernelGGL((scan_bwd_rowbc_kernel<io_t, float, float, true, true, 16, 2>), grid, block, 0, s, p, nullptr, nullptr);
    else hipLaunchKernelGGL((scan_bwd_rowbc_kernel<io_t, float, float, false, true, 16, 2>), grid, block, 0, s, p, nullptr, nullptr);
  } else if (p.z) hipLaunchKernelGGL((scan_bwd_rowbc_kernel<io_t, float, float, true, true>), grid, block, 0, s, p, nullptr, nullptr);
  else hipLaunchKernelGGL((scan_bwd_rowbc_kernel<io_t, float, float, false, true>), grid, block, 0, s, p, nullptr, nullptr);
  SSM_CHECK_LAUNCH("ssm_scan_bwd");
  return SSM_OK;
}

template <typename io_t, typename bc_t, typename out_t>
static int launch_bwd_rowbc(const ScanBwdParams &p, void *dB, void *dC, hipStream_t s) {
  const size_t rows = (size_t)p.batch * p.dim;
  const dim3 grid((unsigned)((rows + BR_WAVES - 1) / BR_WAVES)), block(WAVE * BR_WAVES);
  out_t *b = reinterpret_cast<out_t *>(dB), *c = reinterpret_cast<out_t *>(dC);
  if (p.z) hipLaunchKernelGGL((scan_bwd_rowbc_kernel<io_t, bc_t, out_t, true>), grid, block, 0, s, p, b, c);
  else hipLaunchKernelGGL((scan_bwd_rowbc_kernel<io_t, bc_t, out_t, false>), grid, block, 0, s, p, b, c);
  SSM_CHECK_LAUNCH("ssm_scan_bwd");
  return SSM_OK;
}

}  // namespace ssm
