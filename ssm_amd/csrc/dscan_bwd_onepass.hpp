// Backward of the diagonal chunked scan for the two common calls (float32 dt, a gate of X's shape or none, a
// head's channels in 16, 32 or 64 lanes): per-token B and C of X's shape and type with per-head A and D, or
// (PARAMS) B and C one value per channel -- parameters, as the reference's Mamba2 module passes them,
// src/ssm/modules/mamba2.py:189-199 -- with A and D per head or per channel.
// Every input is read once by the kernel that forms the gradients, no state goes through memory.
//
// A workgroup of 16 waves owns 64 * VEC neighbouring channels of one batch row and walks time backwards in
// rounds of 64 steps, wave w taking steps 4w..4w+3 of the round.  In a round every wave folds its steps twice
// from zero: forwards into (decay product, state) and backwards into the adjoint it would hand to the steps
// before it (mu_t = lambda_t a_t obeys mu_t = a_t (mu_{t+1} + g0_t C_t): the same decays).  The 16 pairs of
// folds meet in LDS (one barrier per round, two buffers); wave w chains the folds of the waves before it from
// the state entering the round on the left, and those of the waves after it from the adjoint entering the round
// on the right (15 links in all, whatever w), which gives it what enters its own steps from both sides, then
// replays its steps forwards (states, kept in registers) and backwards (gradients).  Wave 0's chain ends at the
// round's left edge: it leaves the adjoint there in LDS for everyone's next round.  The state entering a round
// comes from a table written beforehand: by the forward's one-pass kernel, or by that kernel's walk reduced to
// X, B and dt (launch_dscan_round_states).  The reads of the next round are requested before the arithmetic of this one.
#pragma once

namespace ssm {

constexpr int DBO_WAVES = 16, DBO_SEG = 4, DBO_ROUND = DBO_WAVES * DBO_SEG;

// ---- the gradients
template <typename io_t, int VEC, bool HAS_Z>
struct DboRegs {
  float dt[DBO_SEG];
  Word<io_t> x[DBO_SEG], bq[DBO_SEG], cq[DBO_SEG], gq[DBO_SEG], zq[DBO_SEG];
  float enter[VEC];                 // the state entering the round
};

// g_t: element type of dB, dC and dz (io_t, or float).  LPH: lanes that hold one head's channels.
// PARAMS: B and C are held in registers, one value per channel, and their gradients are sums over time like dA's
// and dD's; each channel of a lane has its own decay.
template <typename io_t, typename g_t, int VEC, bool HAS_Z, int LPH, bool PARAMS>
__global__ __launch_bounds__(WAVE *DBO_WAVES) void dscan_bwd_onepass_kernel(const DscanBwdParams p) {
  static_assert(sizeof(io_t) * VEC == 4, "a lane's vector is one register");
  constexpr int AV = PARAMS ? VEC : 1;            // decays per lane
  __shared__ float4 fwd[2][DBO_WAVES][WAVE];     // a wave's four steps per lane: decay product(s), states from zero
  __shared__ float2 rev[2][DBO_WAVES][WAVE];     // ... and the adjoint (times its decay) from zero
  __shared__ float2 left[2][WAVE];               // the adjoint leaving the round, from wave 0 to everyone's next round
  const int wave = wave_id_uniform(), lane = lane_id();
  const int HP = p.heads * p.proj;
  const unsigned ch = ((unsigned)blockIdx.x * WAVE + lane) * VEC;
  const int b = blockIdx.y;
  const int h = (int)ch / p.proj;
  const int L = p.len;
  const int valid = p.lengths ? min(max(p.lengths[b], 0), L) : L;
  float A[AV], A2[AV], Dk[AV], Bc[VEC], Cc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    if (v < AV) {     // per channel (index h*P + p = ch + v) or per head
      A[v] = p.A[p.a_stride_p ? (size_t)ch + v : (size_t)h];
      A2[v] = A[v] * LOG2E;
      Dk[v] = p.Dk ? p.Dk[p.d_stride_p ? (size_t)ch + v : (size_t)h] : 0.0f;
    }
    // constant projections: element strides b_stride_b / c_stride_b are 0 for (H,P) and H*P for (B,H,P)
    Bc[v] = PARAMS ? load_as_f32(p.Bp, p.bc_dtype, (size_t)b * p.b_stride_b + ch + v) : 0.0f;
    Cc[v] = PARAMS ? load_as_f32(p.Cp, p.bc_dtype, (size_t)b * p.c_stride_b + ch + v) : 0.0f;
  }
  // the batch row's part of every tensor: offsets inside it fit 32 bits (checked by the host)
  const size_t row0 = (size_t)b * L;
  const io_t *X = reinterpret_cast<const io_t *>(p.X) + row0 * HP, *G = reinterpret_cast<const io_t *>(p.gy) + row0 * HP;
  const io_t *Bp = reinterpret_cast<const io_t *>(PARAMS ? p.X : p.Bp) + row0 * HP;
  const io_t *Cp = reinterpret_cast<const io_t *>(PARAMS ? p.X : p.Cp) + row0 * HP;
  const io_t *Z = reinterpret_cast<const io_t *>(HAS_Z ? p.z : p.X) + row0 * HP;
  const float *DT = reinterpret_cast<const float *>(p.dt) + row0 * p.heads;
  io_t *dX = reinterpret_cast<io_t *>(p.dX) + row0 * HP;
  g_t *dB = reinterpret_cast<g_t *>(PARAMS ? p.dX : p.dB_t) + row0 * HP, *dC = reinterpret_cast<g_t *>(PARAMS ? p.dX : p.dC_t) + row0 * HP;
  g_t *dZ = reinterpret_cast<g_t *>(HAS_Z ? p.dz_p : p.dX) + row0 * HP;
  float *DDT = p.ddt_direct + row0 * p.heads;
  const int rounds = (L + DBO_ROUND - 1) / DBO_ROUND;
  const float *table = p.round_states + (size_t)b * rounds * HP;

  auto request = [&](DboRegs<io_t, VEC, HAS_Z> &r, int round) {
    const int t0 = round * DBO_ROUND + wave * DBO_SEG;
#pragma unroll
    for (int j = 0; j < DBO_SEG; ++j) {
      const unsigned row = (unsigned)min(t0 + j, L - 1);       // steps past the end read the last row, unused
      const unsigned at = (row * (unsigned)HP + ch) * (unsigned)sizeof(io_t);
      r.dt[j] = *at_bytes<const float>(DT, (row * (unsigned)p.heads + (unsigned)h) * 4u);
      r.x[j] = Word<io_t>{*at_bytes<const unsigned>(X, at)};
      if (!PARAMS) r.bq[j] = Word<io_t>{*at_bytes<const unsigned>(Bp, at)};
      if (!PARAMS) r.cq[j] = Word<io_t>{*at_bytes<const unsigned>(Cp, at)};
      r.gq[j] = Word<io_t>{*at_bytes<const unsigned>(G, at)};
      if (HAS_Z) r.zq[j] = Word<io_t>{*at_bytes<const unsigned>(Z, at)};
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) r.enter[v] = *at_bytes<const float>(table, ((unsigned)round * (unsigned)HP + ch + v) * 4u);
  };

  float accA[VEC], accD[VEC], accB[VEC], accC[VEC], mu_left[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) accA[v] = accD[v] = accB[v] = accC[v] = mu_left[v] = 0.0f;

  auto round_of = [&](DboRegs<io_t, VEC, HAS_Z> &cur, int r) {
    const int q = r & 1;
    const int t0 = r * DBO_ROUND + wave * DBO_SEG;
    float a[AV][DBO_SEG], sg[VEC][DBO_SEG];
    float s[VEC], M[VEC], prod[AV];
#pragma unroll
    for (int v = 0; v < VEC; ++v) s[v] = M[v] = 0.0f;
#pragma unroll
    for (int v = 0; v < AV; ++v) prod[v] = 1.0f;
#pragma unroll
    for (int j = 0; j < DBO_SEG; ++j) {
      const bool live = t0 + j < valid;
      cur.dt[j] = live ? cur.dt[j] : 0.0f;
      cur.x[j].mask(live);
      if (!PARAMS) cur.bq[j].mask(live);
      if (!PARAMS) cur.cq[j].mask(live);
      cur.gq[j].mask(live);
      if (HAS_Z) cur.zq[j].mask(live);
#pragma unroll
      for (int v = 0; v < AV; ++v) {
        a[v][j] = exp2_hw(cur.dt[j] * A2[v]);
        prod[v] *= a[v][j];
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        s[v] = __builtin_fmaf(a[v % AV][j], s[v], cur.dt[j] * (PARAMS ? Bc[v] : cur.bq[j].elem(v)) * cur.x[j].elem(v));
    }
#pragma unroll
    for (int j = DBO_SEG - 1; j >= 0; --j) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        float g0 = cur.gq[j].elem(v);
        if (HAS_Z) {
          const float zz = cur.zq[j].elem(v);
          sg[v][j] = sigmoid_f32(zz);
          g0 *= zz * sg[v][j];
        }
        M[v] = a[v % AV][j] * __builtin_fmaf(g0, PARAMS ? Cc[v] : cur.cq[j].elem(v), M[v]);
      }
    }
    // (one decay per lane: three words to read per link of the forward chain, one per link of the other; two: four, two)
    fwd[q][wave][lane] = AV == 1 ? make_float4(prod[0], s[0], s[VEC - 1], 0.0f) : make_float4(prod[0], prod[AV - 1], s[0], s[VEC - 1]);
    rev[q][wave][lane] = make_float2(M[0], M[VEC - 1]);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < DBO_SEG; ++j) {
      cur.x[j].launder();
      if (!PARAMS) cur.bq[j].launder();
      if (!PARAMS) cur.cq[j].launder();
      cur.gq[j].launder();
      if (HAS_Z) cur.zq[j].launder();
    }
    // the state entering this wave's steps: the folds of the waves before it, from the state entering the round
    float st[VEC][DBO_SEG + 1];
#pragma unroll
    for (int v = 0; v < VEC; ++v) st[v][0] = cur.enter[v];
    for (int w = 0; w < wave; ++w) {
      const float4 f = fwd[q][w][lane];
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        st[v][0] = AV == 1 ? __builtin_fmaf(f.x, st[v][0], v == 0 ? f.y : f.z) : __builtin_fmaf(v == 0 ? f.x : f.y, st[v][0], v == 0 ? f.z : f.w);
    }
    // the adjoint entering them: the folds of the waves after it, from the adjoint that left the round before
    float mu[VEC];
    if (r < rounds - 1) {
      const float2 c = left[q ^ 1][lane];
      mu_left[0] = c.x;
      mu_left[VEC - 1] = c.y;
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) mu[v] = mu_left[v];
    for (int w = DBO_WAVES - 1; w > wave; --w) {
      float pr0, pr1;                                                                 // the decay products
      if constexpr (AV == 1) {
        pr0 = pr1 = fwd[q][w][lane].x;
      } else {
        const float2 pr = *reinterpret_cast<const float2 *>(&fwd[q][w][lane]);
        pr0 = pr.x;
        pr1 = pr.y;
      }
      const float2 f = rev[q][w][lane];
#pragma unroll
      for (int v = 0; v < VEC; ++v) mu[v] = __builtin_fmaf(v % AV == 0 ? pr0 : pr1, mu[v], v == 0 ? f.x : f.y);
    }
    if (wave == 0) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) mu_left[v] = __builtin_fmaf(prod[v % AV], mu[v], M[v]);
      left[q][lane] = make_float2(mu_left[0], mu_left[VEC - 1]);
    }
    // forward replay: st[v][j + 1] = the state after step j
#pragma unroll
    for (int j = 0; j < DBO_SEG; ++j) {
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        st[v][j + 1] = __builtin_fmaf(a[v % AV][j], st[v][j], cur.dt[j] * (PARAMS ? Bc[v] : cur.bq[j].elem(v)) * cur.x[j].elem(v));
    }
    // backward replay; mu[v] is lambda_{t+1} a_{t+1}
#pragma unroll
    for (int j = DBO_SEG - 1; j >= 0; --j) {
      const int t = t0 + j;
      // a step's float32 values are formed at the step, not all in front of the loop
      cur.x[j].launder_after(mu[0]);
      if (!PARAMS) cur.bq[j].launder_after(mu[0]);
      if (!PARAMS) cur.cq[j].launder_after(mu[0]);
      cur.gq[j].launder_after(mu[0]);
      if (HAS_Z) cur.zq[j].launder_after(mu[0]);
      Pack<io_t, VEC> ox;
      Pack<g_t, VEC> ob, oc, oz;
      float ddt = 0.0f;
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float xv = cur.x[j].elem(v), bv = PARAMS ? Bc[v] : cur.bq[j].elem(v), cv = PARAMS ? Cc[v] : cur.cq[j].elem(v);
        const float Av = A[v % AV], Dv = Dk[v % AV], av = a[v % AV][j];
        float g0 = cur.gq[j].elem(v);
        if (HAS_Z) {
          const float zz = cur.zq[j].elem(v);
          const float y0 = __builtin_fmaf(st[v][j + 1], cv, Dv * xv);
          oz.v[v] = from_f32<g_t>(g0 * y0 * sg[v][j] * __builtin_fmaf(zz, 1.0f - sg[v][j], 1.0f));
          g0 *= zz * sg[v][j];
        }
        const float lam = __builtin_fmaf(g0, cv, mu[v]);
        const float ld = lam * cur.dt[j];
        ox.v[v] = from_f32<io_t>(__builtin_fmaf(g0, Dv, ld * bv));
        if (PARAMS) {
          accB[v] = __builtin_fmaf(ld, xv, accB[v]);
          accC[v] = __builtin_fmaf(g0, st[v][j + 1], accC[v]);
        } else {
          ob.v[v] = from_f32<g_t>(ld * xv);
          oc.v[v] = from_f32<g_t>(g0 * st[v][j + 1]);
        }
        const float sa = st[v][j] * av;
        ddt = __builtin_fmaf(lam, __builtin_fmaf(sa, Av, bv * xv), ddt);
        accA[v] = __builtin_fmaf(lam * sa, cur.dt[j], accA[v]);
        accD[v] = __builtin_fmaf(g0, xv, accD[v]);
        mu[v] = lam * av;
      }
      const float head = lane_group_sum_last<LPH>(ddt);
      if (t < L) {
        const unsigned at = (unsigned)t * (unsigned)HP + ch;
        *at_bytes<Pack<io_t, VEC>>(dX, at * (unsigned)sizeof(io_t)) = ox;
        if (!PARAMS) *at_bytes<Pack<g_t, VEC>>(dB, at * (unsigned)sizeof(g_t)) = ob;
        if (!PARAMS) *at_bytes<Pack<g_t, VEC>>(dC, at * (unsigned)sizeof(g_t)) = oc;
        if (HAS_Z) *at_bytes<Pack<g_t, VEC>>(dZ, at * (unsigned)sizeof(g_t)) = oz;
        if ((lane & (LPH - 1)) == LPH - 1) *at_bytes<float>(DDT, ((unsigned)t * (unsigned)p.heads + (unsigned)h) * 4u) = head;
      }
    }
  };

  // two sets of registers take turns: one is worked on while the other's reads are in flight
  DboRegs<io_t, VEC, HAS_Z> ra, rb;
  request(ra, rounds - 1);
  for (int r = rounds - 1; r >= 0; r -= 2) {
    if (r > 0) request(rb, r - 1);
    round_of(ra, r);
    if (r > 0) {
      if (r > 1) request(ra, r - 2);
      round_of(rb, r - 1);
    }
  }

  // sums over time of the whole walk: the 16 waves' shares meet in LDS (after everyone has left the last round)
  __syncthreads();
  constexpr int SUMS = PARAMS ? 4 : 2;                          // per channel: A, D (and B, C)
  float *red = reinterpret_cast<float *>(&fwd[0][0][0]);        // [SUMS VEC][16][64] floats
  static_assert(SUMS * VEC * DBO_WAVES * WAVE * sizeof(float) <= sizeof(fwd), "the sums fit the buffers of the folds");
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    const float mine[4] = {accA[v], accD[v], accB[v], accC[v]};
#pragma unroll
    for (int k = 0; k < SUMS; ++k) red[((SUMS * v + k) * DBO_WAVES + wave) * WAVE + lane] = mine[k];
  }
  __syncthreads();
  if (wave < SUMS) {                                             // wave k adds the k-th sum
    float *const out[4] = {p.pA, p.pD, p.pB, p.pC};
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < DBO_WAVES; ++w) sum += red[((SUMS * v + wave) * DBO_WAVES + w) * WAVE + lane];
      out[wave][(size_t)b * HP + ch + v] = sum;
      if (wave == 0 && p.dinit) p.dinit[(size_t)b * HP + ch + v] = mu_left[v];     // lambda_0 a_0
    }
  }
}

// dA and dD per head: the workgroups' per-channel sums added over batch rows and the head's channels, one wave
// per head, in a fixed order.
__global__ __launch_bounds__(WAVE) void dscan_bwd_head_sums_kernel(const float *pA, const float *pD, float *dA, float *dD,
                                                                   int batch, int heads, int proj) {
  const int h = blockIdx.x, lane = lane_id();
  float sa = 0.0f, sd = 0.0f;
  for (int b = 0; b < batch; ++b) {
    for (int pp = lane; pp < proj; pp += WAVE) {
      const size_t at = ((size_t)b * heads + h) * proj + pp;
      sa += pA[at];
      sd += pD[at];
    }
  }
  sa = wave_sum(sa);
  sd = wave_sum(sd);
  if (lane == 0) {
    dA[h] = sa;
    if (dD) dD[h] = sd;
  }
}

template <typename io_t, typename g_t, int VEC, bool HAS_Z, bool PARAMS>
static void launch_dbo_lph(const DscanBwdParams &p, int lph, hipStream_t s) {
  const dim3 grid((unsigned)((size_t)p.heads * p.proj / (WAVE * VEC)), (unsigned)p.batch);
  const dim3 block(WAVE * DBO_WAVES);
  if (lph == 16) hipLaunchKernelGGL((dscan_bwd_onepass_kernel<io_t, g_t, VEC, HAS_Z, 16, PARAMS>), grid, block, 0, s, p);
  else if (lph == 32) hipLaunchKernelGGL((dscan_bwd_onepass_kernel<io_t, g_t, VEC, HAS_Z, 32, PARAMS>), grid, block, 0, s, p);
  else hipLaunchKernelGGL((dscan_bwd_onepass_kernel<io_t, g_t, VEC, HAS_Z, 64, PARAMS>), grid, block, 0, s, p);
}

// The one-pass backward for one element type.  params: B and C are per-channel constants (their gradients and dz
// then are the only ones whose type grads_io chooses, and without a gate none is).
template <typename io_t, int VEC>
static void launch_bwd_onepass(const DscanBwdParams &p, bool grads_io, bool params, hipStream_t s) {
  const int lph = p.proj / VEC;
  if (params) {
    if (!p.z) launch_dbo_lph<io_t, io_t, VEC, false, true>(p, lph, s);
    else if (grads_io) launch_dbo_lph<io_t, io_t, VEC, true, true>(p, lph, s);
    else launch_dbo_lph<io_t, float, VEC, true, true>(p, lph, s);
  } else if (grads_io) {
    if (p.z) launch_dbo_lph<io_t, io_t, VEC, true, false>(p, lph, s);
    else launch_dbo_lph<io_t, io_t, VEC, false, false>(p, lph, s);
  } else {
    if (p.z) launch_dbo_lph<io_t, float, VEC, true, false>(p, lph, s);
    else launch_dbo_lph<io_t, float, VEC, false, false>(p, lph, s);
  }
}

}  // namespace ssm
