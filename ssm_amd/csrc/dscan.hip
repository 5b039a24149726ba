// Diagonal chunked scan: the operator the reference exposes as `ssd_chunk_scan`.
//
//   s_t = exp(dt_t A) s_{t-1} + dt_t B_t X_t        per (batch, head, p) channel
//   y_t = s_t C_t + D X_t ;  y_t *= silu(z_t) ;  y_t = 0 for t >= len(batch)
//
// Tensors are channels-last, (B, L, H, P): consecutive lanes take consecutive
// channels so every time step is one coalesced access.  Time is cut into
// segments that run in parallel:
//   pass 1  every (segment, channel) folds its steps into (decay product, local state)
//   pass 2  every (segment, channel) rebuilds the state entering it from the folds of
//           the segments before it, then replays its steps and emits y
// which costs one extra read of X/dt/B but fills the device even when B*H*P is
// small.  dt is used as given (no bias, no softplus), as in the reference.
#include "common.hpp"

#include <type_traits>

namespace ssm {

constexpr int DS_THREADS = 256;
constexpr int DS_UNROLL = 8;         // time steps whose reads are in flight together

struct DscanParams {
  const void *X, *dt, *Bp, *Cp, *z, *init;
  const float *A, *Dk;
  const int *lengths;           // (B,) valid steps per batch row, or null
  void *Y;
  float *fold;                  // (B, nseg, H*P, 2): decay product, local state
  int batch, len, heads, proj;
  int x_dtype, dt_dtype, bc_dtype, z_dtype, init_dtype;
  int a_stride_p;               // 1 for A (H,P), 0 for A (H,)
  int d_stride_p;               // 1 for D (H,P), 0 for D (H,)
  long long b_stride_b, b_stride_t, c_stride_b, c_stride_t;   // element strides of B / C (0 = broadcast)
  int z_per_p;                  // 1 for z (B,L,H,P), 0 for z (B,L,H)
  int seg_len, nseg;
  float *round_states;          // (B, ceil(L/64), HP): the state entering every 64 steps, or null (one-pass kernel)
};

__device__ __forceinline__ void ds_store(void *p, int dtype, size_t i, float v) {
  if (dtype == SSM_F32) reinterpret_cast<float *>(p)[i] = v;
  else if (dtype == SSM_BF16) reinterpret_cast<bf16_t *>(p)[i] = from_f32<bf16_t>(v);
  else reinterpret_cast<f16_t *>(p)[i] = from_f32<f16_t>(v);
}

// Loads of the streamed tensors.  io_t = void: the element type is looked up at run time (any mix of
// dtypes); otherwise X, B, C, z and Y all have type io_t and dt is float32, and the loads of a group of
// steps are straight-line code that the compiler can issue together.
template <typename io_t>
__device__ __forceinline__ float ds_load(const void *p, int dtype, size_t i) {
  if constexpr (std::is_void<io_t>::value) return load_as_f32(p, dtype, i);
  else return to_f32(reinterpret_cast<const io_t *>(p)[i]);
}
template <typename io_t>
__device__ __forceinline__ float ds_load_dt(const void *p, int dtype, size_t i) {
  if constexpr (std::is_void<io_t>::value) return load_as_f32(p, dtype, i);
  else return reinterpret_cast<const float *>(p)[i];
}
template <typename io_t>
__device__ __forceinline__ void ds_store_y(void *p, int dtype, size_t i, float v) {
  if constexpr (std::is_void<io_t>::value) ds_store(p, dtype, i, v);
  else reinterpret_cast<io_t *>(p)[i] = from_f32<io_t>(v);
}

template <int PASS, typename io_t>
__global__ __launch_bounds__(DS_THREADS) void dscan_kernel(const DscanParams p) {
  const int HP = p.heads * p.proj;
  const int hp = blockIdx.x * DS_THREADS + threadIdx.x;
  if (hp >= HP) return;
  const int seg = blockIdx.y, b = blockIdx.z;
  const int h = hp / p.proj, pp = hp % p.proj;
  const int valid = p.lengths ? min(max(p.lengths[b], 0), p.len) : p.len;
  const int t_begin = seg * p.seg_len;
  const int t_end = min(p.len, t_begin + p.seg_len);
  const float A2 = p.A[(size_t)h * (p.a_stride_p ? p.proj : 1) + (p.a_stride_p ? pp : 0)] * LOG2E;
  const size_t x_row = (size_t)b * p.len;            // + t, then * HP + hp
  const size_t fold_at = (((size_t)b * p.nseg + seg) * HP + hp) * 2;

  // Time is walked DS_UNROLL steps at a time with all of a group's reads requested before the first is
  // used: one step per trip leaves a wave waiting for memory at every step.
  if (PASS == 1) {
    float prod = 1.0f, s = 0.0f;
    const int stop = min(t_end, valid);
    for (int t0 = t_begin; t0 < stop; t0 += DS_UNROLL) {
      float dtv[DS_UNROLL], xv[DS_UNROLL], bv[DS_UNROLL];
#pragma unroll
      for (int j = 0; j < DS_UNROLL; ++j) {
        const int t = min(t0 + j, stop - 1);
        dtv[j] = ds_load_dt<io_t>(p.dt, p.dt_dtype, (x_row + t) * p.heads + h);
        xv[j] = ds_load<io_t>(p.X, p.x_dtype, (x_row + t) * HP + hp);
        bv[j] = ds_load<io_t>(p.Bp, p.bc_dtype, (size_t)(b * p.b_stride_b + t * p.b_stride_t) + hp);
      }
#pragma unroll
      for (int j = 0; j < DS_UNROLL; ++j) {
        if (t0 + j < stop) {
          const float a = exp2_hw(dtv[j] * A2);
          s = __builtin_fmaf(a, s, dtv[j] * bv[j] * xv[j]);
          prod *= a;
        }
      }
    }
    p.fold[fold_at] = prod;
    p.fold[fold_at + 1] = s;
    return;
  }

  // PASS 2: state entering this segment
  float s = p.init ? load_as_f32(p.init, p.init_dtype, (size_t)b * HP + hp) : 0.0f;
  for (int j = 0; j < seg; ++j) {
    const size_t f = (((size_t)b * p.nseg + j) * HP + hp) * 2;
    s = __builtin_fmaf(p.fold[f], s, p.fold[f + 1]);
  }
  const float Dk = p.Dk ? p.Dk[(size_t)h * (p.d_stride_p ? p.proj : 1) + (p.d_stride_p ? pp : 0)] : 0.0f;
  for (int t0 = t_begin; t0 < t_end; t0 += DS_UNROLL) {
    float dtv[DS_UNROLL], xv[DS_UNROLL], bv[DS_UNROLL], cv[DS_UNROLL], zv[DS_UNROLL];
#pragma unroll
    for (int j = 0; j < DS_UNROLL; ++j) {
      const int t = min(t0 + j, t_end - 1);
      const size_t xi = (x_row + t) * HP + hp;
      dtv[j] = ds_load_dt<io_t>(p.dt, p.dt_dtype, (x_row + t) * p.heads + h);
      xv[j] = ds_load<io_t>(p.X, p.x_dtype, xi);
      bv[j] = ds_load<io_t>(p.Bp, p.bc_dtype, (size_t)(b * p.b_stride_b + t * p.b_stride_t) + hp);
      cv[j] = ds_load<io_t>(p.Cp, p.bc_dtype, (size_t)(b * p.c_stride_b + t * p.c_stride_t) + hp);
      {
        // an absent gate reads X in its place (value dropped): no branch around the read
        const float zraw = ds_load<io_t>(p.z ? p.z : p.X, p.z ? p.z_dtype : p.x_dtype, (p.z && !p.z_per_p) ? (x_row + t) * p.heads + h : xi);
        zv[j] = p.z ? zraw : 0.0f;
      }
    }
#pragma unroll
    for (int j = 0; j < DS_UNROLL; ++j) {
      const int t = t0 + j;
      if (t < t_end) {
        float y = 0.0f;
        if (t < valid) {
          s = __builtin_fmaf(exp2_hw(dtv[j] * A2), s, dtv[j] * bv[j] * xv[j]);
          y = __builtin_fmaf(s, cv[j], Dk * xv[j]);
          if (p.z) y *= silu_f32(zv[j]);
        }
        ds_store_y<io_t>(p.Y, p.x_dtype, (x_row + t) * HP + hp, y);
      }
    }
  }
}

// ---------------------------------------------------------------- one pass
// The common call (per-token B and C of X's shape and type, per-head A and D, gate of X's shape or none) with
// every input read once.  A workgroup of 16 waves owns 64 * VEC neighbouring channels of one batch row (a
// lane VEC of them, so that a wave's access is 128 * VEC bytes of 16-bit elements) and walks time in rounds of
// 128 steps, wave w taking steps 8w..8w+7 of the round: it folds its steps from zero into (decay product, state),
// the 16 folds meet in LDS (one barrier per round, two buffers), wave w chains the folds of the waves before it
// from the state entering the round -- which gives it the state entering its own steps -- and replays its steps
// from the values it still holds in registers.  The last wave's chain ends at the round's right edge: it leaves
// the state there in LDS for everyone's next round.  The reads of the next round are requested before the
// arithmetic of this one.  A workgroup fills a CU's registers (one per CU), so the call is as fast as one
// workgroup's instruction stream: addresses are a uniform base plus a 32-bit offset per lane, steps past a row's
// length are masked only in the rounds that contain any, and two sets of registers take turns without copies.
constexpr int DO_WAVES = 16, DO_SEG = 8, DO_ROUND = DO_WAVES * DO_SEG;

template <typename io_t, int VEC>
struct DoRegs {
  float dt[DO_SEG];
  Word<io_t> x[DO_SEG], bq[DO_SEG], cq[DO_SEG], zq[DO_SEG];
};

// STATES_ONLY: the walk without C, the gate and the output -- only the table of round states is written (the
// backward's own forward sweep when it is called without one).
// PARAMS: the call of the reference's own Mamba2 module (src/ssm/modules/mamba2.py:189-199): B and C are
// parameters, one value per channel ((H,P), or (B,H,P)), kept in registers instead of streamed, and A and D may be
// per channel, so every channel of a lane has its own decay (one per lane otherwise).
template <typename io_t, int VEC, bool HAS_Z, bool STATES_ONLY, bool PARAMS>
__global__ __launch_bounds__(WAVE *DO_WAVES) void dscan_onepass_kernel(const DscanParams p) {
  static_assert(sizeof(io_t) * VEC == 4, "a lane's vector is one register");
  constexpr int AV = PARAMS ? VEC : 1;            // decays per lane
  __shared__ float4 segs[2][DO_WAVES][WAVE];     // a wave's fold per lane: decay product(s), states from zero
  __shared__ float2 right[2][WAVE];
  const int wave = wave_id_uniform(), lane = lane_id();
  const int HP = p.heads * p.proj;
  const unsigned ch = ((unsigned)blockIdx.x * WAVE + lane) * VEC;
  const int b = blockIdx.y;
  const int h = (int)ch / p.proj;
  const int L = p.len;
  const int valid = p.lengths ? min(max(p.lengths[b], 0), L) : L;
  float A2[AV], Dk[AV], Bc[VEC], Cc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    if (v < AV) {     // per channel (index h*P + p = ch + v) or per head
      A2[v] = p.A[p.a_stride_p ? (size_t)ch + v : (size_t)h] * LOG2E;
      Dk[v] = p.Dk ? p.Dk[p.d_stride_p ? (size_t)ch + v : (size_t)h] : 0.0f;
    }
    // constant projections: element strides b_stride_b / c_stride_b are 0 for (H,P) and H*P for (B,H,P)
    Bc[v] = PARAMS ? load_as_f32(p.Bp, p.bc_dtype, (size_t)b * p.b_stride_b + ch + v) : 0.0f;
    Cc[v] = PARAMS ? load_as_f32(p.Cp, p.bc_dtype, (size_t)b * p.c_stride_b + ch + v) : 0.0f;
  }
  // the batch row's part of every tensor: offsets inside it fit 32 bits (checked by the host)
  const size_t row0 = (size_t)b * L;
  const io_t *X = reinterpret_cast<const io_t *>(p.X) + row0 * HP;
  const io_t *Bp = reinterpret_cast<const io_t *>(PARAMS ? p.X : p.Bp) + row0 * HP, *Cp = reinterpret_cast<const io_t *>(PARAMS ? p.X : p.Cp) + row0 * HP;
  const io_t *Z = reinterpret_cast<const io_t *>(HAS_Z ? p.z : p.X) + row0 * HP;
  const float *DT = reinterpret_cast<const float *>(p.dt) + row0 * p.heads;
  io_t *Y = reinterpret_cast<io_t *>(p.Y) + row0 * HP;

  auto request = [&](DoRegs<io_t, VEC> &r, int round) {
    const int t0 = round * DO_ROUND + wave * DO_SEG;
#pragma unroll
    for (int j = 0; j < DO_SEG; ++j) {
      const unsigned row = (unsigned)min(t0 + j, L - 1);       // steps past the end read the last row, unused
      const unsigned at = (row * (unsigned)HP + ch) * (unsigned)sizeof(io_t);
      r.dt[j] = *at_bytes<const float>(DT, (row * (unsigned)p.heads + (unsigned)h) * 4u);
      r.x[j] = Word<io_t>{*at_bytes<const unsigned>(X, at)};
      if (!PARAMS) r.bq[j] = Word<io_t>{*at_bytes<const unsigned>(Bp, at)};
      if (!STATES_ONLY && !PARAMS) r.cq[j] = Word<io_t>{*at_bytes<const unsigned>(Cp, at)};
      if (HAS_Z && !STATES_ONLY) r.zq[j] = Word<io_t>{*at_bytes<const unsigned>(Z, at)};
    }
  };

  const int rounds = (L + DO_ROUND - 1) / DO_ROUND;
  auto round_of = [&](DoRegs<io_t, VEC> &cur, int r) {
    const int q = r & 1;
    const int t0 = r * DO_ROUND + wave * DO_SEG;
    if (t0 + DO_SEG > valid) {
      // the row ends inside these steps (uniform, rare): a dead step reads as zero everywhere -- the identity,
      // nothing added, a zero output
#pragma unroll
      for (int j = 0; j < DO_SEG; ++j) {
        const bool live = t0 + j < valid;
        cur.dt[j] = live ? cur.dt[j] : 0.0f;
        cur.x[j].mask(live);
        if (!PARAMS) cur.bq[j].mask(live);
        if (!STATES_ONLY && !PARAMS) cur.cq[j].mask(live);
      }
    }
    float a[AV][DO_SEG], s[VEC], prod[AV];
#pragma unroll
    for (int v = 0; v < VEC; ++v) s[v] = 0.0f;
#pragma unroll
    for (int v = 0; v < AV; ++v) prod[v] = 1.0f;
#pragma unroll
    for (int j = 0; j < DO_SEG; ++j) {
#pragma unroll
      for (int v = 0; v < AV; ++v) {
        a[v][j] = exp2_hw(cur.dt[j] * A2[v]);
        prod[v] *= a[v][j];
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        s[v] = __builtin_fmaf(a[v % AV][j], s[v], cur.dt[j] * (PARAMS ? Bc[v] : cur.bq[j].elem(v)) * cur.x[j].elem(v));
    }
    // (one decay per lane: three words to read per link; two: four)
    segs[q][wave][lane] = AV == 1 ? make_float4(prod[0], s[0], s[VEC - 1], 0.0f) : make_float4(prod[0], prod[AV - 1], s[0], s[VEC - 1]);
    __syncthreads();
    // the state entering this wave's steps: the folds of the waves before it, from the state entering the round
    float enter[VEC];
    if (r == 0) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) enter[v] = p.init ? load_as_f32(p.init, p.init_dtype, (size_t)b * HP + ch + v) : 0.0f;
    } else {
      const float2 c = right[q ^ 1][lane];
      enter[0] = c.x;
      enter[VEC - 1] = c.y;
    }
    for (int w = 0; w < wave; ++w) {
      const float4 f = segs[q][w][lane];
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        enter[v] = AV == 1 ? __builtin_fmaf(f.x, enter[v], v == 0 ? f.y : f.z) : __builtin_fmaf(v == 0 ? f.x : f.y, enter[v], v == 0 ? f.z : f.w);
    }
    if (wave == DO_WAVES - 1) {
      float leave[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) leave[v] = __builtin_fmaf(prod[v % AV], enter[v], s[v]);
      right[q][lane] = make_float2(leave[0], leave[VEC - 1]);
    }
    if (p.round_states && (wave & (DO_WAVES / 2 - 1)) == 0) {
      // what the backward starts its rounds of 64 steps from: the states entering wave 0's and wave 8's steps
      const int rounds64 = (L + DO_ROUND / 2 - 1) / (DO_ROUND / 2);
      const int k = 2 * r + wave / (DO_WAVES / 2);
      if (k < rounds64) {
        float *table = p.round_states + ((size_t)b * rounds64 + k) * HP + ch;
#pragma unroll
        for (int v = 0; v < VEC; ++v) table[v] = enter[v];
      }
    }
    if (STATES_ONLY) return;
#pragma unroll
    for (int j = 0; j < DO_SEG; ++j) {
      const int t = t0 + j;
      // the float32 values of a step's elements are formed here, step by step, not kept from the fold above
      // and not all in front of the first step
      cur.x[j].launder_after(enter[0]);
      if (!PARAMS) cur.bq[j].launder_after(enter[0]);
      if (!PARAMS) cur.cq[j].launder_after(enter[0]);
      if (HAS_Z) cur.zq[j].launder_after(enter[0]);
      Pack<io_t, VEC> o;
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float xv = cur.x[j].elem(v);
        enter[v] = __builtin_fmaf(a[v % AV][j], enter[v], cur.dt[j] * (PARAMS ? Bc[v] : cur.bq[j].elem(v)) * xv);
        float y = __builtin_fmaf(enter[v], PARAMS ? Cc[v] : cur.cq[j].elem(v), Dk[v % AV] * xv);
        if (HAS_Z) y *= silu_f32(cur.zq[j].elem(v));
        if (PARAMS && t >= valid) y = 0.0f;      // nothing streamed carries the zero of a dead step here
        o.v[v] = from_f32<io_t>(y);
      }
      if (t < L) *at_bytes<Pack<io_t, VEC>>(Y, ((unsigned)t * (unsigned)HP + ch) * (unsigned)sizeof(io_t)) = o;
    }
  };

  // two sets of registers take turns: one is worked on while the other's reads are in flight
  DoRegs<io_t, VEC> ra, rb;
  request(ra, 0);
  for (int r = 0; r < rounds; r += 2) {
    if (r + 1 < rounds) request(rb, r + 1);
    round_of(ra, r);
    if (r + 1 < rounds) {
      if (r + 2 < rounds) request(ra, r + 2);
      round_of(rb, r + 1);
    }
  }
}

template <typename io_t, int VEC>
static void launch_onepass(const DscanParams &p, bool params, hipStream_t s) {
  const dim3 grid((unsigned)((size_t)p.heads * p.proj / (WAVE * VEC)), (unsigned)p.batch);
  const dim3 block(WAVE * DO_WAVES);
  if (params) {
    if (p.z) hipLaunchKernelGGL((dscan_onepass_kernel<io_t, VEC, true, false, true>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((dscan_onepass_kernel<io_t, VEC, false, false, true>), grid, block, 0, s, p);
  } else {
    if (p.z) hipLaunchKernelGGL((dscan_onepass_kernel<io_t, VEC, true, false, false>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((dscan_onepass_kernel<io_t, VEC, false, false, false>), grid, block, 0, s, p);
  }
}

// The table of round states alone, for a call shape the one-pass kernels cover (the caller has checked).
// b_const: B is one value per channel, (H,P) (b_stride_b 0) or (B,H,P) (b_stride_b H*P), of type bc_dtype.
void launch_dscan_round_states(const void *X, const void *dt, const void *Bproj, const float *A, const void *init,
                               int init_dtype, const int *lengths, float *round_states, int batch, int len, int heads,
                               int proj, int x_dtype, bool b_const, int bc_dtype, long long b_stride_b, bool a_per_p,
                               hipStream_t s) {
  DscanParams p{};
  p.X = X; p.dt = dt; p.Bp = Bproj; p.Cp = Bproj; p.A = A; p.init = init; p.init_dtype = init_dtype;
  p.lengths = lengths; p.round_states = round_states;
  p.batch = batch; p.len = len; p.heads = heads; p.proj = proj;
  p.bc_dtype = bc_dtype; p.b_stride_b = p.c_stride_b = b_stride_b; p.a_stride_p = a_per_p ? 1 : 0;
  const int vec = x_dtype == SSM_F32 ? 1 : 2;
  const dim3 grid((unsigned)((size_t)heads * proj / (WAVE * vec)), (unsigned)batch), block(WAVE * DO_WAVES);
#define SSM_STATES(T, V)                                                                                    \
  {                                                                                                         \
    if (b_const) hipLaunchKernelGGL((dscan_onepass_kernel<T, V, false, true, true>), grid, block, 0, s, p); \
    else hipLaunchKernelGGL((dscan_onepass_kernel<T, V, false, true, false>), grid, block, 0, s, p);        \
  }
  if (x_dtype == SSM_BF16) SSM_STATES(bf16_t, 2)
  else if (x_dtype == SSM_F16) SSM_STATES(f16_t, 2)
  else SSM_STATES(float, 1)
#undef SSM_STATES
}

int dscan_segments(int batch, int len, int hp) {
  // enough (segment, channel-block) workgroups to cover ~4 per CU, segments of >= 32 steps
  const int blocks = (hp + DS_THREADS - 1) / DS_THREADS;
  int want = (1024 + batch * blocks - 1) / (batch * blocks);
  const int max_seg = (len + 31) / 32;
  if (want > max_seg) want = max_seg;
  if (want < 1) want = 1;
  return want;
}

}  // namespace ssm

extern "C" size_t ssm_dscan_fwd_workspace_bytes(int batch, int seqlen, int heads, int proj) {
  if (batch <= 0 || seqlen <= 0 || heads <= 0 || proj <= 0) return 0;
  const int nseg = ssm::dscan_segments(batch, seqlen, heads * proj);
  return (size_t)batch * nseg * heads * proj * 2 * sizeof(float);
}

// One pass: float32 dt, a gate of X's shape and type or none, channels in whole waves, vectors aligned, and either
// per-token B and C of X's type with per-head A and D (*params = false), or B and C one value per channel -- (H,P)
// or (B,H,P), any type -- with A and D per head or per channel (*params = true).
static bool dscan_fwd_takes_one_pass(const ssm_dscan_fwd_args *a, bool *params = nullptr) {
  using namespace ssm;
  if (!valid_dtype(a->x_dtype) || !valid_dtype(a->bc_dtype)) return false;
  const long long HP = (long long)a->heads * a->proj;
  const int vec = a->x_dtype == SSM_F32 ? 1 : 2;
  const size_t bytes = (size_t)vec * dtype_size(a->x_dtype);
  const bool streamed = a->b_kind == SSM_CHUNK_BLHP && a->c_kind == SSM_CHUNK_BLHP && a->bc_dtype == a->x_dtype &&
                        !a->a_per_p && !a->d_per_p && aligned_to(a->Bproj, bytes) && aligned_to(a->Cproj, bytes);
  auto per_channel = [](int kind) { return kind == SSM_CHUNK_HP || kind == SSM_CHUNK_BHP; };
  const bool constant = per_channel(a->b_kind) && per_channel(a->c_kind) &&
                        aligned_to(a->Bproj, dtype_size(a->bc_dtype)) && aligned_to(a->Cproj, dtype_size(a->bc_dtype));
  if (params) *params = constant;
  return (streamed || constant) && a->dt_dtype == SSM_F32 && (!a->z || (a->z_dtype == a->x_dtype && a->z_per_p)) &&
         HP % (WAVE * vec) == 0 && a->proj % vec == 0 && (long long)a->seqlen * HP < (1ll << 30) &&
         aligned_to(a->X, bytes) && aligned_to(a->Y, bytes) && (!a->z || aligned_to(a->z, bytes)) && a->batch < 65536;
}

extern "C" int ssm_dscan_fwd_one_pass(const ssm_dscan_fwd_args *a) {
  return a != nullptr && a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->proj > 0 && dscan_fwd_takes_one_pass(a);
}

extern "C" int ssm_dscan_fwd(const ssm_dscan_fwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_dscan_fwd: args is NULL");
  SSM_REQUIRE(a->X && a->dt && a->A && a->Bproj && a->Cproj && a->Y, SSM_ERR_NULL_POINTER,
              "ssm_dscan_fwd: X, dt, A, Bproj, Cproj and Y are required");
  SSM_REQUIRE(a->batch > 0 && a->seqlen > 0 && a->heads > 0 && a->proj > 0, SSM_ERR_BAD_SHAPE,
              "ssm_dscan_fwd: batch=%d seqlen=%d heads=%d proj=%d must all be positive", a->batch, a->seqlen,
              a->heads, a->proj);
  SSM_REQUIRE(valid_dtype(a->x_dtype) && valid_dtype(a->dt_dtype) && valid_dtype(a->bc_dtype) &&
                  (!a->z || valid_dtype(a->z_dtype)) && (!a->initial_states || valid_dtype(a->init_dtype)),
              SSM_ERR_BAD_DTYPE, "ssm_dscan_fwd: unsupported dtype");
  SSM_REQUIRE(a->batch < 65536, SSM_ERR_TOO_LARGE, "ssm_dscan_fwd: batch too large");
  SSM_REQUIRE((size_t)a->batch * a->seqlen * a->heads * a->proj < ((size_t)1 << 40), SSM_ERR_TOO_LARGE,
              "ssm_dscan_fwd: tensor too large");
  auto kind_ok = [](int k) { return k == SSM_CHUNK_HP || k == SSM_CHUNK_BHP || k == SSM_CHUNK_BLHP; };
  SSM_REQUIRE(kind_ok(a->b_kind) && kind_ok(a->c_kind), SSM_ERR_BAD_KIND, "ssm_dscan_fwd: b_kind=%d c_kind=%d",
              a->b_kind, a->c_kind);
  const size_t need = ssm_dscan_fwd_workspace_bytes(a->batch, a->seqlen, a->heads, a->proj);
  SSM_REQUIRE(a->workspace && a->workspace_bytes >= need, SSM_ERR_WORKSPACE,
              "ssm_dscan_fwd: workspace of %zu bytes required", need);

  DscanParams p{};
  p.X = a->X; p.dt = a->dt; p.Bp = a->Bproj; p.Cp = a->Cproj; p.z = a->z; p.init = a->initial_states;
  p.A = a->A; p.Dk = a->Dskip; p.lengths = a->seq_lens; p.Y = a->Y;
  p.fold = reinterpret_cast<float *>(a->workspace);
  p.batch = a->batch; p.len = a->seqlen; p.heads = a->heads; p.proj = a->proj;
  p.x_dtype = a->x_dtype; p.dt_dtype = a->dt_dtype; p.bc_dtype = a->bc_dtype; p.z_dtype = a->z_dtype;
  p.init_dtype = a->init_dtype;
  p.a_stride_p = a->a_per_p ? 1 : 0;
  p.d_stride_p = a->d_per_p ? 1 : 0;
  const long long HP = (long long)a->heads * a->proj;
  auto strides = [&](int kind, long long &sb, long long &st) {
    sb = kind == SSM_CHUNK_HP ? 0 : (kind == SSM_CHUNK_BHP ? HP : HP * a->seqlen);
    st = kind == SSM_CHUNK_BLHP ? HP : 0;
  };
  strides(a->b_kind, p.b_stride_b, p.b_stride_t);
  strides(a->c_kind, p.c_stride_b, p.c_stride_t);
  p.z_per_p = a->z_per_p ? 1 : 0;
  p.nseg = dscan_segments(a->batch, a->seqlen, (int)HP);
  p.seg_len = (a->seqlen + p.nseg - 1) / p.nseg;
  p.nseg = (a->seqlen + p.seg_len - 1) / p.seg_len;

  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  const dim3 grid((unsigned)((HP + DS_THREADS - 1) / DS_THREADS), (unsigned)p.nseg, (unsigned)a->batch);
  const bool typed = a->dt_dtype == SSM_F32 && a->bc_dtype == a->x_dtype && (!a->z || a->z_dtype == a->x_dtype);
  bool params = false;
  const bool one_pass = dscan_fwd_takes_one_pass(a, &params);
  SSM_REQUIRE(!a->round_states || (one_pass && aligned_to(a->round_states, 4)), SSM_ERR_BAD_SHAPE,
              "ssm_dscan_fwd: round_states is only written by the one-pass kernel (ask ssm_dscan_fwd_one_pass first)");
  if (one_pass) {
    p.round_states = a->round_states;
    if (a->x_dtype == SSM_BF16) launch_onepass<bf16_t, 2>(p, params, s);
    else if (a->x_dtype == SSM_F16) launch_onepass<f16_t, 2>(p, params, s);
    else launch_onepass<float, 1>(p, params, s);
    SSM_CHECK_LAUNCH("ssm_dscan_fwd");
    return SSM_OK;
  }
#define SSM_DS_LAUNCH(T)                                                                   \
  {                                                                                        \
    if (p.nseg > 1) hipLaunchKernelGGL((dscan_kernel<1, T>), grid, dim3(DS_THREADS), 0, s, p); \
    hipLaunchKernelGGL((dscan_kernel<2, T>), grid, dim3(DS_THREADS), 0, s, p);             \
  }
  if (typed && a->x_dtype == SSM_BF16) SSM_DS_LAUNCH(bf16_t)
  else if (typed && a->x_dtype == SSM_F16) SSM_DS_LAUNCH(f16_t)
  else if (typed && a->x_dtype == SSM_F32) SSM_DS_LAUNCH(float)
  else SSM_DS_LAUNCH(void)
#undef SSM_DS_LAUNCH
  SSM_CHECK_LAUNCH("ssm_dscan_fwd");
  return SSM_OK;
}
