// Shared device/host helpers for the gfx950 kernels: dtype conversion, vector
// loads, fp32 transcendental helpers, wave64 DPP scans, error reporting.
#pragma once
#include <type_traits>

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/ssm_amd.h"

namespace ssm {

// ---------------------------------------------------------------- host side

void set_error(const char *fmt, ...);   // defined in status.hip

#define SSM_REQUIRE(cond, code, ...)        \
  do {                                      \
    if (!(cond)) {                          \
      ::ssm::set_error(__VA_ARGS__);        \
      return (code);                        \
    }                                       \
  } while (0)

#define SSM_CHECK_LAUNCH(what)                                                  \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess) {                                                     \
      ::ssm::set_error("%s: %s", (what), hipGetErrorString(e_));                \
      return SSM_ERR_LAUNCH;                                                    \
    }                                                                           \
  } while (0)

// Kernel-route selectors travel in the argument structs' `reserved` fields and exist only in a build with
// -DSSM_TEST_HOOKS (include/ssm_amd_testing.h): the shipped library picks kernels by shape and dtype alone and
// rejects a non-zero value.
#ifdef SSM_TEST_HOOKS
#define SSM_RESERVED(a) ((a)->reserved)
#define SSM_CHECK_RESERVED(who, a) do { } while (0)
#else
#define SSM_RESERVED(a) 0
#define SSM_CHECK_RESERVED(who, a) \
  SSM_REQUIRE((a)->reserved == 0, SSM_ERR_BAD_KIND, "%s: reserved must be 0 (kernel selectors need a -DSSM_TEST_HOOKS build)", who)
#endif

inline bool aligned_to(const void *p, size_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; }
inline bool valid_dtype(int d) { return d == SSM_F32 || d == SSM_BF16 || d == SSM_F16; }
inline int dtype_size(int d) { return d == SSM_F32 ? 4 : 2; }

// Raise the dynamic-LDS ceiling of a kernel once (needed above 64 KiB).
template <typename KernelT>
inline hipError_t allow_dynamic_lds(KernelT kernel, size_t bytes) {
  if (bytes <= 48 * 1024) return hipSuccess;
  return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

// Deterministic sums of per-block partials (defined in scan_bwd.hip):
//   rows: out[i]    = sum_{j < count} in[j * inner + i]
//   sum:  out[o][i] = sum_{j < count} in[(o * count + j) * inner + i]
void launch_fold_rows(const float *in, float *out, int count, size_t inner, hipStream_t s);
void launch_fold_sum(const float *in, float *out, size_t outer, int count, size_t inner, hipStream_t s);

// -------------------------------------------------------------- device side

constexpr int WAVE = 64;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }
__device__ __forceinline__ float to_f32(f16_t v) { return (float)v.v; }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t x = __float_as_uint(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);  // quiet NaN
  x += 0x7fffu + ((x >> 16) & 1u);                                              // round to nearest even
  return (uint16_t)(x >> 16);
}

template <typename T> __device__ __forceinline__ T from_f32(float f);
template <> __device__ __forceinline__ float from_f32<float>(float f) { return f; }
// gfx950 converts with round-to-nearest-even in hardware (v_cvt_pk_bf16_f32)
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float f) {
  const __bf16 h = (__bf16)f;
  return bf16_t{__builtin_bit_cast(uint16_t, h)};
}
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float f) { return f16_t{(_Float16)f}; }

// Read element i of a buffer whose dtype is only known at run time (uniform branch).
__device__ __forceinline__ float load_as_f32(const void *p, int dtype, size_t i) {
  if (dtype == SSM_F32) return reinterpret_cast<const float *>(p)[i];
  if (dtype == SSM_BF16) return to_f32(reinterpret_cast<const bf16_t *>(p)[i]);
  return to_f32(reinterpret_cast<const f16_t *>(p)[i]);
}

// A run of K consecutive elements owned by one lane, moved with the widest
// aligned vector access available (16 bytes), or element-wise with bounds.
template <typename T, int K>
struct alignas(sizeof(T) * K >= 16 ? 16 : sizeof(T) * K) Pack { T v[K]; };

template <typename T, int K>
__device__ __forceinline__ void load_run(const T *base, int t, int len, bool vec_ok, float (&out)[K]) {
  constexpr int PIECE = (sizeof(T) * K >= 16) ? (16 / sizeof(T)) : K;   // elements per vector access
  if (vec_ok && t + K <= len) {
#pragma unroll
    for (int j = 0; j < K / PIECE; ++j) {
      Pack<T, PIECE> p = *reinterpret_cast<const Pack<T, PIECE> *>(base + t + j * PIECE);
#pragma unroll
      for (int i = 0; i < PIECE; ++i) out[j * PIECE + i] = to_f32(p.v[i]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < K; ++i) out[i] = (t + i < len) ? to_f32(base[t + i]) : 0.0f;
  }
}

template <typename T, int K>
__device__ __forceinline__ void store_run(T *base, int t, int len, bool vec_ok, const float (&in)[K]) {
  constexpr int PIECE = (sizeof(T) * K >= 16) ? (16 / sizeof(T)) : K;
  if (vec_ok && t + K <= len) {
#pragma unroll
    for (int j = 0; j < K / PIECE; ++j) {
      Pack<T, PIECE> p;
#pragma unroll
      for (int i = 0; i < PIECE; ++i) p.v[i] = from_f32<T>(in[j * PIECE + i]);
      *reinterpret_cast<Pack<T, PIECE> *>(base + t + j * PIECE) = p;
    }
  } else {
#pragma unroll
    for (int i = 0; i < K; ++i)
      if (t + i < len) base[t + i] = from_f32<T>(in[i]);
  }
}

// 2^x on the transcendental unit (v_exp_f32, 1 ulp; results below 2^-126 flush to 0).
__device__ __forceinline__ float exp2_hw(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float log2_hw(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float rcp_hw(float x) { return __builtin_amdgcn_rcpf(x); }

// e^x as 2^(x log2 e): the rounding of the product costs |x| * 6e-8 of relative
// accuracy, negligible for the |x| < 20 these kernels feed it.
__device__ __forceinline__ float exp_f32(float x) { return exp2_hw(x * LOG2E); }

// torch.nn.functional.softplus with its default threshold of 20, branch-free.
// log(1 + e) = log(w) + (e - (w - 1)) / w with w = fl(1 + e): the second term
// restores what the rounding of 1 + e lost, so small results keep full relative
// accuracy (softplus of a very negative number is e itself).
// Above w = 2 the restored term is below half an ulp of the result and is dropped;
// below it, dividing it by w (< 2) would change the result by less than 4e-8 relative.
__device__ __forceinline__ float softplus_f32(float x) {
  const float e = exp_f32(x);
  const float w = 1.0f + e;
  const float lost = w < 2.0f ? e - (w - 1.0f) : 0.0f;
  const float r = __builtin_fmaf(log2_hw(w), LN2, lost);
  return x > 20.0f ? x : r;
}

__device__ __forceinline__ float sigmoid_f32(float x) { return rcp_hw(1.0f + exp_f32(-x)); }
__device__ __forceinline__ float silu_f32(float x) { return x * sigmoid_f32(x); }

// ---- wave64 cross-lane helpers (DPP; rows are 16 lanes) --------------------

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float keep, float src) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(keep), __float_as_int(src), CTRL,
                                                    ROW_MASK, 0xf, false));
}

constexpr int DPP_ROW_SHR1 = 0x111, DPP_ROW_SHR2 = 0x112, DPP_ROW_SHR4 = 0x114, DPP_ROW_SHR8 = 0x118;
constexpr int DPP_ROW_BCAST15 = 0x142, DPP_ROW_BCAST31 = 0x143, DPP_WAVE_SHR1 = 0x138;
constexpr int DPP_ROW_SHL1 = 0x101, DPP_ROW_SHL2 = 0x102, DPP_ROW_SHL4 = 0x104, DPP_ROW_SHL8 = 0x108;
constexpr int DPP_WAVE_SHL1 = 0x130;

// Sum over each group of LPH neighbouring lanes (16, 32 or 64), valid in the group's last lane.
template <int LPH>
__device__ __forceinline__ float lane_group_sum_last(float v) {
  v += dpp_move<DPP_ROW_SHR1, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR2, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR4, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR8, 0xf>(0.0f, v);
  if (LPH >= 32) v += dpp_move<DPP_ROW_BCAST15, 0xa>(0.0f, v);
  if (LPH >= 64) v += dpp_move<DPP_ROW_BCAST31, 0xc>(0.0f, v);
  return v;
}

// Sum over each run of N neighbouring lanes (8 or 16, aligned), valid in the run's last lane.
template <int N>
__device__ __forceinline__ float lane_run_sum_last(float v) {
  static_assert(N == 8 || N == 16, "runs inside a row of 16 lanes");
  v += dpp_move<DPP_ROW_SHR1, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR2, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR4, 0xf>(0.0f, v);
  if (N == 16) v += dpp_move<DPP_ROW_SHR8, 0xf>(0.0f, v);
  return v;
}

// Inclusive scan across the 64 lanes of the pair (a, b) under
//   (a1, b1) then (a2, b2)  ->  (a1 a2, a2 b1 + b2)
// i.e. the composition of the affine maps h -> a h + b, earlier lanes first.
__device__ __forceinline__ void wave_scan_affine(float &a, float &b) {
#define SSM_SCAN_STEP(CTRL, RM)                      \
  {                                                  \
    const float ap = dpp_move<CTRL, RM>(1.0f, a);    \
    const float bp = dpp_move<CTRL, RM>(0.0f, b);    \
    b = __builtin_fmaf(a, bp, b);                    \
    a = a * ap;                                      \
  }
  SSM_SCAN_STEP(DPP_ROW_SHR1, 0xf)
  SSM_SCAN_STEP(DPP_ROW_SHR2, 0xf)
  SSM_SCAN_STEP(DPP_ROW_SHR4, 0xf)
  SSM_SCAN_STEP(DPP_ROW_SHR8, 0xf)
  SSM_SCAN_STEP(DPP_ROW_BCAST15, 0xa)
  SSM_SCAN_STEP(DPP_ROW_BCAST31, 0xc)
#undef SSM_SCAN_STEP
}

// Value of the previous lane (lane 0 receives `first`).
__device__ __forceinline__ float wave_prev(float v, float first) {
  return dpp_move<DPP_WAVE_SHR1, 0xf>(first, v);
}
// Value of the next lane (lane 63 receives `last`).
__device__ __forceinline__ float wave_next(float v, float last) {
  return dpp_move<DPP_WAVE_SHL1, 0xf>(last, v);
}

__device__ __forceinline__ float wave_read_lane(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Sum over the 64 lanes, result valid in every lane (uniform).  Six DPP additions (a running
// sum inside each row of 16, then the row totals passed on: lane 63 ends with everything) and
// one read of lane 63: no trip through the LDS crossbar as with shuffles.
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<DPP_ROW_SHR1, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR2, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR4, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR8, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_BCAST15, 0xa>(0.0f, v);
  v += dpp_move<DPP_ROW_BCAST31, 0xc>(0.0f, v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), WAVE - 1));
}

// Running sum over the lanes: lane l ends with the sum of lanes 0..l (the same steps as wave_sum).
__device__ __forceinline__ float wave_inclusive_sum(float v) {
  v += dpp_move<DPP_ROW_SHR1, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR2, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR4, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_SHR8, 0xf>(0.0f, v);
  v += dpp_move<DPP_ROW_BCAST15, 0xa>(0.0f, v);
  v += dpp_move<DPP_ROW_BCAST31, 0xc>(0.0f, v);
  return v;
}

// One 32-bit register of elements as loaded (two 16-bit elements, or one float), kept as bits until an element is
// used: a register per vector whatever the element type, and the float32 values are formed where they are needed
// instead of being kept.
template <typename io_t>
struct Word {
  unsigned w;
  __device__ __forceinline__ float elem(int v) const;
  // zero when the step is past the row's length: every tensor of a dead step reads as zero, which makes the step
  // the identity that adds nothing and receives nothing
  __device__ __forceinline__ void mask(bool live) { w = live ? w : 0u; }
  // opaque to the compiler from here on: values formed from the bits before are not carried across
  __device__ __forceinline__ void launder() { __asm__ volatile("" : "+v"(w)); }
  // ... and not before `after` has been computed: keeps the conversions of one step of an unrolled loop from
  // being moved in front of the steps before it (where they would all be live at once)
  __device__ __forceinline__ void launder_after(float after) { __asm__ volatile("" : "+v"(w) : "v"(after)); }
};
template <> __device__ __forceinline__ float Word<float>::elem(int) const { return __uint_as_float(w); }
template <> __device__ __forceinline__ float Word<bf16_t>::elem(int v) const {
  return __uint_as_float(v ? (w & 0xffff0000u) : (w << 16));
}
template <> __device__ __forceinline__ float Word<f16_t>::elem(int v) const {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)(v ? (w >> 16) : (w & 0xffffu)));
}

// A wave-uniform base plus a 32-bit byte offset per lane: the form of address the memory instructions take as
// it is (a base in scalar registers, an offset in one vector register), with no 64-bit arithmetic per access.
template <typename T, typename B>
__device__ __forceinline__ T *at_bytes(B *base, unsigned bytes) {
  using C = typename std::conditional<std::is_const<B>::value, const char, char>::type;
  return reinterpret_cast<T *>(reinterpret_cast<C *>(base) + bytes);
}

__device__ __forceinline__ int wave_id_uniform() {
  return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
}
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63); }

}  // namespace ssm
