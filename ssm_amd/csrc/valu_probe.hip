// Issue-rate probe for the vector ALU of gfx950: loops of one instruction pattern with no memory
// traffic, one workgroup per CU (pinned by its LDS request) of 1 to 4 waves per SIMD.  bench.py times
// the launch and divides by the instruction count: the figures behind the instruction-bound estimates
// of the scan kernels (a plain fp32 instruction, a DPP one, a transcendental one, alone and mixed).
#include "common.hpp"

namespace ssm {

typedef float float4v __attribute__((ext_vector_type(4)));
constexpr int PROBE_LDS = 100 * 1024;      // more than half a CU's LDS: one workgroup per CU

template <int KIND>
__global__ __launch_bounds__(1024) void valu_probe_kernel(float *out, long long *clk, int iters, float sB, float sC) {
  extern __shared__ float probe_lds[];
  float r[8], h[8], y = 0.f, dl = -0.001f * (threadIdx.x & 7), du = 0.5f, t, bx;
  for (int i = 0; i < 8; ++i) { r[i] = 0.25f + 0.01f * i + 1e-4f * threadIdx.x; h[i] = 0.f; }
  float4v acc = {0, 0, 0, 0};
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    if constexpr (KIND == 0) {          // 8 independent fma
      asm volatile("v_fma_f32 %0, %0, %8, %9\n v_fma_f32 %1, %1, %8, %9\n v_fma_f32 %2, %2, %8, %9\n v_fma_f32 %3, %3, %8, %9\n"
                   "v_fma_f32 %4, %4, %8, %9\n v_fma_f32 %5, %5, %8, %9\n v_fma_f32 %6, %6, %8, %9\n v_fma_f32 %7, %7, %8, %9\n"
                   : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]) : "v"(du), "v"(dl));
    } else if constexpr (KIND == 1) {   // 8 dependent fma
      asm volatile("v_fma_f32 %0, %0, %1, %2\n v_fma_f32 %0, %0, %1, %2\n v_fma_f32 %0, %0, %1, %2\n v_fma_f32 %0, %0, %1, %2\n"
                   "v_fma_f32 %0, %0, %1, %2\n v_fma_f32 %0, %0, %1, %2\n v_fma_f32 %0, %0, %1, %2\n v_fma_f32 %0, %0, %1, %2\n"
                   : "+v"(r[0]) : "v"(du), "v"(dl));
    } else if constexpr (KIND == 2 || KIND == 3 || KIND == 4) {
#define SSM_PROBE_T8(OP)                                                                                                        \
  asm volatile(OP " %0, %0\n " OP " %1, %1\n " OP " %2, %2\n " OP " %3, %3\n " OP " %4, %4\n " OP " %5, %5\n " OP " %6, %6\n " OP \
                  " %7, %7\n" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
      if constexpr (KIND == 2) { SSM_PROBE_T8("v_exp_f32") } else if constexpr (KIND == 3) { SSM_PROBE_T8("v_log_f32") } else { SSM_PROBE_T8("v_rcp_f32") }
    } else if constexpr (KIND == 5) {   // exp and fma alternating
      asm volatile("v_exp_f32 %0, %0\n v_fma_f32 %4, %4, %8, %9\n v_exp_f32 %1, %1\n v_fma_f32 %5, %5, %8, %9\n"
                   "v_exp_f32 %2, %2\n v_fma_f32 %6, %6, %8, %9\n v_exp_f32 %3, %3\n v_fma_f32 %7, %7, %8, %9\n"
                   : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]) : "v"(du), "v"(dl));
    } else if constexpr (KIND == 6 || KIND == 7) {
      // one step of the scan recurrence for 8 states: mul, exp (KIND 7: mov), mul by a scalar, fma, fmac by a scalar
#define SSM_PROBE_STEP(I, EXPOP) "v_mul_f32 %9, %11, %15\n" EXPOP " %9, %9\n v_mul_f32 %10, %13, %12\n v_fma_f32 %" #I ", %9, %" #I ", %10\n v_fmac_f32 %8, %14, %" #I "\n"
#define SSM_PROBE_STEPS(EXPOP)                                                                                                 \
  asm volatile(SSM_PROBE_STEP(0, EXPOP) SSM_PROBE_STEP(1, EXPOP) SSM_PROBE_STEP(2, EXPOP) SSM_PROBE_STEP(3, EXPOP)             \
               SSM_PROBE_STEP(4, EXPOP) SSM_PROBE_STEP(5, EXPOP) SSM_PROBE_STEP(6, EXPOP) SSM_PROBE_STEP(7, EXPOP)             \
               : "+v"(h[0]), "+v"(h[1]), "+v"(h[2]), "+v"(h[3]), "+v"(h[4]), "+v"(h[5]), "+v"(h[6]), "+v"(h[7]), "+v"(y),      \
                 "=&v"(t), "=&v"(bx) : "v"(dl), "v"(du), "s"(sB), "s"(sC), "v"(r[0]));
      if constexpr (KIND == 6) { SSM_PROBE_STEPS("v_exp_f32") } else { SSM_PROBE_STEPS("v_mov_b32") }
    } else if constexpr (KIND == 8) {   // DPP: multiply by a value broadcast inside each quad
      asm volatile("v_mul_f32_dpp %0, %8, %0 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf\n v_mul_f32_dpp %1, %8, %1 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf\n"
                   "v_mul_f32_dpp %2, %8, %2 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf\n v_mul_f32_dpp %3, %8, %3 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf\n"
                   "v_mul_f32_dpp %4, %8, %4 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf\n v_mul_f32_dpp %5, %8, %5 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf\n"
                   "v_mul_f32_dpp %6, %8, %6 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf\n v_mul_f32_dpp %7, %8, %7 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf\n"
                   : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]) : "v"(du));
    } else if constexpr (KIND == 9) {   // DPP: the fmac / mul pair of a scan step, shifted by one lane of the row
      asm volatile("v_fmac_f32_dpp %1, %1, %0 row_shr:1 row_mask:0xf bank_mask:0xf\n v_fmac_f32_dpp %3, %3, %2 row_shr:1 row_mask:0xf bank_mask:0xf\n"
                   "v_mul_f32_dpp %0, %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf\n v_mul_f32_dpp %2, %2, %2 row_shr:1 row_mask:0xf bank_mask:0xf\n"
                   "v_fmac_f32_dpp %5, %5, %4 row_shr:2 row_mask:0xf bank_mask:0xf\n v_fmac_f32_dpp %7, %7, %6 row_shr:2 row_mask:0xf bank_mask:0xf\n"
                   "v_mul_f32_dpp %4, %4, %4 row_shr:2 row_mask:0xf bank_mask:0xf\n v_mul_f32_dpp %6, %6, %6 row_shr:2 row_mask:0xf bank_mask:0xf\n"
                   : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
    } else if constexpr (KIND == 10) {  // exchanges of wave halves and of 16-lane rows between two registers
      asm volatile("v_permlane32_swap_b32 %0, %1\n v_permlane16_swap_b32 %2, %3\n v_permlane32_swap_b32 %4, %5\n v_permlane16_swap_b32 %6, %7\n"
                   "v_permlane32_swap_b32 %0, %1\n v_permlane16_swap_b32 %2, %3\n v_permlane32_swap_b32 %4, %5\n v_permlane16_swap_b32 %6, %7\n"
                   : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
    } else if constexpr (KIND == 11) {  // 4 state steps (20 instructions) and one fp32 16x16x4 matrix instruction
      asm volatile(SSM_PROBE_STEP(0, "v_exp_f32") SSM_PROBE_STEP(1, "v_exp_f32") SSM_PROBE_STEP(2, "v_exp_f32") SSM_PROBE_STEP(3, "v_exp_f32")
                   : "+v"(h[0]), "+v"(h[1]), "+v"(h[2]), "+v"(h[3]), "+v"(h[4]), "+v"(h[5]), "+v"(h[6]), "+v"(h[7]), "+v"(y),
                     "=&v"(t), "=&v"(bx) : "v"(dl), "v"(du), "s"(sB), "s"(sC), "v"(r[0]));
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(r[1], y, acc, 0, 0, 0);
    } else if constexpr (KIND == 12) {  // 8 conflict-free 8-byte LDS reads
      float2 v[8];
      const float *p = probe_lds + threadIdx.x * 2;
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<const float2 *>(p + ((it + i) & 7) * 2048);
#pragma unroll
      for (int i = 0; i < 8; ++i) y += v[i].x + v[i].y;
    }
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  float s = y + acc[0] + acc[1] + acc[2] + acc[3];
  for (int i = 0; i < 8; ++i) s += r[i] + h[i];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) { clk[0] = c1 - c0; clk[1] = w1 - w0; }
}

template <int KIND>
static int launch_probe(float *out, long long *clk, int grid, int block, int iters, hipStream_t s) {
  auto kernel = valu_probe_kernel<KIND>;
  if (allow_dynamic_lds(kernel, PROBE_LDS) != hipSuccess) {
    (void)hipGetLastError();
    set_error("ssm_probe_valu: cannot reserve %d bytes of LDS", PROBE_LDS);
    return SSM_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), PROBE_LDS, s, out, clk, iters, 0.5f, 0.25f);
  SSM_CHECK_LAUNCH("ssm_probe_valu");
  return SSM_OK;
}

}  // namespace ssm

extern "C" int ssm_probe_valu(int kind, int waves_per_simd, int workgroups, int iters, float *out, long long *clocks,
                              void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(out && clocks, SSM_ERR_NULL_POINTER, "ssm_probe_valu: out and clocks are required");
  SSM_REQUIRE(waves_per_simd >= 1 && waves_per_simd <= 4 && workgroups > 0 && iters > 0, SSM_ERR_BAD_SHAPE,
              "ssm_probe_valu: waves_per_simd=%d (1..4) workgroups=%d iters=%d", waves_per_simd, workgroups, iters);
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  const int block = 256 * waves_per_simd;
  switch (kind) {
#define SSM_PROBE_CASE(K) case K: return launch_probe<K>(out, clocks, workgroups, block, iters, s);
    SSM_PROBE_CASE(0) SSM_PROBE_CASE(1) SSM_PROBE_CASE(2) SSM_PROBE_CASE(3) SSM_PROBE_CASE(4) SSM_PROBE_CASE(5)
    SSM_PROBE_CASE(6) SSM_PROBE_CASE(7) SSM_PROBE_CASE(8) SSM_PROBE_CASE(9) SSM_PROBE_CASE(10) SSM_PROBE_CASE(11)
    SSM_PROBE_CASE(12)
#undef SSM_PROBE_CASE
    default:
      set_error("ssm_probe_valu: unknown kind %d", kind);
      return SSM_ERR_BAD_KIND;
  }
}
