// C-ABI entry point of the forward selective scan: argument validation and
// kernel selection.  The kernels live in scan_fwd_kernel.hpp and are
// instantiated per activation dtype in scan_fwd_{f32,bf16,f16}.hip.
#include "scan_fwd_fast.hpp"

namespace ssm {

extern template int scan_fwd_dispatch<float>(const ScanFwdParams &, int, int, hipStream_t);
extern template int scan_fwd_dispatch<bf16_t>(const ScanFwdParams &, int, int, hipStream_t);
extern template int scan_fwd_dispatch<f16_t>(const ScanFwdParams &, int, int, hipStream_t);

extern template int scan_fwd_fast_dispatch<float, float>(const ScanFwdParams &, int, hipStream_t);
extern template int scan_fwd_fast_dispatch<bf16_t, bf16_t>(const ScanFwdParams &, int, hipStream_t);
extern template int scan_fwd_fast_dispatch<bf16_t, float>(const ScanFwdParams &, int, hipStream_t);
extern template int scan_fwd_fast_dispatch<f16_t, f16_t>(const ScanFwdParams &, int, hipStream_t);
extern template int scan_fwd_fast_dispatch<f16_t, float>(const ScanFwdParams &, int, hipStream_t);

static bool valid_kind(int k) { return k == SSM_PROJ_DN || k == SSM_PROJ_BDN || k == SSM_PROJ_BGNL; }

}  // namespace ssm

extern "C" int ssm_scan_chunk_len(void) { return 512; }

extern "C" int ssm_scan_fwd(const ssm_scan_fwd_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_scan_fwd: args is NULL");
  SSM_REQUIRE(a->u && a->delta && a->A && a->Bproj && a->Cproj && a->out, SSM_ERR_NULL_POINTER,
              "ssm_scan_fwd: u, delta, A, Bproj, Cproj and out are required");
  SSM_REQUIRE(a->batch > 0 && a->dim > 0 && a->seqlen > 0 && a->nstate > 0, SSM_ERR_BAD_SHAPE,
              "ssm_scan_fwd: batch=%d dim=%d seqlen=%d nstate=%d must all be positive", a->batch, a->dim,
              a->seqlen, a->nstate);
  SSM_REQUIRE(a->nstate <= SCAN_MAX_N, SSM_ERR_TOO_LARGE, "ssm_scan_fwd: nstate=%d exceeds %d", a->nstate,
              SCAN_MAX_N);
  SSM_REQUIRE(valid_dtype(a->io_dtype) && valid_dtype(a->bc_dtype), SSM_ERR_BAD_DTYPE,
              "ssm_scan_fwd: io_dtype=%d bc_dtype=%d", a->io_dtype, a->bc_dtype);
  SSM_REQUIRE(valid_kind(a->b_kind) && valid_kind(a->c_kind), SSM_ERR_BAD_KIND, "ssm_scan_fwd: b_kind=%d c_kind=%d",
              a->b_kind, a->c_kind);
  const bool bvary = a->b_kind == SSM_PROJ_BGNL, cvary = a->c_kind == SSM_PROJ_BGNL;
  if (bvary)
    SSM_REQUIRE(a->b_groups > 0 && a->dim % a->b_groups == 0, SSM_ERR_BAD_SHAPE,
                "ssm_scan_fwd: b_groups=%d must divide dim=%d", a->b_groups, a->dim);
  if (cvary)
    SSM_REQUIRE(a->c_groups > 0 && a->dim % a->c_groups == 0, SSM_ERR_BAD_SHAPE,
                "ssm_scan_fwd: c_groups=%d must divide dim=%d", a->c_groups, a->dim);
  const size_t rows_total = (size_t)a->batch * a->dim;
  SSM_REQUIRE(rows_total * (size_t)a->seqlen < ((size_t)1 << 40) && rows_total < ((size_t)1 << 31),
              SSM_ERR_TOO_LARGE, "ssm_scan_fwd: tensor too large");
  const int es = dtype_size(a->io_dtype), bs = dtype_size(a->bc_dtype);
  SSM_REQUIRE(aligned_to(a->u, es) && aligned_to(a->delta, es) && aligned_to(a->out, es) &&
                  (!a->z || aligned_to(a->z, es)) && (!a->last_state || aligned_to(a->last_state, es)) &&
                  aligned_to(a->Bproj, bs) && aligned_to(a->Cproj, bs) && aligned_to(a->A, 4) &&
                  (!a->Dskip || aligned_to(a->Dskip, 4)) && (!a->dt_bias || aligned_to(a->dt_bias, 4)),
              SSM_ERR_ALIGNMENT, "ssm_scan_fwd: a pointer is not aligned to its element size");

  ScanFwdParams p;
  p.u = a->u; p.delta = a->delta; p.z = a->z; p.Bp = a->Bproj; p.Cp = a->Cproj;
  p.A = a->A; p.Dk = a->Dskip; p.bias = a->dt_bias; p.out = a->out; p.last = a->last_state;
  p.chunk_states = a->chunk_states;
  p.batch = a->batch; p.dim = a->dim; p.len = a->seqlen; p.nstate = a->nstate;
  p.bc_dtype = a->bc_dtype;
  p.b_kind = a->b_kind; p.c_kind = a->c_kind;
  p.b_groups = bvary ? a->b_groups : 1; p.c_groups = cvary ? a->c_groups : 1;
  p.softplus = a->delta_softplus ? 1 : 0;
  p.vec_ok = ((size_t)a->seqlen * es) % 16 == 0 && aligned_to(a->u, 16) && aligned_to(a->delta, 16) &&
             aligned_to(a->out, 16) && (!a->z || aligned_to(a->z, 16));
  p.bc_vec_ok = a->seqlen % 4 == 0 && aligned_to(a->Bproj, 4 * bs) && aligned_to(a->Cproj, 4 * bs);

  // channels per workgroup: all must read the same B group and the same C group
  const int per_b = bvary ? a->dim / a->b_groups : a->dim;
  const int per_c = cvary ? a->dim / a->c_groups : a->dim;
  int rows = SCAN_MAX_WAVES;
  while (rows > 1 && (per_b % rows != 0 || per_c % rows != 0)) --rows;      // any divisor, not only powers of two

  // Two channels per wave (tune 1616) pay off once the grid still fills every CU twice.
  const bool pair_ok = bvary && cvary && a->nstate <= 16 && per_b % 16 == 0 && per_c % 16 == 0;
  SSM_CHECK_RESERVED("ssm_scan_fwd", a);
  int tune = SSM_RESERVED(a);               // 0 = automatic
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);

  // The specialised kernel: time-varying B and C of one element type (that of the activations, or fp32), at most
  // 16 states, aligned rows of whole 16-step runs.  A selector of 100000 + v asks for its variant v.
  const bool fast_ok = bvary && cvary && a->nstate <= FAST_N && p.vec_ok && a->seqlen % 16 == 0 &&
                       aligned_to(a->Bproj, 4 * bs) && aligned_to(a->Cproj, 4 * bs) &&
                       (a->bc_dtype == a->io_dtype || a->bc_dtype == SSM_F32);
  if (tune == 0 && fast_ok && a->seqlen > 256) {
    // The variant whose workgroups (48, 24 or 8 channels of one group) still give every CU its share:
    // two rows per wave with 16-step runs and two slabs where 256 such workgroups exist, else 8-step runs at six waves
    // per SIMD, else the smallest workgroup.
    const size_t total = (size_t)a->batch * a->dim;
    // float32 activations: the 8-step runs at six waves per SIMD come out ahead (142.9 against 149.6 us at the
    // headline shape, where twice the bytes per step leave more to wait for); 16-bit: the 16-step runs (120.5 / 133.3)
    const int pref16[3] = {22123, 12121, 11082}, pref32[3] = {12121, 22123, 11082};
    const int *pref = a->io_dtype == SSM_F32 ? pref32 : pref16;
    int pick = 0;
    for (int i = 0; i < 3 && !pick; ++i) {
      const int per_wg = scan_fwd_fast_rows(pref[i]);
      if (per_b % per_wg == 0 && per_c % per_wg == 0 && (total / per_wg >= 256 || i == 2)) pick = pref[i];
    }
    // groups of fewer than 8 channels (down to one per channel): nothing to share, a row per wave
    if (!pick && aligned_to(a->Bproj, 16) && aligned_to(a->Cproj, 16) && ((size_t)a->seqlen * bs) % 16 == 0) pick = 31041;
    if (pick) tune = 100000 + pick;
  }
  // Projections constant in time, (D, N) or (B, D, N): a row per wave with B and C in lanes (variant 31042).
  const bool const_ok = !bvary && !cvary && a->nstate <= FAST_N && p.vec_ok && a->seqlen % 8 == 0;
  if ((tune == 0 && const_ok && a->seqlen > 256) || tune == 100000 + 31042) {
    SSM_REQUIRE(const_ok, SSM_ERR_BAD_KIND, "ssm_scan_fwd: selector %d needs constant projections, at most %d states "
                "and aligned rows of whole 8-step runs", tune, FAST_N);
    switch (a->io_dtype) {
      case SSM_F32: return scan_fwd_fast_dispatch<float, float>(p, 31042, stream);
      case SSM_BF16: return scan_fwd_fast_dispatch<bf16_t, float>(p, 31042, stream);
      default: return scan_fwd_fast_dispatch<f16_t, float>(p, 31042, stream);
    }
  }
  if (tune >= 100000) {
    SSM_REQUIRE(fast_ok, SSM_ERR_BAD_KIND, "ssm_scan_fwd: selector %d needs the shape of the specialised kernel", tune);
    const int v = tune - 100000, per_wg = scan_fwd_fast_rows(v);
    SSM_REQUIRE(per_wg > 0 && per_b % per_wg == 0 && per_c % per_wg == 0, SSM_ERR_BAD_KIND,
                "ssm_scan_fwd: variant %d takes %d channels per workgroup, which must divide a group", v, per_wg);
    const bool bc32 = a->bc_dtype == SSM_F32;
    switch (a->io_dtype) {
      case SSM_F32: return scan_fwd_fast_dispatch<float, float>(p, v, stream);
      case SSM_BF16: return bc32 ? scan_fwd_fast_dispatch<bf16_t, float>(p, v, stream)
                                 : scan_fwd_fast_dispatch<bf16_t, bf16_t>(p, v, stream);
      default: return bc32 ? scan_fwd_fast_dispatch<f16_t, float>(p, v, stream)
                           : scan_fwd_fast_dispatch<f16_t, f16_t>(p, v, stream);
    }
  }
  if (tune == 0) {
    if (a->seqlen <= 256 && !a->chunk_states) tune = 408;
    else tune = a->nstate > 8 ? 816 : 808;
    if (tune != 408 && pair_ok) {
      // Several channels per wave share one staged B/C slab.  Two workgroups of 8 waves are resident per CU;
      // take the number of channels per wave whose grid leaves the fewest of those 512 places idle in its
      // last round (at B=8, D=1536: 3 -> 512 workgroups, one full round; 2 -> 768, the second round half empty).
      const int cand[4] = {3, 2, 4, 6};
      double best = 0.0;
      for (int i = 0; i < 4; ++i) {
        const int per_wg = cand[i] * SCAN_MAX_WAVES;
        if (per_b % per_wg != 0 || per_c % per_wg != 0) continue;
        const size_t wgs = (size_t)a->batch * a->dim / per_wg;
        if (wgs < 512) continue;
        const size_t rounds = (wgs + 511) / 512;
        const double fill = (double)wgs / (double)(rounds * 512);
        if (fill > best + 1e-9) {
          best = fill;
          tune = cand[i] * 800 + 16;
        }
      }
    }
  }
  if (tune == 1616 || tune == 2416 || tune == 3216 || tune == 4816) {        // 2, 3, 4, 6 channels per wave
    const int r = tune / 100;
    if (pair_ok && per_b % r == 0 && per_c % r == 0) rows = r;
    else tune = 816;
  }
  const int steps_per_lane = tune >= 1616 ? 8 : tune / 100;
  if (a->chunk_states)
    SSM_REQUIRE(steps_per_lane * WAVE == ssm_scan_chunk_len(), SSM_ERR_BAD_KIND,
                "ssm_scan_fwd: chunk_states needs a tiling of %d steps per chunk (selectors 808, 816 or 1616)",
                ssm_scan_chunk_len());
  switch (a->io_dtype) {
    case SSM_F32: return scan_fwd_dispatch<float>(p, tune, rows, stream);
    case SSM_BF16: return scan_fwd_dispatch<bf16_t>(p, tune, rows, stream);
    default: return scan_fwd_dispatch<f16_t>(p, tune, rows, stream);
  }
}
