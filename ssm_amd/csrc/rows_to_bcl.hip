// A dense (B, C, L) copy of a (B, C, L)-shaped view whose memory runs channels innermost -- rows of channels, one row
// per time step -- which is what `t.contiguous()` makes of such a view in the reference's Python path, and what
// its blocks hand the scan: `delta = F.linear(...).permute(0, 2, 1)` and `z = gate.permute(0, 2, 1)`
// (src/ssm/modules/mamba1.py:223-228), views that the scan kernels, which walk time, cannot read as they lie.
//
// Pure data movement on the tile of the convolution's rows-in kernels: a workgroup owns 64 channels x 128 steps, a
// thread reads 8 rows of 4 neighbouring channels (the 16 lanes of a row on 128 or 256 contiguous bytes), hands each
// channel's 8 steps to LDS as 16-byte units (unit u of channel group g at unit u ^ (g mod units per row): the
// 16 lanes that write units of 16 groups and the 16 lanes that read 16 units of one row spread over the banks),
// and the units go out along time, 256 contiguous bytes per channel row and 16 lanes.  Elements are moved as
// 2- or 4-byte words whatever their type.
#include "common.hpp"

namespace ssm {

constexpr int TR_CH = 64, TR_STEPS = 128, TR_STRIP = 8, TR_VEC = 4;
constexpr int TR_THREADS = (TR_CH / TR_VEC) * (TR_STEPS / TR_STRIP);   // 256

struct RowsToBclParams {
  const void *src;
  void *dst;
  long long bs, rs;          // elements between batch rows and between time steps of src
  int batch, chans, len;
};

// AL: the rows of dst (L elements each) start on 16-byte boundaries and L is a whole number of 16-byte units.
template <typename W, bool AL>
__global__ __launch_bounds__(TR_THREADS) void rows_to_bcl_kernel(const RowsToBclParams p) {
  constexpr int CH = TR_CH, TT = TR_STEPS, S = TR_STRIP, VEC = TR_VEC;
  constexpr int UNIT = 16 / sizeof(W), UPR = TT / UNIT, UPS = S / UNIT;
  constexpr int GROUPS = CH / VEC;
  __shared__ __attribute__((aligned(16))) W tile[CH * TT];
  const int ttiles = (p.len + TT - 1) / TT, ctiles = (p.chans + CH - 1) / CH;
  int bid = blockIdx.x;
  const int ct = bid % ctiles; bid /= ctiles;
  const int tt = bid % ttiles;
  const int b = bid / ttiles;
  const int cg = threadIdx.x % GROUPS, ts = threadIdx.x / GROUPS;
  const int c_own = ct * CH + cg * VEC;
  const int c0 = c_own < p.chans ? c_own : 0;        // the channel count is a multiple of VEC: a group is all in or all out
  const int t0 = tt * TT + ts * S;
  const W *sb = reinterpret_cast<const W *>(p.src) + (size_t)b * p.bs + c0;
  Pack<W, VEC> raw[S];
#pragma unroll
  for (int j = 0; j < S; ++j) raw[j] = *reinterpret_cast<const Pack<W, VEC> *>(sb + (size_t)min(t0 + j, p.len - 1) * p.rs);
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    Pack<W, UNIT> col[UPS];
#pragma unroll
    for (int j = 0; j < S; ++j) col[j / UNIT].v[j % UNIT] = raw[j].v[i];
    const int r = cg * VEC + i;
#pragma unroll
    for (int h = 0; h < UPS; ++h)
      *reinterpret_cast<Pack<W, UNIT> *>(tile + r * TT + ((ts * UPS + h) ^ (cg % UPR)) * UNIT) = col[h];
  }
  __syncthreads();
  W *db = reinterpret_cast<W *>(p.dst) + (size_t)b * p.chans * p.len;
  for (int v = threadIdx.x; v < CH * UPR; v += TR_THREADS) {
    const int r = v / UPR, u = v % UPR;
    const int c = ct * CH + r, t = tt * TT + u * UNIT;
    if (c >= p.chans || t >= p.len) continue;
    const Pack<W, UNIT> val = *reinterpret_cast<const Pack<W, UNIT> *>(tile + r * TT + (u ^ ((r / VEC) % UPR)) * UNIT);
    W *dst = db + (size_t)c * p.len + t;
    if constexpr (AL) *reinterpret_cast<Pack<W, UNIT> *>(dst) = val;
    else {
#pragma unroll
      for (int e = 0; e < UNIT; ++e)
        if (t + e < p.len) dst[e] = val.v[e];
    }
  }
}

template <typename W>
static void launch_rows_to_bcl(const RowsToBclParams &p, hipStream_t s) {
  const size_t blocks = (size_t)p.batch * ((p.chans + TR_CH - 1) / TR_CH) * ((p.len + TR_STEPS - 1) / TR_STEPS);
  if (p.len % (16 / (int)sizeof(W)) == 0)
    hipLaunchKernelGGL((rows_to_bcl_kernel<W, true>), dim3((unsigned)blocks), dim3(TR_THREADS), 0, s, p);
  else
    hipLaunchKernelGGL((rows_to_bcl_kernel<W, false>), dim3((unsigned)blocks), dim3(TR_THREADS), 0, s, p);
}

}  // namespace ssm

extern "C" int ssm_rows_to_bcl(const ssm_rows_to_bcl_args *a, void *hip_stream) {
  using namespace ssm;
  SSM_REQUIRE(a != nullptr, SSM_ERR_NULL_POINTER, "ssm_rows_to_bcl: args is NULL");
  SSM_REQUIRE(a->src && a->dst, SSM_ERR_NULL_POINTER, "ssm_rows_to_bcl: src and dst are required");
  SSM_REQUIRE(a->batch > 0 && a->channels > 0 && a->seqlen > 0, SSM_ERR_BAD_SHAPE,
              "ssm_rows_to_bcl: batch=%d channels=%d seqlen=%d must all be positive", a->batch, a->channels, a->seqlen);
  SSM_REQUIRE(a->element_size == 2 || a->element_size == 4, SSM_ERR_BAD_DTYPE,
              "ssm_rows_to_bcl: element_size=%d (2 or 4)", a->element_size);
  SSM_REQUIRE(a->channels % TR_VEC == 0, SSM_ERR_BAD_SHAPE,
              "ssm_rows_to_bcl: channels=%d must be a multiple of %d", a->channels, TR_VEC);
  SSM_REQUIRE(a->src_row_stride >= a->channels && a->src_row_stride % TR_VEC == 0 && a->src_batch_stride % TR_VEC == 0 &&
              (a->batch == 1 || a->src_batch_stride >= (long long)(a->seqlen - 1) * a->src_row_stride + a->channels),
              SSM_ERR_BAD_SHAPE, "ssm_rows_to_bcl: src_row_stride=%lld, src_batch_stride=%lld must be multiples of %d, "
              "rows must not overlap", (long long)a->src_row_stride, (long long)a->src_batch_stride, TR_VEC);
  const size_t tiles = (size_t)a->batch * ((a->channels + TR_CH - 1) / TR_CH) * ((a->seqlen + TR_STEPS - 1) / TR_STEPS);
  SSM_REQUIRE(tiles < ((size_t)1 << 31) && (size_t)a->batch * a->channels * a->seqlen < ((size_t)1 << 40),
              SSM_ERR_TOO_LARGE, "ssm_rows_to_bcl: tensor too large");
  SSM_REQUIRE(aligned_to(a->src, (size_t)TR_VEC * a->element_size) && aligned_to(a->dst, 16), SSM_ERR_ALIGNMENT,
              "ssm_rows_to_bcl: src must start on a %d-byte boundary, dst on a 16-byte one", TR_VEC * a->element_size);
  RowsToBclParams p{};
  p.src = a->src; p.dst = a->dst; p.bs = a->src_batch_stride; p.rs = a->src_row_stride;
  p.batch = a->batch; p.chans = a->channels; p.len = a->seqlen;
  hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
  if (a->element_size == 2) launch_rows_to_bcl<uint16_t>(p, s);
  else launch_rows_to_bcl<uint32_t>(p, s);
  SSM_CHECK_LAUNCH("ssm_rows_to_bcl");
  return SSM_OK;
}
