// bf16 MFMA kernels of the state-space-duality family (placeholder: shapes not yet covered).
#include "ssd_common.hpp"

namespace ssm {
bool ssd_bmm_mfma(const SsdBmmParams &, hipStream_t) { return false; }
bool ssd_chunk_state_mfma(const SsdStateParams &, hipStream_t) { return false; }
bool ssd_chunk_scan_mfma(const SsdScanParams &, hipStream_t) { return false; }
}  // namespace ssm
