// Instantiates the forward selective-scan kernels for f16 activations.
#include "scan_fwd_fast.hpp"

namespace ssm {
template int scan_fwd_dispatch<f16_t>(const ScanFwdParams &, int, int, hipStream_t);
template int scan_fwd_fast_dispatch<f16_t, f16_t>(const ScanFwdParams &, int, hipStream_t);
template int scan_fwd_fast_dispatch<f16_t, float>(const ScanFwdParams &, int, hipStream_t);
}
