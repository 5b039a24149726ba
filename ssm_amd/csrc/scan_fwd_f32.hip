// Instantiates the forward selective-scan kernels for f32 activations.
#include "scan_fwd_fast.hpp"

namespace ssm {
template int scan_fwd_dispatch<float>(const ScanFwdParams &, int, int, hipStream_t);
template int scan_fwd_fast_dispatch<float, float>(const ScanFwdParams &, int, hipStream_t);
}
