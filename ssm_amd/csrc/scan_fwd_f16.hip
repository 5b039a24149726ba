// Instantiates the forward selective-scan kernels for f16 activations.
#include "scan_fwd_kernel.hpp"

namespace ssm {
template int scan_fwd_dispatch<f16_t>(const ScanFwdParams &, int, int, hipStream_t);
}
