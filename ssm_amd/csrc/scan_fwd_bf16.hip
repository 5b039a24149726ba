// Instantiates the forward selective-scan kernels for bf16 activations.
#include "scan_fwd_kernel.hpp"

namespace ssm {
template int scan_fwd_dispatch<bf16_t>(const ScanFwdParams &, int, int, hipStream_t);
}
