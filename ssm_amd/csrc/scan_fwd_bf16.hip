// Instantiates the forward selective-scan kernels for bf16 activations.
#include "scan_fwd_fast.hpp"

namespace ssm {
template int scan_fwd_dispatch<bf16_t>(const ScanFwdParams &, int, int, hipStream_t);
template int scan_fwd_fast_dispatch<bf16_t, bf16_t>(const ScanFwdParams &, int, hipStream_t);
template int scan_fwd_fast_dispatch<bf16_t, float>(const ScanFwdParams &, int, hipStream_t);
}
