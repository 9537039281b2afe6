// GEMM+AXPY fast kernels with bf16 output.
#include "launch_impl.hpp"
namespace mi {
template int launch_fast<CfgBig, false, true, MODE_GEMM, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgHalfN, false, true, MODE_GEMM, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgM128, false, true, MODE_GEMM, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgBig, false, false, MODE_GEMM, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
}  // namespace mi
