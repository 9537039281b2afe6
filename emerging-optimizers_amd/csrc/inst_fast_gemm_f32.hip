// GEMM+AXPY fast kernels with float32 output, and the split-K Gram partials of short, wide matrices.
#include "launch_impl.hpp"
namespace mi {
template int launch_fast<CfgBig, false, true, MODE_GEMM, true>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgHalfN, false, true, MODE_GEMM, true>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgM128, false, true, MODE_GEMM, true>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgBig, false, false, MODE_GEMM, true>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgT128, false, false, MODE_GEMM, true>(const GemmParams&, int64_t, hipStream_t, int64_t);
}  // namespace mi
