// Lower-triangle fast kernels, K-strided operands (the memory holds A^T): 256 x 256 and 128 x 128 tiles.
#include "launch_impl.hpp"
namespace mi {
template int launch_fast<CfgBig, true, true, MODE_SYRK, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgT128, true, true, MODE_SYRK, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgT128x2, true, true, MODE_SYRK, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
}  // namespace mi
