// Lower-triangle fast kernels, K-contiguous operands: 256 x 256 and 128 x 128 (two-slot ring, two workgroups per CU) tiles.
#include "launch_impl.hpp"
namespace mi {
template int launch_fast<CfgBig, false, false, MODE_SYRK, false>(const GemmParams&, int64_t, hipStream_t);
template int launch_fast<CfgT128x2, false, false, MODE_SYRK, false>(const GemmParams&, int64_t, hipStream_t);
}  // namespace mi
