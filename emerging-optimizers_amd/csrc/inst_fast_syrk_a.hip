// Lower-triangle fast kernels, K-contiguous operands: 192 x 192 and 128 x 128 (three-slot ring) tiles.
#include "launch_impl.hpp"
namespace mi {
template int launch_fast<CfgSyrk192, false, false, MODE_SYRK, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgT128, false, false, MODE_SYRK, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
}  // namespace mi
