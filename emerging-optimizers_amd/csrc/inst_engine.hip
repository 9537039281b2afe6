// General kernels (any multiple-of-8 shape): three tile classes x the operand layouts and outputs the library uses.
#include "launch_impl.hpp"
namespace mi {
#define MI_ENGINE(P_KS, Q_KS, MODE, OUT_F32)                                                                          \
  template int launch_one<256, 256, 64, 2, 2, P_KS, Q_KS, MODE, OUT_F32>(const GemmParams&, int64_t, hipStream_t);    \
  template int launch_one<128, 128, 64, 2, 2, P_KS, Q_KS, MODE, OUT_F32>(const GemmParams&, int64_t, hipStream_t);    \
  template int launch_one<64, 64, 64, 2, 2, P_KS, Q_KS, MODE, OUT_F32>(const GemmParams&, int64_t, hipStream_t);
MI_ENGINE(false, false, MODE_SYRK, false)
MI_ENGINE(true, true, MODE_SYRK, false)
MI_ENGINE(false, true, MODE_GEMM, false)
MI_ENGINE(false, true, MODE_GEMM, true)
MI_ENGINE(false, false, MODE_GEMM, false)
MI_ENGINE(false, false, MODE_GEMM, true)
#undef MI_ENGINE
}  // namespace mi
