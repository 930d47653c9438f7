// double instantiation of every kernel launcher.
#include "sb_launch_impl.hpp"

namespace sb {
SB_INSTANTIATE_LAUNCHERS(double)

int launch_mfma_probe_f64_4x4x4(hipStream_t st, double *sink, long workgroups, long iters) {
  SB_REQUIRE(sink, "null pointer");
  SB_REQUIRE(workgroups > 0 && workgroups < (1L << 31) && iters > 0 && iters <= (1L << 24), "bad sizes");
  hipLaunchKernelGGL((k_mfma_probe_f64_4x4x4<0>), dim3((unsigned)workgroups), dim3(256), 0, st, sink, iters);
  SB_LAUNCH_CHECK();
  return 0;
}
}  // namespace sb
