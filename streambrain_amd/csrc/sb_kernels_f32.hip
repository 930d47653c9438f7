// float instantiation of every kernel launcher, plus the untyped byte fill.
#include "sb_launch_impl.hpp"

namespace sb {
SB_INSTANTIATE_LAUNCHERS(float)

int launch_fill_bytes(hipStream_t st, void *dst, int value, size_t bytes) {
  if (bytes == 0) return 0;
  SB_REQUIRE(dst, "null pointer");
  const size_t blocks = (bytes + 255) / 256 < 4096 ? (bytes + 255) / 256 : 4096;
  hipLaunchKernelGGL((k_fill_bytes<0>), dim3((unsigned)blocks), dim3(256), 0, st, (uint8_t *)dst,
                     (uint8_t)value, bytes);
  SB_LAUNCH_CHECK();
  return 0;
}
}  // namespace sb
