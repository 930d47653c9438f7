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

int launch_mask_rows(hipStream_t st, int *rows, int *row_cnt, const uint8_t *wmask, long N, long H,
                     long cap, long h0, long count) {
  SB_REQUIRE(rows && row_cnt && wmask, "null pointer");
  SB_REQUIRE(N > 0 && N < (1L << 31) && H > 0, "bad shape");
  SB_REQUIRE(cap > 0 && cap % 16 == 0, "row lists must be padded to a multiple of 16");
  SB_REQUIRE(h0 >= 0 && count > 0 && h0 + count <= H && count < (1L << 31), "hypercolumn range");
  ProfScope prof_(st, K_MASK_ROWS);
  hipLaunchKernelGGL((k_mask_rows<0>), dim3((unsigned)count), dim3(256), 0, st, rows, row_cnt, wmask, N, H, cap,
                     h0);
  SB_LAUNCH_CHECK();
  return 0;
}
}  // namespace sb
