// Prefill GEMM instantiations for 3-bit codes (all survivor counts and group sizes).
#include "cbk_gemm_big.h"

namespace cbk {
int launch_gemm_big_b3(const GbArgs& a, int keep, int group, int blocks, hipStream_t st) {
  return launch_big_bits<3>(a, keep, group, blocks, st);
}
}  // namespace cbk
