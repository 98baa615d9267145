// Prefill GEMM instantiations for 3-bit codes, 64-token tile.
#include "cbk_gemm_big.h"

namespace cbk {
int launch_gemm_big_b3_t1(const GbArgs& a, int keep, int group, int blocks, hipStream_t st) {
  return launch_big_bits<3, 1>(a, keep, group, blocks, st);
}
}  // namespace cbk
