// Prefill GEMM instantiations for 3-bit codes, 128-token tile.
#include "cbk_gemm_big.h"

namespace cbk {
int launch_gemm_big_b3_t2(const GbArgs& a, int keep, int group, int blocks, hipStream_t st) {
  return launch_big_bits<3, 2>(a, keep, group, blocks, st);
}
}  // namespace cbk
