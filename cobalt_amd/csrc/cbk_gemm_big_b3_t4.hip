// Prefill GEMM instantiations for 3-bit codes, 256-token tile.
#include "cbk_gemm_big.h"

namespace cbk {
int launch_gemm_big_b3_t4(const GbArgs& a, int keep, int group, int blocks, hipStream_t st) {
  return launch_big_bits<3, 4>(a, keep, group, blocks, st);
}
}  // namespace cbk
