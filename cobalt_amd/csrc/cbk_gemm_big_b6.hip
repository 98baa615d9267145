// Prefill GEMM instantiations for BLK1632_6 (4-bit nibble stream + plane of high bit pairs;
// 16 of 32 kept, group 128).
#include "cbk_gemm_big.h"

namespace cbk {
int launch_gemm_big_b6(const GbArgs& a, int blocks, hipStream_t st) {
  return launch_big_cfg<6, 16, 128>(a, blocks, st);
}
}  // namespace cbk
