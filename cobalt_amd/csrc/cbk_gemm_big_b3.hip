// Prefill GEMM for 3-bit codes (all survivor counts and group sizes): dispatch over the token
// tile; the instantiations are in cbk_gemm_big_b3_t1/2/4.hip.
#include "cbk_gemm_big.h"

namespace cbk {
int launch_gemm_big_b3_t1(const GbArgs&, int keep, int group, int blocks, hipStream_t);
int launch_gemm_big_b3_t2(const GbArgs&, int keep, int group, int blocks, hipStream_t);
int launch_gemm_big_b3_t4(const GbArgs&, int keep, int group, int blocks, hipStream_t);
int launch_gemm_big_b3(const GbArgs& a, int keep, int group, int blocks, hipStream_t st) {
  return a.ti == 1 ? launch_gemm_big_b3_t1(a, keep, group, blocks, st)
       : a.ti == 2 ? launch_gemm_big_b3_t2(a, keep, group, blocks, st) : launch_gemm_big_b3_t4(a, keep, group, blocks, st);
}
}  // namespace cbk
