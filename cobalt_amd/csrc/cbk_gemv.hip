// MFMA decode GEMV (placeholder until the int8-MFMA kernel lands): takes nothing, so every
// call goes to the generic row kernel.
#include "cbk_device.h"
namespace cbk {
bool gemv_fast_takes(const DMat&, int) { return false; }
size_t gemv_fast_workspace(const DMat&, int) { return 0; }
int launch_gemv_fast(const DMat&, const void*, int, int, int64_t, void*, int, int64_t, const void*, void*,
                     size_t, hipStream_t) { return CBK_ERR_UNSUPPORTED; }
}  // namespace cbk
