// Entry points whose kernels are not written yet: fail loudly.
#include "smr_device.hpp"
extern "C" {
int smr_gemv_allreduce(const void*, const void*, float*, uint32_t*, void*, int, int, int, int, uint32_t*,
                       void*) {
  return smr::fail(SMR_E_UNSUPPORTED, "smr_gemv_allreduce: not built yet");
}
int smr_gemv_flag_blocks(int) { return 0; }
}
