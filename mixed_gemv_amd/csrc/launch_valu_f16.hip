// fp16 instantiations of the VALU GEMV kernel.
#include "gemv_dpp_kernel.h"

namespace mgemv {

hipError_t launch_gemv_f16(const GemvLaunch& g, int bits, int qop, int mb, int gpr) {
  return launch_gemv_act<kActF16>(g, bits, qop, mb, gpr);
}

}  // namespace mgemv
