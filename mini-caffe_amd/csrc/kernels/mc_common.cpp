#include "mc_common.h"
#include "mchip/kernels.h"

namespace mchip {
std::string& last_error() {
  static thread_local std::string msg;
  return msg;
}
}  // namespace mchip

extern "C" const char* mcLastError(void) { return mchip::last_error().c_str(); }
