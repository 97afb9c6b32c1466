// The device builtins header as a string, prepended to every hiprtc translation unit.
#include "codegen.hpp"

namespace ocannl {
const char* builtins_hip_source() {
  static const char text[] =
#include "builtins_hip.inc"
      ;
  return text;
}
}  // namespace ocannl
