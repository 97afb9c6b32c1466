// Compile-time check that the builtins header is valid HIP device code on its own.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "builtins_hip.h"
__global__ void ocannl_builtins_check(uint4x32_t* out, const uint4x32_t* key) {
  uint4x32_t c = uint32_to_uint4x32(threadIdx.x);
  out[threadIdx.x] = arrayjit_threefry4x32_crypto(arrayjit_threefry4x32_light(key[0], c), c);
}
