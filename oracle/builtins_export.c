/* TEST INFRASTRUCTURE.  Non-inline entry points over builtins_cc.h for ctypes-driven tests. */
#include "builtins_cc.h"

void ocn_x_threefry_light(const uint32_t *key, const uint32_t *ctr, uint32_t *out) {
  uint4x32_t k, c; memcpy(k.v, key, 16); memcpy(c.v, ctr, 16);
  uint4x32_t r = arrayjit_threefry4x32_light(k, c); memcpy(out, r.v, 16);
}
void ocn_x_threefry_crypto(const uint32_t *key, const uint32_t *ctr, uint32_t *out) {
  uint4x32_t k, c; memcpy(k.v, key, 16); memcpy(c.v, ctr, 16);
  uint4x32_t r = arrayjit_threefry4x32_crypto(k, c); memcpy(out, r.v, 16);
}
void ocn_x_uint32_to_uint4x32(uint32_t x, uint32_t *out) { uint4x32_t r = uint32_to_uint4x32(x); memcpy(out, r.v, 16); }
void ocn_x_int64_to_uint4x32(int64_t x, uint32_t *out) { uint4x32_t r = int64_to_uint4x32(x); memcpy(out, r.v, 16); }
float ocn_x_u4_to_single(const uint32_t *x) { uint4x32_t k; memcpy(k.v, x, 16); return uint4x32_to_single_uniform(k); }
void ocn_x_u4_to_single_vec(const uint32_t *x, float *out) { uint4x32_t k; memcpy(k.v, x, 16); float4_t r = uint4x32_to_single_uniform_vec(k); memcpy(out, r.v, 16); }
void ocn_x_u4_to_half_vec_as_float(const uint32_t *x, float *out) {
  uint4x32_t k; memcpy(k.v, x, 16); half8_t r = uint4x32_to_half_uniform_vec(k);
  for (int i = 0; i < 8; ++i) out[i] = HALF_TO_FLOAT(r.v[i]);
}
void ocn_x_u4_to_bf16_vec(const uint32_t *x, uint16_t *out) { uint4x32_t k; memcpy(k.v, x, 16); uint16x8_t r = uint4x32_to_bfloat16_uniform_vec(k); memcpy(out, r.v, 16); }
uint16_t ocn_x_u4_to_bf16(const uint32_t *x) { uint4x32_t k; memcpy(k.v, x, 16); return uint4x32_to_bfloat16_uniform(k); }
double ocn_x_u4_to_double(const uint32_t *x) { uint4x32_t k; memcpy(k.v, x, 16); return uint4x32_to_double_uniform(k); }
float ocn_x_bf16_to_single(uint16_t b) { return bfloat16_to_single(b); }
uint16_t ocn_x_single_to_bf16(float f) { return single_to_bfloat16(f); }
float ocn_x_fp8_to_single(uint8_t b) { return fp8_to_single(b); }
uint8_t ocn_x_single_to_fp8(float f) { return single_to_fp8(f); }
float ocn_x_half_bits_to_single(uint16_t h) {
#ifdef __FLT16_MAX__
  _Float16 x; memcpy(&x, &h, 2); return (float)x;
#else
  return half_to_float_emulated(h);
#endif
}
uint16_t ocn_x_single_to_half_bits(float f) {
#ifdef __FLT16_MAX__
  _Float16 x = (_Float16)f; uint16_t h; memcpy(&h, &x, 2); return h;
#else
  return float_to_half_emulated(f);
#endif
}
