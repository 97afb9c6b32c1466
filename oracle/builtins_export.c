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

/* Batched forms for bulk comparisons: n independent (key, counter) pairs / inputs. */
void ocn_x_batch_threefry(int crypto, const uint32_t *keys, const uint32_t *ctrs, uint32_t *out, int n) {
  for (int i = 0; i < n; ++i) {
    uint4x32_t k, c; memcpy(k.v, keys + 4 * i, 16); memcpy(c.v, ctrs + 4 * i, 16);
    uint4x32_t r = crypto ? arrayjit_threefry4x32_crypto(k, c) : arrayjit_threefry4x32_light(k, c);
    memcpy(out + 4 * i, r.v, 16);
  }
}
/* every uniform converter of one uint4x32: 4 floats, 2 doubles, 8 bf16, 8 halves (as float), scalar forms */
void ocn_x_batch_uniform(const uint32_t *xs, float *f4, double *d2, uint16_t *b8, float *h8, float *f1, double *d1,
                         uint16_t *b1, int n) {
  for (int i = 0; i < n; ++i) {
    uint4x32_t k; memcpy(k.v, xs + 4 * i, 16);
    float4_t rf = uint4x32_to_single_uniform_vec(k); memcpy(f4 + 4 * i, rf.v, 16);
    double2_t rd = uint4x32_to_double_uniform_vec(k); memcpy(d2 + 2 * i, rd.v, 16);
    uint16x8_t rb = uint4x32_to_bfloat16_uniform_vec(k); memcpy(b8 + 8 * i, rb.v, 16);
    half8_t rh = uint4x32_to_half_uniform_vec(k);
    for (int j = 0; j < 8; ++j) h8[8 * i + j] = HALF_TO_FLOAT(rh.v[j]);
    f1[i] = uint4x32_to_single_uniform(k); d1[i] = uint4x32_to_double_uniform(k); b1[i] = uint4x32_to_bfloat16_uniform(k);
  }
}
void ocn_x_batch_convert(const float *xs, uint16_t *bf, uint8_t *f8, float *bf_back, float *f8_back, int n) {
  for (int i = 0; i < n; ++i) {
    bf[i] = single_to_bfloat16(xs[i]); f8[i] = single_to_fp8(xs[i]);
    bf_back[i] = bfloat16_to_single(bf[i]); f8_back[i] = fp8_to_single(f8[i]);
  }
}
void ocn_x_batch_spread(const uint32_t *xs, uint32_t *from_u32, uint32_t *from_i64, uint32_t *from_single, int n) {
  for (int i = 0; i < n; ++i) {
    uint4x32_t r = uint32_to_uint4x32(xs[i]); memcpy(from_u32 + 4 * i, r.v, 16);
    int64_t w = (int64_t)(((uint64_t)xs[i] << 32) | xs[(i + 1) % n]);
    r = int64_to_uint4x32(w); memcpy(from_i64 + 4 * i, r.v, 16);
    float f; memcpy(&f, xs + i, 4);
    r = single_to_uint4x32(f); memcpy(from_single + 4 * i, r.v, 16);
  }
}
