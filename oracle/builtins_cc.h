/* TEST INFRASTRUCTURE -- CPU checker, not part of the shipped product path.
 *
 * Restatement of the scalar builtins OCANNL's `cc` backend prepends to generated C
 * (arrayjit/lib/builtins.c:11-743, mirrored as text in arrayjit/lib/builtins_cc.ml).
 * Written afresh from the algorithm descriptions; function NAMES must match because the
 * generated code calls them (arrayjit/lib/ops.ml:579-876).
 *
 *   half emulation            builtins.c:34-152      pinned: exhaustive 2^16 round trip + tests
 *   threefry4x32 light (2)    builtins.c:156-196,284-329  pinned: test/operations/
 *                                                    test_threefry4x32.ml:37-46 and
 *                                                    threefry4x32_demo.ml:31-73
 *   threefry4x32 crypto (20)  builtins.c:199-281     pinned: the reference's own C text of
 *                                                    builtins.c (math.h include down to the
 *                                                    OCaml wrappers) compiled unchanged into
 *                                                    oracle/_ref/builtins_ref.so and compared
 *                                                    bit for bit on 20 000 random key/counter
 *                                                    pairs, as are the light variant, the
 *                                                    uniform converters and the conversions
 *                                                    (tests/test_oracle_builtins.py)
 *   uint4x32 -> uniform       builtins.c:345-528     pinned: same KATs + closed forms
 *   X -> uint4x32             builtins.c:531-606     pinned: same KATs (counter spreading)
 *   bf16 / fp8(E5M2)          builtins.c:611-743     pinned: arrayjit/test/
 *                                                    test_numerical_types.expected:4-33,
 *                                                    compiled reference fixtures (oracle/_ref)
 */
#include <stdio.h>
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>

/* ---- half --------------------------------------------------------------------------- */
#ifdef __FLT16_MAX__
typedef _Float16 ocannl_half_t;
#define HALF_T _Float16
#define HALF_TO_FP(x) (x)
#define FP_TO_HALF(x) (x)
#define HALF_TO_FLOAT(x) ((float)(x))
#define FLOAT_TO_HALF(x) ((_Float16)(x))
#else
#define HALF_T uint16_t
static float half_to_float_emulated(uint16_t h) {
  const uint32_t s = h >> 15, e = (h >> 10) & 31u, m = h & 1023u;
  float r;
  if (e == 31u) r = m ? NAN : INFINITY;
  else if (e == 0u) r = ldexpf((float)m, -24);          /* subnormal: m * 2^-10 * 2^-14 */
  else r = ldexpf((float)(m | 1024u), (int)e - 25);     /* (1 + m/1024) * 2^(e-15) */
  return (s && !(e == 31u && m)) ? -r : r;
}
static uint16_t float_to_half_emulated(float f) {
  /* builtins.c:63-151: sign/exponent/mantissa split of the binary32 pattern; overflow to
     infinity, underflow below 2^-24 to zero, round half to even on the 13 dropped bits
     (with carry into the exponent), subnormals via shifted mantissa with implicit one. */
  uint32_t b; memcpy(&b, &f, 4);
  const uint32_t s = (b >> 16) & 0x8000u;
  const int32_t e = (int32_t)((b >> 23) & 255u) - 127;
  uint32_t m = b & 0x7FFFFFu;
  if (((b >> 23) & 255u) == 255u) return (uint16_t)(s | 0x7C00u | (m ? 0x200u : 0u));
  if (((b >> 23) & 255u) == 0u) return (uint16_t)s;      /* float zero / subnormal -> 0 */
  if (e > 15) return (uint16_t)(s | 0x7C00u);
  if (e < -24) return (uint16_t)s;
  if (e < -14) {
    m |= 0x800000u;
    const int shift = -14 - e + 13;
    uint32_t hm = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (hm & 1u))) hm++;
    return (uint16_t)(s | hm);
  }
  uint32_t he = (uint32_t)(e + 15), hm = m >> 13;
  const uint32_t rem = m & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (hm & 1u))) {
    hm++;
    if (hm == 1024u) { hm = 0; he++; if (he >= 31u) return (uint16_t)(s | 0x7C00u); }
  }
  return (uint16_t)(s | (he << 10) | hm);
}
#define HALF_TO_FP(x) half_to_float_emulated(x)
#define FP_TO_HALF(x) float_to_half_emulated(x)
#define HALF_TO_FLOAT(x) half_to_float_emulated(x)
#define FLOAT_TO_HALF(x) float_to_half_emulated(x)
#endif

/* ---- threefry4x32 ------------------------------------------------------------------- */
typedef struct { uint32_t v[4]; } uint4x32_t;
typedef struct { float v[4]; } float4_t;
typedef struct { double v[2]; } double2_t;
typedef struct { int32_t v[4]; } int32x4_t;
typedef struct { uint32_t v[4]; } uint32x4_t;
typedef struct { int64_t v[2]; } int64x2_t;
typedef struct { uint64_t v[2]; } uint64x2_t;
typedef struct { int8_t v[16]; } int8x16_t;
typedef struct { uint16_t v[8]; } uint16x8_t;
typedef struct { uint8_t v[16]; } uint8x16_t;
typedef struct { HALF_T v[8]; } half8_t;

static inline uint32_t ocn_rotl(uint32_t x, unsigned n) { return (x << n) | (x >> (32u - n)); }

/* One "double round": two mix layers, each followed by exchanging words 1 and 3
   (builtins.c:181-196).  Rotation sets alternate {13,15,26,6} / {17,29,16,24}. */
static inline void ocn_tf_pair(uint32_t x[4], const unsigned r[4]) {
  uint32_t t;
  x[0] += x[1]; x[1] = ocn_rotl(x[1], r[0]) ^ x[0];
  x[2] += x[3]; x[3] = ocn_rotl(x[3], r[1]) ^ x[2];
  t = x[1]; x[1] = x[3]; x[3] = t;
  x[0] += x[1]; x[1] = ocn_rotl(x[1], r[2]) ^ x[0];
  x[2] += x[3]; x[3] = ocn_rotl(x[3], r[3]) ^ x[2];
  t = x[1]; x[1] = x[3]; x[3] = t;
}

/* `groups` blocks of four rounds-equivalents... the reference counts each call above as one
   "round"; the crypto variant applies 20 of them with a key injection after every 4
   (builtins.c:199-281), the light variant 2 with one final injection (builtins.c:284-323). */
static inline uint4x32_t ocn_threefry(uint4x32_t key, uint4x32_t ctr, int n_calls) {
  static const unsigned R0[4] = {13, 15, 26, 6}, R1[4] = {17, 29, 16, 24};
  uint32_t ks[5], x[4];
  ks[4] = 0x1BD11BDAu;
  for (int i = 0; i < 4; ++i) { ks[i] = key.v[i]; ks[4] ^= key.v[i]; x[i] = ctr.v[i] + key.v[i]; }
  if (n_calls == 2) {
    ocn_tf_pair(x, R0); ocn_tf_pair(x, R1);
    for (int i = 0; i < 4; ++i) x[i] += ks[(1 + i) % 5];
    x[3] += 1u;
  } else {
    for (int g = 1; g <= n_calls / 4; ++g) {
      ocn_tf_pair(x, R0); ocn_tf_pair(x, R1); ocn_tf_pair(x, R0); ocn_tf_pair(x, R1);
      for (int i = 0; i < 4; ++i) x[i] += ks[(g + i) % 5];
      x[3] += (uint32_t)g;
    }
  }
  uint4x32_t out; for (int i = 0; i < 4; ++i) out.v[i] = x[i];
  return out;
}
static inline uint4x32_t arrayjit_threefry4x32_crypto(uint4x32_t key, uint4x32_t counter) {
  return ocn_threefry(key, counter, 20);
}
static inline uint4x32_t arrayjit_threefry4x32_light(uint4x32_t key, uint4x32_t counter) {
  return ocn_threefry(key, counter, 2);
}
static inline uint4x32_t arrayjit_threefry4x32(uint4x32_t key, uint4x32_t counter) {
  return ocn_threefry(key, counter, 2);  /* default = light, builtins.c:326-329 */
}

/* ---- uint4x32 -> uniform ------------------------------------------------------------ */
static inline float uint32_to_single_uniform(uint32_t x) { return (float)(x >> 8) * 0x1p-24f; }
static inline double uint32_to_double_uniform(uint32_t x) { return (double)x * 0x1p-32; }
static inline uint64_t ocn_lo64(uint4x32_t x) { return ((uint64_t)x.v[1] << 32) | x.v[0]; }
static inline uint64_t ocn_hi64(uint4x32_t x) { return ((uint64_t)x.v[3] << 32) | x.v[2]; }
static inline uint16_t ocn_bf16_rne_bits(float f) {
  /* explicit guard/sticky rounding used by the uniform converters (builtins.c:397-406) */
  uint32_t b; memcpy(&b, &f, 4);
  uint16_t r = (uint16_t)(b >> 16);
  if ((b & 0x8000u) && ((b & 0x7FFFu) || (r & 1u))) r++;
  return r;
}
static inline float uint4x32_to_single_uniform(uint4x32_t x) { return uint32_to_single_uniform(x.v[0]); }
static inline double uint4x32_to_double_uniform(uint4x32_t x) { return (double)ocn_lo64(x) * 0x1p-64; }
static inline int32_t uint4x32_to_int32_uniform(uint4x32_t x) { return (int32_t)x.v[0]; }
static inline int64_t uint4x32_to_int64_uniform(uint4x32_t x) { return (int64_t)ocn_lo64(x); }
static inline uint32_t uint4x32_to_uint32_uniform(uint4x32_t x) { return x.v[0]; }
static inline uint64_t uint4x32_to_uint64_uniform(uint4x32_t x) { return ocn_lo64(x); }
static inline int8_t uint4x32_to_byte_uniform(uint4x32_t x) { return (int8_t)(x.v[0] & 0xFFu); }
static inline uint16_t uint4x32_to_uint16_uniform(uint4x32_t x) { return (uint16_t)(x.v[0] & 0xFFFFu); }
static inline uint16_t uint4x32_to_bfloat16_uniform(uint4x32_t x) {
  return ocn_bf16_rne_bits(uint32_to_single_uniform(x.v[0]));
}
static inline HALF_T uint4x32_to_half_uniform(uint4x32_t x) {
  return FLOAT_TO_HALF((float)(x.v[0] & 0xFFFFu) * 0x1p-16f);
}
static inline uint8_t uint4x32_to_fp8_uniform(uint4x32_t x) { return (uint8_t)(x.v[0] & 0xFFu); }

static inline float4_t uint4x32_to_single_uniform_vec(uint4x32_t x) {
  float4_t r; for (int i = 0; i < 4; ++i) r.v[i] = uint32_to_single_uniform(x.v[i]); return r;
}
static inline double2_t uint4x32_to_double_uniform_vec(uint4x32_t x) {
  double2_t r; r.v[0] = (double)ocn_lo64(x) * 0x1p-64; r.v[1] = (double)ocn_hi64(x) * 0x1p-64; return r;
}
static inline int32x4_t uint4x32_to_int32_uniform_vec(uint4x32_t x) {
  int32x4_t r; for (int i = 0; i < 4; ++i) r.v[i] = (int32_t)x.v[i]; return r;
}
static inline uint32x4_t uint4x32_to_uint32_uniform_vec(uint4x32_t x) {
  uint32x4_t r; for (int i = 0; i < 4; ++i) r.v[i] = x.v[i]; return r;
}
static inline int64x2_t uint4x32_to_int64_uniform_vec(uint4x32_t x) {
  int64x2_t r; r.v[0] = (int64_t)ocn_lo64(x); r.v[1] = (int64_t)ocn_hi64(x); return r;
}
static inline uint64x2_t uint4x32_to_uint64_uniform_vec(uint4x32_t x) {
  uint64x2_t r; r.v[0] = ocn_lo64(x); r.v[1] = ocn_hi64(x); return r;
}
static inline int8x16_t uint4x32_to_byte_uniform_vec(uint4x32_t x) {
  int8x16_t r; for (int i = 0; i < 16; ++i) r.v[i] = (int8_t)((x.v[i / 4] >> (8 * (i % 4))) & 0xFFu); return r;
}
static inline uint16x8_t uint4x32_to_uint16_uniform_vec(uint4x32_t x) {
  uint16x8_t r; for (int i = 0; i < 8; ++i) r.v[i] = (uint16_t)((x.v[i / 2] >> (16 * (i % 2))) & 0xFFFFu); return r;
}
static inline uint16x8_t uint4x32_to_bfloat16_uniform_vec(uint4x32_t x) {
  uint16x8_t r;
  for (int i = 0; i < 8; ++i)
    r.v[i] = ocn_bf16_rne_bits((float)((x.v[i / 2] >> (16 * (i % 2))) & 0xFFFFu) * 0x1p-16f);
  return r;
}
static inline half8_t uint4x32_to_half_uniform_vec(uint4x32_t x) {
  half8_t r;
  for (int i = 0; i < 8; ++i)
    r.v[i] = FLOAT_TO_HALF((float)((x.v[i / 2] >> (16 * (i % 2))) & 0xFFFFu) * 0x1p-16f);
  return r;
}
static inline uint8x16_t uint4x32_to_fp8_uniform_vec(uint4x32_t x) {
  uint8x16_t r; for (int i = 0; i < 16; ++i) r.v[i] = (uint8_t)((x.v[i / 4] >> (8 * (i % 4))) & 0xFFu); return r;
}

/* ---- X -> uint4x32 ------------------------------------------------------------------- */
static inline uint4x32_t ocn_u4(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  uint4x32_t r; r.v[0] = a; r.v[1] = b; r.v[2] = c; r.v[3] = d; return r;
}
/* 32-bit integers are spread over the four words so that consecutive counters differ in
   every word (builtins.c:545-576): x, x^golden, x^mmix, x^rot16(x). */
static inline uint4x32_t uint32_to_uint4x32(uint32_t x) {
  return ocn_u4(x, x ^ 0x9E3779B9u, x ^ 0x6C078965u, x ^ ocn_rotl(x, 16));
}
static inline uint4x32_t int32_to_uint4x32(int32_t x) { return uint32_to_uint4x32((uint32_t)x); }
static inline uint4x32_t uint64_to_uint4x32(uint64_t x) { return ocn_u4((uint32_t)x, (uint32_t)(x >> 32), 0, 0); }
static inline uint4x32_t int64_to_uint4x32(int64_t x) { return uint64_to_uint4x32((uint64_t)x); }
static inline uint4x32_t single_to_uint4x32(float x) { uint32_t b; memcpy(&b, &x, 4); return ocn_u4(b, 0, 0, 0); }
static inline uint4x32_t double_to_uint4x32(double x) { uint64_t b; memcpy(&b, &x, 8); return uint64_to_uint4x32(b); }
static inline uint4x32_t byte_to_uint4x32(unsigned char x) { return ocn_u4(x, 0, 0, 0); }
static inline uint4x32_t uint16_to_uint4x32(uint16_t x) { return ocn_u4(x, 0, 0, 0); }
static inline uint4x32_t bfloat16_to_uint4x32(uint16_t x) { return ocn_u4(x, 0, 0, 0); }
static inline uint4x32_t half_to_uint4x32(uint16_t x) { return ocn_u4(x, 0, 0, 0); }
static inline uint4x32_t fp8_to_uint4x32(uint8_t x) { return ocn_u4(x, 0, 0, 0); }

/* ---- bf16 / fp8 ---------------------------------------------------------------------- */
static inline float bfloat16_to_single(uint16_t b) {
  uint32_t w = (uint32_t)b << 16; float f; memcpy(&f, &w, 4); return f;
}
/* round-to-nearest-even by adding 0x7FFF + lsb; NaN payloads are not special-cased
   (builtins.c:620-627). */
static inline uint16_t single_to_bfloat16(float f) {
  uint32_t w; memcpy(&w, &f, 4);
  return (uint16_t)((w + 0x7FFFu + ((w >> 16) & 1u)) >> 16);
}
/* E5M2, bias 15 (builtins.c:646-743) */
static inline float fp8_to_single(uint8_t v) {
  if (v == 0) return 0.0f;
  const uint32_t s = v >> 7, e = (v >> 2) & 31u, m = v & 3u;
  float r;
  if (e == 31u) { if (m) return NAN; r = INFINITY; }
  else if (e == 0u) r = ldexpf((float)m / 4.0f, -14);
  else r = (1.0f + (float)m * 0.25f) * ldexpf(1.0f, (int)e - 15);
  return s ? -r : r;
}
static inline uint8_t single_to_fp8(float f) {
  if (f == 0.0f) return 0;
  const uint32_t s = (f < 0) ? 1u : 0u;
  f = fabsf(f);
  if (isinf(f)) return (uint8_t)((s << 7) | 0x7Cu);
  if (isnan(f)) return (uint8_t)((s << 7) | 0x7Fu);
  int ev; float mf = frexpf(f, &ev);           /* f = mf * 2^ev, mf in [0.5, 1) */
  const int e = ev + 14;
  if (e < 0) return (uint8_t)(s << 7);
  if (e > 30) return (uint8_t)((s << 7) | 0x7Cu);
  uint32_t mb;
  if (e == 0) {
    mb = (uint32_t)(f * ldexpf(1.0f, 14) * 4.0f + 0.5f);
    if (mb > 3u) mb = 3u;
    return (uint8_t)((s << 7) | mb);
  }
  mb = (uint32_t)((mf - 0.5f) * 4.0f + 0.5f);   /* NB: reference maps [0.5,1) to 2 bits so */
  if (mb > 3u) mb = 3u;                         /* only mantissa codes 0..2 are produced   */
  return (uint8_t)((s << 7) | (((uint32_t)e & 31u) << 2) | (mb & 3u));
}
