// Device-side scalar builtins prepended to every generated HIP module.
//
// Same names and results as the C builtins OCANNL's generated code calls
// (arrayjit/lib/builtins.c:11-743; call sites are produced from arrayjit/lib/ops.ml:579-876), so
// that a routine computes on gfx950 what the `cc` backend computes on the host:
//   bf16 <-> float  builtins.c:611-627      fp8 (E5M2) <-> float  builtins.c:646-743
//   half            native _Float16 (builtins.c:12-21 "HAS_NATIVE_FLOAT16" arm)
//   threefry4x32    builtins.c:156-329      uint4x32 -> uniform   builtins.c:345-528
//   X -> uint4x32   builtins.c:531-606
// This text is compiled by hiprtc (which predeclares the fixed-width integer types and the math
// library) and, for a syntax check, by hipcc via builtins_check.hip.
#pragma once

#ifdef __HIPCC_RTC__
typedef unsigned int uint32_t;
typedef int int32_t;
typedef unsigned long long uint64_t;
typedef long long int64_t;
#endif

#define OCN_DEV __device__ __forceinline__
#ifndef INFINITY
#define INFINITY __builtin_huge_valf()
#endif
#ifndef NAN
#define NAN __builtin_nanf("")
#endif

#define HALF_T _Float16
#define HALF_TO_FP(x) (x)
#define FP_TO_HALF(x) (x)
#define HALF_TO_FLOAT(x) ((float)(x))
#define FLOAT_TO_HALF(x) ((_Float16)(x))

struct uint4x32_t { uint32_t v[4]; };
struct float4_t { float v[4]; };
struct double2_t { double v[2]; };
struct int32x4_t { int32_t v[4]; };
struct uint32x4_t { uint32_t v[4]; };
struct int64x2_t { long long v[2]; };
struct uint64x2_t { uint64_t v[2]; };
struct int8x16_t { signed char v[16]; };
struct uint16x8_t { unsigned short v[8]; };
struct uint8x16_t { unsigned char v[16]; };
struct half8_t { _Float16 v[8]; };

// ---- bf16 / fp8 ---------------------------------------------------------------------------------
OCN_DEV float bfloat16_to_single(unsigned short b) { return __uint_as_float(((uint32_t)b) << 16); }
// Round to nearest even through the integer add of the host code (builtins.c:620-627), NaN
// included: three VALU operations (bit extract, three-operand add, shift), and the shift folds into
// the mask of a following bfloat16_to_single.  (The hardware conversion gives the same bits for every
// non-NaN input but needs a NaN guard around it to stay exact, which costs more than it saves.)
OCN_DEV unsigned short single_to_bfloat16(float f) {
  const uint32_t w = __float_as_uint(f);
  return (unsigned short)((w + 0x7FFFu + ((w >> 16) & 1u)) >> 16);
}
OCN_DEV float fp8_to_single(unsigned char v) {
  if (v == 0) return 0.0f;
  const uint32_t sgn = v >> 7, e = (v >> 2) & 31u, m = v & 3u;
  float r;
  if (e == 31u) { if (m) return NAN; r = INFINITY; }
  else if (e == 0u) r = ldexpf((float)m * 0.25f, -14);
  else r = (1.0f + (float)m * 0.25f) * ldexpf(1.0f, (int)e - 15);
  return sgn ? -r : r;
}
OCN_DEV unsigned char single_to_fp8(float f) {
  if (f == 0.0f) return 0;
  const uint32_t sgn = f < 0 ? 1u : 0u;
  f = fabsf(f);
  if (isinf(f)) return (unsigned char)((sgn << 7) | 0x7Cu);
  if (isnan(f)) return (unsigned char)((sgn << 7) | 0x7Fu);
  int ev;
  const float mf = frexpf(f, &ev);
  const int e = ev + 14;
  if (e < 0) return (unsigned char)(sgn << 7);
  if (e > 30) return (unsigned char)((sgn << 7) | 0x7Cu);
  uint32_t mb;
  if (e == 0) {
    mb = (uint32_t)(f * 16384.0f * 4.0f + 0.5f);
    if (mb > 3u) mb = 3u;
    return (unsigned char)((sgn << 7) | mb);
  }
  mb = (uint32_t)((mf - 0.5f) * 4.0f + 0.5f);
  if (mb > 3u) mb = 3u;
  return (unsigned char)((sgn << 7) | (((uint32_t)e & 31u) << 2) | mb);
}

// ---- threefry4x32 -------------------------------------------------------------------------------
OCN_DEV uint32_t ocn_rotl32(uint32_t x, uint32_t n) { return (x << n) | (x >> (32u - n)); }
#define OCN_TF_MIX(x, ra, rb)                                   \
  x.v[0] += x.v[1]; x.v[1] = ocn_rotl32(x.v[1], ra) ^ x.v[0];   \
  x.v[2] += x.v[3]; x.v[3] = ocn_rotl32(x.v[3], rb) ^ x.v[2];   \
  { const uint32_t t_ = x.v[1]; x.v[1] = x.v[3]; x.v[3] = t_; }
// The reference's "round" = two mix+swap layers; rotation sets alternate (builtins.c:163-196).
#define OCN_TF_EVEN(x) OCN_TF_MIX(x, 13u, 15u) OCN_TF_MIX(x, 26u, 6u)
#define OCN_TF_ODD(x) OCN_TF_MIX(x, 17u, 29u) OCN_TF_MIX(x, 16u, 24u)
OCN_DEV uint4x32_t arrayjit_threefry4x32_light(uint4x32_t key, uint4x32_t ctr) {
  const uint32_t k4 = key.v[0] ^ key.v[1] ^ key.v[2] ^ key.v[3] ^ 0x1BD11BDAu;
  uint4x32_t x;
  for (int i = 0; i < 4; ++i) x.v[i] = ctr.v[i] + key.v[i];
  OCN_TF_EVEN(x) OCN_TF_ODD(x)
  x.v[0] += key.v[1]; x.v[1] += key.v[2]; x.v[2] += key.v[3]; x.v[3] += k4 + 1u;
  return x;
}
OCN_DEV uint4x32_t arrayjit_threefry4x32_crypto(uint4x32_t key, uint4x32_t ctr) {
  uint32_t ks[5];
  ks[4] = 0x1BD11BDAu;
  uint4x32_t x;
  for (int i = 0; i < 4; ++i) { ks[i] = key.v[i]; ks[4] ^= key.v[i]; x.v[i] = ctr.v[i] + key.v[i]; }
#pragma unroll
  for (uint32_t g = 1; g <= 5; ++g) {   // 20 "rounds", key injection after every 4 (builtins.c:199-281)
    OCN_TF_EVEN(x) OCN_TF_ODD(x) OCN_TF_EVEN(x) OCN_TF_ODD(x)
    for (uint32_t i = 0; i < 4; ++i) x.v[i] += ks[(g + i) % 5u];
    x.v[3] += g;
  }
  return x;
}
OCN_DEV uint4x32_t arrayjit_threefry4x32(uint4x32_t key, uint4x32_t ctr) {
  return arrayjit_threefry4x32_light(key, ctr);
}

// ---- uint4x32 -> uniform ------------------------------------------------------------------------
OCN_DEV float uint32_to_single_uniform(uint32_t x) { return (float)(x >> 8) * 5.9604644775390625e-08f; }
OCN_DEV double uint32_to_double_uniform(uint32_t x) { return (double)x * 2.3283064365386963e-10; }
OCN_DEV uint64_t ocn_lo64(uint4x32_t x) { return ((uint64_t)x.v[1] << 32) | x.v[0]; }
OCN_DEV uint64_t ocn_hi64(uint4x32_t x) { return ((uint64_t)x.v[3] << 32) | x.v[2]; }
OCN_DEV unsigned short ocn_bf16_guard_round(float f) {   // builtins.c:397-406
  const uint32_t b = __float_as_uint(f);
  unsigned short r = (unsigned short)(b >> 16);
  if ((b & 0x8000u) && ((b & 0x7FFFu) || (r & 1u))) r++;
  return r;
}
OCN_DEV float ocn_u16_unit(uint32_t w, int hi) { return (float)((w >> (hi ? 16 : 0)) & 0xFFFFu) * 1.52587890625e-05f; }
OCN_DEV float uint4x32_to_single_uniform(uint4x32_t x) { return uint32_to_single_uniform(x.v[0]); }
OCN_DEV double uint4x32_to_double_uniform(uint4x32_t x) { return (double)ocn_lo64(x) * 5.421010862427522e-20; }
OCN_DEV int uint4x32_to_int32_uniform(uint4x32_t x) { return (int)x.v[0]; }
OCN_DEV long long uint4x32_to_int64_uniform(uint4x32_t x) { return (long long)ocn_lo64(x); }
OCN_DEV uint32_t uint4x32_to_uint32_uniform(uint4x32_t x) { return x.v[0]; }
OCN_DEV uint64_t uint4x32_to_uint64_uniform(uint4x32_t x) { return ocn_lo64(x); }
OCN_DEV signed char uint4x32_to_byte_uniform(uint4x32_t x) { return (signed char)(x.v[0] & 0xFFu); }
OCN_DEV unsigned short uint4x32_to_uint16_uniform(uint4x32_t x) { return (unsigned short)(x.v[0] & 0xFFFFu); }
OCN_DEV unsigned short uint4x32_to_bfloat16_uniform(uint4x32_t x) { return ocn_bf16_guard_round(uint32_to_single_uniform(x.v[0])); }
OCN_DEV _Float16 uint4x32_to_half_uniform(uint4x32_t x) { return (_Float16)ocn_u16_unit(x.v[0], 0); }
OCN_DEV unsigned char uint4x32_to_fp8_uniform(uint4x32_t x) { return (unsigned char)(x.v[0] & 0xFFu); }

OCN_DEV float4_t uint4x32_to_single_uniform_vec(uint4x32_t x) {
  float4_t r; for (int i = 0; i < 4; ++i) r.v[i] = uint32_to_single_uniform(x.v[i]); return r; }
OCN_DEV double2_t uint4x32_to_double_uniform_vec(uint4x32_t x) {
  double2_t r; r.v[0] = (double)ocn_lo64(x) * 5.421010862427522e-20; r.v[1] = (double)ocn_hi64(x) * 5.421010862427522e-20; return r; }
OCN_DEV int32x4_t uint4x32_to_int32_uniform_vec(uint4x32_t x) {
  int32x4_t r; for (int i = 0; i < 4; ++i) r.v[i] = (int32_t)x.v[i]; return r; }
OCN_DEV uint32x4_t uint4x32_to_uint32_uniform_vec(uint4x32_t x) {
  uint32x4_t r; for (int i = 0; i < 4; ++i) r.v[i] = x.v[i]; return r; }
OCN_DEV int64x2_t uint4x32_to_int64_uniform_vec(uint4x32_t x) {
  int64x2_t r; r.v[0] = (long long)ocn_lo64(x); r.v[1] = (long long)ocn_hi64(x); return r; }
OCN_DEV uint64x2_t uint4x32_to_uint64_uniform_vec(uint4x32_t x) {
  uint64x2_t r; r.v[0] = ocn_lo64(x); r.v[1] = ocn_hi64(x); return r; }
OCN_DEV int8x16_t uint4x32_to_byte_uniform_vec(uint4x32_t x) {
  int8x16_t r; for (int i = 0; i < 16; ++i) r.v[i] = (signed char)((x.v[i >> 2] >> (8 * (i & 3))) & 0xFFu); return r; }
OCN_DEV uint16x8_t uint4x32_to_uint16_uniform_vec(uint4x32_t x) {
  uint16x8_t r; for (int i = 0; i < 8; ++i) r.v[i] = (unsigned short)((x.v[i >> 1] >> (16 * (i & 1))) & 0xFFFFu); return r; }
OCN_DEV uint16x8_t uint4x32_to_bfloat16_uniform_vec(uint4x32_t x) {
  uint16x8_t r; for (int i = 0; i < 8; ++i) r.v[i] = ocn_bf16_guard_round(ocn_u16_unit(x.v[i >> 1], i & 1)); return r; }
OCN_DEV half8_t uint4x32_to_half_uniform_vec(uint4x32_t x) {
  half8_t r; for (int i = 0; i < 8; ++i) r.v[i] = (_Float16)ocn_u16_unit(x.v[i >> 1], i & 1); return r; }
OCN_DEV uint8x16_t uint4x32_to_fp8_uniform_vec(uint4x32_t x) {
  uint8x16_t r; for (int i = 0; i < 16; ++i) r.v[i] = (unsigned char)((x.v[i >> 2] >> (8 * (i & 3))) & 0xFFu); return r; }

// ---- X -> uint4x32 ------------------------------------------------------------------------------
OCN_DEV uint4x32_t ocn_u4(uint32_t a, uint32_t b, uint32_t c, uint32_t d) { uint4x32_t r; r.v[0] = a; r.v[1] = b; r.v[2] = c; r.v[3] = d; return r; }
// 32-bit counters are spread over all four words (builtins.c:545-576)
OCN_DEV uint4x32_t uint32_to_uint4x32(uint32_t x) { return ocn_u4(x, x ^ 0x9E3779B9u, x ^ 0x6C078965u, x ^ ocn_rotl32(x, 16u)); }
OCN_DEV uint4x32_t int32_to_uint4x32(int x) { return uint32_to_uint4x32((uint32_t)x); }
OCN_DEV uint4x32_t uint64_to_uint4x32(uint64_t x) { return ocn_u4((uint32_t)x, (uint32_t)(x >> 32), 0u, 0u); }
OCN_DEV uint4x32_t int64_to_uint4x32(long long x) { return uint64_to_uint4x32((uint64_t)x); }
OCN_DEV uint4x32_t single_to_uint4x32(float x) { return ocn_u4(__float_as_uint(x), 0u, 0u, 0u); }
OCN_DEV uint4x32_t double_to_uint4x32(double x) { return uint64_to_uint4x32((uint64_t)__double_as_longlong(x)); }
OCN_DEV uint4x32_t byte_to_uint4x32(unsigned char x) { return ocn_u4(x, 0u, 0u, 0u); }
OCN_DEV uint4x32_t uint16_to_uint4x32(unsigned short x) { return ocn_u4(x, 0u, 0u, 0u); }
OCN_DEV uint4x32_t bfloat16_to_uint4x32(unsigned short x) { return ocn_u4(x, 0u, 0u, 0u); }
OCN_DEV uint4x32_t half_to_uint4x32(unsigned short x) { return ocn_u4(x, 0u, 0u, 0u); }
OCN_DEV uint4x32_t fp8_to_uint4x32(unsigned char x) { return ocn_u4(x, 0u, 0u, 0u); }

// ---- lane-group combine used by cooperative reductions ------------------------------------------
OCN_DEV float ocn_xshfl(float v, int m) { return __shfl_xor(v, m, 64); }
OCN_DEV double ocn_xshfl(double v, int m) { return __shfl_xor(v, m, 64); }

// ---- a contraction as the prologue of a row-wise kernel ---------------------------------------------
// xs[32][T] = A[32][K] * B[T][K]^T for a workgroup of NW waves: bf16 operands, both unit-stride
// along K, fp32 accumulation on the matrix cores (v_mfma_f32_32x32x16_bf16), results rounded to XT
// (bf16 bits or float) in LDS.  The workgroup's NW waves take the T / 32 column tiles in turn.  The MFMA
// fragments come straight from memory: a lane supplies row (lane % 32) of its operand at
// k = 8 * (lane / 32) .. + 7 of each 16-k sub-step (16 bytes), and receives column (lane % 32) of the
// 32 x 32 result at rows 8 * (e / 4) + 4 * (lane / 32) + e % 4.
typedef __bf16 ocn_bf16x8 __attribute__((ext_vector_type(8)));
typedef float ocn_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int ocn_u32x4 __attribute__((ext_vector_type(4)));

OCN_DEV void ocn_rowtile_put(unsigned short* p, float v) { *p = single_to_bfloat16(v); }
OCN_DEV void ocn_rowtile_put(float* p, float v) { *p = v; }

template <int T, int K, int NW, typename XT, int XS = T>   // XS: elements from row to row of xs
__device__ __forceinline__ void ocn_rowtile_contract(const unsigned short* __restrict__ a, long long a_row,
                                                     const unsigned short* __restrict__ b, long long b_row, XT* xs) {
  static_assert(T % 32 == 0 && K % 16 == 0 && K <= 128, "row tile: T in steps of 32, K in steps of 16 up to 128");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;   // NW waves share the T / 32 column tiles
  constexpr int KS = K / 16;
  if (wave >= T / 32) return;
  ocn_bf16x8 af[KS];
  const unsigned short* ap = a + (long long)(lane & 31) * a_row + (lane >> 5) * 8;
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) af[kk] = __builtin_bit_cast(ocn_bf16x8, *reinterpret_cast<const ocn_u32x4*>(ap + kk * 16));
#pragma unroll
  for (int t = 0; t < (T / 32 + NW - 1) / NW; ++t) {
    const int n0 = (wave + t * NW) * 32;
    if (n0 >= T) break;
    const unsigned short* bp = b + (long long)(n0 + (lane & 31)) * b_row + (lane >> 5) * 8;
    ocn_bf16x8 bf[KS];
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) bf[kk] = __builtin_bit_cast(ocn_bf16x8, *reinterpret_cast<const ocn_u32x4*>(bp + kk * 16));
    ocn_f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk], bf[kk], acc, 0, 0, 0);
    XT* out = xs + ((lane >> 5) * 4) * XS + n0 + (lane & 31);
#pragma unroll
    for (int e = 0; e < 16; ++e) ocn_rowtile_put(out + ((e >> 2) * 8 + (e & 3)) * XS, acc[e]);
  }
}

// Row group with a contraction epilogue: the workgroup's 32 finished rows y[32][T] (bf16 bits in LDS,
// YS elements from row to row) times b[T][N] (bf16 in memory, unit stride along n, b_row elements from
// t to t + 1) give c[32][N] (c_row elements from row to row; `copy`, when given, receives the same
// values as bf16 at the same offsets).  Wave w takes the 32-column block w % (N / 32) and part
// w / (N / 32) of the KP parts of T; with KP > 1 the partial results meet in `ps` (LDS, KP x 32 x N
// floats) and are added in a fixed order.  Every wave of the workgroup calls it (it holds a barrier).
OCN_DEV void ocn_rowtile_put4(unsigned short* p, const float* v) {
  typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
  u32x2 w;
  w[0] = (unsigned int)single_to_bfloat16(v[0]) | ((unsigned int)single_to_bfloat16(v[1]) << 16);
  w[1] = (unsigned int)single_to_bfloat16(v[2]) | ((unsigned int)single_to_bfloat16(v[3]) << 16);
  *reinterpret_cast<u32x2*>(p) = w;
}
OCN_DEV void ocn_rowtile_put4(float* p, const float* v) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  f32x4 w;
  w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
  *reinterpret_cast<f32x4*>(p) = w;
}

template <int T, int N, int NW, int KP, int YS, typename CT>
__device__ __forceinline__ void ocn_rowtile_project(const unsigned short* ys, const unsigned short* __restrict__ b, long long b_row,
                                                    float* ps, CT* __restrict__ c, long long c_row, unsigned short* __restrict__ copy) {
  static_assert(T % (16 * KP) == 0 && N % 32 == 0 && (N / 32) * KP <= NW, "row-tile epilogue: shape");
  constexpr int NB = N / 32, KS = T / 16 / KP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave < NB * KP) {
    const int nb = wave % NB, kp = wave / NB;
    ocn_f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
    const unsigned short* yp = ys + (lane & 31) * YS + kp * (KS * 16) + (lane >> 5) * 8;
    const unsigned short* bp = b + (long long)(kp * (KS * 16) + (lane >> 5) * 8) * b_row + nb * 32 + (lane & 31);
#pragma unroll 4
    for (int kk = 0; kk < KS; ++kk) {
      const ocn_bf16x8 af = __builtin_bit_cast(ocn_bf16x8, *reinterpret_cast<const ocn_u32x4*>(yp + kk * 16));
      ocn_u32x4 bw;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        bw[j] = (unsigned int)bp[(long long)(kk * 16 + 2 * j) * b_row] | ((unsigned int)bp[(long long)(kk * 16 + 2 * j + 1) * b_row] << 16);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, __builtin_bit_cast(ocn_bf16x8, bw), acc, 0, 0, 0);
    }
    const int col = nb * 32 + (lane & 31);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int row = (e >> 2) * 8 + (e & 3) + (lane >> 5) * 4;
      if (KP > 1) ps[(kp * 32 + row) * N + col] = acc[e];
      else {
        ocn_rowtile_put(c + row * c_row + col, acc[e]);
        if (copy) copy[row * c_row + col] = single_to_bfloat16(acc[e]);
      }
    }
  }
  if (KP > 1) {
    __syncthreads();
    for (int idx = threadIdx.x; idx < 32 * N / 4; idx += NW * 64) {
      const int row = idx / (N / 4), c4 = (idx % (N / 4)) * 4;
      float v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = ps[row * N + c4 + q];
#pragma unroll
      for (int p = 1; p < KP; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] += ps[(p * 32 + row) * N + c4 + q];
      ocn_rowtile_put4(c + row * c_row + c4, v);
      if (copy) ocn_rowtile_put4(copy + row * c_row + c4, v);
    }
  }
}
