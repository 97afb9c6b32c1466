// Device-side helpers shared by the MFMA contraction kernels (gemm.hip, gemm_dtl.hpp): register
// types, batch / group decoding, the XCD-aware tile order, register staging of operand tiles, the
// ds_read_b64_tr_b16 fragment read and the epilogue that takes a wave's accumulator tiles to memory.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>
#include <utility>

#include "gemm.hpp"

namespace ocannl {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Compile-time loop: the accumulator array is only ever indexed by constants, so it stays in
// registers whatever the unroller decides.  The loop bodies are lambdas that must be inlined too
// (a body left as a call would take the accumulators' address and push them to scratch memory).
#define OCN_LAMBDA_INLINE __attribute__((always_inline))
template <int N, typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl<N>(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

constexpr int kThreads = 256;
constexpr int kBK = 64;        // K elements per stage (bf16 compute)
constexpr int kPad = 8;        // bf16 elements of row padding (16 bytes)
constexpr int kBKf = 32;       // K elements per stage (fp32 compute)
constexpr int kPadf = 4;       // floats of row padding (16 bytes)

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
// fp32 -> bf16, round to nearest even, in hardware (v_cvt_pk_bf16_f32).  Equal to
// single_to_bfloat16 for every input that is not a NaN.
__device__ __forceinline__ unsigned f2bf(float f) { return __builtin_bit_cast(unsigned short, (__bf16)f); }
__device__ __forceinline__ unsigned pack2(float lo, float hi) {
  return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{lo, hi}, bf16x2_t));
}

// Raw staging type of 8 consecutive source elements: bf16 sources travel as one 16-byte vector,
// fp32 sources as two; the fp32 -> bf16 rounding happens when the registers are written to LDS, so
// that the global loads stay in flight while the previous tile is being multiplied.
template <typename T> struct Raw8;
template <> struct Raw8<unsigned short> {
  u32x4 v;
  __device__ __forceinline__ void zero() { v = u32x4{0, 0, 0, 0}; }
  __device__ __forceinline__ void load(const unsigned short* p) { v = *reinterpret_cast<const u32x4*>(p); }
  __device__ __forceinline__ u32x4 bf16() const { return v; }
};
template <> struct Raw8<float> {
  f32x4 lo, hi;
  __device__ __forceinline__ void zero() { lo = f32x4{0, 0, 0, 0}; hi = lo; }
  __device__ __forceinline__ void load(const float* p) {
    lo = *reinterpret_cast<const f32x4*>(p);
    hi = *reinterpret_cast<const f32x4*>(p + 4);
  }
  __device__ __forceinline__ u32x4 bf16() const {
    return u32x4{pack2(lo.x, lo.y), pack2(lo.z, lo.w), pack2(hi.x, hi.y), pack2(hi.z, hi.w)};
  }
};

// Batch index -> element offsets.  Written with constant array indices only: a runtime index into
// the by-value argument struct would force the whole struct into scratch memory.
__device__ __forceinline__ void decode_batch(const GemmArgs& g, long z, long& ao, long& bo, long& co) {
  ao = bo = co = 0;
  if (g.nbatch > 2) { const long e = g.batch_ext[2], q = z % e; z /= e; ao += q * g.a_batch[2]; bo += q * g.b_batch[2]; co += q * g.c_batch[2]; }
  if (g.nbatch > 1) { const long e = g.batch_ext[1], q = z % e; z /= e; ao += q * g.a_batch[1]; bo += q * g.b_batch[1]; co += q * g.c_batch[1]; }
  if (g.nbatch > 0) { const long e = g.batch_ext[0], q = z % e; ao += q * g.a_batch[0]; bo += q * g.b_batch[0]; co += q * g.c_batch[0]; }
}

// Grouped launch: blockIdx.z = group * batches + batch.  Returns the batch index and the operands of
// the group (constant array indices only, as above).
__device__ __forceinline__ long decode_group(const GemmArgs& g, long z, const void*& a, const void*& b, void*& c, void*& c2) {
  a = g.a; b = g.b; c = g.c; c2 = g.c2;
  if (g.ngroups > 1) {
    const long grp = z / g.batches;
    z -= grp * g.batches;
    if (grp == 1) { a = g.a_more[0]; b = g.b_more[0]; c = g.c_more[0]; c2 = g.c2_more[0]; }
    else if (grp == 2) { a = g.a_more[1]; b = g.b_more[1]; c = g.c_more[1]; c2 = g.c2_more[1]; }
    else if (grp == 3) { a = g.a_more[2]; b = g.b_more[2]; c = g.c_more[2]; c2 = g.c2_more[2]; }
  }
  return z;
}

// XCD-aware tile order.  Consecutive hardware workgroup ids land on different XCDs (id % 8), each
// with its own L2.  The tile grid is cut into xcd_m x (8 / xcd_m) rectangles, one per XCD, chosen
// on the host so that the operand panels shared inside a rectangle are the expensive ones
// (fewest bytes re-read across XCDs).  Inside its rectangle an XCD walks column-bands of 8
// row-tiles, so that tiles running at the same time share B panels.
// `nx`: the number of XCDs the tile grid is spread over (8, or fewer when the members of a grouped
// launch each keep to their own XCDs); wg % nx then names the XCD among them.
__device__ __forceinline__ void tile_of_block(long wg, long tiles_m, long tiles_n, int xcd_m, int nx, long& tm, long& tn) {
  long t = wg, rm = tiles_m, rn = tiles_n, m_off = 0, n_off = 0;
  if (xcd_m > 0) {
    const int xcd_n = nx / xcd_m;
    const long x = wg % nx;
    rm = tiles_m / xcd_m; rn = tiles_n / xcd_n;
    m_off = (x / xcd_n) * rm; n_off = (x % xcd_n) * rn;
    t = wg / nx;
  }
  constexpr long kGroup = 8;
  const long band = kGroup * rn;
  const long g = t / band;
  const long first_m = g * kGroup;
  const long gm = (rm - first_m) < kGroup ? (rm - first_m) : kGroup;
  const long r = t % band;
  tm = m_off + first_m + r % gm;
  tn = n_off + r / gm;
}

// Workgroup -> (tile-grid workgroup id, z index = member * batches + batch, XCDs sharing the grid).
// Grouped launches with member_xcds > 0 give each member XCDs of its own (member m owns XCDs
// m * member_xcds ... ): its operand panels then fill 8 / ngroups L2 caches instead of all eight.
// The hardware deals workgroups to the XCDs round robin in dispatch order (x fastest, then z here:
// such launches have no split along y).
__device__ __forceinline__ void place_workgroup(const GemmArgs& g, long& wg, long& z, int& nx) {
  wg = blockIdx.x; z = blockIdx.z; nx = 8;
  if (g.member_xcds > 0) {
    const long linear = z * gridDim.x + wg;
    const long xcd = linear & 7, slot = linear >> 3;
    nx = g.member_xcds;
    z = xcd / nx;                 // the member (one batch entry each)
    wg = slot * nx + xcd % nx;
  }
}

// ---- staging one operand tile: global -> registers -> LDS --------------------------------------
// ROWS x kBK tile starting at (row0, k0); a thread owns 16-byte chunks (8 elements, converted to
// bf16 on the way to LDS).
//   K-contiguous operand:   chunk = 8 k of one row;  LDS holds [row][k], row stride kBK + kPad.
//   row-contiguous operand: chunk = 8 rows of one k; LDS holds [k][row], row stride ROWS + kPadT --
//     the tile is NOT transposed on the way in: the MFMA fragments are read with
//     ds_read_b64_tr_b16, which hands a lane the four k values of its own row (see tr_fragment).
// Either way global loads and LDS writes are plain 16-byte accesses, adjacent lanes adjacent.
constexpr int kPadT = 32;   // bf16 elements of padding per k-row of a [k][row] tile: consecutive k
                            // rows start 64 bytes apart modulo the 256-byte bank cycle

template <int ROWS, bool KC>
constexpr int lds_tile_elems() { return KC ? ROWS * (kBK + kPad) : kBK * (ROWS + kPadT); }

template <int ROWS, typename T, bool KC>
struct Stager {
  static constexpr int kChunks = ROWS * (kBK / 8) / kThreads;   // chunks per thread
  static constexpr int kPerLine = KC ? kBK / 8 : ROWS / 8;       // chunks per contiguous line
  static constexpr int kLineStride = KC ? kBK + kPad : ROWS + kPadT;   // LDS elements per line
  static constexpr int kLinesPerOp = kThreads / kPerLine;        // lines covered by one op of the workgroup
  Raw8<T> regs[kChunks];

  // checked version for ragged tiles: `rows` / `K` are the operand's extents
  __device__ __forceinline__ void load(const T* base, long ld, long row0, long k0, long rows, long K, int tid) {
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int c = tid + kThreads * j;
      const long line = c / kPerLine, pos = (c % kPerLine) * 8;
      regs[j].zero();
      if (KC) { if (row0 + line < rows && k0 + pos < K) regs[j].load(base + (row0 + line) * ld + k0 + pos); }
      else    { if (k0 + line < K && row0 + pos < rows) regs[j].load(base + (k0 + line) * ld + row0 + pos); }
    }
  }

  __device__ __forceinline__ void store(unsigned short* lds, int tid) const {
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int c = tid + kThreads * j;
      *reinterpret_cast<u32x4*>(lds + (c / kPerLine) * kLineStride + (c % kPerLine) * 8) = regs[j].bf16();
    }
  }

  // The same work cut into single instructions for the interleaved main loop of full tiles (no
  // bounds checks): kOps loads, then kOps LDS writes, in matching order.  An address is a part
  // that is uniform over the workgroup (tile origin, op number: scalar registers / immediates) plus
  // one per-thread 32-bit offset computed once by init_ops().
  static constexpr int kOps = kChunks;
  unsigned goff, loff;

  __device__ __forceinline__ void init_ops(long ld, int tid) {
    goff = (unsigned)((tid / kPerLine) * ld + (tid % kPerLine) * 8);
    loff = (tid / kPerLine) * kLineStride + (tid % kPerLine) * 8;
  }

  // `origin` points at the tile's first element: uniform.
  template <int I>
  __device__ __forceinline__ void load_op(const T* origin, long ld) {
    regs[I].load(origin + (long)(I * kLinesPerOp) * ld + goff);
  }

  template <int I>
  __device__ __forceinline__ void store_op(unsigned short* lds) const {
    *reinterpret_cast<u32x4*>(lds + loff + I * kLinesPerOp * kLineStride) = regs[I].bf16();
  }
};

// MFMA fragment (row = lane % 32 of a 32-row block, k = 8 * (lane / 32) + 0..7 of a 16-k sub-step)
// out of a [k][row] tile.  ds_read_b64_tr_b16 works on groups of 16 lanes: lane p of a group
// supplies the address of four consecutive 16-bit words, and receives word p % 4 of the chunks
// supplied by lanes p / 4, p / 4 + 4, p / 4 + 8, p / 4 + 12.  With lane 4 j + q pointing at
// (k = j, rows 4 q .. 4 q + 3), lane p gets row p at k = 0..3: its own row, four consecutive k.
// `tile` points at (k = 0, row = 0) of the 16-k sub-step and the 32-row block.
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ unsigned tr_lane_offset(int lane, int line_stride) {
  const int p = lane & 15;
  return (unsigned)(((lane >> 5) * 8 + (p >> 2)) * line_stride + ((lane >> 4) & 1) * 16 + (p & 3) * 4);
}
__device__ __forceinline__ bf16x8 tr_fragment(const unsigned short* at_lane, int line_stride) {
  typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(at_lane));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(at_lane + 4 * line_stride));
  return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// ---- epilogue -----------------------------------------------------------------------------------
// One wave's block of TM x TN accumulator tiles -> memory, one row of tiles (32 x TN*32) at a
// time.  In a 32x32 tile the lane holds column lane % 32 and register e holds row
// 8 * (e / 4) + 4 * (lane / 32) + e % 4, so one store instruction writes two 32-element row
// pieces.  The address of an element splits into a part that is uniform over the wave (tile
// origin + compile-time row/column: scalar registers) and one 32-bit per-lane offset computed
// once.  ACC loads the whole row of tiles before the first store, so that TN * 16 reads are in
// flight; CHECK guards ragged edges.
// kOutF32Copy: fp32 result plus its bf16 rounding at the same element offset of a second tensor.
enum : int { kOutF32 = 0, kOutBf16 = 1, kOutF32Copy = 2 };

// bf16 bits <-> float, as the generated code converts them
__device__ __forceinline__ float bf2f(unsigned b) { return __uint_as_float(b << 16); }

template <int TN, int OUT, bool ACC, bool CHECK>
__device__ __forceinline__ void store_tile_row(f32x16 (&acc)[TN], void* origin, long ld, int lane,
                                               long rows_left, long cols_left, void* origin2 = nullptr,
                                               const unsigned short* bias = nullptr, unsigned short* relu_out = nullptr,
                                               bool relu_c = false) {
  using T = typename std::conditional<OUT == kOutBf16, unsigned short, float>::type;
  T* const base = static_cast<T*>(origin);
  unsigned short* const base2 = static_cast<unsigned short*>(origin2);
  const unsigned col = lane & 31, rb = (lane >> 5) * 4;
  const unsigned loff = rb * (unsigned)ld + col;
  // Pin the tiles to accumulation registers up to this point: without it the register allocator
  // may move all accumulators of the block into ordinary registers right after the main loop and
  // spill most of them.
  static_assert(TN == 1 || TN == 2 || TN == 4, "tile rows of 1, 2 or 4 tiles");
  if constexpr (TN == 1) asm volatile("" : "+a"(acc[0]));
  else asm volatile("" : "+a"(acc[0]), "+a"(acc[1]));
  if constexpr (TN == 4) asm volatile("" : "+a"(acc[2]), "+a"(acc[3]));
  float old[ACC ? TN : 1][16];
  if (ACC) {
    static_for<TN>([&](auto jc) OCN_LAMBDA_INLINE {
      static_for<16>([&](auto ec) OCN_LAMBDA_INLINE {
        constexpr int j = decltype(jc)::value, e = decltype(ec)::value, r = (e >> 2) * 8 + (e & 3);
        const T* p = base + (long)r * ld + j * 32;
        float o = 0.0f;
        if (!CHECK || ((long)(r + rb) < rows_left && (long)(j * 32 + col) < cols_left)) {
          if (OUT == kOutBf16) o = __uint_as_float(((unsigned)p[loff]) << 16);
          else o = p[loff];
        }
        old[ACC ? j : 0][e] = o;
      });
    });
  }
  static_for<TN>([&](auto jc) OCN_LAMBDA_INLINE {
    static_for<16>([&](auto ec) OCN_LAMBDA_INLINE {
      constexpr int j = decltype(jc)::value, e = decltype(ec)::value, r = (e >> 2) * 8 + (e & 3);
      T* p = base + (long)r * ld + j * 32;
      float v = acc[j][e];
      if (ACC) v += old[ACC ? j : 0][e];
      if (!CHECK || ((long)(r + rb) < rows_left && (long)(j * 32 + col) < cols_left)) {
        if (OUT == kOutBf16) {
          unsigned b = f2bf(v);
          if (!ACC && bias) b = f2bf(bf2f(b) + bf2f(bias[j * 32 + col]));   // (bias: at the tile row's first column)
          if (!ACC && relu_c) b = ((b & 0x8000u) || (b & 0x7FFFu) > 0x7F80u) ? 0u : b;
          p[loff] = (unsigned short)b;
          if (!ACC && relu_out) (relu_out + (long)r * ld + j * 32)[loff] = (unsigned short)(((b & 0x8000u) || (b & 0x7FFFu) > 0x7F80u) ? 0u : b);   // fmaxf(0, y): negatives and NaN give +0
        }
        else p[loff] = v;
        if (OUT == kOutF32Copy) (base2 + (long)r * ld + j * 32)[loff] = (unsigned short)f2bf(v);
      }
    });
    __builtin_amdgcn_sched_barrier(0);   // one tile's registers at a time
  });
}

// The same row of tiles through LDS, for full tiles whose rows start on 16-byte boundaries: the
// accumulators go to this wave's staging area as fp32 [32][TN * 32] (ds_write_b32, a half-wave per
// 128-byte row piece), come back row-wise as 16-byte chunks, and every lane stores 16 bytes (four
// fp32 or eight bf16 results) next to its neighbours' -- an eighth (a quarter) of the store
// instructions of the direct form, each covering whole cache lines.  `stage` holds 32 * (TN * 32 + 4)
// floats of this wave's own; LDS operations of one wave complete in order, so no barrier is needed.
template <int TN, int OUT, bool ACC>
__device__ __forceinline__ void store_tile_row_wide(f32x16 (&acc)[TN], float* stage, void* origin, long ld, int lane,
                                                    void* origin2 = nullptr, const unsigned short* bias = nullptr,
                                                    unsigned short* relu_out = nullptr, bool relu_c = false) {
  constexpr int CW = TN * 32, LS = CW + 4;
  static_assert(TN == 1 || TN == 2 || TN == 4, "tile rows of 1, 2 or 4 tiles");
  if constexpr (TN == 1) asm volatile("" : "+a"(acc[0]));
  else asm volatile("" : "+a"(acc[0]), "+a"(acc[1]));
  if constexpr (TN == 4) asm volatile("" : "+a"(acc[2]), "+a"(acc[3]));
  float* const wr = stage + ((lane >> 5) * 4) * LS + (lane & 31);
  static_for<TN>([&](auto jc) OCN_LAMBDA_INLINE {
    static_for<16>([&](auto ec) OCN_LAMBDA_INLINE {
      constexpr int j = decltype(jc)::value, e = decltype(ec)::value, r = (e >> 2) * 8 + (e & 3);
      wr[r * LS + j * 32] = acc[j][e];
    });
  });
  constexpr int VEC = OUT == kOutBf16 ? 8 : 4;     // results per lane
  constexpr int LPR = CW / VEC, RPP = 64 / LPR;    // lanes per row, rows per pass
  const int rr = lane / LPR, cc = (lane % LPR) * VEC;
  const float* const rd = stage + rr * LS + cc;
  const unsigned goff = (unsigned)rr * (unsigned)ld + (unsigned)cc;
  static_for<32 / RPP>([&](auto pc) OCN_LAMBDA_INLINE {
    constexpr int p = decltype(pc)::value;
    const long row_off = (long)(p * RPP) * ld;     // uniform
    f32x4 v0 = *reinterpret_cast<const f32x4*>(rd + p * RPP * LS);
    if constexpr (OUT == kOutBf16) {
      f32x4 v1 = *reinterpret_cast<const f32x4*>(rd + p * RPP * LS + 4);
      u32x4* const dst = reinterpret_cast<u32x4*>(static_cast<unsigned short*>(origin) + row_off + goff);
      if (ACC) {
        const u32x4 o = *dst;
        v0 += f32x4{__uint_as_float(o.x << 16), __uint_as_float(o.x & 0xFFFF0000u), __uint_as_float(o.y << 16), __uint_as_float(o.y & 0xFFFF0000u)};
        v1 += f32x4{__uint_as_float(o.z << 16), __uint_as_float(o.z & 0xFFFF0000u), __uint_as_float(o.w << 16), __uint_as_float(o.w & 0xFFFF0000u)};
      }
      u32x4 out = u32x4{pack2(v0.x, v0.y), pack2(v0.z, v0.w), pack2(v1.x, v1.y), pack2(v1.z, v1.w)};
      if (!ACC && bias) {
        // x rounded to bf16 (above), then y = bf16(x + bias[n]): eight columns per lane
        const u32x4 bb = *reinterpret_cast<const u32x4*>(bias + cc);
        auto add2 = [](unsigned x, unsigned b) { return pack2(__uint_as_float(x << 16) + __uint_as_float(b << 16),
                                                               __uint_as_float(x & 0xFFFF0000u) + __uint_as_float(b & 0xFFFF0000u)); };
        out = u32x4{add2(out.x, bb.x), add2(out.y, bb.y), add2(out.z, bb.z), add2(out.w, bb.w)};
      }
      // relu on bf16 bits, as fmaxf(0, y) gives it: negatives (and NaN) become +0
      auto relu2 = [](unsigned x) {
        const unsigned lo = x & 0xFFFFu, hi = x >> 16;
        const unsigned rl = ((lo & 0x8000u) || (lo & 0x7FFFu) > 0x7F80u) ? 0u : lo;
        const unsigned rh = ((hi & 0x8000u) || (hi & 0x7FFFu) > 0x7F80u) ? 0u : hi;
        return rl | (rh << 16);
      };
      if (!ACC && relu_c) out = u32x4{relu2(out.x), relu2(out.y), relu2(out.z), relu2(out.w)};
      *dst = out;
      if (!ACC && relu_out) *reinterpret_cast<u32x4*>(relu_out + row_off + goff) = u32x4{relu2(out.x), relu2(out.y), relu2(out.z), relu2(out.w)};
    } else {
      f32x4* const dst = reinterpret_cast<f32x4*>(static_cast<float*>(origin) + row_off + goff);
      if (ACC) v0 += *dst;
      *dst = v0;
      if constexpr (OUT == kOutF32Copy) {
        typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
        *reinterpret_cast<u32x2*>(static_cast<unsigned short*>(origin2) + row_off + goff) = u32x2{pack2(v0.x, v0.y), pack2(v0.z, v0.w)};
      }
    }
  });
  __builtin_amdgcn_sched_barrier(0);
}

// (m, n) is the origin of the wave's block.  The variant is picked per row of tiles with a
// wave-uniform switch: that bounds what the compiler can hoist above the branch to one row's
// registers (hoisting all 256 accumulator reads above one up-front branch spills them).
// `stage`: this wave's own LDS area of at least 32 * (TN * 32 + 4) floats, free once the main loop
// has passed its last barrier.
template <int TM, int TN>
__device__ __forceinline__ void epilogue(const GemmArgs& g, void* cbase, void* c2base, f32x16 (&acc)[TM][TN], long m, long n, long co, int lane,
                                         float* stage) {
  const long rows_left = g.M - m, cols_left = g.N - n;
  if (rows_left <= 0 || cols_left <= 0) return;
  const bool full = rows_left >= TM * 32 && cols_left >= TN * 32;
  const bool to_ws = g.splits > 1;   // split-K partial sums go to the workspace [batch][split][M][N]
  const bool bf = !to_ws && g.c_is_bf16;
  const long ld = to_ws ? g.N : g.c_row;
  const long first = to_ws ? (((long)blockIdx.z * g.splits + blockIdx.y) * g.M + m) * g.N + n : co + m * g.c_row + n;
  char* const origin = (to_ws ? reinterpret_cast<char*>(g.ws) : static_cast<char*>(cbase)) + first * (bf ? 2 : 4);
  const bool copy = !to_ws && !bf && c2base != nullptr;   // (with split-K the reduction pass writes the copy)
  char* const origin2 = copy ? static_cast<char*>(c2base) + first * 2 : nullptr;
  // 16-byte stores need rows that start on 16-byte boundaries (and 8-byte ones for the bf16 copy)
  const bool wide = full && ((reinterpret_cast<unsigned long>(origin) | (unsigned long)(ld * (bf ? 2 : 4))) & 15) == 0 &&
                    (!copy || ((reinterpret_cast<unsigned long>(origin2) | (unsigned long)(ld * 2)) & 7) == 0) &&
                    (!g.relu_out || ((reinterpret_cast<unsigned long>(g.relu_out) + (unsigned long)first * 2) & 15) == 0) &&
                    (!g.bias || ((reinterpret_cast<unsigned long>(g.bias) + (unsigned long)n * 2) & 15) == 0) &&
                    (unsigned long)ld * 32 < 0x100000000ul;
  // fp32 results already leave as 128-byte row pieces per half-wave and go out directly (measured:
  // staging them gains nothing, the burst of a tile's results is bound by the memory system); bf16
  // results and bf16 copies would leave as 2-byte elements and take the staged form
  const int variant = (copy ? 8 : bf ? 4 : 0) + ((!to_ws && g.accumulate) ? 2 : 0) + ((copy || bf) ? (wide ? 0 : 1) : (full ? 0 : 1));
  // folded consumers (bf16 results, stored, not accumulated): bias at this block's first column, relu output at its origin
  const bool epi = bf && !g.accumulate;
  const unsigned short* const bias = epi && g.bias ? static_cast<const unsigned short*>(g.bias) + n : nullptr;
  char* const origin3 = epi && g.relu_out ? static_cast<char*>(g.relu_out) + first * 2 : nullptr;
  const bool relu_c = epi && g.relu_c;
  static_for<TM>([&](auto ic) OCN_LAMBDA_INLINE {
    constexpr int i = decltype(ic)::value;
    void* o = origin + (long)i * 32 * ld * (bf ? 2 : 4);
    void* o2 = origin2 + (long)i * 32 * ld * 2;
    void* o3 = origin3 ? origin3 + (long)i * 32 * ld * 2 : nullptr;
    const long rl = rows_left - i * 32;
    switch (variant) {
      case 0: store_tile_row<TN, kOutF32, false, false>(acc[i], o, ld, lane, rl, cols_left); break;
      case 1: store_tile_row<TN, kOutF32, false, true>(acc[i], o, ld, lane, rl, cols_left); break;
      case 2: store_tile_row<TN, kOutF32, true, false>(acc[i], o, ld, lane, rl, cols_left); break;
      case 3: store_tile_row<TN, kOutF32, true, true>(acc[i], o, ld, lane, rl, cols_left); break;
      case 4: store_tile_row_wide<TN, kOutBf16, false>(acc[i], stage, o, ld, lane, nullptr, bias, reinterpret_cast<unsigned short*>(o3), relu_c); break;
      case 5: store_tile_row<TN, kOutBf16, false, true>(acc[i], o, ld, lane, rl, cols_left, nullptr, bias, reinterpret_cast<unsigned short*>(o3), relu_c); break;
      case 6: store_tile_row_wide<TN, kOutBf16, true>(acc[i], stage, o, ld, lane); break;
      case 7: store_tile_row<TN, kOutBf16, true, true>(acc[i], o, ld, lane, rl, cols_left); break;
      case 8: store_tile_row_wide<TN, kOutF32Copy, false>(acc[i], stage, o, ld, lane, o2); break;
      case 9: store_tile_row<TN, kOutF32Copy, false, true>(acc[i], o, ld, lane, rl, cols_left, o2); break;
      case 10: store_tile_row_wide<TN, kOutF32Copy, true>(acc[i], stage, o, ld, lane, o2); break;
      default: store_tile_row<TN, kOutF32Copy, true, true>(acc[i], o, ld, lane, rl, cols_left, o2); break;
    }
    __builtin_amdgcn_sched_barrier(0);
  });
}

// Sums the split-K partials in split order (deterministic) and applies them to C.
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const GemmArgs g) {
  const long n4 = g.N / 4;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= g.M * n4) return;
  const long m = idx / n4, n = (idx % n4) * 4;
  long ao, bo, co;
  const void *abase, *bbase;
  void *cbase, *c2base;
  decode_batch(g, decode_group(g, blockIdx.z, abase, bbase, cbase, c2base), ao, bo, co);
  f32x4 sum = {0, 0, 0, 0};
  for (int sp = 0; sp < g.splits; ++sp)
    sum += *reinterpret_cast<const f32x4*>(g.ws + (((long)blockIdx.z * g.splits + sp) * g.M + m) * g.N + n);
  const long off = co + m * g.c_row + n;
  if (g.c_is_bf16) {
    unsigned short* C = static_cast<unsigned short*>(cbase);
    for (int q = 0; q < 4; ++q) {
      float v = sum[q];
      if (g.accumulate) v += __uint_as_float(((unsigned)C[off + q]) << 16);
      C[off + q] = (unsigned short)f2bf(v);
    }
  } else {
    float* C = static_cast<float*>(cbase);
    f32x4 v = sum;
    if (g.accumulate) v += *reinterpret_cast<const f32x4*>(C + off);
    *reinterpret_cast<f32x4*>(C + off) = v;
    if (c2base) {
      unsigned short* C2 = static_cast<unsigned short*>(c2base);
      for (int q = 0; q < 4; ++q) C2[off + q] = (unsigned short)f2bf(v[q]);
    }
  }
}


// Launches `kernel` over the tile grid of `a` (x: tiles, y: K splits, z: members x batch entries) and,
// after a K split, the reduction pass.
template <typename K>
hipError_t launch(K kernel, size_t smem, int BM, int BN, GemmArgs a, hipStream_t s, hipEvent_t after_main) {
  static thread_local const void* configured[128];
  static thread_local int n_configured = 0;
  bool done = false;
  for (int i = 0; i < n_configured; ++i) done |= configured[i] == (const void*)kernel;
  if (!done) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    if (n_configured < 128) configured[n_configured++] = (const void*)kernel;
  }
  const long tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  long nb = 1;
  for (int i = 0; i < a.nbatch; ++i) nb *= a.batch_ext[i];
  if (a.ngroups < 1 || a.ngroups > 4 || a.npairs < 1 || a.npairs > 4 || (a.npairs > 1 && a.ngroups > 1)) return hipErrorInvalidValue;
  a.batches = (int)nb;
  nb *= a.ngroups;
  if (tiles <= 0 || tiles > 0x7FFFFFFFL || nb <= 0 || nb > 65535) return hipErrorInvalidValue;
  if (a.splits > 1 && (!a.ws || a.N % 4 != 0)) return hipErrorInvalidValue;   // (the reduction pass adds four columns per thread)
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)a.splits, (unsigned)nb), dim3(kThreads), smem, s, a);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess && after_main) e = hipEventRecord(after_main, s);
  if (e != hipSuccess || a.splits <= 1) return e;
  const long groups = a.M * (a.N / 4);
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((groups + 255) / 256), 1, (unsigned)nb), dim3(256), 0, s, a);
  return hipGetLastError();
}


}  // namespace
}  // namespace ocannl
