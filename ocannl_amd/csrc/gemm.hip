// Hand-written CDNA4 (gfx950) MFMA kernels for OCANNL's `+*` contractions:
//     C[batch, m, n] (+)= sum_k A[batch, m, k] * B[batch, n, k]
// i.e. the loop nests `c[..] := fma(a[..], b[..], c[..])` that Assignments.to_low_level emits for
// matmul / einsum and their gradients (arrayjit/lib/assignments.ml:311-488,
// tensor/operation.ml:77-99), which the reference runs as a serial scalar loop.
//
// Layout freedom: each operand is unit-stride either along K or along its row dimension (M for A,
// N for B) with an arbitrary leading stride, plus up to three batch strides -- this covers the
// forward (both K-contiguous), dX (B row-contiguous) and dW (both row-contiguous) forms and the
// attention contractions on [b, s, h, d] tensors without any transposition pass.
//
// Kernel structure (bf16 compute, fp32 accumulate):
//   * 256 threads = 4 wavefronts in a 2x2 grid; block tile BM x BN, K step 64;
//   * global -> registers (16-byte loads) -> LDS, double buffered, one barrier per K step; a
//     K-contiguous operand is held [row][k] (rows padded by 16 bytes: ds_read_b128 of 16 rows hits
//     distinct banks), a row-contiguous operand stays [k][row] as it lies in memory and its MFMA
//     fragments are read with ds_read_b64_tr_b16 -- no transposition anywhere; fp32 sources are
//     rounded to bf16 (RNE) on the way to LDS;
//   * v_mfma_f32_32x32x16_bf16, each wavefront owns a (BM/2) x (BN/2) sub-tile;
//   * workgroup ids are remapped so that each XCD (ids are dealt round-robin over 8 XCDs) works on
//     a compact band of tiles and shares B/A panels through its own L2.
// fp32 compute uses v_mfma_f32_32x32x2_f32 with the same staging.
#include <hip/hip_runtime.h>

#include <cstdio>
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
                                               const unsigned short* bias = nullptr, unsigned short* relu_out = nullptr) {
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
                                                    unsigned short* relu_out = nullptr) {
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
      *dst = out;
      if (!ACC && relu_out) {
        // relu on bf16 bits, as fmaxf(0, y) gives it: negatives (and NaN) become +0
        auto relu2 = [](unsigned x) {
          const unsigned lo = x & 0xFFFFu, hi = x >> 16;
          const unsigned rl = ((lo & 0x8000u) || (lo & 0x7FFFu) > 0x7F80u) ? 0u : lo;
          const unsigned rh = ((hi & 0x8000u) || (hi & 0x7FFFu) > 0x7F80u) ? 0u : hi;
          return rl | (rh << 16);
        };
        *reinterpret_cast<u32x4*>(relu_out + row_off + goff) = u32x4{relu2(out.x), relu2(out.y), relu2(out.z), relu2(out.w)};
      }
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
      case 4: store_tile_row_wide<TN, kOutBf16, false>(acc[i], stage, o, ld, lane, nullptr, bias, reinterpret_cast<unsigned short*>(o3)); break;
      case 5: store_tile_row<TN, kOutBf16, false, true>(acc[i], o, ld, lane, rl, cols_left, nullptr, bias, reinterpret_cast<unsigned short*>(o3)); break;
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

// One wavefront per SIMD for the 256x256 tile (the 256 accumulator registers live in AGPRs and the
// whole 512-register budget is available); two for the 128x128 tile.
// PF = 2: global loads run two K stages ahead in two register sets, for launches of at most one
// workgroup per CU, where nothing else hides the HBM latency of a stage; that needs the whole
// register file, so one wavefront per SIMD.
// CHAIN: the launch accumulates several operand pairs into one C (`c =+ a_p * b_p`, p < npairs):
// the K pipeline runs once per pair and the accumulators stay in registers in between.  Only the
// 128x128 tile with two register sets is built that way (the loop around the pipeline costs
// registers that the other variants do not have).
template <int BM, int BN, typename AT, typename BT, bool A_KC, bool B_KC, int PF, bool CHAIN = false>
__global__ void __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu((BM < 256 && sizeof(AT) == 2 && sizeof(BT) == 2 && PF == 1) ? 2 : 1,
                                   (BM >= 256 || PF > 1) ? 1 : 2)))
gemm_bf16_kernel(const GemmArgs g) {
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 32, TN = WN / 32;
  constexpr int kAT = lds_tile_elems<BM, A_KC>(), kBT = lds_tile_elems<BN, B_KC>();   // one stage of each operand
  constexpr int kAS = Stager<BM, AT, A_KC>::kLineStride, kBS = Stager<BN, BT, B_KC>::kLineStride;
  extern __shared__ __align__(16) unsigned short smem[];
  unsigned short* const As0 = smem;
  unsigned short* const Bs0 = smem + 2 * kAT;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
  const long tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
  long tmi, tni, wg, zz;
  int nx;
  place_workgroup(g, wg, zz, nx);
  tile_of_block(wg, tiles_m, tiles_n, g.xcd_m, nx, tmi, tni);
  const long m0 = tmi * BM, n0 = tni * BN;
  long ao, bo, co;
  const void *abase, *bbase;
  void *cbase, *c2base;
  decode_batch(g, decode_group(g, zz, abase, bbase, cbase, c2base), ao, bo, co);
  const AT* A = static_cast<const AT*>(abase) + ao;
  const BT* B = static_cast<const BT*>(bbase) + bo;
  const long lda = A_KC ? g.a_row : g.a_k, ldb = B_KC ? g.b_row : g.b_k;

  // per-lane offsets of the MFMA fragments inside a stage of each operand
  const unsigned a_frag = A_KC ? (unsigned)((wm0 + (lane & 31)) * kAS + (lane >> 5) * 8) : (unsigned)wm0 + tr_lane_offset(lane, kAS);
  const unsigned b_frag = B_KC ? (unsigned)((wn0 + (lane & 31)) * kBS + (lane >> 5) * 8) : (unsigned)wn0 + tr_lane_offset(lane, kBS);
  // fragment of 32-row block `blk`, 16-k sub-step `kk`, from the stage starting at `stage`
  auto a_fragment = [&](const unsigned short* stage, int blk, int kk) OCN_LAMBDA_INLINE -> bf16x8 {
    if constexpr (A_KC) return *reinterpret_cast<const bf16x8*>(stage + a_frag + blk * 32 * kAS + kk * 16);
    else return tr_fragment(stage + a_frag + kk * 16 * kAS + blk * 32, kAS);
  };
  auto b_fragment = [&](const unsigned short* stage, int blk, int kk) OCN_LAMBDA_INLINE -> bf16x8 {
    if constexpr (B_KC) return *reinterpret_cast<const bf16x8*>(stage + b_frag + blk * 32 * kBS + kk * 16);
    else return tr_fragment(stage + b_frag + kk * 16 * kBS + blk * 32, kBS);
  };

  f32x16 acc[TM][TN];
  static_for<TM>([&](auto ic) OCN_LAMBDA_INLINE {
    static_for<TN>([&](auto jc) OCN_LAMBDA_INLINE {
      static_for<16>([&](auto ec) OCN_LAMBDA_INLINE { acc[decltype(ic)::value][decltype(jc)::value][decltype(ec)::value] = 0.0f; });
    });
  });

  // split-K: blockIdx.y owns a contiguous range of K steps
  const long all_steps = (g.K + kBK - 1) / kBK;
  const long per_split = (all_steps + g.splits - 1) / g.splits;
  const long kbeg = (long)blockIdx.y * per_split * kBK;
  const long kend = (kbeg + per_split * kBK) < g.K ? (kbeg + per_split * kBK) : g.K;
  const long ksteps = kend > kbeg ? (kend - kbeg + kBK - 1) / kBK : 0;

  // Software pipeline.  LDS is double buffered; global loads run kPF tiles ahead of the tile being
  // multiplied, held in kPF register sets (one or two).
  constexpr int kPF = PF;
  static_assert(PF == 1 || (PF == 2 && sizeof(AT) == 2 && sizeof(BT) == 2), "two register sets: bf16 sources only");
  Stager<BM, AT, A_KC> sa[kPF];
  Stager<BN, BT, B_KC> sb[kPF];
  static_assert(!CHAIN || (BM == 128 && PF == 2), "chains: 128x128 tiles with two register sets");
  // (the pipeline is a lambda so that the variants without chains hold no loop statement around it:
  // a loop with one trip still cost the 256x256 variants registers)
  auto pipeline = [&]() __attribute__((always_inline)) {
  sa[0].load(A, lda, m0, kbeg, g.M, kend, tid);
  sb[0].load(B, ldb, n0, kbeg, g.N, kend, tid);
  if (kPF > 1) {
    sa[kPF - 1].load(A, lda, m0, kbeg + kBK, g.M, kend, tid);
    sb[kPF - 1].load(B, ldb, n0, kbeg + kBK, g.N, kend, tid);
  }
  sa[0].store(As0, tid);
  sb[0].store(Bs0, tid);
  __syncthreads();

  // one K step; `par` = ks % kPF is a compile-time constant so that the register sets are
  // addressed statically
  auto step = [&](long ks, auto par_c) __attribute__((always_inline)) {
    constexpr int par = decltype(par_c)::value;
    const int cur = ks & 1;
    // register set `par` held tile ks (already in LDS): refill it with tile ks + kPF
    if (ks + kPF < ksteps) {
      sa[par].load(A, lda, m0, kbeg + (ks + kPF) * kBK, g.M, kend, tid);
      sb[par].load(B, ldb, n0, kbeg + (ks + kPF) * kBK, g.N, kend, tid);
    }
    __builtin_amdgcn_sched_barrier(0);   // the loads are issued before the MFMA block, not sunk below it
    const unsigned short* as = As0 + cur * kAT;
    const unsigned short* bs = Bs0 + cur * kBT;
    // fragments are double buffered: the LDS reads of sub-step kk + 1 are issued before the MFMAs
    // of sub-step kk, so that a lone wave per SIMD does not sit out the LDS latency every time
    bf16x8 af[2][TM], bf[2][TN];
    auto read_frags = [&](auto kkc) OCN_LAMBDA_INLINE {
      constexpr int kk = decltype(kkc)::value, fb = kk & 1;
      static_for<TM>([&](auto ic) OCN_LAMBDA_INLINE {
        constexpr int i = decltype(ic)::value;
        af[fb][i] = a_fragment(as, i, kk);
      });
      static_for<TN>([&](auto jc) OCN_LAMBDA_INLINE {
        constexpr int j = decltype(jc)::value;
        bf[fb][j] = b_fragment(bs, j, kk);
      });
    };
    read_frags(std::integral_constant<int, 0>{});
    static_for<kBK / 16>([&](auto kkc) OCN_LAMBDA_INLINE {
      constexpr int kk = decltype(kkc)::value, fb = kk & 1;
      if constexpr (kk + 1 < kBK / 16) {
        read_frags(std::integral_constant<int, kk + 1>{});
        __builtin_amdgcn_sched_barrier(0);
      }
      static_for<TM>([&](auto ic) OCN_LAMBDA_INLINE {
        static_for<TN>([&](auto jc) OCN_LAMBDA_INLINE {
          constexpr int i = decltype(ic)::value, j = decltype(jc)::value;
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[fb][i], bf[fb][j], acc[i][j], 0, 0, 0);
        });
      });
    });
    __builtin_amdgcn_sched_barrier(0);
    // tile ks + 1 sits in the other register set (or, with one set, in the one just refilled)
    if (ks + 1 < ksteps) {
      constexpr int nxt = (par + 1) % kPF;
      sa[nxt].store(As0 + (cur ^ 1) * kAT, tid);
      sb[nxt].store(Bs0 + (cur ^ 1) * kBT, tid);
    }
    __syncthreads();
  };
  // Interleaved K step for full tiles: one basic block in which the other instructions are placed
  // between the MFMAs by hand (and pinned there), so that they issue while the matrix pipe is busy
  // -- with one wave per SIMD nothing else would hide them.  Global loads of tile ks + 1 go with
  // the first half of the MFMAs, its LDS writes with the second half, the LDS reads of the next
  // sub-step's fragments with the current sub-step.
  auto fast_step = [&](long ks, auto loads_c, auto stores_c, auto par_c) __attribute__((always_inline)) {
    constexpr bool kLoads = decltype(loads_c)::value, kStores = decltype(stores_c)::value;
    constexpr int kLoadSet = decltype(par_c)::value, kStoreSet = (kLoadSet + 1) % kPF;   // tile ks + kPF in, tile ks + 1 out
    constexpr int kSub = kBK / 16, kPer = TM * TN, kAll = kSub * kPer, kHalf = kAll / 2;
    constexpr int kA = Stager<BM, AT, A_KC>::kOps, kL = kA + Stager<BN, BT, B_KC>::kOps, kR = TM + TN;
    const int cur = ks & 1;
    const long kn = kbeg + (ks + kPF) * kBK;
    const AT* const a_next = A_KC ? A + m0 * lda + kn : A + kn * lda + m0;
    const BT* const b_next = B_KC ? B + n0 * ldb + kn : B + kn * ldb + n0;
    unsigned short* const an = As0 + (cur ^ 1) * kAT;
    unsigned short* const bn = Bs0 + (cur ^ 1) * kBT;
    const unsigned short* as = As0 + cur * kAT;
    const unsigned short* bs = Bs0 + cur * kBT;
    bf16x8 af[2][TM], bf[2][TN];
    auto read_frag = [&](auto kkc, auto rc) OCN_LAMBDA_INLINE {
      constexpr int kk = decltype(kkc)::value, r = decltype(rc)::value, fb = kk & 1;
      if constexpr (r < TM) af[fb][r] = a_fragment(as, r, kk);
      else bf[fb][r - TM] = b_fragment(bs, r - TM, kk);
    };
    static_for<kR>([&](auto rc) OCN_LAMBDA_INLINE { read_frag(std::integral_constant<int, 0>{}, rc); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<kAll>([&](auto mc) OCN_LAMBDA_INLINE {
      constexpr int m = decltype(mc)::value, kk = m / kPer, idx = m % kPer, i = idx / TN, j = idx % TN, fb = kk & 1;
      if constexpr (kk + 1 < kSub) {
        static_for<(idx + 1) * kR / kPer - idx * kR / kPer>([&](auto rc) OCN_LAMBDA_INLINE {
          read_frag(std::integral_constant<int, kk + 1>{}, std::integral_constant<int, idx * kR / kPer + decltype(rc)::value>{});
        });
      }
      if constexpr (kLoads && m < kHalf) {
        static_for<(m + 1) * kL / kHalf - m * kL / kHalf>([&](auto oc) OCN_LAMBDA_INLINE {
          constexpr int o = m * kL / kHalf + decltype(oc)::value;
          if constexpr (o < kA) sa[kLoadSet].template load_op<o>(a_next, lda);
          else sb[kLoadSet].template load_op<o - kA>(b_next, ldb);
        });
      }
      if constexpr (kStores && m >= kHalf) {
        static_for<(m - kHalf + 1) * kL / kHalf - (m - kHalf) * kL / kHalf>([&](auto oc) OCN_LAMBDA_INLINE {
          constexpr int o = (m - kHalf) * kL / kHalf + decltype(oc)::value;
          if constexpr (o < kA) sa[kStoreSet].template store_op<o>(an);
          else sb[kStoreSet].template store_op<o - kA>(bn);
        });
      }
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[fb][i], bf[fb][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    });
    __syncthreads();
  };

  static_for<kPF>([&](auto p) OCN_LAMBDA_INLINE { sa[decltype(p)::value].init_ops(lda, tid); sb[decltype(p)::value].init_ops(ldb, tid); });
  // (fp32 sources stage twice the registers: with double-buffered fragments on top the loop
  // spills, so they keep the plain loop)
  constexpr bool kInterleave = sizeof(AT) == 2 && sizeof(BT) == 2 && kPF <= 2;
  const bool full_tile = kInterleave && m0 + BM <= g.M && n0 + BN <= g.N && ksteps > 0 && kbeg + ksteps * kBK <= kend;
  if constexpr (kInterleave) {
    if (full_tile) {
      using Y = std::true_type; using N = std::false_type;
      using P0 = std::integral_constant<int, 0>; using P1 = std::integral_constant<int, 1 % kPF>;
      if constexpr (kPF == 1) {
        for (long ks = 0; ks + 1 < ksteps; ++ks) fast_step(ks, Y{}, Y{}, P0{});
        fast_step(ksteps - 1, N{}, N{}, P0{});
      } else {
        // two register sets: steps come in pairs so that the set numbers are compile-time constants
        long ks = 0;
        for (; ks + 3 < ksteps; ks += 2) { fast_step(ks, Y{}, Y{}, P0{}); fast_step(ks + 1, Y{}, Y{}, P1{}); }
        const long rem = ksteps - ks;   // 1, 2 or 3 steps left; ks is even
        if (rem == 3) { fast_step(ks, Y{}, Y{}, P0{}); fast_step(ks + 1, N{}, Y{}, P1{}); fast_step(ks + 2, N{}, N{}, P0{}); }
        else if (rem == 2) { fast_step(ks, N{}, Y{}, P0{}); fast_step(ks + 1, N{}, N{}, P1{}); }
        else fast_step(ks, N{}, N{}, P0{});
      }
    }
  }
  if (!full_tile) {
    long ks = 0;
    for (; ks + kPF <= ksteps; ks += kPF) static_for<kPF>([&](auto p) OCN_LAMBDA_INLINE { step(ks + decltype(p)::value, p); });
    static_for<kPF>([&](auto p) OCN_LAMBDA_INLINE { if (ks + decltype(p)::value < ksteps) step(ks + decltype(p)::value, p); });
  }
  };   // pipeline
  if constexpr (CHAIN) {
    for (int pair = 0; pair < g.npairs; ++pair) {
      if (pair > 0) {
        A = static_cast<const AT*>(pair == 1 ? g.a_more[0] : pair == 2 ? g.a_more[1] : g.a_more[2]) + ao;
        B = static_cast<const BT*>(pair == 1 ? g.b_more[0] : pair == 2 ? g.b_more[1] : g.b_more[2]) + bo;
      }
      pipeline();
    }
  } else {
    pipeline();
  }

  // (every wave has passed the last barrier of the main loop: the operand stages are free)
  epilogue<TM, TN>(g, cbase, c2base, acc, m0 + wm0, n0 + wn0, co, lane,
                   reinterpret_cast<float*>(smem) + wave * ((kAT + kBT) / 4));
}

// ---- fp32 compute -------------------------------------------------------------------------------
// v_mfma_f32_32x32x2_f32: a lane supplies one float of its row per instruction; instruction q of a
// group of four multiplies k = q (lanes 0-31) and k = 4 + q (lanes 32-63) of an 8-k sub-step -- A
// and B use the same assignment, so the sum is complete.
//   K-contiguous operand:   LDS [row][k], row stride kBKf + kPadf: a lane reads its four k with one
//     ds_read_b128.
//   row-contiguous operand: LDS [k][row] as it lies in memory, row stride ROWS + kPadTf: a lane
//     reads its four k with four ds_read_b32 (lanes of a half read 32 consecutive floats; the two
//     halves sit 4 k-rows = 32 banks apart): no transposition anywhere.
constexpr int kPadTf = 8;

template <int ROWS, bool KC>
constexpr int lds_tile_floats() { return KC ? ROWS * (kBKf + kPadf) : kBKf * (ROWS + kPadTf); }

template <int ROWS, bool KC>
struct StagerF {
  static constexpr int kChunks = ROWS * (kBKf / 4) / kThreads;   // 16-byte chunks per thread
  static constexpr int kPerLine = KC ? kBKf / 4 : ROWS / 4;      // chunks per contiguous line
  static constexpr int kLineStride = KC ? kBKf + kPadf : ROWS + kPadTf;
  f32x4 regs[kChunks];

  __device__ __forceinline__ void load(const float* base, long ld, long row0, long k0, long rows, long K, int tid) {
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int c = tid + kThreads * j;
      const long line = c / kPerLine, pos = (c % kPerLine) * 4;
      f32x4 v = {0, 0, 0, 0};
      if (KC) { if (row0 + line < rows && k0 + pos < K) v = *reinterpret_cast<const f32x4*>(base + (row0 + line) * ld + k0 + pos); }
      else    { if (k0 + line < K && row0 + pos < rows) v = *reinterpret_cast<const f32x4*>(base + (k0 + line) * ld + row0 + pos); }
      regs[j] = v;
    }
  }

  __device__ __forceinline__ void store(float* lds, int tid) const {
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int c = tid + kThreads * j;
      *reinterpret_cast<f32x4*>(lds + (c / kPerLine) * kLineStride + (c % kPerLine) * 4) = regs[j];
    }
  }
};

template <int BM, int BN, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, BM >= 256 ? 1 : 2)))
gemm_f32_kernel(const GemmArgs g) {
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 32, TN = WN / 32;
  constexpr int kAT = lds_tile_floats<BM, A_KC>(), kBT = lds_tile_floats<BN, B_KC>();
  constexpr int kAS = StagerF<BM, A_KC>::kLineStride, kBS = StagerF<BN, B_KC>::kLineStride;
  extern __shared__ __align__(16) unsigned short smem[];
  float* fsm = reinterpret_cast<float*>(smem);
  float* const As0 = fsm;
  float* const Bs0 = fsm + 2 * kAT;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
  const long tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
  long tmi, tni, wg, zz;
  int nx;
  place_workgroup(g, wg, zz, nx);
  tile_of_block(wg, tiles_m, tiles_n, g.xcd_m, nx, tmi, tni);
  const long m0 = tmi * BM, n0 = tni * BN;
  long ao, bo, co;
  const void *abase, *bbase;
  void *cbase, *c2base;
  decode_batch(g, decode_group(g, zz, abase, bbase, cbase, c2base), ao, bo, co);
  const float* A = static_cast<const float*>(abase) + ao;
  const float* B = static_cast<const float*>(bbase) + bo;
  const long lda = A_KC ? g.a_row : g.a_k, ldb = B_KC ? g.b_row : g.b_k;

  f32x16 acc[TM][TN];
  static_for<TM>([&](auto ic) OCN_LAMBDA_INLINE {
    static_for<TN>([&](auto jc) OCN_LAMBDA_INLINE {
      static_for<16>([&](auto ec) OCN_LAMBDA_INLINE { acc[decltype(ic)::value][decltype(jc)::value][decltype(ec)::value] = 0.0f; });
    });
  });

  StagerF<BM, A_KC> sa;
  StagerF<BN, B_KC> sb;
  // split-K: blockIdx.y owns a contiguous range of K steps
  const long all_steps = (g.K + kBKf - 1) / kBKf;
  const long per_split = (all_steps + g.splits - 1) / g.splits;
  const long kbeg = (long)blockIdx.y * per_split * kBKf;
  const long kend = (kbeg + per_split * kBKf) < g.K ? (kbeg + per_split * kBKf) : g.K;
  sa.load(A, lda, m0, kbeg, g.M, kend, tid);
  sb.load(B, ldb, n0, kbeg, g.N, kend, tid);
  sa.store(As0, tid);
  sb.store(Bs0, tid);
  __syncthreads();

  const long ksteps = kend > kbeg ? (kend - kbeg + kBKf - 1) / kBKf : 0;
  for (long ks = 0; ks < ksteps; ++ks) {
    const int cur = ks & 1;
    const bool more = ks + 1 < ksteps;
    if (more) {
      sa.load(A, lda, m0, kbeg + (ks + 1) * kBKf, g.M, kend, tid);
      sb.load(B, ldb, n0, kbeg + (ks + 1) * kBKf, g.N, kend, tid);
    }
    const float* as = As0 + cur * kAT + (A_KC ? (wm0 + (lane & 31)) * kAS + (lane >> 5) * 4 : (lane >> 5) * 4 * kAS + wm0 + (lane & 31));
    const float* bs = Bs0 + cur * kBT + (B_KC ? (wn0 + (lane & 31)) * kBS + (lane >> 5) * 4 : (lane >> 5) * 4 * kBS + wn0 + (lane & 31));
#pragma unroll
    for (int kk = 0; kk < kBKf / 8; ++kk) {
      f32x4 af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        if (A_KC) af[i] = *reinterpret_cast<const f32x4*>(as + i * 32 * kAS + kk * 8);
        else {
          const float* p = as + kk * 8 * kAS + i * 32;
          af[i] = f32x4{p[0], p[kAS], p[2 * kAS], p[3 * kAS]};
        }
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if (B_KC) bf[j] = *reinterpret_cast<const f32x4*>(bs + j * 32 * kBS + kk * 8);
        else {
          const float* p = bs + kk * 8 * kBS + j * 32;
          bf[j] = f32x4{p[0], p[kBS], p[2 * kBS], p[3 * kBS]};
        }
      }
      static_for<4>([&](auto qc) OCN_LAMBDA_INLINE {
        static_for<TM>([&](auto ic) OCN_LAMBDA_INLINE {
          static_for<TN>([&](auto jc) OCN_LAMBDA_INLINE {
            constexpr int q = decltype(qc)::value, i = decltype(ic)::value, j = decltype(jc)::value;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][q], bf[j][q], acc[i][j], 0, 0, 0);
          });
        });
      });
    }
    if (more) {
      sa.store(As0 + (cur ^ 1) * kAT, tid);
      sb.store(Bs0 + (cur ^ 1) * kBT, tid);
    }
    __syncthreads();
  }

  epilogue<TM, TN>(g, cbase, c2base, acc, m0 + wm0, n0 + wn0, co, lane, fsm + wave * ((kAT + kBT) / 2));
}

template <int BM, int BN, bool A_KC, bool B_KC>
constexpr size_t bf16_smem() { return 2ull * (lds_tile_elems<BM, A_KC>() + lds_tile_elems<BN, B_KC>()) * sizeof(unsigned short); }
template <int BM, int BN, bool A_KC, bool B_KC>
constexpr size_t f32_smem() { return 2ull * (lds_tile_floats<BM, A_KC>() + lds_tile_floats<BN, B_KC>()) * sizeof(float); }

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

// Tile grids of one launch along z: batch entries times grouped contractions.
long batch_count(const GemmDesc& d) {
  long nb = 1 + (long)d.group.size();
  for (int i = 0; i < d.nbatch; ++i) nb *= d.batch_ext[i];
  return nb;
}


// Tile size and split-K factor, from a measured sweep on MI355X (bf16 operands).  256x256 tiles
// (one workgroup per CU) win only when the output alone gives >= 256 of them and K runs at least
// 8 stages (below that a launch is all prologue and epilogue); anything else
// runs 128x128 tiles, two workgroups per CU, and when those are fewer than 256 K is split
// towards ~512 workgroups (~256 for bf16 sources), never below 8 K stages per split.  Splits are summed in index order by
// splitk_reduce_kernel (deterministic).
struct TileConfig { bool big; int splits; int prefetch; bool narrow = false; };

TileConfig tile_config(const GemmDesc& d) {
  const long nb = batch_count(d);
  const long t256 = ((d.M + 255) / 256) * ((d.N + 255) / 256) * nb;
  const long t128 = ((d.M + 127) / 128) * ((d.N + 127) / 128) * nb;
  TileConfig c;
  const bool bf16_sources = d.a.prec == Prec::Bfloat16 && d.b.prec == Prec::Bfloat16;
  if (d.more.empty() && t256 >= 256 && d.M > 128 && d.N > 128 && d.K >= 512) { c.big = true; c.splits = 1; }
  else {
    c.big = false;
    long s = 1;
    // bf16 sources: towards one workgroup per CU, which then loads two stages ahead (below);
    // otherwise towards two per CU
    const long target = bf16_sources ? 256 : 512;
    if (t128 < 256 && d.epi_bias < 0 && d.epi_relu < 0) {   // (folded consumers are applied by the contraction's own epilogue)
      while (s * 2 * t128 <= target && s * 2 <= d.K / 512 && s < 64) s *= 2;
    }
    c.splits = (int)s;
  }
  // two stages of global loads in flight when the launch puts at most one workgroup on a CU and
  // each runs at least 8 K stages (measured: 8192x512x2048 bf16 595 -> 738 TFLOP/s)
  c.prefetch = (!c.big && bf16_sources && t128 * c.splits <= 256 && d.K / c.splits >= 512) ? 2 : 1;
  if (!d.more.empty()) c.prefetch = 2;   // the only variant built for chains
  // results of at most 64 columns (the attention products against V, K, Q: N = head size) take a
  // 128 x 64 tile: with 128 columns half of every tile would be masked and the launch would run the
  // checked loop for ragged tiles
  c.narrow = !c.big && bf16_sources && d.more.empty() && d.N <= 64 && d.N > 16;
  return c;
}
bool narrow_tile(const GemmDesc& d) { return tile_config(d).narrow; }

bool big_tile(const GemmDesc& d) { return tile_config(d).big; }
int split_count(const GemmDesc& d) { return tile_config(d).splits; }
int prefetch_depth(const GemmDesc& d) { return tile_config(d).prefetch; }

template <typename K>
hipError_t launch(K kernel, size_t smem, int BM, int BN, GemmArgs a, hipStream_t s, hipEvent_t after_main) {
  static thread_local const void* configured[64];
  static thread_local int n_configured = 0;
  bool done = false;
  for (int i = 0; i < n_configured; ++i) done |= configured[i] == (const void*)kernel;
  if (!done) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    if (n_configured < 64) configured[n_configured++] = (const void*)kernel;
  }
  const long tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  long nb = 1;
  for (int i = 0; i < a.nbatch; ++i) nb *= a.batch_ext[i];
  if (a.ngroups < 1 || a.ngroups > 4 || a.npairs < 1 || a.npairs > 4 || (a.npairs > 1 && a.ngroups > 1)) return hipErrorInvalidValue;
  a.batches = (int)nb;
  nb *= a.ngroups;
  if (tiles <= 0 || tiles > 0x7FFFFFFFL || nb <= 0 || nb > 65535) return hipErrorInvalidValue;
  if (a.splits > 1 && !a.ws) return hipErrorInvalidValue;
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)a.splits, (unsigned)nb), dim3(kThreads), smem, s, a);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess && after_main) e = hipEventRecord(after_main, s);
  if (e != hipSuccess || a.splits <= 1) return e;
  const long groups = a.M * (a.N / 4);
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((groups + 255) / 256), 1, (unsigned)nb), dim3(256), 0, s, a);
  return hipGetLastError();
}

template <int BM, int BN, typename AT, typename BT, int PF = 1, bool CHAIN = false>
hipError_t launch_bf16_layout(bool akc, bool bkc, const GemmArgs& a, hipStream_t s, hipEvent_t ev) {
  if (akc && bkc) return launch(gemm_bf16_kernel<BM, BN, AT, BT, true, true, PF, CHAIN>, bf16_smem<BM, BN, true, true>(), BM, BN, a, s, ev);
  if (akc && !bkc) return launch(gemm_bf16_kernel<BM, BN, AT, BT, true, false, PF, CHAIN>, bf16_smem<BM, BN, true, false>(), BM, BN, a, s, ev);
  if (!akc && bkc) return launch(gemm_bf16_kernel<BM, BN, AT, BT, false, true, PF, CHAIN>, bf16_smem<BM, BN, false, true>(), BM, BN, a, s, ev);
  return launch(gemm_bf16_kernel<BM, BN, AT, BT, false, false, PF, CHAIN>, bf16_smem<BM, BN, false, false>(), BM, BN, a, s, ev);
}

template <int BM, int BN>
hipError_t launch_f32_layout(bool akc, bool bkc, const GemmArgs& a, hipStream_t s, hipEvent_t ev) {
  if (akc && bkc) return launch(gemm_f32_kernel<BM, BN, true, true>, f32_smem<BM, BN, true, true>(), BM, BN, a, s, ev);
  if (akc && !bkc) return launch(gemm_f32_kernel<BM, BN, true, false>, f32_smem<BM, BN, true, false>(), BM, BN, a, s, ev);
  if (!akc && bkc) return launch(gemm_f32_kernel<BM, BN, false, true>, f32_smem<BM, BN, false, true>(), BM, BN, a, s, ev);
  return launch(gemm_f32_kernel<BM, BN, false, false>, f32_smem<BM, BN, false, false>(), BM, BN, a, s, ev);
}

bool a_kcontig(const GemmDesc& d) { return d.a.s_k == 1 || d.K == 1; }
bool b_kcontig(const GemmDesc& d) { return d.b.s_k == 1 || d.K == 1; }

}  // namespace

const char* gemm_kernel_name(const GemmDesc& d) {
  // the instantiation as a profiler prints it (without namespaces)
  static thread_local char buf[128];
  const bool af = d.a.prec == Prec::Single, bf = d.b.prec == Prec::Single;
  const int tile = big_tile(d) ? 256 : 128, tile_n = narrow_tile(d) ? 64 : tile;
  const char* tf[2] = {"false", "true"};
  if (af && bf)
    snprintf(buf, sizeof buf, "gemm_f32_kernel<%d, %d, %s, %s>", tile, tile, tf[a_kcontig(d)], tf[b_kcontig(d)]);
  else
    snprintf(buf, sizeof buf, "gemm_bf16_kernel<%d, %d, %s, %s, %s, %s, %d, %s>", tile, tile_n, af ? "float" : "unsigned short",
             bf ? "float" : "unsigned short", tf[a_kcontig(d)], tf[b_kcontig(d)], prefetch_depth(d), tf[!d.more.empty()]);
  return buf;
}

size_t gemm_workspace_bytes(const GemmDesc& d) {
  const int sp = split_count(d);
  return sp > 1 ? (size_t)sp * (size_t)batch_count(d) * (size_t)d.M * (size_t)d.N * sizeof(float) : 0;
}

hipError_t launch_gemm(const GemmDesc& d, const GemmArgs& a_in, void* workspace, hipStream_t s, hipEvent_t ev) {
  GemmArgs a = a_in;
  a.splits = split_count(d);
  a.ws = static_cast<float*>(workspace);
  const bool akc = a_kcontig(d), bkc = b_kcontig(d);
  const bool big = big_tile(d);
  {
    // XCD partition: every A panel is read by each of the xcd_n rectangle columns, every B panel
    // by each of the xcd_m rows
    const long tile = big ? 256 : 128, tile_n = narrow_tile(d) ? 64 : tile;
    const long tiles_m = (d.M + tile - 1) / tile, tiles_n = (d.N + tile_n - 1) / tile_n;
    const double a_bytes = (double)d.M * prec_in_bytes(d.a.prec), b_bytes = (double)d.N * prec_in_bytes(d.b.prec);
    // a grouped launch of 2 or 4 unbatched members without a K split: each member on 4 or 2 XCDs of
    // its own, so that its panels are fetched into that many L2 caches instead of all eight
    const int members = 1 + (int)d.group.size();
    int nx = 8;
    a.member_xcds = 0;
    if ((members == 2 || members == 4) && d.nbatch == 0 && a.splits == 1 && (tiles_m * tiles_n) % (8 / members) == 0) {
      nx = 8 / members;
      a.member_xcds = nx;
    }
    a.xcd_m = 0;
    double best = 0;
    for (int xm = 1; xm <= nx; xm *= 2) {
      const int xn = nx / xm;
      if (tiles_m % xm || tiles_n % xn) continue;
      const double cost = a_bytes * xn + b_bytes * xm;
      if (a.xcd_m == 0 || cost < best) { a.xcd_m = xm; best = cost; }
    }
  }
  const bool af = d.a.prec == Prec::Single, bf = d.b.prec == Prec::Single;
  if (af && bf) return big ? launch_f32_layout<256, 256>(akc, bkc, a, s, ev) : launch_f32_layout<128, 128>(akc, bkc, a, s, ev);
  if (a.npairs > 1 && (af || bf)) return hipErrorInvalidValue;   // chains: bf16 operands only
  if (!af && !bf) {
    if (a.npairs > 1) return launch_bf16_layout<128, 128, unsigned short, unsigned short, 2, true>(akc, bkc, a, s, ev);
    if (big) return launch_bf16_layout<256, 256, unsigned short, unsigned short>(akc, bkc, a, s, ev);
    if (narrow_tile(d))
      return prefetch_depth(d) == 2 ? launch_bf16_layout<128, 64, unsigned short, unsigned short, 2>(akc, bkc, a, s, ev)
                                    : launch_bf16_layout<128, 64, unsigned short, unsigned short>(akc, bkc, a, s, ev);
    return prefetch_depth(d) == 2 ? launch_bf16_layout<128, 128, unsigned short, unsigned short, 2>(akc, bkc, a, s, ev)
                                  : launch_bf16_layout<128, 128, unsigned short, unsigned short>(akc, bkc, a, s, ev);
  }
  if (af && !bf)
    return big ? launch_bf16_layout<256, 256, float, unsigned short>(akc, bkc, a, s, ev)
               : launch_bf16_layout<128, 128, float, unsigned short>(akc, bkc, a, s, ev);
  return big ? launch_bf16_layout<256, 256, unsigned short, float>(akc, bkc, a, s, ev)
             : launch_bf16_layout<128, 128, unsigned short, float>(akc, bkc, a, s, ev);
}

}  // namespace ocannl
