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
#include "gemm_common.hpp"

namespace ocannl {

// gemm_dtl.hip: the direct-to-LDS instance of that shape (one of those dtl_shape() names).
hipError_t launch_gemm_dtl(int bm, int bn, int bk, int ns, bool akc, bool bkc, const GemmArgs& a, hipStream_t s, hipEvent_t ev);

namespace {


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

// ---- the direct-to-LDS kernel (gemm_dtl.hpp) -----------------------------------------------------
// Shape of the instance for a contraction, or bm = 0 when the register-staged kernels take it: bf16
// operands, full tiles, every K split a whole number of at least NS - 1 steps.  256 x 256 tiles run
// four stages of 32 k (128 KB of LDS); 128 x 128 tiles five stages of 64 k when the launch puts at
// most one workgroup on a compute unit -- what such a launch lacks is loads in flight -- and four
// stages of 32 k (64 KB: two workgroups per compute unit) otherwise; 128 x 64 tiles (results of at
// most 64 columns: short-K batched products of attention) four stages of 32 k (48 KB: three
// workgroups per compute unit, measured 2 % of a transformer step against five stages of 64 k).
struct DtlShape { int bm = 0, bn = 0, bk = 0, ns = 0; };

DtlShape dtl_shape(const GemmDesc& d) {
  DtlShape none, s;
  if (d.a.prec != Prec::Bfloat16 || d.b.prec != Prec::Bfloat16 || !d.more.empty()) return none;
  const TileConfig c = tile_config(d);
  if (c.big) s = {256, 256, 32, 4};
  else if (c.narrow) s = {128, 64, 32, 4};
  else {
    const long t128 = ((d.M + 127) / 128) * ((d.N + 127) / 128) * batch_count(d);
    if (t128 * c.splits <= 256) s = {128, 128, 64, 5};
    else s = {128, 128, 32, 4};
  }
  if (d.M % s.bm || d.N % s.bn || d.K % s.bk) return none;
  const long steps = d.K / s.bk;
  if (steps % c.splits || steps / c.splits < s.ns - 1) return none;
  return s;
}

// Operand addresses and strides as the direct loads need them: 16-byte aligned bases and lines, lane
// offsets within 32 bits.
bool dtl_operands_ok(const GemmArgs& a, bool akc, bool bkc) {
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const int64_t lda = akc ? a.a_row : a.a_k, ldb = bkc ? a.b_row : a.b_k;
  if (!aligned(a.a) || !aligned(a.b) || lda % 8 || ldb % 8 || lda <= 0 || ldb <= 0 || lda >= (1 << 24) || ldb >= (1 << 24)) return false;
  if ((akc ? a.a_k : a.a_row) != 1 || (bkc ? a.b_k : a.b_row) != 1) return false;
  for (int i = 0; i < a.nbatch; ++i) if (a.a_batch[i] % 8 || a.b_batch[i] % 8) return false;
  for (int g = 1; g < a.ngroups; ++g) if (!aligned(a.a_more[g - 1]) || !aligned(a.b_more[g - 1])) return false;
  return true;
}

}  // namespace

const char* gemm_kernel_name(const GemmDesc& d) {
  // the instantiation as a profiler prints it (without namespaces)
  static thread_local char buf[128];
  const bool af = d.a.prec == Prec::Single, bf = d.b.prec == Prec::Single;
  const int tile = big_tile(d) ? 256 : 128, tile_n = narrow_tile(d) ? 64 : tile;
  const char* tf[2] = {"false", "true"};
  const DtlShape ds = dtl_shape(d);
  if (af && bf)
    snprintf(buf, sizeof buf, "gemm_f32_kernel<%d, %d, %s, %s>", tile, tile, tf[a_kcontig(d)], tf[b_kcontig(d)]);
  else if (ds.bm)   // (operands that turn out misaligned at launch take the register-staged kernel instead)
    snprintf(buf, sizeof buf, "gemm_bf16_dtl_kernel<%d, %d, %d, %d, %s, %s>", ds.bm, ds.bn, ds.bk, ds.ns, tf[a_kcontig(d)], tf[b_kcontig(d)]);
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
    const DtlShape ds = dtl_shape(d);
    if (ds.bm && a.npairs == 1 && dtl_operands_ok(a, akc, bkc)) {
      return launch_gemm_dtl(ds.bm, ds.bn, ds.bk, ds.ns, akc, bkc, a, s, ev);
    }
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
