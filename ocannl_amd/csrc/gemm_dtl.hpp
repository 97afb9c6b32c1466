// bf16 contraction kernel whose operand tiles go from global memory straight into LDS
// (global_load_lds_dwordx4: no staging registers, no LDS store instructions), so that NS >= 3
// stages of K can be in flight per workgroup.  For full tiles of bf16 operands only (M % BM == 0,
// N % BN == 0, every K split a multiple of BK, 16-byte aligned rows); launch_gemm sends everything
// else to the register-staged kernels.
//
// A wave-wide direct load moves 64 x 16 bytes and lands them at consecutive LDS addresses in lane
// order: padding between rows is not available, so bank conflicts are avoided by choosing WHICH
// 16-byte chunk of the tile a lane fetches (an XOR swizzle of the chunk position):
//   K-contiguous operand, tile held [row][k], row = BK * 2 bytes (64 or 128):
//     chunk c of row r sits at position c ^ ((r / RP) & (CPR - 1)) of its row, RP = rows per 256
//     bytes, CPR = chunks per row: the ds_read_b128 of 16 consecutive rows at one k touch 16
//     different 16-byte bank groups.
//   row-contiguous operand, tile held [k][row] as it lies in memory, k-line = ROWS * 2 bytes:
//     chunk c of k-line kl sits at position c ^ ((kl & 3) << 2) (ROWS >= 128) or
//     c ^ (((kl >> 1) & 1) << 2) (ROWS = 64): the four k-lines that one ds_read_b64_tr_b16 of 32
//     lanes touches land in four different 64-byte bank groups.
// The 1 KB blocks of a tile are dealt to the four waves round robin (block b to wave b % 4), which
// makes the swizzle term of a lane independent of the block: one 32-bit lane offset per operand.
//
// Pipeline (one barrier per K step, placed ahead of the LAST 16-k sub-step of the step): at that
// point every wave has issued all fragment reads of the previous step, so its stage is free: the
// loads of K step ks + NS - 1 go there, and the first fragments of step ks + 1 (whose stage the
// wait ahead of the barrier has seen land) are read under the MFMAs of the last sub-step -- the
// matrix pipe never waits for LDS latency at a step boundary.
#pragma once
#include "gemm_common.hpp"

namespace ocannl {
namespace {

// One wave-wide direct load: 16 bytes per lane from `base + voff` (base uniform, voff a per-lane
// byte offset) to LDS byte address `lds + 16 * lane` (lds uniform).  Written as assembly so that the
// compiler's wait-count insertion does not see an LDS write it would wait for ahead of every LDS
// read; the waits are placed by hand (dtl_wait).  The instruction needs one wait state after the
// write of M0.
__device__ __forceinline__ void dtl_load16(const void* base, unsigned voff, unsigned lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds), "v"(voff), "s"(base) : "memory");
}
// At most N vector-memory operations of this wave still in flight (they complete in order).
template <int N>
__device__ __forceinline__ void dtl_wait() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __forceinline__ void lds_wait_all() { asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); }

// A pointer that is the same in every lane, moved to scalar registers.
template <typename T>
__device__ __forceinline__ const T* uniform_ptr(const T* p) {
  const unsigned long v = reinterpret_cast<unsigned long>(p);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  return reinterpret_cast<const T*>(((unsigned long)hi << 32) | lo);
}

template <int ROWS, int BK, bool KC>
struct DtlTile {
  static constexpr int kBytes = ROWS * BK * 2;
  static constexpr int kOps = kBytes / 1024 / 4;   // direct loads per wave and stage
  static_assert(kBytes % 4096 == 0, "a tile is a whole number of 1 KB blocks per wave");
  // K-contiguous
  static constexpr int kRowBytes = BK * 2, kCPR = BK / 8, kRP = 256 / kRowBytes, kRPB = 1024 / kRowBytes;
  // row-contiguous
  static constexpr int kLineBytes = ROWS * 2, kCPL = kLineBytes / 16, kLPB = 1024 / kLineBytes;
  static_assert(KC || ROWS == 64 || ROWS == 128 || ROWS == 256, "k-lines of 128, 256 or 512 bytes");
  static_assert(BK == 32 || BK == 64, "rows of 64 or 128 bytes");

  // rows (KC) or k-lines (!KC) between the blocks that consecutive loads of one wave fetch
  static constexpr int kOpLines = (KC ? kRPB : kLPB) * 4;

  // per-lane byte offset into global memory of the chunk this lane fetches in the wave's first block
  // (`ld`: elements between rows / k-lines)
  static __device__ __forceinline__ unsigned lane_goff(int wave, int lane, long ld) {
    if constexpr (KC) {
      const int r = kRPB * wave + lane / kCPR;
      const int c = (lane % kCPR) ^ ((r / kRP) & (kCPR - 1));
      return (unsigned)((r * ld + c * 8) * 2);
    } else {
      const int kl = kLPB * wave + lane / kCPL;
      const int sw = ROWS >= 128 ? (kl & 3) << 2 : ((kl >> 1) & 1) << 2;
      const int c = (lane % kCPL) ^ sw;
      return (unsigned)((kl * ld + c * 8) * 2);
    }
  }

  // per-lane byte offset of the MFMA fragment of 32-row block 0, sub-step 0, inside the tile; `w0`:
  // first row of the wave's block of rows
  static __device__ __forceinline__ unsigned lane_frag(int lane, int w0) {
    if constexpr (KC) {
      const int r = lane & 31;
      const int sw = (r / kRP) & (kCPR - 1);
      return (unsigned)((w0 + r) * kRowBytes + (((lane >> 5) ^ sw) * 16));
    } else {
      const int p = lane & 15;
      const int sw = ROWS >= 128 ? (p >> 2) & 3 : (p >> 3) & 1;
      return (unsigned)(((lane >> 5) * 8 + (p >> 2)) * kLineBytes + ((w0 * 2 + ((lane >> 4) & 1) * 32 + (p & 3) * 8) ^ (sw * 64)));
    }
  }

  // fragment of 32-row block `blk`, 16-k sub-step `kk`; `tile`: the tile's first byte in LDS
  template <int BLK, int KK>
  static __device__ __forceinline__ bf16x8 fragment(const unsigned char* tile, unsigned frag) {
    if constexpr (KC) {
      return *reinterpret_cast<const bf16x8*>(tile + (frag ^ (unsigned)(KK * 32)) + BLK * 32 * kRowBytes);
    } else {
      return tr_fragment(reinterpret_cast<const unsigned short*>(tile + (frag ^ (unsigned)(BLK * 64)) + KK * 16 * kLineBytes), kLineBytes / 2);
    }
  }
};

template <int BM, int BN, int BK, int NS>
constexpr size_t dtl_smem() { return (size_t)NS * (BM + BN) * BK * 2; }

template <int BM, int BN, int BK, int NS, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, (BM * BN >= 256 * 256) ? 1 : 2)))
gemm_bf16_dtl_kernel(const GemmArgs g) {
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 32, TN = WN / 32;
  using TA = DtlTile<BM, BK, A_KC>;
  using TB = DtlTile<BN, BK, B_KC>;
  constexpr int kStage = TA::kBytes + TB::kBytes;
  constexpr int kOps = TA::kOps + TB::kOps;
  constexpr int kSub = BK / 16, kPer = TM * TN, kR = TM + TN;
  static_assert(NS >= 3, "the barrier ahead of the last sub-step needs three stages");
  static_assert((NS - 2) * kOps < 64, "loads in flight fit the counter");
  extern __shared__ __align__(16) unsigned short smem[];
  unsigned char* const lds = reinterpret_cast<unsigned char*>(smem);
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) void*)smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
  const long tiles_m = g.M / BM, tiles_n = g.N / BN;
  long tmi, tni, wg, zz;
  int nx;
  place_workgroup(g, wg, zz, nx);
  tile_of_block(wg, tiles_m, tiles_n, g.xcd_m, nx, tmi, tni);
  const long m0 = tmi * BM, n0 = tni * BN;
  long ao, bo, co;
  const void *abase, *bbase;
  void *cbase, *c2base;
  decode_batch(g, decode_group(g, zz, abase, bbase, cbase, c2base), ao, bo, co);
  const long lda = A_KC ? g.a_row : g.a_k, ldb = B_KC ? g.b_row : g.b_k;

  // split-K: blockIdx.y owns a contiguous range of K steps
  const long all_steps = g.K / BK;
  const long per_split = (all_steps + g.splits - 1) / g.splits;
  const long sbeg = (long)blockIdx.y * per_split;
  const long send = sbeg + per_split < all_steps ? sbeg + per_split : all_steps;
  const int ksteps = send > sbeg ? (int)(send - sbeg) : 0;

  // uniform source of the next stage to fetch (first element of the tile at that K step), advanced per stage
  // (the batch decoding divides in vector registers: the addresses are uniform, say so)
  const unsigned short* a_src = uniform_ptr(static_cast<const unsigned short*>(abase) + ao + (A_KC ? m0 * lda + sbeg * BK : sbeg * BK * lda + m0));
  const unsigned short* b_src = uniform_ptr(static_cast<const unsigned short*>(bbase) + bo + (B_KC ? n0 * ldb + sbeg * BK : sbeg * BK * ldb + n0));
  const long a_adv = A_KC ? BK : BK * lda, b_adv = B_KC ? BK : BK * ldb;
  const long a_op = (long)TA::kOpLines * lda, b_op = (long)TB::kOpLines * ldb;   // elements between a wave's loads
  const unsigned a_goff = TA::lane_goff(wave, lane, lda), b_goff = TB::lane_goff(wave, lane, ldb);
  unsigned fetch_lds = lds0 + wave * 1024;   // LDS byte address of this wave's first block in the stage being fetched
  int fetch_stage = 0;
  auto advance_fetch = [&]() OCN_LAMBDA_INLINE {
    a_src += a_adv; b_src += b_adv;
    ++fetch_stage; fetch_lds += kStage;
    if (fetch_stage == NS) { fetch_stage = 0; fetch_lds -= NS * kStage; }
  };
  // load number `o` of the stage being fetched (compile-time): A's blocks, then B's
  auto fetch_op = [&](auto oc) OCN_LAMBDA_INLINE {
    constexpr int o = decltype(oc)::value;
    if constexpr (o < TA::kOps) dtl_load16(a_src + o * a_op, a_goff, fetch_lds + o * 4096);
    else dtl_load16(b_src + (o - TA::kOps) * b_op, b_goff, fetch_lds + TA::kBytes + (o - TA::kOps) * 4096);
  };

  const unsigned a_frag = TA::lane_frag(lane, wm0), b_frag = TB::lane_frag(lane, wn0);
  f32x16 acc[TM][TN];
  static_for<TM>([&](auto ic) OCN_LAMBDA_INLINE {
    static_for<TN>([&](auto jc) OCN_LAMBDA_INLINE {
      static_for<16>([&](auto ec) OCN_LAMBDA_INLINE { acc[decltype(ic)::value][decltype(jc)::value][decltype(ec)::value] = 0.0f; });
    });
  });
  bf16x8 af[2][TM], bf[2][TN];
  // fragment number r (A's blocks, then B's) of sub-step kk from the stage starting at `st`
  auto read_frag = [&](const unsigned char* st, auto kkc, auto rc) OCN_LAMBDA_INLINE {
    constexpr int kk = decltype(kkc)::value, r = decltype(rc)::value, fb = kk & 1;
    if constexpr (r < TM) af[fb][r] = TA::template fragment<r, kk>(st, a_frag);
    else bf[fb][r - TM] = TB::template fragment<r - TM, kk>(st + TA::kBytes, b_frag);
  };

  // The kOps loads of a stage are spread evenly over the kAll MFMAs that follow the barrier that
  // frees its slot: load o goes ahead of MFMA number o * kAll / kOps of that window, which covers
  // the last sub-step of one K step (the "tail" part of the stage) and the sub-steps ahead of the
  // barrier of the next (its "head" part) -- clumped loads would fill the memory pipeline's queue
  // and stall the MFMAs behind them.
  constexpr int kAll = kSub * kPer;
  auto fetch_at = [&](auto wc) OCN_LAMBDA_INLINE {
    static_for<kOps>([&](auto oc) OCN_LAMBDA_INLINE {
      constexpr int o = decltype(oc)::value;
      if constexpr (o * kAll / kOps == decltype(wc)::value) fetch_op(oc);
    });
  };
  // One K step on the stage starting at `st`.  kHead: the sub-steps ahead of the barrier issue the
  // head part of the stage being fetched, which is then complete.  kWait >= 0: ahead of the last
  // sub-step, wait until at most kWait loads are in flight (the next stage has landed) and meet the
  // other waves; then, under the MFMAs of the last sub-step, issue the tail part of a further stage
  // (kTail) and read the first fragments of the next stage (kNext), which starts at `nx`.
  auto step = [&](const unsigned char* st, const unsigned char* nx, auto head_c, auto wait_c, auto tail_c, auto next_c) OCN_LAMBDA_INLINE {
    constexpr int kWait = decltype(wait_c)::value;
    constexpr bool kHead = decltype(head_c)::value, kTail = decltype(tail_c)::value, kNext = decltype(next_c)::value;
    static_for<kSub>([&](auto kkc) OCN_LAMBDA_INLINE {
      constexpr int kk = decltype(kkc)::value, fb = kk & 1;
      constexpr bool last = kk + 1 == kSub;
      if constexpr (last) {
        if constexpr (kHead) advance_fetch();
        if constexpr (kWait >= 0) {
          dtl_wait<kWait>();
          lds_wait_all();
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      static_for<kPer>([&](auto mc) OCN_LAMBDA_INLINE {
        constexpr int idx = decltype(mc)::value, i = idx / TN, j = idx % TN;
        constexpr int r0 = idx * kR / kPer, r1 = (idx + 1) * kR / kPer;
        if constexpr (!last) {
          static_for<r1 - r0>([&](auto rc) OCN_LAMBDA_INLINE {
            read_frag(st, std::integral_constant<int, kk + 1>{}, std::integral_constant<int, r0 + decltype(rc)::value>{});
          });
          if constexpr (kHead) fetch_at(std::integral_constant<int, (kk + 1) * kPer + idx>{});
        } else {
          if constexpr (kNext) {
            static_for<r1 - r0>([&](auto rc) OCN_LAMBDA_INLINE {
              read_frag(nx, std::integral_constant<int, 0>{}, std::integral_constant<int, r0 + decltype(rc)::value>{});
            });
          }
          if constexpr (kTail) fetch_at(std::integral_constant<int, idx>{});
        }
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[fb][i], bf[fb][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  using Y = std::true_type; using N = std::false_type;
  auto fetch_stage_now = [&]() OCN_LAMBDA_INLINE {
    static_for<kOps>([&](auto oc) OCN_LAMBDA_INLINE { fetch_op(oc); });
    advance_fetch();
  };
  auto first_frags = [&](const unsigned char* st) OCN_LAMBDA_INLINE {
    static_for<kR>([&](auto rc) OCN_LAMBDA_INLINE { read_frag(st, std::integral_constant<int, 0>{}, rc); });
  };

  if (ksteps >= NS - 1) {
    // prologue: stages 0 .. NS - 3, then what the tail of a step does: wait for stage 0, barrier,
    // fetch stage NS - 2, first fragments
    static_for<NS - 2>([&](auto) OCN_LAMBDA_INLINE { fetch_stage_now(); });
    dtl_wait<(NS - 3) * kOps>();
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    static_for<kPer>([&](auto wc) OCN_LAMBDA_INLINE { fetch_at(wc); });   // tail part of stage NS - 2
    first_frags(lds);
    int cur = 0;   // stage of the step being multiplied
    auto stage_ptr = [&](int s) OCN_LAMBDA_INLINE { return lds + s * kStage; };
    auto next_of = [&](int s) OCN_LAMBDA_INLINE { return s + 1 == NS ? 0 : s + 1; };
    int ks = 0;
    for (; ks + NS - 1 < ksteps; ++ks) {
      const int nxt = next_of(cur);
      step(stage_ptr(cur), stage_ptr(nxt), Y{}, std::integral_constant<int, (NS - 3) * kOps>{}, Y{}, Y{});
      cur = nxt;
    }
    // NS - 1 steps are left: the first completes the last stage's fetch, then nothing more to fetch.
    // With `rem` steps left (this one included), the stages after the next one that are still in
    // flight number min(NS - 3, rem - 2).
    static_for<NS - 1>([&](auto tc) OCN_LAMBDA_INLINE {
      constexpr int rem = NS - 1 - decltype(tc)::value;
      using Head = std::integral_constant<bool, rem == NS - 1>;
      const int nxt = next_of(cur);
      if constexpr (rem > 1) {
        constexpr int fl = (rem - 2) < (NS - 3) ? (rem - 2) : (NS - 3);
        step(stage_ptr(cur), stage_ptr(nxt), Head{}, std::integral_constant<int, fl * kOps>{}, N{}, Y{});
      } else {
        step(stage_ptr(cur), stage_ptr(nxt), Head{}, std::integral_constant<int, -1>{}, N{}, N{});
      }
      cur = nxt;
    });
  }
  // (launch_gemm sends a contraction with fewer than NS - 1 K steps per split to the other kernels)
  // every wave's fragment reads are complete (the MFMAs that consume them were issued) once all
  // waves have passed this barrier: the stages are free for the epilogue's staging area
  lds_wait_all();
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  constexpr int kStageFloats = 32 * (TN * 32 + 4);
  static_assert((size_t)4 * kStageFloats * 4 <= dtl_smem<BM, BN, BK, NS>(), "epilogue staging fits the operand stages");
  epilogue<TM, TN>(g, cbase, c2base, acc, m0 + wm0, n0 + wn0, co, lane, reinterpret_cast<float*>(smem) + wave * kStageFloats);
}

}  // namespace
}  // namespace ocannl
