// Launch interface of the hand-written CDNA4 MFMA contraction kernels (gemm.hip).
#pragma once
#include <hip/hip_runtime.h>

#include "plan.hpp"

namespace ocannl {

// Device-side view of one strided-batched contraction.
struct GemmArgs {
  const void* a;
  const void* b;
  void* c;
  int64_t M, N, K;
  int64_t a_row, a_k, b_row, b_k, c_row;   // element strides; C is unit-stride along N
  int nbatch;
  int64_t batch_ext[3];
  int64_t a_batch[3], b_batch[3], c_batch[3];
  int accumulate;    // beta = 1
  int c_is_bf16;
  int xcd_m;         // tile-grid rows of the XCD partition (set by launch_gemm; 0: none)
  int member_xcds;   // > 0: every member of a grouped launch keeps to this many XCDs of its own (set by launch_gemm)
  int splits;        // split-K factor (set by launch_gemm)
  float* ws;         // split-K workspace [batch][split][M][N] (set by launch_gemm)
  // One launch may cover up to four independent contractions of identical shapes, strides and
  // precisions: member g > 0 uses a_more / b_more / c_more[g - 1], and the grid's z axis is
  // member * batches + batch.
  int ngroups;       // >= 1
  // A chain `c =+ a_p * b_p` into the same C (bf16 operands): K runs over a / b, then over
  // a_more[p - 1] / b_more[p - 1].  Never together with ngroups > 1.
  int npairs;        // >= 1
  int batches;       // product of batch_ext (set by launch_gemm)
  const void* a_more[3];
  const void* b_more[3];
  void* c_more[3];
  // When not null: a bf16 tensor of C's shape that receives the rounded result at the same element
  // offsets (C must be fp32).  It feeds later bf16 contractions that read C.
  void* c2;
  void* c2_more[3];
  // Epilogue fusion (bf16 C, no accumulation, no K split): when `bias` is not null the stored value is
  // bf16(bf16(acc) + bias[n]) (bias: bf16, indexed by the column); when `relu_out` is not null, relu of
  // the stored value also goes to that tensor at the same element offsets; with `relu_c` set the stored
  // value itself is the relu (C is the only tensor written).
  const void* bias;
  void* relu_out;
  int relu_c;
};

// Picks the kernel instance for the operand precisions / layouts and launches it on `stream`.
// Returns hipErrorInvalidValue for a combination the planner should not have produced.
// `workspace` must hold gemm_workspace_bytes(desc) bytes (may be null when that is 0).
// `after_main`, when not null, is recorded on the stream right after the contraction kernel itself
// (before the split-K reduction, if one follows), for per-kernel timing.
hipError_t launch_gemm(const GemmDesc& desc, const GemmArgs& args, void* workspace, hipStream_t stream,
                       hipEvent_t after_main = nullptr);

// Bytes of split-K workspace this contraction needs (0 when K is not split).
size_t gemm_workspace_bytes(const GemmDesc& desc);

// Name of the instance launch_gemm would pick (for kernel_info and profiles).
const char* gemm_kernel_name(const GemmDesc& desc);

}  // namespace ocannl
