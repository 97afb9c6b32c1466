// Planner: splits a routine's loop nest into device kernels.
//
// The reference's GPU backends print the whole routine as ONE serial function run by one thread
// (arrayjit/lib/cuda_backend.ml:359-360,1043).  Here every top-level statement of the routine
// (arrayjit/lib/low_level.mli:22-51) becomes a *phase*; each phase is classified as
//   * Fill         -- Zero_out of a node (c_syntax.ml:468-479)
//   * Contraction  -- an accumulating `c[..] := fma(a[..], b[..], c[..])` nest
//                     (arrayjit/lib/assignments.ml:431-432, low_level.ml:1631-1634) big enough for
//                     the hand-written MFMA kernels
//   * Generic      -- anything else: a generated kernel with one thread (or one cooperating lane
//                     group) per point of the nest's parallel index space.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "llir.hpp"

namespace ocannl {

// One strided operand of a contraction, in elements.
struct GemmOperand {
  int node = -1;
  Prec prec = Prec::Single;
  int64_t offset = 0;                                  // constant part of the element offset
  std::vector<std::pair<int, int64_t>> static_terms;   // (static symbol, stride): added at launch
  int64_t s_row = 0;     // stride along M (A, C) or N (B)
  int64_t s_k = 0;       // stride along K (A, B); for C: stride along N
  int64_t s_batch[3] = {0, 0, 0};
};

// C[batch, m, n] (+)= sum_k A[batch, m, k] * B[batch, n, k], all strides explicit.
struct GemmDesc {
  GemmOperand a, b, c;
  int64_t M = 1, N = 1, K = 1;
  int nbatch = 0;
  int64_t batch_ext[3] = {1, 1, 1};
  bool accumulate = false;   // beta = 1: add into existing C (gradient accumulation `=+`)
  // Independent contractions of the same shapes, strides and precisions (the q / k / v projections of
  // one input, their weight gradients) that ride in the same launch: {a, b, c} per extra member.  A
  // small contraction alone puts at most one workgroup on a compute unit; several together let
  // workgroups hide each other's memory latency.
  // Further operand pairs of the same shapes, strides and precisions whose products go to the same C
  // (`c =+ a_i * b_i` statements: the input gradient of a tensor that feeds several projections): one
  // launch runs K over the first pair, then over these, and reads and writes C once.
  std::vector<std::pair<GemmOperand, GemmOperand>> more;
  struct Member { GemmOperand a, b, c; int c_copy = -1; };
  std::vector<Member> group;
  // >= 0: a bf16 scratch tensor of C's shape that the epilogue fills with the rounded result (C is
  // fp32 and written whole): it feeds later bf16 contractions that read C, in place of a conversion pass
  int c_copy = -1;
  // Pointwise consumers folded into the epilogue (bf16 results only; never with a K split, a group or a
  // chain).  The optimiser inlines the product `x = a * b` into `y := x + bias[n]` (either order) and
  // `z := relu(y)` reads y (lib/nn_blocks.ml:108-135, an mlp layer): the kernel then rounds x as the
  // inlined scalar would be, adds the bias, rounds again and stores that as C (= y), and stores relu of
  // it to `epi_relu`.  -1: absent.
  int epi_bias = -1;     // vector indexed by n, bf16
  int epi_relu = -1;     // tensor of C's shape and precision that receives relu(C); C itself: the stored value is the relu
  double flops() const {
    double f = 2.0 * (double)M * (double)N * (double)K * (double)(1 + group.size()) * (double)(1 + more.size());
    for (int i = 0; i < nbatch; ++i) f *= (double)batch_ext[i];
    return f;
  }
};

struct Phase {
  enum Kind { Generic, Fill, Contraction } kind = Generic;
  std::string label;          // human-readable, from the nearest preceding comment
  // Generic
  StmtP stmt;                 // the statement this phase runs
  std::vector<int> par_syms;  // parallel loop symbols, slowest first
  std::vector<int64_t> par_from, par_ext;
  std::vector<int> seq_syms;  // chain symbols that stay sequential inside a thread, outer first
  std::vector<int64_t> seq_from, seq_to;
  Block inner;                // body below the perfect-nest chain
  int coop_lanes = 1;         // >1: that many adjacent lanes share one output (tree-combined)
  // coop_lanes > 1 with no sequential chain loops: the lanes split the innermost loop of this
  // inlined scalar reduction `v { v := c; for.. { v := accum(v, e) } }` inside the statement
  const Scalar* coop_scope = nullptr;
  Binop coop_accum = Binop::Add;
  bool fused_zero_init = false;  // the preceding Zero_out of the target was folded in (beta = 0)
  // second half of a split reduction: adds the slices' partial sums, which lie one output tensor apart
  bool sums_partials = false;
  // Row group (kind Generic, `members` non-empty): consecutive phases that all work row by row
  // over the same rows -- pointwise over (rows x T), reductions of a row of T elements, per-row
  // scalars -- and whose mutual dependencies stay inside a row.  They run as ONE kernel in which a
  // group of `coop_lanes` lanes owns a row and executes the members in order (values pass through
  // memory, with a workgroup fence in between, and are read back from cache).
  std::vector<Phase> members;
  std::vector<int64_t> row_outer_ext;   // extents of the row index space, slowest first
  int64_t row_len = 0;                  // T
  enum RowRole : uint8_t { RowPointwise, RowReduce, RowScalar } row_role = RowPointwise;   // as a member
  std::vector<int> row_outer_syms;      // as a member: this phase's symbols for the outer axes, slowest first
  int row_sym = -1;                     // as a member: its symbol for the position in the row (-1: none)
  // Serial group (kind Generic, `serial_members` non-empty): a routine whose phases are all tiny runs
  // as ONE kernel of a single workgroup that executes the phases in order with a barrier in between
  // (dozens of launches of a few microseconds each would otherwise be pure launch latency).
  std::vector<Phase> serial_members;
  // Serial group: tensors whose first touch in the kernel is a store to all of their elements are
  // shadowed in LDS (node -> index of the member that makes the shadow valid): later members read
  // the shadow instead of waiting on global memory; every store still goes to global memory too.
  std::map<int, int> serial_shadows;
  // Parallel group (kind Generic, `parallel_members` non-empty): consecutive small phases that do not
  // depend on one another (the updates of many small parameters) run as ONE kernel in which every
  // member owns a range of workgroups.
  std::vector<Phase> parallel_members;
  // Row group with a contraction prologue (members non-empty, fused_x >= 0): the tensor `fused_x` that
  // the members read row by row -- the result of a `+*` contraction with a short K (attention scores
  // Q K^T, their gradient dOut V^T) -- is not read from memory: the kernel computes 32 rows of it on
  // the matrix cores into LDS (a workgroup owns 32 consecutive positions of outer axis `fused_m_axis`,
  // the other outer axes fixed), then its four waves run the members over eight rows each.  When the
  // tensor is a context node, or something later reads it, the rows are stored as well.
  int fused_x = -1;
  bool fused_x_store = false;
  GemmOperand fused_a, fused_b;                       // node, precision, constant offset (strides below)
  std::vector<int64_t> fused_a_stride, fused_b_stride;   // element stride per outer axis of the group
  int64_t fused_b_row = 0;                            // stride of B along the row position
  int64_t fused_k = 0;                                // contracted extent (unit stride in both operands)
  int fused_m_axis = -1;
  int fused_waves = 16;                               // waves per workgroup (each takes 32 / fused_waves of the rows)
  // ... and a contraction epilogue (proj_y >= 0; only with a prologue, whose 32-row workgroups it shares):
  // `c[o.., n] = sum_t y[o.., t] * b[.., t, n]`, where y is what a member of the group stores per row
  // position -- attention weights times V, the gradient of the scores times K -- is taken out of the
  // plan as well: the rows of y stay in LDS as bf16 and the workgroup multiplies its 32 x T tile with
  // b on the matrix cores.  b and c are unit-stride along n.
  int proj_y = -1;
  GemmOperand proj_b, proj_c;                           // node, precision, constant offset
  std::vector<int64_t> proj_b_stride, proj_c_stride;    // element stride per outer axis of the group
  int64_t proj_b_row = 0;                               // stride of b along t
  int64_t proj_n = 0;
  int proj_kp = 1;                                      // parts of T that separate waves sum up (partial results meet in LDS)
  int proj_c_copy = -1;                                 // bf16 copy of an fp32 c, stored alongside
  // Fill
  int fill_node = -1;
  // Contraction
  GemmDesc gemm;
  // Launch order across the device's two queues.  stream 1: this contraction is off the critical path
  // (nothing reads its result or rewrites its operands for a while: weight gradients wait for the
  // optimiser) and runs on the side queue, next to the phases that follow it on the main one.
  // wait_for: phases of the side queue that this phase must see finished before it starts.
  int stream = 0;
  std::vector<int> wait_for;
  // debug logging: the routine's top-level comments since the previous phase, logged ahead of this one
  std::vector<std::string> comments_before;
  // accounting (algorithmic): distinct elements read + written, and flops
  double bytes = 0, flops = 0;
};

struct PlanOptions {
  int64_t min_mfma_flops = 1 << 22;   // below this a contraction stays a generic kernel
  bool enable_mfma = true;
  bool enable_coop = true;
  bool enable_row_groups = true;
  bool enable_serial_group = true;   // tiny routines as one single-workgroup kernel
  bool group_contractions = true;   // independent contractions of equal shapes as one launch
  bool merge_chains = true;         // `c =+ a_i * b_i` chains of equal shapes as one launch
  bool enable_parallel_groups = true;   // consecutive independent small phases as one launch
  bool large_models = false;        // 64-bit offsets in generated kernels even when every node is small
  // debug_log_from_routines (arrayjit/lib/utils.ml:591, c_syntax.ml:493-535): every statement logs what
  // it computes.  The reference runs a routine as one thread, so its log is in program order; here
  // every top-level statement becomes a kernel of ONE thread that walks its loops in order, and none
  // of the fusing rewrites applies.
  bool debug_log = false;
  // row groups: a lane takes runs of four neighbouring row positions, for 16-byte accesses.  Off:
  // measured on the transformer step the wide accesses were 5-8% slower than one position per lane
  // per unrolled iteration (these kernels are bound by the memory system, not by instruction count).
  bool row_vec4 = false;
  // plain runs replay a captured HIP graph of the routine's kernels.  Off by default: measured on
  // MI355X / ROCm 7.2 it pays only for a routine of about ten tiny kernels (half-moons step as ten
  // launches: 40 -> 26 us); nine kernels of the char-MLP step went 36 -> 42 us and the 127 kernels of
  // the transformer step 3.68 -> 3.73 ms.
  bool use_graphs = false;
  int group_window = 1 << 30;        // contractions share a launch only when at most this many phases apart
  // contractions off the critical path run on a second queue beside the rest (side_queue=1).  Off:
  // measured on the transformer step it gains 0.9 % (3.528 -> 3.495 ms), less than the step varies from
  // box to box, and every per-kernel duration (profilers, event brackets) becomes a time on a shared chip
  bool side_queue = false;
  bool side_queue_generated = false;  // ... and generated kernels of a few MB that nothing waits for (side_queue=2): measured, no gain
  bool fuse_epilogues = true;        // bias / relu consumers of an inlined contraction run in the contraction's epilogue
  bool fuse_row_contractions = true; // a short-K contraction feeding a row group runs as that kernel's prologue ...
  int row_tile_waves = 0;            // waves per workgroup of those kernels (4, 8 or 16); 0: 16 for rows of at most 512, else 8
  bool fuse_row_projections = true;   // contraction epilogue of a row group with a prologue (see Phase::proj_y)
  bool fuse_stored_rows = false;     // ... also when its result has to be stored anyway (a context node): measured slower
  // a sub-expression that recomputes what an earlier statement stored (the reference's optimiser inlines a
  // tensor into every reader at the assigned position: the backward pass of a relu holds the whole
  // contraction behind its argument again) reads the stored tensor instead (reuse.cpp)
  bool reuse_stored = true;
  bool enable_bf16_copies = true;   // keep bf16 copies of fp32 operands of mixed contractions (written by the producing kernels)
};

struct Plan {
  std::vector<Phase> phases;
  std::vector<Node> scratch;   // nodes invented by the planner (de-virtualised contraction results)
  // fp32 node -> bf16 scratch copy kept in step by every generated store to the node (a store to
  // the node also stores the rounded value to the copy): the copy feeds bf16 contractions
  std::map<int, int> mirrors;
  bool large_index = false;    // generated kernels compute offsets in 64 bits
  bool use_graphs = false;     // plain runs are replayed from a captured HIP graph
  bool row_vec4 = false;       // row groups: a lane takes runs of four neighbouring row positions (16-byte accesses)
  bool debug_log = false;      // generated kernels print what they compute (and take an `int log_id` argument)
  std::vector<std::string> trailing_comments;   // debug logging: comments after the last phase
};

Plan make_plan(Routine& r, const PlanOptions& opt);

// Rewrites, in place, sub-expressions of later statements that recompute a value an earlier statement
// stored (see reuse.cpp); returns how many it replaced.
int reuse_stored_values(Routine& r);

// Positions of ph.par_syms ordered by their stride in the first array the phase writes, slowest
// first: adjacent threads take adjacent values of the last one (coalesced stores).
std::vector<size_t> store_order(const Routine& r, const Phase& ph);

}  // namespace ocannl
