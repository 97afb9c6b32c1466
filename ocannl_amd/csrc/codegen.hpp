// HIP source generation for the generic (non-MFMA) phases of a routine.
//
// The scalar expression printer follows the reference's C printer rule for rule -- evaluate every
// operation in the precision of the enclosing destination, convert on load, compute reduced
// precisions in float with a conversion around each single operation
// (arrayjit/lib/c_syntax.ml:706-855, arrayjit/lib/cc_backend.ml:169-323, tables
// arrayjit/lib/ops.ml:579-876) -- while the statement printer differs by design: instead of one
// serial function (c_syntax.ml:1021-1210) each phase becomes a __global__ kernel whose threads own
// the points of the phase's parallel index space.
#pragma once
#include <string>
#include <vector>

#include "plan.hpp"

namespace ocannl {

struct KernelParam {
  enum Kind { NodePtr, StaticIdx, MergeBuffer, LogId } kind;   // LogId: `int log_id`, the prefix of the run's log lines
  int id;   // node id (NodePtr; MergeBuffer: the node whose layout the buffer has) or static symbol
};

struct GeneratedKernel {
  std::string name;
  std::vector<KernelParam> params;
  uint64_t threads = 0;      // total threads wanted (points x cooperating lanes)
  int block = 256;
  int phase_index = -1;
};

struct GeneratedModule {
  std::string source;                      // builtins + all kernels
  std::vector<GeneratedKernel> kernels;    // one per generic phase, in phase order
};

const char* builtins_hip_source();

GeneratedModule generate_module(const Routine& r, const Plan& plan);

// C type of a precision as the reference's printer declares it (Ops.c_typ_of_prec, ops.ml:324-337),
// with the host's spelling of the half type: what the parameter lines of a routine's log show.
const char* c_typ_name(Prec p);

}  // namespace ocannl
