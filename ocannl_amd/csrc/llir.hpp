// Loop IR received across the backend boundary: the C++ image of OCANNL's
// Low_level.optimized (arrayjit/lib/low_level.mli:22-68,160-166), Indexing.axis_index
// (arrayjit/lib/indexing.ml:104-120) and the tensor-node fields a device backend reads
// (arrayjit/lib/tnode.ml:33-64).  Parsed from the S-expression wire text the OCaml stub emits.
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace ocannl {

// Error classes mirroring the reference's exception split (arrayjit/lib/cuda_backend.ml:1017-1035):
// User_error for user mistakes, Invalid_argument for internal misuse.
struct UserError : std::runtime_error { using std::runtime_error::runtime_error; };
struct InvalidArgument : std::runtime_error { using std::runtime_error::runtime_error; };

enum class Prec : uint8_t {
  Void, Byte, Uint16, Int32, Uint32, Int64, Uint64, Uint4x32, Half, Bfloat16, Fp8, Single, Double
};
Prec prec_of_string(const std::string& s);
const char* prec_string(Prec p);       // Ops.prec_string, ops.ml:122-135
int prec_in_bytes(Prec p);             // Ops.prec_in_bytes, ops.ml:209-222
inline bool prec_is_intish(Prec p) {   // the integer-like arm of the ops.ml syntax tables
  return p == Prec::Byte || p == Prec::Uint16 || p == Prec::Int32 || p == Prec::Uint32 ||
         p == Prec::Int64 || p == Prec::Uint64 || p == Prec::Fp8;
}

enum class Mode : uint8_t { Ctx, Local, Virtual };

struct Node {
  int id = 0;
  std::string ident;
  Prec prec = Prec::Single;
  Mode mode = Mode::Ctx;
  bool zero_initialized_by_code = false;
  bool read_only = false;
  std::vector<int64_t> dims;
  int64_t num_elems() const { int64_t n = 1; for (auto d : dims) n *= d; return n; }
  int64_t size_in_bytes() const { return num_elems() * prec_in_bytes(prec); }
};

struct AxisIndex {
  enum Kind : uint8_t { Fixed, Iter, Affine } kind = Fixed;
  int64_t fixed = 0;                             // Fixed
  int sym = 0;                                   // Iter
  std::vector<std::pair<int64_t, int>> terms;    // Affine: (coeff, sym)
  int64_t offset = 0;                            // Affine
  bool operator==(const AxisIndex& o) const {
    return kind == o.kind && fixed == o.fixed && sym == o.sym && terms == o.terms && offset == o.offset;
  }
  bool mentions(int s) const {
    if (kind == Iter) return sym == s;
    if (kind == Affine) for (auto& t : terms) if (t.second == s) return true;
    return false;
  }
};
using Indices = std::vector<AxisIndex>;

enum class Binop : uint8_t { Arg1, Arg2, Add, Sub, Mul, Div, Pow, ReluGate, Sat01Gate, Max, Min, Mod,
                             Lt, Eq, Ne, Or, And, ThreefryCrypto, ThreefryLight };
enum class Unop : uint8_t { Id, Relu, Sat01, Exp, Log, Exp2, Log2, Sin, Cos, Sqrt, Recip, RecipSqrt,
                            Neg, Trunc, Tanh, Not, Uniform1 };
enum class Ternop : uint8_t { Where, Fma, Mul3 };

struct Stmt;
using StmtP = std::shared_ptr<Stmt>;
using Block = std::vector<StmtP>;

struct ScopeId { int node = 0; int scope = 0;
  bool operator==(const ScopeId& o) const { return node == o.node && scope == o.scope; }
  bool operator<(const ScopeId& o) const { return node != o.node ? node < o.node : scope < o.scope; } };

struct Scalar;
using ScalarP = std::shared_ptr<Scalar>;
struct Scalar {
  enum Kind : uint8_t { Get, GetDyn, GetMerge, GetLocal, LocalScope, Const, Bits, Index, Un, Bin, Tern } kind;
  int node = 0;              // Get / GetDyn / GetMerge
  Indices idcs;
  int dyn_axis = 0;          // GetDyn
  Prec arg_prec = Prec::Void;  // GetDyn index prec, Un argument prec, Tern first-argument prec
  ScopeId scope;             // GetLocal / LocalScope
  Block body;                // LocalScope
  double cst = 0;            // Const
  int64_t bits = 0;          // Bits
  AxisIndex index;           // Index
  Unop un{}; Binop bin{}; Ternop tern{};
  ScalarP a, b, c;
};

struct Stmt {
  enum Kind : uint8_t { Comment, For, ZeroOut, Set, SetVec, SetLocal, DeclareLocal } kind;
  std::string text;          // Comment; Set: its `debug` text when the routine was serialised with one
  int sym = 0; int64_t from = 0, to = 0;  // For (inclusive bounds, c_syntax.ml:450-456)
  Block body;                // For
  int node = 0;              // ZeroOut / Set / SetVec
  Indices idcs;
  ScalarP value;             // Set / SetLocal / SetVec argument
  int length = 0;            // SetVec
  Prec arg_prec = Prec::Void;  // SetVec
  ScopeId scope;             // SetLocal / DeclareLocal
  bool needs_init = false;   // DeclareLocal
};

struct StaticSym { int sym; int64_t range; /* -1: unbounded */ };

struct Routine {
  std::string name;
  std::vector<StaticSym> statics;
  int merge_node = -1;
  std::map<int, Node> nodes;
  std::vector<int> node_order;
  Block body;
  const Node& node(int id) const {
    auto it = nodes.find(id);
    if (it == nodes.end()) throw InvalidArgument("LLIR: unknown node id " + std::to_string(id));
    return it->second;
  }
  bool is_static(int sym) const { for (auto& s : statics) if (s.sym == sym) return true; return false; }
};

// Low_level.scalar_precision (arrayjit/lib/low_level.ml:76-90)
Prec scalar_precision(const Routine& r, const Scalar& s);

// Parses one or more "(routine ...)" forms.
std::vector<Routine> parse_routines(const char* text, size_t len);

inline std::string sym_ident(int s) { return "i" + std::to_string(s); }

}  // namespace ocannl
