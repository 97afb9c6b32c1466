#include "codegen.hpp"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <functional>
#include <set>
#include <sstream>

namespace ocannl {
namespace {

// ------------------------------------------------------------------------------------------------
// syntax tables (arrayjit/lib/ops.ml)
// ------------------------------------------------------------------------------------------------

const char* c_typ(Prec p) {   // Ops.c_typ_of_prec, ops.ml:324-337 (HALF_T = _Float16 on device)
  switch (p) {
    case Prec::Byte: return "unsigned char";
    case Prec::Uint16: return "unsigned short";
    case Prec::Int32: return "int";
    case Prec::Uint32: return "uint32_t";
    case Prec::Int64: return "long long";
    case Prec::Uint64: return "uint64_t";
    case Prec::Uint4x32: return "uint4x32_t";
    case Prec::Half: return "HALF_T";
    case Prec::Bfloat16: return "unsigned short";
    case Prec::Fp8: return "unsigned char";
    case Prec::Single: return "float";
    case Prec::Double: return "double";
    case Prec::Void: return "void";
  }
  return "void";
}

std::string c_vec_typ(int length, Prec p) {   // Ops.c_vec_typ_of_prec, ops.ml:339-351
  if (p == Prec::Single && length == 4) return "float4_t";
  if (p == Prec::Double && length == 2) return "double2_t";
  if (p == Prec::Int32 && length == 4) return "int32x4_t";
  if (p == Prec::Uint32 && length == 4) return "uint32x4_t";
  if (p == Prec::Int64 && length == 2) return "int64x2_t";
  if (p == Prec::Uint64 && length == 2) return "uint64x2_t";
  if ((p == Prec::Byte || p == Prec::Fp8) && length == 16) return "int8x16_t";
  if ((p == Prec::Uint16 || p == Prec::Bfloat16) && length == 8) return "uint16x8_t";
  if (p == Prec::Half && length == 8) return "half8_t";
  if (length == 1) return c_typ(p);
  throw InvalidArgument("vector type: invalid (precision, length) combination");
}

bool plain_int(Prec p) {
  return p == Prec::Byte || p == Prec::Uint16 || p == Prec::Int32 || p == Prec::Uint32 ||
         p == Prec::Int64 || p == Prec::Uint64;
}
bool dbl_or_intish(Prec p) { return p == Prec::Double || prec_is_intish(p); }

using Pair = std::pair<std::string, std::string>;

Pair convert_precision(Prec f, Prec t) {   // Ops.c_convert_precision, ops.ml:808-876
  if (f == t) return {"", ""};
  using P = Prec;
  if (f == P::Bfloat16 && t == P::Single) return {"bfloat16_to_single(", ")"};
  if (f == P::Single && t == P::Bfloat16) return {"single_to_bfloat16(", ")"};
  if (f == P::Bfloat16 && t == P::Double) return {"(double)bfloat16_to_single(", ")"};
  if (f == P::Double && t == P::Bfloat16) return {"single_to_bfloat16((float)", ")"};
  if (f == P::Fp8 && t == P::Single) return {"fp8_to_single(", ")"};
  if (f == P::Single && t == P::Fp8) return {"single_to_fp8(", ")"};
  if (f == P::Fp8 && t == P::Double) return {"(double)fp8_to_single(", ")"};
  if (f == P::Double && t == P::Fp8) return {"single_to_fp8((float)", ")"};
  if (f == P::Bfloat16 && t == P::Half) return {"FLOAT_TO_HALF(bfloat16_to_single(", "))"};
  if (f == P::Half && t == P::Bfloat16) return {"single_to_bfloat16(HALF_TO_FLOAT(", "))"};
  if (f == P::Bfloat16 && plain_int(t)) return {std::string("(") + c_typ(t) + ")bfloat16_to_single(", ")"};
  if (plain_int(f) && t == P::Bfloat16) return {"single_to_bfloat16((float)", ")"};
  if (f == P::Fp8 && t == P::Half) return {"FLOAT_TO_HALF(fp8_to_single(", "))"};
  if (f == P::Half && t == P::Fp8) return {"single_to_fp8(HALF_TO_FLOAT(", "))"};
  if (f == P::Fp8 && plain_int(t)) return {std::string("(") + c_typ(t) + ")fp8_to_single(", ")"};
  if (plain_int(f) && t == P::Fp8) return {"single_to_fp8((float)", ")"};
  if (f == P::Bfloat16 && t == P::Fp8) return {"single_to_fp8(bfloat16_to_single(", "))"};
  if (f == P::Fp8 && t == P::Bfloat16) return {"single_to_bfloat16(fp8_to_single(", "))"};
  if (f == P::Half && t == P::Single) return {"HALF_TO_FLOAT(", ")"};
  if (f == P::Single && t == P::Half) return {"FLOAT_TO_HALF(", ")"};
  if (f == P::Half && t == P::Double) return {"(double)HALF_TO_FLOAT(", ")"};
  if (f == P::Double && t == P::Half) return {"FLOAT_TO_HALF((float)", ")"};
  if (f == P::Half && plain_int(t)) return {std::string("(") + c_typ(t) + ")HALF_TO_FLOAT(", ")"};
  if (plain_int(f) && t == P::Half) return {"FLOAT_TO_HALF((float)", ")"};
  if (f == P::Uint4x32) return {std::string("uint4x32_to_") + prec_string(t) + "(", ")"};
  if (t == P::Uint4x32) return {std::string(prec_string(f)) + "_to_uint4x32(", ")"};
  return {std::string("(") + c_typ(t) + ")(", ")"};
}

struct Syn3 { std::string p, i, s; };
struct Syn4 { std::string p, i1, i2, s; };

Syn3 binop_syntax(Prec prec, Binop op) {   // Ops.binop_c_syntax, ops.ml:579-630
  const bool ii = prec_is_intish(prec);
  switch (op) {
    case Binop::Add: return {"(", " +", ")"};
    case Binop::Sub: return {"(", " -", ")"};
    case Binop::Mul: return {"(", " *", ")"};
    case Binop::Div: return {"(", " /", ")"};
    case Binop::Pow:
      if (prec == Prec::Double) return {"pow(", ",", ")"};
      if (ii) throw InvalidArgument("ToPowOf not supported for integer precisions");
      return {"powf(", ",", ")"};
    case Binop::ReluGate: return ii ? Syn3{"(", " > 0 ?", " : 0)"} : Syn3{"(", " > 0.0 ?", " : 0.0)"};
    case Binop::Sat01Gate:
      if (ii) return {"(abs(", " ) > 0 ? 0 : (", "))"};
      if (prec == Prec::Single) return {"(fabsf(floorf(", ")) > 0.0 ? 0.0 : (", "))"};
      return {"(fabs(floor(", ")) > 0.0 ? 0.0 : (", "))"};
    case Binop::Max: return dbl_or_intish(prec) ? Syn3{"fmax(", ",", ")"} : Syn3{"fmaxf(", ",", ")"};
    case Binop::Min: return dbl_or_intish(prec) ? Syn3{"fmin(", ",", ")"} : Syn3{"fminf(", ",", ")"};
    case Binop::Mod: return {"(", " %", ")"};
    case Binop::Lt: return {"(", " <", ")"};
    case Binop::Eq: return {"(", " ==", ")"};
    case Binop::Ne: return {"(", " !=", ")"};
    case Binop::Or: return {"(", " ||", ")"};
    case Binop::And: return {"(", " &&", ")"};
    case Binop::ThreefryCrypto: return {"arrayjit_threefry4x32_crypto(", ",", ")"};
    case Binop::ThreefryLight: return {"arrayjit_threefry4x32_light(", ",", ")"};
    default: throw InvalidArgument("binop syntax: Arg1/Arg2 are not operators");
  }
}

Pair unop_syntax(Prec prec, Unop op) {   // Ops.unop_c_syntax, ops.ml:688-782
  const bool wide = dbl_or_intish(prec), ii = prec_is_intish(prec);
  const std::string fmax = wide ? "fmax" : "fmaxf", fmin = wide ? "fmin" : "fminf";
  auto libm = [&](const char* n) -> Pair { return {std::string(n) + (wide ? "(" : "f("), ")"}; };
  switch (op) {
    case Unop::Id: return {"", ""};
    case Unop::Relu: return ii ? Pair{"fmax(0, ", ")"} : Pair{fmax + "(0.0, ", ")"};
    case Unop::Sat01: return ii ? Pair{"fmax(0, fmin(1, ", "))"} : Pair{fmax + "(0.0, " + fmin + "(1.0, ", "))"};
    case Unop::Exp: return libm("exp");
    case Unop::Log: return libm("log");
    case Unop::Exp2: return libm("exp2");
    case Unop::Log2: return libm("log2");
    case Unop::Sin: return libm("sin");
    case Unop::Cos: return libm("cos");
    case Unop::Sqrt: return libm("sqrt");
    case Unop::Recip:
      if (ii) throw InvalidArgument("Recip not supported for integer precisions");
      return {"(1.0 / (", "))"};
    case Unop::RecipSqrt:
      if (ii) throw InvalidArgument("Recip_sqrt not supported for integer precisions");
      return prec == Prec::Double ? Pair{"(1.0 / sqrt(", "))"} : Pair{"(1.0 / sqrtf(", "))"};
    case Unop::Neg: return {"(-(", "))"};
    case Unop::Trunc: return prec == Prec::Double ? Pair{"trunc(", ")"} : Pair{"truncf(", ")"};
    case Unop::Tanh:
      if (ii) throw InvalidArgument("Tanh_approx not supported for integer precisions");
      return {"tanhf(", ")"};
    case Unop::Not: return {"(", " == 0.0 ? 1.0 : 0.0)"};
    case Unop::Uniform1:
      if (prec == Prec::Uint4x32) throw InvalidArgument("Uint4x32_to_prec_uniform1 not supported for Uint4x32");
      return {std::string("uint4x32_to_") + prec_string(prec) + "_uniform(", ")"};
  }
  return {"", ""};
}

Syn4 ternop_syntax(Prec prec, Ternop op) {   // Ops.ternop_c_syntax, ops.ml:793-806
  switch (op) {
    case Ternop::Where:
      return prec_is_intish(prec) ? Syn4{"((", ") != 0 ? (", ") : (", "))"} : Syn4{"((", ") != 0.0 ? (", ") : (", "))"};
    case Ternop::Fma: return dbl_or_intish(prec) ? Syn4{"fma(", ",", ",", ")"} : Syn4{"fmaf(", ",", ",", ")"};
    case Ternop::Mul3: return {"((", ") * (", ") * (", "))"};
  }
  return {};
}

// cc_backend.ml:169-323: reduced precisions compute in float
bool via_float(Prec p, std::string* to_f, std::string* from_f) {
  if (p == Prec::Bfloat16) { *to_f = "bfloat16_to_single("; *from_f = "single_to_bfloat16("; return true; }
  if (p == Prec::Half) { *to_f = "HALF_TO_FP("; *from_f = "FP_TO_HALF("; return true; }
  if (p == Prec::Fp8) { *to_f = "fp8_to_single("; *from_f = "single_to_fp8("; return true; }
  return false;
}

std::string emit_ternop(Prec prec, Ternop op, const std::string& a, const std::string& b, const std::string& c) {
  std::string tf, ff;
  // bf16 `where`: the result is one of two bf16 values, and rounding a widened bf16 value gives it back
  // (its low 16 bits are zero: the rounding increment cannot carry), so the choice is made on the bits
  // (the condition is widened as the reference writes it, cc_backend.ml:169-186)
  if (op == Ternop::Where && prec == Prec::Bfloat16) return "((bfloat16_to_single(" + a + ")) != 0.0 ? (" + b + ") : (" + c + "))";
  if (via_float(prec, &tf, &ff)) {
    Syn4 s = ternop_syntax(Prec::Single, op);
    return ff + s.p + tf + a + ")" + s.i1 + " " + tf + b + ")" + s.i2 + " " + tf + c + ")" + s.s + ")";
  }
  Syn4 s = ternop_syntax(prec, op);
  return s.p + a + s.i1 + " " + b + s.i2 + " " + c + s.s;
}

std::string emit_binop(Prec prec, Binop op, const std::string& a, const std::string& b) {
  if (op == Binop::ThreefryCrypto || op == Binop::ThreefryLight) {
    if (prec != Prec::Uint4x32) throw UserError("threefry4x32 on non-uint4x32 precision");
    return std::string(op == Binop::ThreefryCrypto ? "arrayjit_threefry4x32_crypto(" : "arrayjit_threefry4x32_light(") +
           a + ", " + b + ")";
  }
  std::string tf, ff;
  if (via_float(prec, &tf, &ff)) {
    Syn3 s = binop_syntax(Prec::Single, op);
    return ff + s.p + tf + a + ")" + s.i + " " + tf + b + ")" + s.s + ")";
  }
  Syn3 s = binop_syntax(prec, op);
  return s.p + a + s.i + " " + b + s.s;
}

std::string emit_unop(Prec prec, Unop op, const std::string& a) {
  std::string tf, ff;
  if (via_float(prec, &tf, &ff)) {
    Pair s = unop_syntax(Prec::Single, op);
    return ff + s.first + tf + a + ")" + s.second + ")";
  }
  Pair s = unop_syntax(prec, op);
  return s.first + a + s.second;
}

std::string axis_str(const AxisIndex& a) {   // Doc_helpers.pp_axis_index, indexing.ml:454-476
  if (a.kind == AxisIndex::Iter) return sym_ident(a.sym);
  if (a.kind == AxisIndex::Fixed) return std::to_string(a.fixed);
  std::string out;
  for (auto& t : a.terms) {
    if (!out.empty()) out += "+";
    out += t.first == 1 ? sym_ident(t.second) : std::to_string(t.first) + "*" + sym_ident(t.second);
  }
  if (a.offset > 0) out += (out.empty() ? "" : "+") + std::to_string(a.offset);
  else if (a.offset < 0) out += (out.empty() ? "" : "+") + ("-" + std::to_string(-a.offset));
  return out.empty() ? "0" : out;
}

std::string offset_str(const Indices& idcs, const std::vector<int64_t>& dims, int dyn_axis = -1,
                       const std::string& dyn = "") {   // pp_array_offset, c_syntax.ml:367-397
  if (idcs.empty()) return "0";
  auto part = [&](size_t i) { return (int)i == dyn_axis ? dyn : axis_str(idcs[i]); };
  std::string doc = part(0);
  for (size_t i = 1; i < idcs.size(); ++i) doc = "(" + doc + ") * " + std::to_string(dims[i]) + " + " + part(i);
  return doc;
}

std::string const_str(double c) {
  if (std::isinf(c)) return c > 0 ? "INFINITY" : "(-INFINITY)";
  if (std::isnan(c)) return "NAN";
  char buf[64];
  std::snprintf(buf, sizeof buf, "%.16g", c);
  return buf;
}

// low_level.ml:1998-2037
bool reads_scope_before_set(const ScopeId& target, const Block& body) {
  std::function<bool(const Scalar&)> sc_reads;
  std::function<bool(const Block&)> blk_reads = [&](const Block& b) {
    for (auto& s : b) {
      if (s->kind == Stmt::For && blk_reads(s->body)) return true;
      if ((s->kind == Stmt::Set || s->kind == Stmt::SetVec || s->kind == Stmt::SetLocal) && sc_reads(*s->value)) return true;
    }
    return false;
  };
  sc_reads = [&](const Scalar& s) -> bool {
    switch (s.kind) {
      case Scalar::GetLocal: return s.scope == target;
      case Scalar::LocalScope: return blk_reads(s.body);
      case Scalar::GetDyn: case Scalar::Un: return sc_reads(*s.a);
      case Scalar::Bin: return sc_reads(*s.a) || sc_reads(*s.b);
      case Scalar::Tern: return sc_reads(*s.a) || sc_reads(*s.b) || sc_reads(*s.c);
      default: return false;
    }
  };
  enum R { Read, Written, Neither };
  std::function<R(const Block&)> scan = [&](const Block& b) -> R {
    for (auto& s : b) {
      R r = Neither;
      switch (s->kind) {
        case Stmt::Set: case Stmt::SetVec: r = sc_reads(*s->value) ? Read : Neither; break;
        case Stmt::SetLocal: r = sc_reads(*s->value) ? Read : (s->scope == target ? Written : Neither); break;
        case Stmt::For: { R in = scan(s->body); r = in == Written ? (s->from <= s->to ? Written : Neither) : in; break; }
        default: break;
      }
      if (r != Neither) return r;
    }
    return Neither;
  };
  return scan(body) != Written;
}

// ------------------------------------------------------------------------------------------------
// statement / scalar printer
// ------------------------------------------------------------------------------------------------

std::string neutral_literal(Binop accum, bool dbl);
std::string combine_expr(Binop accum, bool dbl, const std::string& a, const std::string& b);

struct Printer {
  const Routine& r;
  std::set<int> used_nodes;
  std::set<int> used_statics;
  bool used_merge = false;
  std::map<int, std::string> shadow;   // serial group: node -> LDS array every store is copied to
  std::set<int> shadow_live;           // ... and whose contents reads may use by now
  // type of loop iterators and offsets: 64-bit when a node is too large for 32-bit offsets
  // (the `large_models` setting, c_syntax.ml:111-112)
  std::string idx_t = "uint32_t";
  // when set, this inlined scalar reduction is shared by `coop_lanes` adjacent lanes (lane id in
  // `lane_`): they stride its innermost loop, accumulate in float and combine by butterfly
  // shuffles; the enclosing store is done by lane 0
  const Scalar* coop_scope = nullptr;
  int coop_lanes = 1;
  Binop coop_accum = Binop::Add;
  std::string store_guard;   // prefix of plain stores ("if (lane_ == 0) " when one lane stores for a group)
  // Row groups with short rows keep what they produce in registers: a node written inside the
  // group is also kept in `cache_name` (an array indexed by the unrolled row iteration `it_` for
  // row-position values, a scalar every lane holds for per-row values) and later reads of it
  // inside the group use that instead of memory.
  bool row_vec4 = false;                    // see row_loop
  int row_iters = 0;                        // > 0: loops over the row position run `it_` = 0..row_iters-1, unrolled
  std::map<int, std::string> cache_name;    // node -> register expression
  std::set<int> cache_defined;              // nodes whose cache holds the current value
  // nodes whose store the member being printed leaves to a later member of the group that writes the
  // same elements again (the registers are kept in step all the same)
  std::set<int> skip_store;
  // `lhs = value;` with the cache kept in step
  const std::map<int, int>* mirrors = nullptr;   // fp32 node -> bf16 copy stored alongside (Plan::mirrors)
  std::string store_line(int node, const std::string& lhs, const std::string& value, const std::string& guard) {
    std::string mirror_lhs;
    if (mirrors) {
      auto m = mirrors->find(node);
      if (m != mirrors->end()) {
        used_nodes.insert(m->second);
        mirror_lhs = r.node(m->second).ident + lhs.substr(lhs.find('['));   // same dims: same offset
      }
    }
    auto sh = shadow.find(node);
    if (sh != shadow.end()) {
      // (a shadowed tensor has no bf16 mirror: mirrors belong to matrix-core contractions, which a
      // serial group does not contain)
      const std::string sh_lhs = sh->second + lhs.substr(lhs.find('['));
      auto itc = cache_name.find(node);
      if (itc == cache_name.end()) {
        const std::string t = "m" + std::to_string(fresh++) + "_";
        return "{ const " + std::string(c_typ(r.node(node).prec)) + " " + t + " = " + value + "; " + guard + "{ " + lhs + " = " + t +
               "; " + sh_lhs + " = " + t + "; } }";
      }
      cache_defined.insert(node);
      return itc->second + " = " + value + "; " + guard + "{ " + lhs + " = " + itc->second + "; " + sh_lhs + " = " + itc->second + "; }";
    }
    auto it = cache_name.find(node);
    if (it == cache_name.end()) {
      if (mirror_lhs.empty()) return guard + lhs + " = " + value + ";";
      const std::string t = "m" + std::to_string(fresh++) + "_";
      return "{ const " + std::string(c_typ(r.node(node).prec)) + " " + t + " = " + value + "; " + guard + "{ " + lhs + " = " + t +
             "; " + mirror_lhs + " = single_to_bfloat16(" + t + "); } }";
    }
    cache_defined.insert(node);
    if (skip_store.count(node)) return it->second + " = " + value + ";";
    std::string line = it->second + " = " + value + "; " + guard + "{ " + lhs + " = " + it->second + ";";
    if (!mirror_lhs.empty()) line += " " + mirror_lhs + " = single_to_bfloat16(" + it->second + ");";
    return line + " }";
  }
  // Lines that leave in `var` (of every lane) the combination of the lane group's partial values:
  // xor butterfly inside a wave; a group of 256 lanes is a whole workgroup, whose four waves
  // exchange their results through LDS (`red_`, declared by the kernel) and combine them in a
  // fixed order.
  void group_reduce(const std::string& var, Binop accum, bool dbl, int lanes, const std::string& ind,
                    std::vector<std::string>& out) {
    for (int o = std::min(lanes, 64) / 2; o > 0; o >>= 1)
      out.push_back(ind + var + " = " + combine_expr(accum, dbl, var, "ocn_xshfl(" + var + ", " + std::to_string(o) + ")") + ";");
    if (lanes > 64) {
      const std::string red = dbl ? "redd_" : "red_";
      out.push_back(ind + "if ((threadIdx.x & 63u) == 0) " + red + "[threadIdx.x >> 6] = " + var + ";");
      out.push_back(ind + "__syncthreads();");
      out.push_back(ind + var + " = " + combine_expr(accum, dbl, combine_expr(accum, dbl, red + "[0]", red + "[1]"),
                                                    combine_expr(accum, dbl, red + "[2]", red + "[3]")) + ";");
      out.push_back(ind + "__syncthreads();");
    }
  }

  // the row position that unrolled iteration `it_` of a lane stands for
  std::string row_pos(int lanes) const {
    if (row_vec4 && row_iters % 4 == 0) return "lane_ * 4u + (it_ & 3u) + (it_ >> 2) * " + std::to_string(lanes * 4) + "u";
    return "lane_ + it_ * " + std::to_string(lanes);
  }
  // header of a loop over the row position shared by `lanes` lanes
  std::string row_loop(const std::string& sym, int64_t from, int64_t to, int lanes, const std::string& ind) {
    if (row_iters > 0 && from == 0) {
      const std::string head = ind + "_Pragma(\"unroll\") for (uint32_t it_ = 0; it_ < " + std::to_string(row_iters) + "; ++it_) { const " +
                               idx_t + " " + sym + " = ";
      // a lane takes runs of four neighbouring positions, so that the unrolled loads and stores of a
      // unit-stride tensor combine into 16-byte (fp32) or 8-byte (bf16) accesses
      return head + row_pos(lanes) + ";";
    }
    return ind + "for (" + idx_t + " " + sym + " = " + std::to_string(from) + " + lane_; " + sym + " <= " + std::to_string(to) +
           "; " + sym + " += " + std::to_string(lanes) + ") {";
  }
  // row group with a contraction prologue: reads of this node come from the LDS tile `xs_` that the
  // kernel computed itself: [row of the tile][row position]
  int lds_node = -1;
  std::string lds_row;
  int64_t lds_ld = 0;
  // ---- debug logging (debug_log_from_routines; c_syntax.ml:493-535 and debug_float, :857-) ----------
  // A statement prints `# <its text>` and `<lhs>[<offset>]{=<old value>} = <new value> = <expression
  // with the value of every read in braces>`, as the reference's generated code does; every line starts
  // with the run's log id and ends in `$` for a newline (cuda_backend.ml:874-893), for the host to split.
  bool debug_log = false;
  struct Dbg { std::string fmt; std::vector<std::string> args; };
  static std::string lit(const std::string& t) {   // text inside a C string literal that is a printf format
    std::string o;
    for (char ch : t) {
      if (ch == '%') o += "%%";
      else if (ch == '"') o += "\\\"";
      else if (ch == '\\') o += "\\\\";
      else if (ch == '\n') o += "$";
      else o += ch;
    }
    return o;
  }
  static bool loggable(Prec p) { return p != Prec::Uint4x32 && p != Prec::Void; }
  std::string as_double(Prec from, const std::string& e) { Pair c = convert_precision(from, Prec::Double); return c.first + e + c.second; }
  // op syntax around already-formatted sub-expressions: print it around placeholders, escape, put them back
  std::string wrap_fmt(const std::string& with_marks, const std::vector<std::string>& subs) {
    std::string o = lit(with_marks);
    for (size_t i = 0; i < subs.size(); ++i) {
      const std::string mark = std::string("\001") + (char)('A' + i) + "\001";
      for (size_t at = o.find(mark); at != std::string::npos; at = o.find(mark, at + subs[i].size())) o.replace(at, mark.size(), subs[i]);
    }
    return o;
  }
  Dbg dbg(Prec prec, const Scalar& s) {
    Dbg d;
    switch (s.kind) {
      case Scalar::LocalScope: case Scalar::GetLocal: {
        const Prec sp = r.node(s.scope.node).prec;
        Pair c = convert_precision(sp, prec);
        const std::string v = c.first + scope_name(s.scope) + c.second;
        d.fmt = lit(v) + "{=%g}";
        d.args.push_back(loggable(prec) ? as_double(prec, v) : "0.0");
        return d;
      }
      case Scalar::Get: case Scalar::GetMerge: {
        const Node& n = r.node(s.node);
        Pair c = convert_precision(n.prec, prec);
        const std::string name = s.kind == Scalar::GetMerge ? "merge_buffer" : n.ident;
        const std::string off = offset_str(s.idcs, n.dims);
        d.fmt = lit(c.first + name) + "[%u]" + lit(c.second) + "{=%g}";
        d.args.push_back("(unsigned)(" + off + ")");
        d.args.push_back(loggable(prec) && loggable(n.prec) ? as_double(prec, c.first + name + "[" + off + "]" + c.second) : "0.0");
        return d;
      }
      case Scalar::GetDyn: {   // the table is not dereferenced in the log: the index value is what is shown
        std::vector<Def> defs;
        d.fmt = lit(r.node(s.node).ident + "@dyn_idx") + "{=%g}";
        d.args.push_back(as_double(s.arg_prec, scalar(s.arg_prec, *s.a, "", defs)));
        return d;
      }
      case Scalar::Const: { Pair c = convert_precision(Prec::Double, prec); d.fmt = lit(c.first + const_str(s.cst) + c.second); return d; }
      case Scalar::Bits: { Pair c = convert_precision(Prec::Int64, prec); d.fmt = lit(c.first + std::to_string((long long)s.bits) + "LL" + c.second); return d; }
      case Scalar::Index: d.fmt = lit(axis_str(s.index)); return d;
      case Scalar::Un: {
        Dbg a = dbg(s.un == Unop::Uniform1 ? s.arg_prec : prec, *s.a);
        d.fmt = wrap_fmt(emit_unop(prec, s.un, "\001A\001"), {a.fmt});
        d.args = a.args;
        return d;
      }
      case Scalar::Bin: {
        if (s.bin == Binop::Arg1) return dbg(prec, *s.a);
        if (s.bin == Binop::Arg2) return dbg(prec, *s.b);
        Dbg a = dbg(prec, *s.a), b = dbg(prec, *s.b);
        d.fmt = wrap_fmt(emit_binop(prec, s.bin, "\001A\001", "\001B\001"), {a.fmt, b.fmt});
        d.args = a.args; d.args.insert(d.args.end(), b.args.begin(), b.args.end());
        return d;
      }
      case Scalar::Tern: {
        Dbg a = dbg(s.tern == Ternop::Where ? s.arg_prec : prec, *s.a), b = dbg(prec, *s.b), c = dbg(prec, *s.c);
        d.fmt = wrap_fmt(emit_ternop(prec, s.tern, "\001A\001", "\001B\001", "\001C\001"), {a.fmt, b.fmt, c.fmt});
        d.args = a.args; d.args.insert(d.args.end(), b.args.begin(), b.args.end()); d.args.insert(d.args.end(), c.args.begin(), c.args.end());
        return d;
      }
    }
    return d;
  }
  std::string log_call(const std::string& fmt, const std::vector<std::string>& args) {
    std::string c = "printf(\"%d: " + fmt + "$\", log_id";
    for (auto& a : args) c += ", " + a;
    return c + ");";
  }
  // when set, a read of exactly this (node, indices) prints as `self_name`
  const Stmt* self_set = nullptr;
  std::string self_name;
  int fresh = 0;

  explicit Printer(const Routine& rr) : r(rr) {}

  std::string scope_name(const ScopeId& s) { return "v" + std::to_string(s.scope) + "_" + r.node(s.node).ident; }
  void note_idx(const AxisIndex& a) {
    if (a.kind == AxisIndex::Iter && r.is_static(a.sym)) used_statics.insert(a.sym);
    if (a.kind == AxisIndex::Affine) for (auto& t : a.terms) if (r.is_static(t.second)) used_statics.insert(t.second);
  }
  void note(int node, const Indices& idcs) {
    if (r.node(node).mode == Mode::Virtual)
      throw InvalidArgument("hip backend: access to virtual node " + r.node(node).ident + " survived optimisation");
    used_nodes.insert(node);
    for (auto& a : idcs) note_idx(a);
  }
  std::string init_zero(Prec p) { Pair c = convert_precision(Prec::Int32, p); return " = " + c.first + "0" + c.second; }

  struct Def { int scope; std::vector<std::string> lines; };

  // An operand of a C conditional (`where`, `relu_gate`) that reads memory is loaded ahead of the
  // statement: written inside `c ? x[i] : 0` the load would wait for the condition -- two dependent
  // trips to memory per element (the relu backward pass of the transformer step ran at 3.2 TB/s).
  // Only reads through loop iterators and fixed positions are moved: those are in range whatever the
  // condition says.  Same value either way.
  static bool safe_reads(const Scalar& s, bool* any) {
    switch (s.kind) {
      case Scalar::Get:
        for (auto& ix : s.idcs) if (ix.kind != AxisIndex::Iter && ix.kind != AxisIndex::Fixed) return false;
        *any = true;
        return true;
      case Scalar::Const: case Scalar::Bits: case Scalar::GetLocal: case Scalar::Index: return true;
      case Scalar::Un: return s.un != Unop::Uniform1 && safe_reads(*s.a, any);
      case Scalar::Bin: return safe_reads(*s.a, any) && safe_reads(*s.b, any);
      case Scalar::Tern: return safe_reads(*s.a, any) && safe_reads(*s.b, any) && safe_reads(*s.c, any);
      default: return false;
    }
  }
  int hoisted = 1;
  std::string eager(Prec prec, const Scalar& s, const std::string& expr, const std::string& ind, std::vector<Def>& defs) {
    bool any = false;
    if (debug_log || !safe_reads(s, &any) || !any) return expr;
    const std::string t = "w" + std::to_string(fresh++) + "_";
    Def d; d.scope = -(++hoisted);   // (definitions of one scope id are printed once: give each load its own)
    d.lines.push_back(ind + "const " + c_typ(prec) + " " + t + " = " + expr + ";");
    defs.push_back(std::move(d));
    return t;
  }

  std::string scalar(Prec prec, const Scalar& s, const std::string& ind, std::vector<Def>& defs) {
    switch (s.kind) {
      case Scalar::LocalScope: {
        const Prec sp = r.node(s.scope.node).prec;
        if (&s == coop_scope) return coop_reduction(prec, s, ind, defs);
        Def d; d.scope = s.scope.scope;
        d.lines.push_back(ind + c_typ(sp) + " " + scope_name(s.scope) +
                          (reads_scope_before_set(s.scope, s.body) ? init_zero(sp) : "") + ";");
        block(s.body, ind, d.lines);
        defs.push_back(std::move(d));
        Pair c = convert_precision(sp, prec);
        return c.first + scope_name(s.scope) + c.second;
      }
      case Scalar::GetLocal: {
        Pair c = convert_precision(r.node(s.scope.node).prec, prec);
        return c.first + scope_name(s.scope) + c.second;
      }
      case Scalar::GetMerge: {
        const Node& n = r.node(s.node);
        for (auto& a : s.idcs) note_idx(a);
        used_merge = true;
        Pair c = convert_precision(n.prec, prec);
        return c.first + "merge_buffer[" + offset_str(s.idcs, n.dims) + "]" + c.second;
      }
      case Scalar::Get: {
        const Node& n = r.node(s.node);
        Pair c = convert_precision(n.prec, prec);
        if (self_set && s.node == self_set->node && s.idcs == self_set->idcs) return c.first + self_name + c.second;
        if (s.node == lds_node) {
          note_idx(s.idcs.back());
          return c.first + "xs_[" + lds_row + " * " + std::to_string(lds_ld) + "u + " + axis_str(s.idcs.back()) + "]" + c.second;
        }
        if (cache_defined.count(s.node)) return c.first + cache_name.at(s.node) + c.second;
        note(s.node, s.idcs);
        if (shadow_live.count(s.node)) return c.first + shadow.at(s.node) + "[" + offset_str(s.idcs, n.dims) + "]" + c.second;
        return c.first + n.ident + "[" + offset_str(s.idcs, n.dims) + "]" + c.second;
      }
      case Scalar::GetDyn: {
        const Node& n = r.node(s.node);
        note(s.node, s.idcs);
        Pair c = convert_precision(n.prec, prec);
        // (c_syntax.ml:753-768 prints the index value in its own precision and casts that.  For bf16 and
        // fp8 that is the storage integer, 16512 for an id of 4.0, and the load leaves the table --
        // here it would fault the GPU: those two are read as the numbers they stand for.)
        const Prec ip = s.arg_prec == Prec::Bfloat16 || s.arg_prec == Prec::Fp8 ? Prec::Single : s.arg_prec;
        std::string dyn = std::string("((") + idx_t + ")(" + scalar(ip, *s.a, ind, defs) + "))";
        return c.first + n.ident + "[" + offset_str(s.idcs, n.dims, s.dyn_axis, dyn) + "]" + c.second;
      }
      case Scalar::Const: {
        Pair c = convert_precision(Prec::Double, prec);
        const std::string cs = const_str(s.cst);
        if (c.first.empty() && s.cst < 0.0 && !std::isinf(s.cst)) return "(" + cs + ")" + c.second;
        return c.first + cs + c.second;
      }
      case Scalar::Bits: {
        Pair c = convert_precision(Prec::Int64, prec);
        return c.first + std::to_string((long long)s.bits) + "LL" + c.second;
      }
      case Scalar::Index: {
        note_idx(s.index);
        Pair c = convert_precision(idx_t == "uint64_t" ? Prec::Uint64 : Prec::Uint32, prec);
        return c.first + axis_str(s.index) + c.second;
      }
      case Scalar::Tern: {
        // Where is heterogeneous: its condition keeps its own precision (c_syntax.ml:798-829)
        std::string a = scalar(s.tern == Ternop::Where ? s.arg_prec : prec, *s.a, ind, defs);
        std::string b = scalar(prec, *s.b, ind, defs);
        std::string c = scalar(prec, *s.c, ind, defs);
        if (s.tern == Ternop::Where) { b = eager(prec, *s.b, b, ind, defs); c = eager(prec, *s.c, c, ind, defs); }
        return emit_ternop(prec, s.tern, a, b, c);
      }
      case Scalar::Bin: {
        if (s.bin == Binop::Arg1) return scalar(prec, *s.a, ind, defs);
        if (s.bin == Binop::Arg2) return scalar(prec, *s.b, ind, defs);
        std::string a = scalar(prec, *s.a, ind, defs);
        std::string b = scalar(prec, *s.b, ind, defs);
        if (s.bin == Binop::ReluGate) b = eager(prec, *s.b, b, ind, defs);
        return emit_binop(prec, s.bin, a, b);
      }
      case Scalar::Un: {
        std::string a = scalar(s.un == Unop::Uniform1 ? s.arg_prec : prec, *s.a, ind, defs);
        return emit_unop(prec, s.un, a);
      }
    }
    return "";
  }

  // `v { v := neutral; for k1.. for kn { v := accum(v, e) } }` computed by a group of lanes.
  std::string coop_reduction(Prec prec, const Scalar& s, const std::string& ind, std::vector<Def>& defs) {
    const Prec sp = r.node(s.scope.node).prec;
    const bool dbl = sp == Prec::Double;
    const Prec accP = dbl ? Prec::Double : Prec::Single;
    const std::string part = "part" + std::to_string(s.scope.scope) + "_";
    auto only = [](const Block& b) -> const Stmt* {   // the single non-comment statement
      const Stmt* one = nullptr;
      for (auto& x : b) if (x->kind != Stmt::Comment) { if (one) return nullptr; one = x.get(); }
      return one;
    };
    const Stmt* loop = nullptr;
    for (auto& x : s.body) if (x->kind == Stmt::For) loop = x.get();
    std::vector<const Stmt*> loops;
    const Stmt* upd = nullptr;
    for (const Stmt* cur = loop; cur;) {
      loops.push_back(cur);
      const Stmt* in = only(cur->body);
      if (in && in->kind == Stmt::For) { cur = in; continue; }
      upd = in;
      break;
    }
    if (!upd || upd->kind != Stmt::SetLocal) throw InvalidArgument("codegen: cooperative scope lost its shape");
    Def d; d.scope = s.scope.scope;
    d.lines.push_back(ind + (dbl ? "double " : "float ") + part + " = " + neutral_literal(coop_accum, dbl) + ";");
    std::string ci = ind;
    for (size_t i = 0; i < loops.size(); ++i) {
      const std::string sy = sym_ident(loops[i]->sym);
      if (i + 1 == loops.size())
        d.lines.push_back(row_loop(sy, loops[i]->from, loops[i]->to, coop_lanes, ci));
      else
        d.lines.push_back(ci + "for (" + idx_t + " " + sy + " = " + std::to_string(loops[i]->from) + "; " + sy + " <= " +
                          std::to_string(loops[i]->to) + "; ++" + sy + ") {");
      ci += "  ";
    }
    auto widen = [&](const std::string& e) { Pair c = convert_precision(sp, accP); return c.first + e + c.second; };
    auto is_v = [&](const Scalar& x) { return x.kind == Scalar::GetLocal && x.scope == s.scope; };
    const Scalar& v = *upd->value;
    std::vector<Def> inner_defs;
    std::string line;
    if (v.kind == Scalar::Tern) {
      const std::string a = scalar(sp, *v.a, ci + "  ", inner_defs), b = scalar(sp, *v.b, ci + "  ", inner_defs);
      line = part + " = " + (dbl ? "fma(" : "fmaf(") + widen(a) + ", " + widen(b) + ", " + part + ");";
    } else {
      const std::string e = scalar(sp, is_v(*v.a) ? *v.b : *v.a, ci + "  ", inner_defs);
      line = part + " = " + combine_expr(coop_accum, dbl, part, widen(e)) + ";";
    }
    with_defs(inner_defs, {line}, ci, d.lines);
    for (size_t i = 0; i < loops.size(); ++i) { ci.resize(ci.size() - 2); d.lines.push_back(ci + "}"); }
    group_reduce(part, coop_accum, dbl, coop_lanes, ind, d.lines);
    Pair narrow = convert_precision(accP, sp);
    d.lines.push_back(ind + c_typ(sp) + " " + scope_name(s.scope) + " = " + narrow.first + part + narrow.second + ";");
    defs.push_back(std::move(d));
    Pair c = convert_precision(sp, prec);
    return c.first + scope_name(s.scope) + c.second;
  }

  void with_defs(std::vector<Def>& defs, const std::vector<std::string>& lines, const std::string& ind,
                 std::vector<std::string>& out) {
    if (defs.empty()) { for (auto& l : lines) out.push_back(ind + l); return; }
    std::stable_sort(defs.begin(), defs.end(), [](const Def& a, const Def& b) { return a.scope < b.scope; });
    out.push_back(ind + "{");
    int last = -1; bool first = true;
    for (auto& d : defs) {
      if (!first && d.scope == last) continue;   // c_syntax.ml:406-409 dedup by scope id
      first = false; last = d.scope;
      for (auto& l : d.lines) out.push_back(l);
    }
    for (auto& l : lines) out.push_back(ind + "  " + l);
    out.push_back(ind + "}");
  }

  void stmt(const Stmt& c, const std::string& ind, std::vector<std::string>& out) {
    switch (c.kind) {
      case Stmt::Comment:
        if (debug_log) out.push_back(ind + log_call("COMMENT: " + lit(c.text), {}));
        else out.push_back(ind + "/* " + c.text + " */");
        break;
      case Stmt::For: {
        const std::string s = sym_ident(c.sym);
        out.push_back(ind + "for (" + idx_t + " " + s + " = " + std::to_string(c.from) + "; " + s + " <= " +
                      std::to_string(c.to) + "; ++" + s + ") {");
        if (debug_log) out.push_back(ind + "  " + log_call("index " + s + " = %d", {"(int)(" + s + ")"}));   // c_syntax.ml:458-465
        block(c.body, ind + "  ", out);
        out.push_back(ind + "}");
        break;
      }
      case Stmt::ZeroOut: {
        // a re-zero reached inside a kernel: plain serial loop over the node (c_syntax.ml:476-479)
        const Node& n = r.node(c.node);
        used_nodes.insert(c.node);
        const std::string v = "z" + std::to_string(fresh++);
        Pair cv = convert_precision(Prec::Double, n.prec);
        if (debug_log && loggable(n.prec)) {
          // every element logs `# <ident> := 0` and its value line (c_syntax.ml:476-479; the loops over
          // the axes print as one loop over the flat offset, index lines left out)
          const std::string zero = cv.first + "0" + cv.second, lhs = n.ident + "[" + v + "]";
          out.push_back(ind + "for (" + idx_t + " " + v + " = 0; " + v + " < " + std::to_string(n.num_elems()) + "; ++" + v + ") {");
          out.push_back(ind + "  " + log_call("# " + lit(n.ident + " := 0"), {}));
          out.push_back(ind + "  " + log_call(lit(n.ident) + "[%u]{=%g} = %g = " + lit(zero),
                                              {"(unsigned)(" + v + ")", as_double(n.prec, lhs), as_double(n.prec, zero)}));
          out.push_back(ind + "  " + lhs + " = " + zero + ";");
          out.push_back(ind + "}");
          break;
        }
        out.push_back(ind + "for (" + idx_t + " " + v + " = 0; " + v + " < " + std::to_string(n.num_elems()) + "; ++" + v +
                      ") " + n.ident + "[" + v + "] = " + cv.first + "0" + cv.second + ";");
        break;
      }
      case Stmt::Set: {
        const Node& n = r.node(c.node);
        note(c.node, c.idcs);
        std::vector<Def> defs;
        std::string v = scalar(n.prec, *c.value, ind + "  ", defs);
        if (debug_log && loggable(n.prec)) {
          // { T new_set_v = value; log "# text"; log "lhs[off]{=old} = new = expression{=values}"; lhs[off] = new_set_v; }
          const std::string off = offset_str(c.idcs, n.dims), lhs = n.ident + "[" + off + "]";
          Dbg d = dbg(n.prec, *c.value);
          std::vector<std::string> args{"(unsigned)(" + off + ")", as_double(n.prec, lhs), as_double(n.prec, "new_set_v")};
          args.insert(args.end(), d.args.begin(), d.args.end());
          std::vector<std::string> lines{std::string(c_typ(n.prec)) + " new_set_v = " + v + ";"};
          if (!c.text.empty()) lines.push_back(log_call("# " + lit(c.text), {}));
          lines.push_back(log_call(lit(n.ident) + "[%u]{=%g} = %g = " + d.fmt, args));
          lines.push_back(store_line(c.node, lhs, "new_set_v", store_guard));
          if (defs.empty()) { out.push_back(ind + "{"); for (auto& l : lines) out.push_back(ind + "  " + l); out.push_back(ind + "}"); }
          else with_defs(defs, lines, ind, out);
          break;
        }
        with_defs(defs, {store_line(c.node, n.ident + "[" + offset_str(c.idcs, n.dims) + "]", v, store_guard)}, ind, out);
        break;
      }
      case Stmt::SetVec: {
        const Node& n = r.node(c.node);
        note(c.node, c.idcs);
        std::vector<Def> defs;
        std::string a = scalar(c.arg_prec, *c.value, ind + "  ", defs);
        if (n.prec == Prec::Uint4x32) throw InvalidArgument("Uint4x32_to_prec_uniform not supported for Uint4x32");
        std::vector<std::string> lines;
        lines.push_back(c_vec_typ(c.length, n.prec) + " vec_result = uint4x32_to_" + prec_string(n.prec) +
                        "_uniform_vec(" + a + ");");
        for (int i = 0; i < c.length; ++i) {
          std::string off;
          const AxisIndex& last = c.idcs.back();
          if (last.kind == AxisIndex::Fixed) {
            Indices el = c.idcs; el.back().fixed += i;
            off = offset_str(el, n.dims);
          } else off = offset_str(c.idcs, n.dims) + " + " + std::to_string(i);
          lines.push_back(n.ident + "[" + off + "] = " +
                          (c.length == 1 ? std::string("vec_result") : "vec_result.v[" + std::to_string(i) + "]") + ";");
        }
        if (debug_log && loggable(n.prec) && c.length > 1) {
          // `# text`, then per element `ident[offset]{=old} = vec_result.v[i] = new` (c_syntax.ml:590-640),
          // ahead of the stores
          std::vector<std::string> logs;
          if (!c.text.empty()) logs.push_back(log_call("# " + lit(c.text), {}));
          for (int i = 0; i < c.length; ++i) {
            const std::string& store = lines[1 + i];
            const std::string lhs = store.substr(0, store.find(" = "));
            const std::string off = lhs.substr(lhs.find('[') + 1, lhs.size() - lhs.find('[') - 2);
            const std::string lane = "vec_result.v[" + std::to_string(i) + "]";
            logs.push_back(log_call(lit(n.ident) + "[%u]{=%g} = " + lit(lane) + " = %g",
                                    {"(unsigned)(" + off + ")", as_double(n.prec, lhs), as_double(n.prec, lane)}));
          }
          lines.insert(lines.begin() + 1, logs.begin(), logs.end());
        }
        // always a block here: several statements of one kernel may declare vec_result
        out.push_back(ind + "{");
        std::vector<std::string> inner;
        with_defs(defs, lines, ind + "  ", inner);
        for (auto& l : inner) out.push_back(l);
        out.push_back(ind + "}");
        break;
      }
      case Stmt::SetLocal: {
        std::vector<Def> defs;
        const Prec sp = r.node(c.scope.node).prec;
        std::string v = scalar(sp, *c.value, ind + "  ", defs);
        if (debug_log && loggable(sp)) {
          const std::string name = scope_name(c.scope);
          Dbg d = dbg(sp, *c.value);
          std::vector<std::string> args{as_double(sp, name), as_double(sp, "new_set_v")};
          args.insert(args.end(), d.args.begin(), d.args.end());
          std::vector<std::string> lines{std::string(c_typ(sp)) + " new_set_v = " + v + ";",
                                         log_call("# local " + lit(name + " := " + v), {}),
                                         log_call(lit(name) + "{=%g} = %g = " + d.fmt, args), name + " = new_set_v;"};
          if (defs.empty()) { out.push_back(ind + "{"); for (auto& l : lines) out.push_back(ind + "  " + l); out.push_back(ind + "}"); }
          else with_defs(defs, lines, ind, out);
          break;
        }
        with_defs(defs, {scope_name(c.scope) + " = " + v + ";"}, ind, out);
        break;
      }
      case Stmt::DeclareLocal: {
        const Prec p = r.node(c.scope.node).prec;
        out.push_back(ind + c_typ(p) + " " + scope_name(c.scope) + (c.needs_init ? init_zero(p) : "") + ";");
        break;
      }
    }
  }

  void block(const Block& b, const std::string& ind, std::vector<std::string>& out) {
    for (auto& s : b) stmt(*s, ind, out);
  }
};

// In a row group whose rows stay in registers: does a later member store the very elements member
// `mi` stores (the same tensor through the same row indices)?  Readers in between take the value
// from the registers, so the earlier store never reaches anyone.
bool row_store_is_overwritten(const Phase& q, size_t mi) {
  const Phase& m = q.members[mi];
  if (m.row_role != Phase::RowPointwise || m.inner.size() != 1 || m.inner[0]->kind != Stmt::Set) return false;
  const Stmt& st = *m.inner[0];
  // -3: constant, -1: position in the row, k >= 0: outer axis k of the group, -2: anything else
  auto role = [](const Phase& ph, const AxisIndex& ix, long long* fixed) -> int {
    if (ix.kind == AxisIndex::Fixed) { *fixed = ix.fixed; return -3; }
    if (ix.kind != AxisIndex::Iter) return -2;
    if (ix.sym == ph.row_sym) return -1;
    for (size_t k = 0; k < ph.row_outer_syms.size(); ++k) if (ph.row_outer_syms[k] == ix.sym) return (int)k;
    return -2;
  };
  for (size_t mj = mi + 1; mj < q.members.size(); ++mj) {
    const Phase& o = q.members[mj];
    if (o.row_role != Phase::RowPointwise || o.inner.size() != 1 || o.inner[0]->kind != Stmt::Set) continue;
    const Stmt& ot = *o.inner[0];
    if (ot.node != st.node || ot.idcs.size() != st.idcs.size()) continue;
    bool same = true;
    for (size_t p = 0; p < st.idcs.size() && same; ++p) {
      long long fa = 0, fb = 0;
      const int ra = role(m, st.idcs[p], &fa), rb = role(o, ot.idcs[p], &fb);
      same = ra != -2 && ra == rb && fa == fb;
    }
    if (same) return true;
  }
  return false;
}

std::string neutral_literal(Binop accum, bool dbl) {
  switch (accum) {
    case Binop::Max: return dbl ? "(-__builtin_huge_val())" : "(-INFINITY)";
    case Binop::Min: return dbl ? "__builtin_huge_val()" : "INFINITY";
    default: return dbl ? "0.0" : "0.0f";
  }
}

std::string combine_expr(Binop accum, bool dbl, const std::string& a, const std::string& b) {
  switch (accum) {
    case Binop::Max: return std::string(dbl ? "fmax(" : "fmaxf(") + a + ", " + b + ")";
    case Binop::Min: return std::string(dbl ? "fmin(" : "fminf(") + a + ", " + b + ")";
    default: return "(" + a + " + " + b + ")";
  }
}

}  // namespace

namespace {

// Statements of one phase for a thread whose parallel symbols are already defined.  G > 1: the
// thread is lane `lane_` of a group of G sharing the point.  `lane0_store`: plain stores are done
// by lane 0 only (per-row scalars inside a row group).
void emit_phase_statements(const Routine& r, Printer& pr, const Phase& ph, int G, bool lane0_store,
                           const std::string& ind, std::vector<std::string>& body) {
  Binop accum = Binop::Add;
  bool is_reduction = false;
  const Stmt* set = nullptr;
  if ((!ph.seq_syms.empty() || ph.fused_zero_init) && ph.inner.size() == 1 && ph.inner[0]->kind == Stmt::Set) {
    set = ph.inner[0].get();
    const Scalar& v = *set->value;
    auto is_self = [&](const Scalar& s) { return s.kind == Scalar::Get && s.node == set->node && s.idcs == set->idcs; };
    if (v.kind == Scalar::Tern && v.tern == Ternop::Fma && is_self(*v.c)) { is_reduction = true; accum = Binop::Add; }
    else if (v.kind == Scalar::Bin && (v.bin == Binop::Add || v.bin == Binop::Max || v.bin == Binop::Min) &&
             (is_self(*v.a) || is_self(*v.b))) { is_reduction = true; accum = v.bin; }
    // the accumulator lives in a register across the sequential loops only when they all update
    // one and the same element (not so for sums of symbols on an axis, convolution-style)
    for (auto& ix : set->idcs) for (int q : ph.seq_syms) if (ix.mentions(q)) is_reduction = false;
  }
  auto open_seq_loops = [&](std::string& cur_ind, bool coop_last) {
    for (size_t i = 0; i < ph.seq_syms.size(); ++i) {
      const std::string s = sym_ident(ph.seq_syms[i]);
      if (coop_last && i + 1 == ph.seq_syms.size())
        body.push_back(pr.row_loop(s, ph.seq_from[i], ph.seq_to[i], G, cur_ind));
      else
        body.push_back(cur_ind + "for (" + pr.idx_t + " " + s + " = " + std::to_string(ph.seq_from[i]) + "; " + s + " <= " +
                       std::to_string(ph.seq_to[i]) + "; ++" + s + ") {");
      cur_ind += "  ";
    }
  };
  auto close_seq_loops = [&](std::string& cur_ind) {
    for (size_t i = 0; i < ph.seq_syms.size(); ++i) { cur_ind.resize(cur_ind.size() - 2); body.push_back(cur_ind + "}"); }
  };
  const bool guard = lane0_store || ph.coop_scope;
  const std::string lane0 = guard && G > 1 ? "if (lane_ == 0) " : "";

  if (is_reduction && G > 1 && !ph.coop_scope && !ph.seq_syms.empty()) {
    // lanes of a group stride the innermost sequential loop; partials are combined by butterfly
    // shuffles in a fixed order (deterministic), accumulating in float (double for double).
    const Node& n = r.node(set->node);
    pr.note(set->node, set->idcs);
    const bool dbl = n.prec == Prec::Double;
    const std::string accT = dbl ? "double" : "float";
    const Prec accP = dbl ? Prec::Double : Prec::Single;
    body.push_back(ind + accT + " part_ = " + neutral_literal(accum, dbl) + ";");
    std::string ci = ind;
    open_seq_loops(ci, true);
    const Scalar& v = *set->value;
    std::vector<Printer::Def> defs;
    std::vector<std::string> lines;
    auto widen = [&](const std::string& e) { Pair c = convert_precision(n.prec, accP); return c.first + e + c.second; };
    if (v.kind == Scalar::Tern) {
      std::string a = pr.scalar(n.prec, *v.a, ci + "  ", defs), b = pr.scalar(n.prec, *v.b, ci + "  ", defs);
      lines.push_back(std::string("part_ = ") + (dbl ? "fma(" : "fmaf(") + widen(a) + ", " + widen(b) + ", part_);");
    } else {
      auto is_self = [&](const Scalar& s) { return s.kind == Scalar::Get && s.node == set->node && s.idcs == set->idcs; };
      const Scalar& e = is_self(*v.a) ? *v.b : *v.a;
      std::string es = pr.scalar(n.prec, e, ci + "  ", defs);
      lines.push_back("part_ = " + combine_expr(accum, dbl, "part_", widen(es)) + ";");
    }
    pr.with_defs(defs, lines, ci, body);
    close_seq_loops(ci);
    pr.group_reduce("part_", accum, dbl, G, ind, body);
    const std::string lhs = n.ident + "[" + offset_str(set->idcs, n.dims) + "]";
    Pair narrow = convert_precision(accP, n.prec);
    Pair wide = convert_precision(n.prec, accP);
    // (every lane holds the combined value after the butterfly)
    if (ph.fused_zero_init)
      body.push_back(ind + pr.store_line(set->node, lhs, narrow.first + "part_" + narrow.second, "if (lane_ == 0) "));
    else {
      const std::string old_v = pr.cache_defined.count(set->node) ? pr.cache_name.at(set->node) : lhs;
      body.push_back(ind + pr.store_line(set->node, lhs, narrow.first +
                     combine_expr(accum, dbl, wide.first + old_v + wide.second, "part_") + narrow.second, "if (lane_ == 0) "));
    }
  } else if (is_reduction) {
    // one thread per output element, sequential loops in the reference's order: for fp32 this is
    // the same operation sequence as the `cc` backend's serial loop.
    const Node& n = r.node(set->node);
    pr.note(set->node, set->idcs);
    const std::string lhs = n.ident + "[" + offset_str(set->idcs, n.dims) + "]";
    Pair zero = convert_precision(Prec::Double, n.prec);
    const std::string old_v = pr.cache_defined.count(set->node) ? pr.cache_name.at(set->node) : lhs;
    body.push_back(ind + c_typ(n.prec) + " acc_ = " + (ph.fused_zero_init ? zero.first + "0" + zero.second : old_v) + ";");
    std::string ci = ind;
    open_seq_loops(ci, false);
    pr.self_set = set; pr.self_name = "acc_";
    if (ph.coop_scope && G > 1) { pr.coop_scope = ph.coop_scope; pr.coop_lanes = G; pr.coop_accum = ph.coop_accum; }
    std::vector<Printer::Def> defs;
    std::string v = pr.scalar(n.prec, *set->value, ci + "  ", defs);
    pr.with_defs(defs, {"acc_ = " + v + ";"}, ci, body);
    pr.self_set = nullptr;
    close_seq_loops(ci);
    body.push_back(ind + pr.store_line(set->node, lhs, "acc_", lane0));
    pr.coop_scope = nullptr;
  } else {
    if (ph.fused_zero_init) throw InvalidArgument("planner: fused zero-init on a non-reduction phase");
    std::string ci = ind;
    open_seq_loops(ci, false);
    if (ph.coop_scope && G > 1) { pr.coop_scope = ph.coop_scope; pr.coop_lanes = G; pr.coop_accum = ph.coop_accum; }
    pr.store_guard = lane0;
    pr.block(ph.inner, ci, body);
    pr.store_guard.clear();
    pr.coop_scope = nullptr;
    close_seq_loops(ci);
  }
}

}  // namespace

GeneratedModule generate_module(const Routine& r, const Plan& plan) {
  GeneratedModule mod;
  std::ostringstream src;
  src << builtins_hip_source() << "\n";
  int kidx = 0;
  for (size_t pi = 0; pi < plan.phases.size(); ++pi) {
    const Phase& ph = plan.phases[pi];
    if (ph.kind != Phase::Generic) continue;
    Printer pr(r);
    if (plan.large_index) pr.idx_t = "uint64_t";
    pr.mirrors = &plan.mirrors;
    pr.debug_log = plan.debug_log;
    pr.row_vec4 = plan.row_vec4;
    std::vector<std::string> body;
    const std::string ind = "  ";

    int fused_block = 0;   // > 0: the kernel is a row group with a contraction prologue and wants this workgroup size
    // one phase for the thread (or loop iteration) identified by gtid_; `skip` leaves it
    auto emit_points = [&](const Phase& q, const std::string& pind, const std::string& skip) {
      const int QG = q.coop_lanes;
      uint64_t QP = 1;
      if (QG > 1) {
        body.push_back(pind + "const uint32_t lane_ = (uint32_t)(gtid_ % " + std::to_string(QG) + "u);");
        body.push_back(pind + "uint64_t pt_ = gtid_ / " + std::to_string(QG) + "u;");
      } else {
        body.push_back(pind + "uint64_t pt_ = gtid_;");
      }
      if (!q.members.empty() && q.fused_x >= 0) {
        // ---- row group with a contraction prologue: a workgroup owns 32 rows (consecutive along outer
        //      axis fused_m_axis); it computes their part of x into LDS on the matrix cores, then each of
        //      its four waves runs the members over eight of the rows
        const Node& xn = r.node(q.fused_x);
        const size_t n = q.row_outer_ext.size();
        const int ma = q.fused_m_axis;
        QP = 1;
        for (size_t k = 0; k < n; ++k) QP *= (uint64_t)(k == (size_t)ma ? q.row_outer_ext[k] / 32 : q.row_outer_ext[k]);
        // 16 waves of two rows each for short rows; long rows keep more of what they produce in
        // registers and take 8 waves of four rows
        const int NW = q.fused_waves, RPW = 32 / NW;
        fused_block = NW * 64;
        body.pop_back(); body.pop_back();   // (lane_ / pt_ as laid out for lane groups: redone per workgroup)
        body.push_back(pind + "const uint32_t lane_ = threadIdx.x & 63u, wave_ = threadIdx.x >> 6;");
        body.push_back(pind + "uint64_t pt_ = gtid_ / " + std::to_string(fused_block) + "u;");
        body.push_back(pind + "if (pt_ >= " + std::to_string(QP) + "ull) " + skip + ";");
        for (int k = (int)n - 1; k >= 0; --k) {
          const std::string ext = std::to_string(k == ma ? q.row_outer_ext[k] / 32 : q.row_outer_ext[k]) + "ull";
          std::string line = pind + "const " + pr.idx_t + " t" + std::to_string(k) + "_ = (" + pr.idx_t + ")(";
          if (k == 0) line += "pt_);";
          else line += "pt_ % " + ext + "); pt_ /= " + ext + ";";
          body.push_back(line);
        }
        const std::string xt = c_typ(xn.prec);
        // rows of the tile lie 16 bytes more than a row apart where the static LDS budget allows: with a
        // power-of-two row the 32 rows a matrix-core fragment read touches (one row per lane) would all
        // start in the same banks
        const int64_t xbytes = prec_in_bytes(xn.prec);
        const int64_t ps_bytes = (q.proj_y >= 0 && q.proj_kp > 1) ? (int64_t)q.proj_kp * 32 * q.proj_n * 4 : 0;
        const int64_t xpad = (32 * (q.row_len + 16 / xbytes) * xbytes + ps_bytes <= 65536) ? 16 / xbytes : 0;
        const int64_t xld = q.row_len + xpad;
        body.push_back(pind + "__shared__ __attribute__((aligned(16))) " + xt + " xs_[" + std::to_string(32 * xld) + "];");
        {
          pr.used_nodes.insert(q.fused_a.node); pr.used_nodes.insert(q.fused_b.node);
          std::string ao = std::to_string(q.fused_a.offset) + "ull", bo = std::to_string(q.fused_b.offset) + "ull";
          for (size_t k = 0; k < n; ++k) {
            const std::string tk = "(uint64_t)t" + std::to_string(k) + "_" + (k == (size_t)ma ? " * 32ull" : "");
            if (q.fused_a_stride[k]) ao += " + " + tk + " * " + std::to_string(q.fused_a_stride[k]) + "ull";
            if (q.fused_b_stride[k]) bo += " + " + tk + " * " + std::to_string(q.fused_b_stride[k]) + "ull";
          }
          body.push_back(pind + "ocn_rowtile_contract<" + std::to_string(q.row_len) + ", " + std::to_string(q.fused_k) + ", " +
                         std::to_string(NW) + ", " + xt + ", " + std::to_string(xld) + ">(" +
                         r.node(q.fused_a.node).ident + " + (" + ao + "), " + std::to_string(q.fused_a_stride[ma]) + "ll, " +
                         r.node(q.fused_b.node).ident + " + (" + bo + "), " + std::to_string(q.fused_b_row) + "ll, xs_);");
        }
        body.push_back(pind + "__syncthreads();");
        if (q.row_len % 64 != 0 || q.row_len / 64 > 16 || QG != 64) throw InvalidArgument("planner: fused row group of a shape the kernel does not take");
        pr.row_iters = (int)(q.row_len / 64);
        for (auto& m : q.members) {
          const Stmt& st = *m.inner[0];
          if (pr.cache_name.count(st.node)) continue;
          const Node& wn = r.node(st.node);
          bool per_position = false;
          for (auto& ix : st.idcs) if (ix.kind == AxisIndex::Iter && ix.sym == m.row_sym && m.row_role == Phase::RowPointwise) per_position = true;
          const std::string base = "c" + std::to_string(st.node) + "_";
          if (per_position) {
            body.push_back(pind + c_typ(wn.prec) + " " + base + "[" + std::to_string(pr.row_iters) + "];");
            pr.cache_name[st.node] = base + "[it_]";
          } else {
            body.push_back(pind + c_typ(wn.prec) + " " + base + ";");
            pr.cache_name[st.node] = base;
          }
        }
        // the rows of a wave are independent: unrolled (while what they keep in registers stays small), the
        // loads, shuffles and stores of one row fill the waits of the other
        const int row_unroll = RPW * pr.row_iters <= 16 ? RPW : pr.row_iters <= 8 ? 2 : 1;
        body.push_back(pind + (row_unroll > 1 ? "_Pragma(\"unroll " + std::to_string(row_unroll) + "\") " : "") +
                       "for (uint32_t rl_ = 0; rl_ < " + std::to_string(RPW) + "u; ++rl_) {");
        const std::string rind = pind + "  ";
        for (size_t k = 0; k < n; ++k)
          body.push_back(rind + "const " + pr.idx_t + " row" + std::to_string(k) + "_ = t" + std::to_string(k) + "_" +
                         (k == (size_t)ma ? " * 32u + wave_ * " + std::to_string(RPW) + "u + rl_;" : ";"));
        pr.lds_node = q.fused_x; pr.lds_row = "(wave_ * " + std::to_string(RPW) + "u + rl_)"; pr.lds_ld = xld;
        if (q.fused_x_store) {
          // x is visible outside the kernel: its rows go to memory as well (adjacent lanes adjacent elements)
          pr.used_nodes.insert(q.fused_x);
          std::string off;
          for (size_t k = 0; k < n; ++k) off = k == 0 ? "(uint64_t)row0_" : "(" + off + ") * " + std::to_string(q.row_outer_ext[k]) + "ull + row" + std::to_string(k) + "_";
          body.push_back(rind + "_Pragma(\"unroll\") for (uint32_t it_ = 0; it_ < " + std::to_string(pr.row_iters) + "; ++it_) " + xn.ident +
                         "[(" + off + ") * " + std::to_string(q.row_len) + "ull + lane_ + it_ * 64u] = xs_[" + pr.lds_row + " * " +
                         std::to_string(xld) + "u + lane_ + it_ * 64u];");
        }
        for (size_t mi = 0; mi < q.members.size(); ++mi) {
          const Phase& m = q.members[mi];
          body.push_back(rind + "{  /* " + m.label + " */");
          const std::string mi_ind = rind + "  ";
          for (size_t k = 0; k < m.row_outer_syms.size(); ++k)
            body.push_back(mi_ind + "const " + pr.idx_t + " " + sym_ident(m.row_outer_syms[k]) + " = row" + std::to_string(k) + "_;");
          pr.skip_store.clear();
          if (row_store_is_overwritten(q, mi) && pr.cache_name.count(m.inner[0]->node)) pr.skip_store.insert(m.inner[0]->node);
          if (m.row_role == Phase::RowPointwise) {
            body.push_back(pr.row_loop(sym_ident(m.row_sym), 0, q.row_len - 1, QG, mi_ind));
            emit_phase_statements(r, pr, m, 1, false, mi_ind + "  ", body);
            body.push_back(mi_ind + "}");
          } else {
            emit_phase_statements(r, pr, m, QG, true, mi_ind, body);
          }
          pr.skip_store.clear();
          body.push_back(rind + "}");
        }
        // contraction epilogue: the finished row of y replaces the row of x in LDS, as bf16 (the wave owns
        // both; a row of y takes at most the bytes of a row of x)
        const int64_t ys = xld * xbytes / 2;   // row stride of y in LDS, in bf16 elements
        if (q.proj_y >= 0) {
          auto yc = pr.cache_name.find(q.proj_y);
          if (yc == pr.cache_name.end() || yc->second.find("[it_]") == std::string::npos) throw InvalidArgument("planner: row-group epilogue over a tensor the group does not keep");
          const std::string bits = r.node(q.proj_y).prec == Prec::Bfloat16 ? yc->second : "single_to_bfloat16(" + yc->second + ")";
          body.push_back(rind + "_Pragma(\"unroll\") for (uint32_t it_ = 0; it_ < " + std::to_string(pr.row_iters) + "; ++it_) ((unsigned short*)xs_)[" +
                         pr.lds_row + " * " + std::to_string(ys) + "u + " + pr.row_pos(QG) + "] = " + bits + ";");
        }
        body.push_back(pind + "}");
        if (q.proj_y >= 0) {
          const int NB = (int)(q.proj_n / 32);
          const int KP = q.proj_kp;
          if (KP < 1 || KP * NB > NW || (q.row_len / 16) % KP != 0) throw InvalidArgument("planner: row-group epilogue split the kernel does not take");
          pr.used_nodes.insert(q.proj_b.node); pr.used_nodes.insert(q.proj_c.node);
          if (q.proj_c_copy >= 0) pr.used_nodes.insert(q.proj_c_copy);
          std::string bo = std::to_string(q.proj_b.offset) + "ull", co = std::to_string(q.proj_c.offset) + "ull";
          for (size_t k = 0; k < n; ++k) {
            const std::string tk = "(uint64_t)t" + std::to_string(k) + "_" + (k == (size_t)ma ? " * 32ull" : "");
            if (q.proj_b_stride[k]) bo += " + " + tk + " * " + std::to_string(q.proj_b_stride[k]) + "ull";
            if (q.proj_c_stride[k]) co += " + " + tk + " * " + std::to_string(q.proj_c_stride[k]) + "ull";
          }
          if (KP > 1) body.push_back(pind + "__shared__ __attribute__((aligned(16))) float ps_[" + std::to_string((int64_t)KP * 32 * q.proj_n) + "];");
          body.push_back(pind + "__syncthreads();");
          body.push_back(pind + "ocn_rowtile_project<" + std::to_string(q.row_len) + ", " + std::to_string(q.proj_n) + ", " + std::to_string(NW) + ", " +
                         std::to_string(KP) + ", " + std::to_string(ys) + ">((const unsigned short*)xs_, " +
                         r.node(q.proj_b.node).ident + " + (" + bo + "), " + std::to_string(q.proj_b_row) + "ll, " +
                         (KP > 1 ? "ps_" : "(float*)0") + ", " + r.node(q.proj_c.node).ident + " + (" + co + "), " +
                         std::to_string(q.proj_c_stride[ma]) + "ll, " +
                         (q.proj_c_copy >= 0 ? r.node(q.proj_c_copy).ident + " + (" + co + ")" : std::string("(unsigned short*)0")) + ");");
        }
        pr.lds_node = -1;
        pr.row_iters = 0; pr.cache_name.clear(); pr.cache_defined.clear();
        return (uint64_t)(QP * (uint64_t)fused_block);
      }
      if (!q.members.empty()) {
        // ---- row group: a lane group owns one row and runs the member phases in order
        for (auto e : q.row_outer_ext) QP *= (uint64_t)e;
        body.push_back(pind + "if (pt_ >= " + std::to_string(QP) + "ull) " + skip + ";");
        const size_t n = q.row_outer_ext.size();
        for (int k = (int)n - 1; k >= 0; --k) {
          const std::string ext = std::to_string(q.row_outer_ext[k]) + "ull";
          std::string line = pind + "const " + pr.idx_t + " row" + std::to_string(k) + "_ = (" + pr.idx_t + ")(";
          if (k == 0) line += "pt_);";
          else line += "pt_ % " + ext + "); pt_ /= " + ext + ";";
          body.push_back(line);
        }
        if (QG > 64) body.push_back(pind + "__shared__ float red_[4]; __shared__ double redd_[4];");
        // short rows: everything the group produces stays in registers as well (no read-back)
        const bool cached = q.row_len % QG == 0 && q.row_len / QG <= 16;
        if (cached) {
          pr.row_iters = (int)(q.row_len / QG);
          for (auto& m : q.members) {
            const Stmt& st = *m.inner[0];
            if (pr.cache_name.count(st.node)) continue;
            const Node& wn = r.node(st.node);
            bool per_position = false;
            for (auto& ix : st.idcs) if (ix.kind == AxisIndex::Iter && ix.sym == m.row_sym && m.row_role == Phase::RowPointwise) per_position = true;
            const std::string base = "c" + std::to_string(st.node) + "_";
            if (per_position) {
              body.push_back(pind + c_typ(wn.prec) + " " + base + "[" + std::to_string(pr.row_iters) + "];");
              pr.cache_name[st.node] = base + "[it_]";
            } else {
              body.push_back(pind + c_typ(wn.prec) + " " + base + ";");
              pr.cache_name[st.node] = base;
            }
          }
        }
        for (size_t mi = 0; mi < q.members.size(); ++mi) {
          const Phase& m = q.members[mi];
          if (mi && !cached) body.push_back(pind + "__builtin_amdgcn_fence(__ATOMIC_RELEASE, \"workgroup\"); "
                                                   "__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, \"workgroup\");");
          body.push_back(pind + "{  /* " + m.label + " */");
          const std::string mi_ind = pind + "  ";
          for (size_t k = 0; k < m.row_outer_syms.size(); ++k)
            body.push_back(mi_ind + "const " + pr.idx_t + " " + sym_ident(m.row_outer_syms[k]) + " = row" + std::to_string(k) + "_;");
          pr.skip_store.clear();
          if (cached && row_store_is_overwritten(q, mi) && pr.cache_name.count(m.inner[0]->node)) pr.skip_store.insert(m.inner[0]->node);
          if (m.row_role == Phase::RowPointwise) {
            body.push_back(pr.row_loop(sym_ident(m.row_sym), 0, q.row_len - 1, QG, mi_ind));
            emit_phase_statements(r, pr, m, 1, false, mi_ind + "  ", body);
            body.push_back(mi_ind + "}");
          } else {
            emit_phase_statements(r, pr, m, QG, true, mi_ind, body);
          }
          pr.skip_store.clear();
          body.push_back(pind + "}");
        }
        pr.row_iters = 0; pr.cache_name.clear(); pr.cache_defined.clear();
      } else {
        // --- point decode: the symbol with the smallest stride in the first written array varies
        //     fastest across adjacent threads (coalesced stores)
        std::vector<size_t> order = store_order(r, q);
        for (auto e : q.par_ext) QP *= (uint64_t)e;
        body.push_back(pind + "if (pt_ >= " + std::to_string(QP) + "ull) " + skip + ";");
        for (int k = (int)order.size() - 1; k >= 0; --k) {
          const size_t i = order[k];
          const std::string sy = sym_ident(q.par_syms[i]);
          const std::string ext = std::to_string(q.par_ext[i]) + "ull";
          std::string line = pind + "const " + pr.idx_t + " " + sy + " = (" + pr.idx_t + ")(" + std::to_string(q.par_from[i]) + " + ";
          if (k == 0) line += "pt_);";
          else line += "pt_ % " + ext + "); pt_ /= " + ext + ";";
          body.push_back(line);
        }
        if (QG > 1 && !q.coop_scope && q.seq_syms.empty()) throw InvalidArgument("planner: lane group without a reduction to share");
        if (QG > 64) body.push_back(pind + "__shared__ float red_[4]; __shared__ double redd_[4];");
        emit_phase_statements(r, pr, q, QG, false, pind, body);
      }
      return QP * (uint64_t)QG;
    };

    uint64_t total_threads = 0;
    if (!ph.serial_members.empty()) {
      // ---- the whole routine in one workgroup: phases in order, a barrier after each
      for (auto& kv : ph.serial_shadows) {
        const Node& sn = r.node(kv.first);
        pr.shadow[kv.first] = "sh_" + sn.ident;
        body.push_back(ind + "__shared__ " + c_typ(sn.prec) + " sh_" + sn.ident + "[" + std::to_string(sn.num_elems()) + "];");
      }
      for (size_t qi = 0; qi < ph.serial_members.size(); ++qi) {
        const Phase& q = ph.serial_members[qi];
        for (auto& kv : ph.serial_shadows) if (kv.second < (int)qi) pr.shadow_live.insert(kv.first);
        body.push_back(ind + "/* " + q.label + " */");
        if (q.kind == Phase::Fill) {
          const Node& fn = r.node(q.fill_node);
          pr.used_nodes.insert(q.fill_node);
          Pair cv = convert_precision(Prec::Double, fn.prec);
          const std::string zero = cv.first + "0" + cv.second;
          std::string line = ind + "for (" + pr.idx_t + " z_ = threadIdx.x; z_ < " + std::to_string(fn.num_elems()) + "ull; z_ += 256u) ";
          if (pr.shadow.count(q.fill_node)) line += "{ " + fn.ident + "[z_] = " + zero + "; " + pr.shadow.at(q.fill_node) + "[z_] = " + zero + "; }";
          else line += fn.ident + "[z_] = " + zero + ";";
          body.push_back(line);
        } else {
          uint64_t qt = (uint64_t)q.coop_lanes;
          for (auto e : (q.members.empty() ? q.par_ext : q.row_outer_ext)) qt *= (uint64_t)e;
          const uint64_t rounded = (qt + 255) / 256 * 256;
          body.push_back(ind + "for (uint64_t gtid_ = threadIdx.x; gtid_ < " + std::to_string(rounded) + "ull; gtid_ += 256u) {");
          emit_points(q, ind + "  ", "continue");
          body.push_back(ind + "}");
        }
        body.push_back(ind + "__syncthreads();");
      }
      pr.shadow.clear(); pr.shadow_live.clear();
      total_threads = 256;
    } else if (!ph.parallel_members.empty()) {
      // ---- independent phases side by side: every member owns a range of whole workgroups
      body.push_back(ind + "const uint64_t g_ = ((uint64_t)blockIdx.y * gridDim.x + blockIdx.x) * blockDim.x + threadIdx.x;");
      uint64_t first = 0;
      for (auto& q : ph.parallel_members) {
        uint64_t qt = (uint64_t)q.coop_lanes;
        for (auto e : (q.members.empty() ? q.par_ext : q.row_outer_ext)) qt *= (uint64_t)e;
        const uint64_t end = first + (qt + 255) / 256 * 256;
        body.push_back(ind + (first ? "else if" : "if") + " (g_ < " + std::to_string(end) + "ull) {  /* " + q.label + " */");
        body.push_back(ind + "  const uint64_t gtid_ = g_ - " + std::to_string(first) + "ull;");
        emit_points(q, ind + "  ", "return");
        body.push_back(ind + "}");
        first = end;
      }
      total_threads = first;
    } else {
      body.push_back(ind + "const uint64_t gtid_ = ((uint64_t)blockIdx.y * gridDim.x + blockIdx.x) * blockDim.x + threadIdx.x;");
      total_threads = emit_points(ph, ind, "return");
    }

    if (plan.debug_log) {
      // one thread runs the phase (the planner kept every loop sequential); the routine's top-level
      // comments since the previous phase come first, those after the last phase at the very end
      std::vector<std::string> head;
      for (auto& t : ph.comments_before) head.push_back(ind + "if (gtid_ == 0) " + pr.log_call("COMMENT: " + Printer::lit(t), {}));
      body.insert(body.begin() + 1, head.begin(), head.end());   // (after the line that defines gtid_)
      bool last_generic = true;
      for (size_t q = pi + 1; q < plan.phases.size(); ++q) last_generic = last_generic && plan.phases[q].kind != Phase::Generic;
      if (last_generic) for (auto& t : plan.trailing_comments) body.push_back(ind + pr.log_call("COMMENT: " + Printer::lit(t), {}));
    }
    GeneratedKernel gk;
    gk.name = r.name + "_k" + std::to_string(kidx++);
    gk.phase_index = (int)pi;
    gk.threads = total_threads;
    gk.block = fused_block > 0 ? fused_block : 256;
    std::vector<std::string> decls;
    for (int id : r.node_order) {
      if (!pr.used_nodes.count(id)) continue;
      const Node& n = r.node(id);
      decls.push_back(std::string(c_typ(n.prec)) + " * __restrict__ " + n.ident);
      gk.params.push_back({KernelParam::NodePtr, id});
    }
    for (int id : pr.used_nodes) {   // planner-made scratch nodes are not in node_order
      if (std::find(r.node_order.begin(), r.node_order.end(), id) != r.node_order.end()) continue;
      const Node& n = r.node(id);
      decls.push_back(std::string(c_typ(n.prec)) + " * __restrict__ " + n.ident);
      gk.params.push_back({KernelParam::NodePtr, id});
    }
    if (pr.used_merge) {
      if (r.merge_node < 0) throw InvalidArgument("hip backend: routine " + r.name + " reads a merge buffer it does not declare");
      decls.push_back(std::string("const ") + c_typ(r.node(r.merge_node).prec) + " * __restrict__ merge_buffer");
      gk.params.push_back({KernelParam::MergeBuffer, r.merge_node});
    }
    for (auto& s : r.statics) {
      if (!pr.used_statics.count(s.sym)) continue;
      // integer arguments are 64 bits wide under large_models (c_syntax.ml:111-112 `arg_int_prefix`)
      decls.push_back(std::string(plan.large_index ? "const uint64_t " : "const uint32_t ") + sym_ident(s.sym));
      gk.params.push_back({KernelParam::StaticIdx, s.sym});
    }
    if (plan.debug_log) { decls.push_back("const int log_id"); gk.params.push_back({KernelParam::LogId, 0}); }
    src << "/* phase " << pi << ": " << ph.label << " */\n";
    src << "extern \"C\" __global__ void __launch_bounds__(" << gk.block << ") " << gk.name << "(";
    for (size_t i = 0; i < decls.size(); ++i) src << (i ? ", " : "") << decls[i];
    src << ") {\n";
    for (auto& l : body) src << l << "\n";
    src << "}\n\n";
    mod.kernels.push_back(std::move(gk));
  }
  mod.source = src.str();
  return mod;
}

const char* c_typ_name(Prec p) { return p == Prec::Half ? "HALF_T" : c_typ(p); }

}  // namespace ocannl
