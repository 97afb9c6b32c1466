#include "llir.hpp"

#include <cctype>
#include <cmath>
#include <cstdlib>
#include <cstring>

namespace ocannl {

static const char* kPrecNames[] = {"void", "byte", "uint16", "int32", "uint32", "int64", "uint64",
                                   "uint4x32", "half", "bfloat16", "fp8", "single", "double"};
static const int kPrecBytes[] = {0, 1, 2, 4, 4, 8, 8, 16, 2, 2, 1, 4, 8};

Prec prec_of_string(const std::string& s) {
  for (int i = 0; i < 13; ++i)
    if (s == kPrecNames[i]) return static_cast<Prec>(i);
  throw InvalidArgument("LLIR: unknown precision " + s);
}
const char* prec_string(Prec p) { return kPrecNames[static_cast<int>(p)]; }
int prec_in_bytes(Prec p) { return kPrecBytes[static_cast<int>(p)]; }

// ---------------------------------------------------------------------------------------------
// S-expressions
// ---------------------------------------------------------------------------------------------
namespace {

struct Sx {
  bool atom = false;
  bool quoted = false;
  std::string s;
  std::vector<Sx> kids;
  const Sx& at(size_t i) const {
    if (atom || i >= kids.size()) throw InvalidArgument("LLIR: malformed form near '" + head() + "'");
    return kids[i];
  }
  std::string head() const { return (!atom && !kids.empty() && kids[0].atom) ? kids[0].s : s; }
  size_t size() const { return kids.size(); }
};

struct Reader {
  const char* p;
  const char* end;
  void skip() { while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p; }
  Sx read() {
    skip();
    if (p >= end) throw InvalidArgument("LLIR: unexpected end of input");
    Sx x;
    if (*p == '(') {
      ++p;
      for (;;) {
        skip();
        if (p >= end) throw InvalidArgument("LLIR: unbalanced parenthesis");
        if (*p == ')') { ++p; break; }
        x.kids.push_back(read());
      }
      return x;
    }
    if (*p == ')') throw InvalidArgument("LLIR: unexpected ')'");
    x.atom = true;
    if (*p == '"') {
      x.quoted = true;
      ++p;
      while (p < end && *p != '"') {
        if (*p == '\\' && p + 1 < end) ++p;
        x.s.push_back(*p++);
      }
      if (p >= end) throw InvalidArgument("LLIR: unterminated string");
      ++p;
      return x;
    }
    while (p < end && *p != '(' && *p != ')' && *p != ' ' && *p != '\n' && *p != '\t' && *p != '\r')
      x.s.push_back(*p++);
    return x;
  }
};

int64_t to_int(const Sx& x) {
  if (!x.atom) throw InvalidArgument("LLIR: expected an integer");
  char* e = nullptr;
  long long v = std::strtoll(x.s.c_str(), &e, 10);
  if (e == x.s.c_str() || *e) throw InvalidArgument("LLIR: bad integer '" + x.s + "'");
  return v;
}

double to_double(const Sx& x) {
  if (!x.atom) throw InvalidArgument("LLIR: expected a float");
  if (x.s == "inf") return HUGE_VAL;
  if (x.s == "-inf") return -HUGE_VAL;
  char* e = nullptr;
  double v = std::strtod(x.s.c_str(), &e);  // accepts C99 hex floats, "nan"
  if (e == x.s.c_str() || *e) throw InvalidArgument("LLIR: bad float '" + x.s + "'");
  return v;
}

template <class E>
E lookup(const char* const* names, int n, const std::string& s, const char* what) {
  for (int i = 0; i < n; ++i)
    if (s == names[i]) return static_cast<E>(i);
  throw InvalidArgument(std::string("LLIR: unknown ") + what + " '" + s + "'");
}

const char* kBinops[] = {"arg1", "arg2", "add", "sub", "mul", "div", "pow", "relu_gate", "sat01_gate",
                         "max", "min", "mod", "lt", "eq", "ne", "or", "and", "threefry4x32_crypto",
                         "threefry4x32_light"};
const char* kUnops[] = {"id", "relu", "sat01", "exp", "log", "exp2", "log2", "sin", "cos", "sqrt",
                        "recip", "recip_sqrt", "neg", "trunc", "tanh", "not",
                        "uint4x32_to_prec_uniform1"};
const char* kTernops[] = {"where", "fma", "mul3"};

AxisIndex parse_index(const Sx& x) {
  AxisIndex a;
  const std::string h = x.head();
  if (h == "fixed") { a.kind = AxisIndex::Fixed; a.fixed = to_int(x.at(1)); }
  else if (h == "it") { a.kind = AxisIndex::Iter; a.sym = (int)to_int(x.at(1)); }
  // Sub_axis (indexing.ml:116): an axis spanned by an adjacent multi-axis index adds nothing to the
  // offset (indexing.ml:429) -- position 0 of its axis
  else if (h == "sub") { a.kind = AxisIndex::Fixed; a.fixed = 0; }
  else if (h == "affine") {
    a.kind = AxisIndex::Affine;
    for (auto& t : x.at(1).kids) a.terms.emplace_back(to_int(t.at(0)), (int)to_int(t.at(1)));
    a.offset = to_int(x.at(2));
  } else throw InvalidArgument("LLIR: unknown index form '" + h + "'");
  return a;
}

Indices parse_indices(const Sx& x) {
  Indices r;
  if (x.atom) throw InvalidArgument("LLIR: expected an index list");
  for (auto& k : x.kids) r.push_back(parse_index(k));
  return r;
}

Block parse_block(const Sx& x);

ScalarP parse_scalar(const Sx& x) {
  auto s = std::make_shared<Scalar>();
  const std::string h = x.head();
  if (h == "get") { s->kind = Scalar::Get; s->node = (int)to_int(x.at(1)); s->idcs = parse_indices(x.at(2)); }
  else if (h == "get_merge") { s->kind = Scalar::GetMerge; s->node = (int)to_int(x.at(1)); s->idcs = parse_indices(x.at(2)); }
  else if (h == "get_dyn") {
    s->kind = Scalar::GetDyn; s->node = (int)to_int(x.at(1)); s->idcs = parse_indices(x.at(2));
    s->dyn_axis = (int)to_int(x.at(3)); s->arg_prec = prec_of_string(x.at(4).s); s->a = parse_scalar(x.at(5));
  } else if (h == "get_local") { s->kind = Scalar::GetLocal; s->scope = {(int)to_int(x.at(1)), (int)to_int(x.at(2))}; }
  else if (h == "local_scope") {
    s->kind = Scalar::LocalScope; s->scope = {(int)to_int(x.at(1)), (int)to_int(x.at(2))};
    s->body = parse_block(x.at(3));
  } else if (h == "const") { s->kind = Scalar::Const; s->cst = to_double(x.at(1)); }
  else if (h == "bits") { s->kind = Scalar::Bits; s->bits = to_int(x.at(1)); }
  else if (h == "index") { s->kind = Scalar::Index; s->index = parse_index(x.at(1)); }
  else if (h == "unop") {
    s->kind = Scalar::Un; s->un = lookup<Unop>(kUnops, 17, x.at(1).s, "unop");
    s->arg_prec = prec_of_string(x.at(2).s); s->a = parse_scalar(x.at(3));
  } else if (h == "binop") {
    s->kind = Scalar::Bin; s->bin = lookup<Binop>(kBinops, 19, x.at(1).s, "binop");
    s->a = parse_scalar(x.at(2)); s->b = parse_scalar(x.at(3));
  } else if (h == "ternop") {
    s->kind = Scalar::Tern; s->tern = lookup<Ternop>(kTernops, 3, x.at(1).s, "ternop");
    s->arg_prec = prec_of_string(x.at(2).s);
    s->a = parse_scalar(x.at(3)); s->b = parse_scalar(x.at(4)); s->c = parse_scalar(x.at(5));
  } else throw InvalidArgument("LLIR: unknown scalar form '" + h + "'");
  return s;
}

StmtP parse_stmt(const Sx& x) {
  auto s = std::make_shared<Stmt>();
  const std::string h = x.head();
  if (h == "comment") { s->kind = Stmt::Comment; s->text = x.at(1).s; }
  else if (h == "for") {
    s->kind = Stmt::For; s->sym = (int)to_int(x.at(1)); s->from = to_int(x.at(2)); s->to = to_int(x.at(3));
    s->body = parse_block(x.at(4));
  } else if (h == "zero_out") { s->kind = Stmt::ZeroOut; s->node = (int)to_int(x.at(1)); }
  else if (h == "set") {
    s->kind = Stmt::Set; s->node = (int)to_int(x.at(1)); s->idcs = parse_indices(x.at(2));
    s->value = parse_scalar(x.at(3));
    if (x.kids.size() > 4) s->text = x.at(4).s;   // Low_level.Set's `debug` field: the statement as text
  } else if (h == "set_vec") {
    s->kind = Stmt::SetVec; s->node = (int)to_int(x.at(1)); s->idcs = parse_indices(x.at(2));
    s->length = (int)to_int(x.at(3));
    if (x.at(4).s != "uint4x32_to_prec_uniform") throw InvalidArgument("LLIR: unknown vec_unop " + x.at(4).s);
    s->arg_prec = prec_of_string(x.at(5).s); s->value = parse_scalar(x.at(6));
  } else if (h == "set_local") {
    s->kind = Stmt::SetLocal; s->scope = {(int)to_int(x.at(1)), (int)to_int(x.at(2))};
    s->value = parse_scalar(x.at(3));
  } else if (h == "declare_local") {
    s->kind = Stmt::DeclareLocal; s->scope = {(int)to_int(x.at(1)), (int)to_int(x.at(2))};
    s->needs_init = to_int(x.at(3)) != 0;
  } else throw InvalidArgument("LLIR: unknown statement form '" + h + "'");
  return s;
}

Block parse_block(const Sx& x) {
  Block b;
  if (x.atom) throw InvalidArgument("LLIR: expected a statement list");
  for (auto& k : x.kids) b.push_back(parse_stmt(k));
  return b;
}

void check_scalar(const Routine& r, const Scalar& s);
void check_block(const Routine& r, const Block& b);

void check_access(const Routine& r, int node, const Indices& idcs, const char* what) {
  const Node& n = r.node(node);
  if (idcs.size() != n.dims.size())
    throw InvalidArgument(std::string("LLIR: ") + what + " of " + n.ident + " has " +
                          std::to_string(idcs.size()) + " indices for " + std::to_string(n.dims.size()) + " axes");
}

void check_scalar(const Routine& r, const Scalar& s) {
  switch (s.kind) {
    case Scalar::Get: case Scalar::GetMerge: check_access(r, s.node, s.idcs, "read"); break;
    case Scalar::GetDyn:
      check_access(r, s.node, s.idcs, "gather");
      if (s.dyn_axis < 0 || s.dyn_axis >= (int)s.idcs.size()) throw InvalidArgument("LLIR: bad dyn_axis");
      check_scalar(r, *s.a); break;
    case Scalar::GetLocal: r.node(s.scope.node); break;
    case Scalar::LocalScope: r.node(s.scope.node); check_block(r, s.body); break;
    case Scalar::Un: check_scalar(r, *s.a); break;
    case Scalar::Bin: check_scalar(r, *s.a); check_scalar(r, *s.b); break;
    case Scalar::Tern: check_scalar(r, *s.a); check_scalar(r, *s.b); check_scalar(r, *s.c); break;
    default: break;
  }
}

void check_block(const Routine& r, const Block& b) {
  for (auto& s : b) {
    switch (s->kind) {
      case Stmt::For: check_block(r, s->body); break;
      case Stmt::ZeroOut: r.node(s->node); break;
      case Stmt::Set: check_access(r, s->node, s->idcs, "write"); check_scalar(r, *s->value); break;
      case Stmt::SetVec: check_access(r, s->node, s->idcs, "write"); check_scalar(r, *s->value); break;
      case Stmt::SetLocal: r.node(s->scope.node); check_scalar(r, *s->value); break;
      case Stmt::DeclareLocal: r.node(s->scope.node); break;
      default: break;
    }
  }
}

Routine parse_routine(const Sx& x) {
  if (x.head() != "routine") throw InvalidArgument("LLIR: expected (routine ...)");
  Routine r;
  r.name = x.at(1).s;
  for (char c : r.name)
    if (!(std::isalnum((unsigned char)c) || c == '_')) throw InvalidArgument("LLIR: routine name must be a C identifier");
  for (size_t i = 2; i < x.size(); ++i) {
    const Sx& f = x.kids[i];
    const std::string h = f.head();
    if (h == "static") {
      for (size_t k = 1; k < f.size(); ++k)
        r.statics.push_back({(int)to_int(f.kids[k].at(0)), to_int(f.kids[k].at(1))});
    } else if (h == "merge") {
      r.merge_node = (int)to_int(f.at(1));
    } else if (h == "nodes") {
      for (size_t k = 1; k < f.size(); ++k) {
        const Sx& n = f.kids[k];
        Node nd;
        nd.id = (int)to_int(n.at(0));
        nd.ident = n.at(1).s;
        nd.prec = prec_of_string(n.at(2).s);
        const std::string m = n.at(3).s;
        nd.mode = m == "ctx" ? Mode::Ctx : m == "local" ? Mode::Local : m == "virtual" ? Mode::Virtual
                  : throw InvalidArgument("LLIR: unknown memory mode " + m);
        nd.zero_initialized_by_code = to_int(n.at(4)) != 0;
        nd.read_only = to_int(n.at(5)) != 0;
        for (auto& d : n.at(6).kids) {
          nd.dims.push_back(to_int(d));
          if (nd.dims.back() <= 0) throw InvalidArgument("LLIR: non-positive dimension in " + nd.ident);
        }
        if (r.nodes.count(nd.id)) throw InvalidArgument("LLIR: duplicate node id");
        r.node_order.push_back(nd.id);
        r.nodes.emplace(nd.id, std::move(nd));
      }
    } else if (h == "body") {
      for (size_t k = 1; k < f.size(); ++k) r.body.push_back(parse_stmt(f.kids[k]));
    } else throw InvalidArgument("LLIR: unknown routine section '" + h + "'");
  }
  check_block(r, r.body);
  return r;
}

}  // namespace

Prec scalar_precision(const Routine& r, const Scalar& s) {
  switch (s.kind) {
    case Scalar::Get: case Scalar::GetDyn: case Scalar::GetMerge: return r.node(s.node).prec;
    case Scalar::GetLocal: case Scalar::LocalScope: return r.node(s.scope.node).prec;
    case Scalar::Const: return Prec::Single;
    case Scalar::Bits: return Prec::Int64;
    case Scalar::Index: return Prec::Uint32;
    case Scalar::Tern: return s.arg_prec;
    case Scalar::Bin: return scalar_precision(r, *s.a);
    case Scalar::Un: return s.arg_prec;
  }
  return Prec::Void;
}

std::vector<Routine> parse_routines(const char* text, size_t len) {
  Reader rd{text, text + len};
  std::vector<Routine> out;
  for (;;) {
    rd.skip();
    if (rd.p >= rd.end) break;
    out.push_back(parse_routine(rd.read()));
  }
  if (out.empty()) throw InvalidArgument("LLIR: no routine in input");
  return out;
}

}  // namespace ocannl
