// Reuse of values that the routine has already stored.
//
// The reference's optimiser does not count a read at the very position being assigned as a visit
// (arrayjit/lib/low_level.ml:496-552 with inline_complex_computations, the default), so a tensor that
// is computed once per cell is inlined into EVERY reader of that kind and recomputed there -- with
// whatever its own definition had inlined.  The reference's own golden shows it
// (test/einsum/moons_demo_variant.expected:39-44: the product `w1 * x`, the sum with the bias and the
// gradient of the relu are all virtual, only relu(..) is stored): the backward statement of a relu,
// `g1 =+ relu_gate(v1, g)` (tensor/operation.ml:172-178), then holds the whole contraction that computes
// v1 a second time, per element.  For a serial C loop that is twice the work; for a routine cut into
// kernels it turns a pointwise statement into a K-long loop per element (8 ms instead of 45 us per
// feed-forward block of the transformer step).
//
// This pass, run on the routine before planning, finds such recomputations and reads what is in memory
// instead:
//   * `T[p..] := E` stored earlier, and a later statement holds a sub-expression structurally equal
//     to E (up to the names of loop symbols and scopes) that contains an inlined reduction: it becomes
//     `T[..]`;
//   * `T[p..] := relu(E)` stored earlier, and a later `relu_gate(E', g)` with E' equal to E: the
//     condition E' > 0 holds exactly when T > 0 (relu(x) = fmaxf(0, x): negative, zero and NaN all give a
//     value that is not > 0), so E' becomes `T[..]`.
// Equal means: same operations, constants, precisions, tensor nodes and index structure, evaluated in
// the same precision; and no statement between the two writes T or anything E reads.
#include <functional>
#include <map>
#include <set>
#include <sstream>

#include "plan.hpp"

namespace ocannl {
namespace {

// Canonical text of an expression: free loop symbols are numbered in order of first appearance (q0,
// q1, ..), symbols bound by loops inside scopes likewise (b0, ..), scopes too (s0, ..).
struct Canon {
  std::map<int, int> free_syms, bound_syms;
  std::map<ScopeId, int> scopes;
  std::vector<int> free_order;      // the symbols behind q0, q1, ..
  std::set<int> reads;              // nodes read
  bool has_reduction = false;       // a loop inside a scope
  bool ok = true;                   // nothing the comparison cannot see through
  std::ostringstream out;

  void sym(int s) {
    auto b = bound_syms.find(s);
    if (b != bound_syms.end()) { out << "b" << b->second; return; }
    auto f = free_syms.find(s);
    if (f == free_syms.end()) { f = free_syms.emplace(s, (int)free_syms.size()).first; free_order.push_back(s); }
    out << "q" << f->second;
  }
  void index(const AxisIndex& a) {
    if (a.kind == AxisIndex::Fixed) out << "#" << a.fixed;
    else if (a.kind == AxisIndex::Iter) sym(a.sym);
    else { out << "aff("; for (auto& t : a.terms) { out << t.first << "*"; sym(t.second); out << "+"; } out << a.offset << ")"; }
  }
  void indices(const Indices& ix) { out << "["; for (auto& a : ix) { index(a); out << ","; } out << "]"; }
  void scope(const ScopeId& s) {
    auto it = scopes.find(s);
    if (it == scopes.end()) it = scopes.emplace(s, (int)scopes.size()).first;
    out << "s" << it->second << ":" << s.node;   // (the scope's node fixes its precision)
  }
  void block(const Block& b) {
    for (auto& sp : b) {
      const Stmt& c = *sp;
      switch (c.kind) {
        case Stmt::Comment: break;
        case Stmt::For: {
          has_reduction = true;
          const int id = (int)bound_syms.size();
          bound_syms[c.sym] = id;
          out << "for(b" << id << "," << c.from << "," << c.to << "){"; block(c.body); out << "}";
          break;
        }
        case Stmt::SetLocal: out << "setl("; scope(c.scope); out << ","; scalar(*c.value); out << ");"; break;
        case Stmt::DeclareLocal: out << "decl("; scope(c.scope); out << "," << c.needs_init << ");"; break;
        default: ok = false; break;   // stores to tensors inside a scope: not a pure value
      }
    }
  }
  void scalar(const Scalar& s) {
    switch (s.kind) {
      case Scalar::Get: reads.insert(s.node); out << "get(" << s.node; indices(s.idcs); out << ")"; break;
      case Scalar::GetMerge: ok = false; break;
      case Scalar::GetDyn:
        reads.insert(s.node);
        out << "dyn(" << s.node; indices(s.idcs); out << "," << s.dyn_axis << "," << (int)s.arg_prec << ","; scalar(*s.a); out << ")";
        break;
      case Scalar::GetLocal: out << "getl("; scope(s.scope); out << ")"; break;
      case Scalar::LocalScope: out << "scope("; scope(s.scope); out << "){"; block(s.body); out << "}"; break;
      case Scalar::Const: { uint64_t bits; static_assert(sizeof bits == sizeof s.cst, ""); __builtin_memcpy(&bits, &s.cst, 8); out << "c" << bits; break; }
      case Scalar::Bits: out << "B" << s.bits; break;
      case Scalar::Index: out << "idx("; index(s.index); out << ")"; break;
      case Scalar::Un: out << "u" << (int)s.un << ":" << (int)s.arg_prec << "("; scalar(*s.a); out << ")"; break;
      case Scalar::Bin: out << "o" << (int)s.bin << "("; scalar(*s.a); out << ","; scalar(*s.b); out << ")"; break;
      case Scalar::Tern: out << "t" << (int)s.tern << ":" << (int)s.arg_prec << "("; scalar(*s.a); out << ","; scalar(*s.b); out << ","; scalar(*s.c); out << ")"; break;
    }
  }
};

// A scope whose body is the single statement `v := e` with e not reading v: the value e, evaluated in
// the scope's precision (how the lowering keeps a value of another precision rounded to its own first).
const Scalar* unwrap(const Routine& r, const Scalar& s, Prec* prec) {
  const Scalar* cur = &s;
  for (;;) {
    if (cur->kind != Scalar::LocalScope) return cur;
    const Stmt* only = nullptr;
    int n = 0;
    for (auto& sp : cur->body) if (sp->kind != Stmt::Comment) { only = sp.get(); ++n; }
    if (n != 1 || only->kind != Stmt::SetLocal || !(only->scope == cur->scope)) return cur;
    bool reads_self = false;
    std::function<void(const Scalar&)> w = [&](const Scalar& x) {
      if (x.kind == Scalar::GetLocal && x.scope == cur->scope) reads_self = true;
      if (x.kind == Scalar::LocalScope) for (auto& sp : x.body) if (sp->value) w(*sp->value);
      if (x.a) w(*x.a); if (x.b) w(*x.b); if (x.c) w(*x.c);
    };
    w(*only->value);
    if (reads_self) return cur;
    *prec = r.node(cur->scope.node).prec;
    cur = only->value.get();
  }
}

// A value computed (and rounded) in precision `from` is the same number after a store to a tensor of
// precision `to` and the read back: equal precisions, or a wider floating-point type.
bool stores_exactly(Prec from, Prec to) {
  auto rank = [](Prec p) { return p == Prec::Double ? 3 : p == Prec::Single ? 2 : (p == Prec::Bfloat16 || p == Prec::Half) ? 1 : 0; };
  if (rank(from) == 0 || rank(to) == 0) return false;   // integer-like and 8-bit types: not taken
  return from == to || rank(to) > rank(from);
}

struct Stored {
  int node;                       // T
  std::vector<int> pos_of_free;   // free symbol q_k of E stands at this position of T's index tuple
  std::set<int> reads;            // what E reads
  size_t at;                      // index of the defining top-level statement
};

void written_nodes(const Block& b, std::set<int>& out) {
  for (auto& sp : b) {
    if (sp->kind == Stmt::For) written_nodes(sp->body, out);
    else if (sp->kind == Stmt::Set || sp->kind == Stmt::SetVec || sp->kind == Stmt::ZeroOut) out.insert(sp->node);
    std::function<void(const Scalar&)> w = [&](const Scalar& x) {
      if (x.kind == Scalar::LocalScope) written_nodes(x.body, out);
      if (x.a) w(*x.a); if (x.b) w(*x.b); if (x.c) w(*x.c);
    };
    if (sp->value) w(*sp->value);
  }
}

}  // namespace

int reuse_stored_values(Routine& r) {
  // top-level statements and what each writes
  std::vector<std::set<int>> writes(r.body.size());
  for (size_t i = 0; i < r.body.size(); ++i) written_nodes({r.body[i]}, writes[i]);
  std::map<std::string, Stored> plain, through_relu;   // key: "<evaluation precision>|<canonical text>"
  int replaced = 0;

  auto still_valid = [&](const Stored& st, size_t use) {
    for (size_t q = st.at + 1; q < use; ++q) {
      if (writes[q].count(st.node)) return false;
      for (int n : st.reads) if (writes[q].count(n)) return false;
    }
    // (the using statement itself may store to T or to an operand only after reading: not assumed)
    if (writes[use].count(st.node)) return false;
    for (int n : st.reads) if (writes[use].count(n)) return false;
    return true;
  };

  for (size_t i = 0; i < r.body.size(); ++i) {
    // the statement as a perfect chain of loops around one Set
    std::vector<const Stmt*> chain;
    Stmt* set = nullptr;
    {
      Stmt* cur = r.body[i].get();
      for (;;) {
        if (cur->kind == Stmt::Set) { set = cur; break; }
        if (cur->kind != Stmt::For) break;
        Stmt* next = nullptr;
        int n = 0;
        for (auto& sp : cur->body) if (sp->kind != Stmt::Comment) { next = sp.get(); ++n; }
        if (n != 1) break;
        chain.push_back(cur);
        cur = next;
      }
    }
    if (!set) continue;

    // ---- use: rewrite sub-expressions that recompute a stored value
    // (ranges of the loop symbols around the sub-expression being looked at: the stored tensor is only
    // known over its own extents, whatever the extents of the operands are)
    std::map<int, std::pair<int64_t, int64_t>> range;
    for (const Stmt* l : chain) range[l->sym] = {l->from, l->to};
    auto inside = [&](const Stored& st, const Canon& c) {
      const Node& t = r.node(st.node);
      for (size_t k = 0; k < c.free_order.size(); ++k) {
        auto it = range.find(c.free_order[k]);
        if (it == range.end() || it->second.first < 0 || it->second.second > t.dims[st.pos_of_free[k]] - 1) return false;
      }
      return true;
    };
    std::function<void(ScalarP&, Prec, bool)> visit = [&](ScalarP& sp, Prec prec, bool gate_arg) {
      Prec eval = prec;
      const Scalar* e = unwrap(r, *sp, &eval);
      Canon c;
      c.scalar(*e);
      if (c.ok && c.has_reduction) {
        const std::string key = std::to_string((int)eval) + "|" + c.out.str();
        const Stored* hit = nullptr;
        auto it = plain.find(key);
        if (it != plain.end() && still_valid(it->second, i)) hit = &it->second;
        if (!hit && gate_arg) {
          it = through_relu.find(key);
          if (it != through_relu.end() && still_valid(it->second, i)) hit = &it->second;
        }
        if (hit && hit->pos_of_free.size() == c.free_order.size() && inside(*hit, c)) {
          auto g = std::make_shared<Scalar>();
          g->kind = Scalar::Get; g->node = hit->node;
          g->idcs.resize(r.node(hit->node).dims.size());
          for (auto& a : g->idcs) { a.kind = AxisIndex::Fixed; a.fixed = 0; }
          for (size_t k = 0; k < c.free_order.size(); ++k) {
            AxisIndex& a = g->idcs[hit->pos_of_free[k]];
            a.kind = AxisIndex::Iter; a.sym = c.free_order[k];
          }
          sp = g;
          ++replaced;
          return;
        }
      }
      Scalar& s = *sp;   // (descend into the expression as written, wrappers included)
      switch (s.kind) {
        case Scalar::Un: visit(s.a, s.un == Unop::Uniform1 ? s.arg_prec : prec, false); break;
        case Scalar::Bin:
          visit(s.a, prec, s.bin == Binop::ReluGate);
          visit(s.b, prec, false);
          break;
        case Scalar::Tern:
          visit(s.a, s.tern == Ternop::Where ? s.arg_prec : prec, false);
          visit(s.b, prec, false);
          visit(s.c, prec, false);
          break;
        case Scalar::LocalScope: {
          const Prec sp_prec = r.node(s.scope.node).prec;
          std::function<void(Block&)> blk = [&](Block& b) {
            for (auto& st : b) {
              if (st->kind == Stmt::For) { range[st->sym] = {st->from, st->to}; blk(st->body); range.erase(st->sym); }
              else if (st->kind == Stmt::SetLocal && st->value) visit(st->value, sp_prec, false);
            }
          };
          blk(s.body);
          break;
        }
        default: break;
      }
    };
    visit(set->value, r.node(set->node).prec, false);

    // ---- definition: `T[p..] := E` or `T[p..] := relu(E)` over the whole of T, E holding a reduction
    const Node& tn = r.node(set->node);
    if (tn.mode == Mode::Virtual) continue;
    bool whole = set->idcs.size() == tn.dims.size() && chain.size() == tn.dims.size();
    std::map<int, int> pos_of_sym;
    for (size_t p = 0; p < set->idcs.size() && whole; ++p) {
      const AxisIndex& a = set->idcs[p];
      if (a.kind != AxisIndex::Iter || pos_of_sym.count(a.sym)) { whole = false; break; }
      const Stmt* loop = nullptr;
      for (const Stmt* l : chain) if (l->sym == a.sym) loop = l;
      if (!loop || loop->from != 0 || loop->to != tn.dims[p] - 1) { whole = false; break; }
      pos_of_sym[a.sym] = (int)p;
    }
    if (!whole) continue;
    // `keeps`: only the sign of the value is asked for later (the relu form), which a store in bf16, with
    // the exponent range of fp32, keeps as well
    auto record = [&](const Scalar& value, Prec prec, std::map<std::string, Stored>& table, bool keeps) {
      Prec eval = prec;
      const Scalar* e = unwrap(r, value, &eval);
      Canon c;
      c.scalar(*e);
      if (!c.ok || !c.has_reduction || c.reads.count(set->node)) return;
      if (!stores_exactly(eval, tn.prec) && !(keeps && eval == Prec::Single && tn.prec == Prec::Bfloat16)) return;
      Stored st;
      st.node = set->node; st.reads = c.reads; st.at = i;
      for (int s : c.free_order) {
        auto it = pos_of_sym.find(s);
        if (it == pos_of_sym.end()) return;   // (a static index or a symbol that is not an axis of T)
        st.pos_of_free.push_back(it->second);
      }
      if (st.pos_of_free.size() != tn.dims.size()) return;   // every axis of T has to be addressed
      table[std::to_string((int)eval) + "|" + c.out.str()] = st;
    };
    record(*set->value, tn.prec, plain, false);
    if (set->value->kind == Scalar::Un && set->value->un == Unop::Relu && stores_exactly(tn.prec, tn.prec))
      record(*set->value->a, tn.prec, through_relu, true);
  }
  return replaced;
}

}  // namespace ocannl
