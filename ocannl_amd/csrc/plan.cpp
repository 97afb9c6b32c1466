#include "plan.hpp"

#include <algorithm>
#include <cmath>
#include <functional>
#include <set>

namespace ocannl {
namespace {

Block strip_comments(const Block& b, std::string* last_comment);

struct Access {
  int node;
  const Indices* idcs;
  bool write;
  int vec_len;   // >0 for Set_from_vec writes
};

void scalar_accesses(const Scalar& s, std::vector<Access>& out, bool& foreign_local_write,
                     std::set<ScopeId>& declared);
void block_accesses(const Block& b, std::vector<Access>& out, bool& whole_array_write,
                    bool& foreign_local_write, std::set<ScopeId>& declared) {
  for (auto& sp : b) {
    const Stmt& s = *sp;
    switch (s.kind) {
      case Stmt::Comment: break;
      case Stmt::For: block_accesses(s.body, out, whole_array_write, foreign_local_write, declared); break;
      case Stmt::ZeroOut: whole_array_write = true; break;
      case Stmt::Set:
        out.push_back({s.node, &s.idcs, true, 0});
        scalar_accesses(*s.value, out, foreign_local_write, declared);
        break;
      case Stmt::SetVec:
        out.push_back({s.node, &s.idcs, true, s.length});
        scalar_accesses(*s.value, out, foreign_local_write, declared);
        break;
      case Stmt::SetLocal:
        if (!declared.count(s.scope)) foreign_local_write = true;
        scalar_accesses(*s.value, out, foreign_local_write, declared);
        break;
      case Stmt::DeclareLocal: declared.insert(s.scope); break;
    }
  }
}

void scalar_accesses(const Scalar& s, std::vector<Access>& out, bool& flw, std::set<ScopeId>& declared) {
  switch (s.kind) {
    case Scalar::Get: case Scalar::GetMerge: out.push_back({s.node, &s.idcs, false, 0}); break;
    case Scalar::GetDyn:
      out.push_back({s.node, &s.idcs, false, 0});
      scalar_accesses(*s.a, out, flw, declared);
      break;
    case Scalar::LocalScope: {
      declared.insert(s.scope);
      bool whole = false;
      block_accesses(s.body, out, whole, flw, declared);
      break;
    }
    case Scalar::Un: scalar_accesses(*s.a, out, flw, declared); break;
    case Scalar::Bin: scalar_accesses(*s.a, out, flw, declared); scalar_accesses(*s.b, out, flw, declared); break;
    case Scalar::Tern:
      scalar_accesses(*s.a, out, flw, declared); scalar_accesses(*s.b, out, flw, declared);
      scalar_accesses(*s.c, out, flw, declared);
      break;
    default: break;
  }
}

// Axis at which `idcs` is driven by `sym` alone: Iterator sym, or a one-term Affine c*sym+o.
int axis_of(const Indices& idcs, int sym) {
  for (size_t p = 0; p < idcs.size(); ++p) {
    const AxisIndex& a = idcs[p];
    if (a.kind == AxisIndex::Iter && a.sym == sym) return (int)p;
    if (a.kind == AxisIndex::Affine)
      for (auto& t : a.terms) if (t.second == sym && t.first != 0) return (int)p;
  }
  return -1;
}

// A chain symbol is parallel when every array written below the chain is touched, in every access
// (reads included), through one and the same index expression driven by that symbol on one and the
// same axis: different values of the symbol then work on disjoint slices.
// A sum of loop symbols on one axis (`stride * o + k`, convolution-style) sends distinct tuples of
// symbol values to distinct positions only when the coefficients form a mixed radix over the extents:
// sorted by magnitude, each coefficient exceeds the reach of all smaller terms together.  Symbols
// without an extent (static indices) are constants here.
bool affine_is_injective(const AxisIndex& e, const std::map<int, int64_t>& ext, int64_t unit_run = 1) {
  std::vector<std::pair<int64_t, int64_t>> terms;   // (|coefficient|, extent)
  if (unit_run > 1) terms.push_back({1, unit_run});   // a vector access covers [e, e + unit_run)
  for (auto& t : e.terms) {
    auto it = ext.find(t.second);
    if (it == ext.end() || it->second <= 1) continue;
    if (t.first == 0) return false;
    terms.push_back({std::abs(t.first), it->second});
  }
  std::sort(terms.begin(), terms.end());
  int64_t reach = 0;   // largest offset the smaller terms can add up to
  for (auto& t : terms) {
    if (t.first <= reach) return false;
    reach += t.first * (t.second - 1);
  }
  return true;
}

bool symbol_is_parallel(int sym, const std::vector<Access>& acc, const std::map<int, int64_t>& ext) {
  std::set<int> written;
  for (auto& a : acc) if (a.write) written.insert(a.node);
  for (int w : written) {
    int axis = -1;
    const AxisIndex* expr = nullptr;
    for (auto& a : acc) {
      if (a.node != w) continue;
      int p = axis_of(*a.idcs, sym);
      if (p < 0) return false;
      const AxisIndex& e = (*a.idcs)[p];
      if (a.vec_len > 0 && p == (int)a.idcs->size() - 1) {
        // a vector write covers [e, e+len): needs a stride of at least len along sym
        if (!(e.kind == AxisIndex::Affine && affine_is_injective(e, ext, a.vec_len))) return false;
      }
      // the symbol must not also appear on another axis of this access
      for (size_t q = 0; q < a.idcs->size(); ++q)
        if ((int)q != p && (*a.idcs)[q].mentions(sym)) return false;
      // threads of different symbols sharing the axis must not meet on one element
      if (a.write && e.kind == AxisIndex::Affine && !affine_is_injective(e, ext)) return false;
      if (axis < 0) { axis = p; expr = &e; }
      else if (axis != p || !(*expr == e)) return false;
    }
  }
  return true;
}

bool same_indices(const Indices& a, const Indices& b) { return a == b; }

int64_t row_major_stride(const Node& n, size_t axis) {
  int64_t s = 1;
  for (size_t q = axis + 1; q < n.dims.size(); ++q) s *= n.dims[q];
  return s;
}

struct Strides {
  std::map<int, int64_t> by_sym;
  int64_t offset = 0;
  std::vector<std::pair<int, int64_t>> statics;
  bool ok = true;
};

Strides strides_of(const Routine& r, int node, const Indices& idcs) {
  Strides st;
  const Node& n = r.node(node);
  for (size_t p = 0; p < idcs.size(); ++p) {
    const int64_t rs = row_major_stride(n, p);
    const AxisIndex& a = idcs[p];
    if (a.kind == AxisIndex::Fixed) st.offset += a.fixed * rs;
    else if (a.kind == AxisIndex::Iter) {
      if (r.is_static(a.sym)) st.statics.emplace_back(a.sym, rs);
      else st.by_sym[a.sym] += rs;
    } else {
      for (auto& t : a.terms) {
        if (r.is_static(t.second)) st.statics.emplace_back(t.second, t.first * rs);
        else st.by_sym[t.second] += t.first * rs;
      }
      st.offset += a.offset * rs;
    }
  }
  return st;
}

int64_t get_stride(const Strides& s, int sym) {
  auto it = s.by_sym.find(sym);
  return it == s.by_sym.end() ? 0 : it->second;
}

bool mfma_prec(Prec p) { return p == Prec::Single || p == Prec::Bfloat16; }

// Recognises `for.. { c[L] := fma(a[A], b[B], c[L]) }` (either operand order; also
// `(a*b) + c`), fills a strided-batched GEMM descriptor.  Returns false to leave the phase generic.
bool match_contraction(const Routine& r, Phase& ph, const PlanOptions& opt) {
  if (!opt.enable_mfma) return false;
  if (ph.inner.size() != 1 || ph.inner[0]->kind != Stmt::Set) return false;
  const Stmt& set = *ph.inner[0];
  const Scalar& v = *set.value;
  const Scalar *pa = nullptr, *pb = nullptr, *pc = nullptr;
  if (v.kind == Scalar::Tern && v.tern == Ternop::Fma) { pa = v.a.get(); pb = v.b.get(); pc = v.c.get(); }
  else if (v.kind == Scalar::Bin && v.bin == Binop::Add) {
    const Scalar* l = v.a.get(); const Scalar* rr = v.b.get();
    if (rr->kind == Scalar::Bin && rr->bin == Binop::Mul) { pc = l; pa = rr->a.get(); pb = rr->b.get(); }
    else if (l->kind == Scalar::Bin && l->bin == Binop::Mul) { pc = rr; pa = l->a.get(); pb = l->b.get(); }
    else return false;
  } else return false;
  if (pa->kind != Scalar::Get || pb->kind != Scalar::Get || pc->kind != Scalar::Get) return false;
  if (pc->node != set.node || !same_indices(pc->idcs, set.idcs)) return false;
  if (pa->node == set.node || pb->node == set.node) return false;
  const Node &na = r.node(pa->node), &nb = r.node(pb->node), &nc = r.node(set.node);
  if (!mfma_prec(na.prec) || !mfma_prec(nb.prec) || !mfma_prec(nc.prec)) return false;

  Strides sa = strides_of(r, pa->node, pa->idcs), sb = strides_of(r, pb->node, pb->idcs),
          sc = strides_of(r, set.node, set.idcs);

  struct Sym { int sym; int64_t ext, a, b, c; };
  std::vector<Sym> batch, ms, ns, ks;
  auto add_chain = [&](int sym, int64_t from, int64_t ext) -> bool {
    if (from != 0) return false;
    if (ext == 1) return true;  // degenerate loops contribute nothing
    Sym s{sym, ext, get_stride(sa, sym), get_stride(sb, sym), get_stride(sc, sym)};
    if (s.a < 0 || s.b < 0 || s.c < 0) return false;
    const bool ia = s.a != 0, ib = s.b != 0, ic = s.c != 0;
    if (ic && ia && ib) batch.push_back(s);
    else if (ic && ia) ms.push_back(s);
    else if (ic && ib) ns.push_back(s);
    else if (ia && ib) ks.push_back(s);
    else return false;
    return true;
  };
  for (size_t i = 0; i < ph.par_syms.size(); ++i)
    if (!add_chain(ph.par_syms[i], ph.par_from[i], ph.par_ext[i])) return false;
  for (size_t i = 0; i < ph.seq_syms.size(); ++i)
    if (!add_chain(ph.seq_syms[i], ph.seq_from[i], ph.seq_to[i] - ph.seq_from[i] + 1)) return false;

  // merge symbols of one class that are contiguous in all three tensors
  auto merge = [&](std::vector<Sym>& v, bool by_a) {
    std::sort(v.begin(), v.end(), [&](const Sym& x, const Sym& y) {
      return by_a ? x.a > y.a : x.c > y.c; });
    for (size_t i = 0; i + 1 < v.size();) {
      Sym &o = v[i], &in = v[i + 1];
      if (o.a == in.ext * in.a && o.b == in.ext * in.b && o.c == in.ext * in.c) {
        in.ext *= o.ext;
        v.erase(v.begin() + i);
      } else ++i;
    }
  };
  merge(batch, false); merge(ms, false); merge(ns, false); merge(ks, true);
  // surplus M / N symbols become batch dimensions (the other operand is re-read: stride 0)
  while (ms.size() > 1) { batch.push_back(ms.front()); ms.erase(ms.begin()); }
  while (ns.size() > 1) { batch.push_back(ns.front()); ns.erase(ns.begin()); }
  if (ks.size() > 1 || batch.size() > 3) return false;
  // The kernels store (or read-add-write) every (batch, m, n) cell from its own lane with no atomics:
  // distinct cells must be distinct elements of C.  An accumulation through overlapping windows
  // (the input gradient of a convolution: x_grad[stride * o + k] with stride < window) is not that,
  // and stays a generated kernel, which has the same one-to-one test per axis.
  {
    std::vector<std::pair<int64_t, int64_t>> cells;   // (C stride, extent)
    for (auto* v : {&batch, &ms, &ns}) for (auto& s : *v) cells.push_back({s.c, s.ext});
    std::sort(cells.begin(), cells.end());
    int64_t reach = 0;
    for (auto& c : cells) {
      if (c.first <= reach) return false;
      reach += c.first * (c.second - 1);
    }
  }

  GemmDesc g;
  g.M = ms.empty() ? 1 : ms[0].ext;
  g.N = ns.empty() ? 1 : ns[0].ext;
  g.K = ks.empty() ? 1 : ks[0].ext;
  g.a.node = pa->node; g.a.prec = na.prec; g.a.offset = sa.offset; g.a.static_terms = sa.statics;
  g.b.node = pb->node; g.b.prec = nb.prec; g.b.offset = sb.offset; g.b.static_terms = sb.statics;
  g.c.node = set.node; g.c.prec = nc.prec; g.c.offset = sc.offset; g.c.static_terms = sc.statics;
  g.a.s_row = ms.empty() ? 0 : ms[0].a;  g.a.s_k = ks.empty() ? 0 : ks[0].a;
  g.b.s_row = ns.empty() ? 0 : ns[0].b;  g.b.s_k = ks.empty() ? 0 : ks[0].b;
  g.c.s_row = ms.empty() ? 0 : ms[0].c;  g.c.s_k = ns.empty() ? 0 : ns[0].c;
  g.nbatch = (int)batch.size();
  for (int i = 0; i < g.nbatch; ++i) {
    g.batch_ext[i] = batch[i].ext;
    g.a.s_batch[i] = batch[i].a; g.b.s_batch[i] = batch[i].b; g.c.s_batch[i] = batch[i].c;
  }
  if (g.flops() < (double)opt.min_mfma_flops) return false;
  if (g.M < 16 || g.N < 16 || g.K < 8) return false;   // matrix-vector shapes stay generic
  {
    int64_t nb = 1;   // the batch is the launch grid's z extent
    for (int i = 0; i < g.nbatch; ++i) nb *= g.batch_ext[i];
    if (nb > 65535) return false;
  }

  // C must be contiguous along N; if it is contiguous along M instead, compute the transpose.
  if (g.c.s_k != 1) {
    if (g.c.s_row != 1) return false;
    std::swap(g.a, g.b);
    std::swap(g.M, g.N);
    std::swap(g.c.s_row, g.c.s_k);
  }
  // each operand: unit stride along K or along its row dimension; vector-load alignment
  const bool f32_compute = g.a.prec == Prec::Single && g.b.prec == Prec::Single;
  auto operand_ok = [&](const GemmOperand& o, int64_t rows) {
    // staging moves 8-element (bf16 compute) or 4-element (fp32 compute) chunks
    const int vec = f32_compute ? 4 : 8;
    if (o.s_k != 1 && o.s_row != 1) return false;
    const int64_t ld = o.s_k == 1 ? o.s_row : o.s_k;
    if (rows > 1 && g.K > 1 && ld % vec) return false;
    if (o.offset % vec) return false;
    for (auto& t : o.static_terms) if (t.second % vec) return false;
    for (int i = 0; i < g.nbatch; ++i) if (o.s_batch[i] % vec) return false;
    const int64_t contig = o.s_k == 1 ? g.K : rows;
    if (contig % vec) return false;
    return true;
  };
  if (!operand_ok(g.a, g.M) || !operand_ok(g.b, g.N)) return false;
  {
    const int vec = 4;
    if (g.c.s_row % vec || g.c.offset % vec || g.N % vec) return false;
    for (auto& t : g.c.static_terms) if (t.second % vec) return false;
    for (int i = 0; i < g.nbatch; ++i) if (g.c.s_batch[i] % vec) return false;
  }
  g.accumulate = !ph.fused_zero_init;
  ph.kind = Phase::Contraction;
  ph.gemm = g;
  ph.flops = g.flops();
  return true;
}

// Is the phase `lhs[L] := accum(lhs[L], e)` / `fma(a, b, lhs[L])` with an associative, commutative
// accum and `e` free of lhs?  Then sequential chain loops may be split across lanes.
bool reduction_shape(const Routine& r, const Phase& ph, Binop* accum_out) {
  if (ph.inner.size() != 1 || ph.inner[0]->kind != Stmt::Set) return false;
  const Stmt& set = *ph.inner[0];
  const Scalar& v = *set.value;
  // the accumulated element must be the same through all sequential loops
  for (auto& ix : set.idcs) for (int q : ph.seq_syms) if (ix.mentions(q)) return false;
  auto is_self = [&](const Scalar& s) {
    return s.kind == Scalar::Get && s.node == set.node && same_indices(s.idcs, set.idcs); };
  std::function<bool(const Scalar&)> reads_lhs = [&](const Scalar& s) -> bool {
    switch (s.kind) {
      case Scalar::Get: case Scalar::GetMerge: return s.node == set.node;
      case Scalar::GetDyn: return s.node == set.node || reads_lhs(*s.a);
      case Scalar::LocalScope: {
        std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
        block_accesses(s.body, acc, w, f, d);
        for (auto& a : acc) if (a.node == set.node) return true;
        return false;
      }
      case Scalar::Un: return reads_lhs(*s.a);
      case Scalar::Bin: return reads_lhs(*s.a) || reads_lhs(*s.b);
      case Scalar::Tern: return reads_lhs(*s.a) || reads_lhs(*s.b) || reads_lhs(*s.c);
      default: return false;
    }
  };
  if (v.kind == Scalar::Tern && v.tern == Ternop::Fma) {
    if (!is_self(*v.c) || reads_lhs(*v.a) || reads_lhs(*v.b)) return false;
    *accum_out = Binop::Add;
    return true;
  }
  if (v.kind == Scalar::Bin && (v.bin == Binop::Add || v.bin == Binop::Max || v.bin == Binop::Min)) {
    if (is_self(*v.a) && !reads_lhs(*v.b)) { *accum_out = v.bin; return true; }
    if (is_self(*v.b) && !reads_lhs(*v.a)) { *accum_out = v.bin; return true; }
  }
  (void)r;
  return false;
}

// The inlined scalar reduction form `v { v := const; for k1.. for kn { v := accum(v, e) } }`
// (low_level.ml:1165-1316) with e free of v.  Fills the reduction loops (outer first) and the update.
bool scope_reduction(const Scalar& ls, std::vector<const Stmt*>& loops, const Stmt*& init, const Stmt*& upd,
                     Binop* accum) {
  if (ls.kind != Scalar::LocalScope) return false;
  Block body = strip_comments(ls.body, nullptr);
  if (body.size() != 2 || body[0]->kind != Stmt::SetLocal || !(body[0]->scope == ls.scope)) return false;
  if (body[0]->value->kind != Scalar::Const || body[1]->kind != Stmt::For) return false;
  init = body[0].get();
  const Stmt* cur = body[1].get();
  upd = nullptr;
  for (;;) {
    loops.push_back(cur);
    Block b2 = strip_comments(cur->body, nullptr);
    if (b2.size() != 1) return false;
    if (b2[0]->kind == Stmt::For) { cur = b2[0].get(); continue; }
    if (b2[0]->kind == Stmt::SetLocal && b2[0]->scope == ls.scope) upd = b2[0].get();
    break;
  }
  if (!upd) return false;
  std::function<bool(const Scalar&)> mentions = [&](const Scalar& s) -> bool {
    if (s.kind == Scalar::GetLocal) return s.scope == ls.scope;
    if (s.kind == Scalar::LocalScope) return true;   // nested scopes: leave alone
    return (s.a && mentions(*s.a)) || (s.b && mentions(*s.b)) || (s.c && mentions(*s.c));
  };
  auto is_v = [&](const Scalar& s) { return s.kind == Scalar::GetLocal && s.scope == ls.scope; };
  const Scalar& v = *upd->value;
  if (v.kind == Scalar::Tern && v.tern == Ternop::Fma && is_v(*v.c) && !mentions(*v.a) && !mentions(*v.b)) {
    *accum = Binop::Add;
  } else if (v.kind == Scalar::Bin && (v.bin == Binop::Add || v.bin == Binop::Max || v.bin == Binop::Min) &&
             ((is_v(*v.a) && !mentions(*v.b)) || (is_v(*v.b) && !mentions(*v.a)))) {
    *accum = v.bin;
  } else return false;
  const double c0 = init->value->cst;
  if (*accum == Binop::Add && c0 != 0.0) return false;
  if (*accum == Binop::Max && !(std::isinf(c0) && c0 < 0)) return false;
  if (*accum == Binop::Min && !(std::isinf(c0) && c0 > 0)) return false;
  for (const Stmt* l : loops) if (l->to < l->from) return false;
  return true;
}

// A pointwise statement whose value holds one inlined scalar reduction: lanes may share it.
void choose_scope_coop(const Routine& r, Phase& ph) {
  if (ph.inner.size() != 1 || ph.inner[0]->kind != Stmt::Set) return;
  std::vector<const Scalar*> found;
  std::function<void(const Scalar&)> walk = [&](const Scalar& s) {
    if (s.kind == Scalar::LocalScope) { found.push_back(&s); return; }
    if (s.a) walk(*s.a);
    if (s.b) walk(*s.b);
    if (s.c) walk(*s.c);
  };
  walk(*ph.inner[0]->value);
  if (found.size() != 1) return;
  std::vector<const Stmt*> loops; const Stmt* init = nullptr; const Stmt* upd = nullptr; Binop accum;
  if (!scope_reduction(*found[0], loops, init, upd, &accum)) return;
  const Prec p = r.node(found[0]->scope.node).prec;
  if (!(p == Prec::Single || p == Prec::Double || p == Prec::Bfloat16 || p == Prec::Half)) return;
  int64_t P = 1, R = 1;
  for (auto e : ph.par_ext) P *= e;
  for (const Stmt* l : loops) R *= l->to - l->from + 1;
  const int64_t rext = loops.back()->to - loops.back()->from + 1;
  // one thread per point walks its own row: adjacent threads are a whole row apart, so sharing
  // the row between adjacent lanes is what makes the reads coalesce
  std::vector<Access> acc; bool f = false; std::set<ScopeId> d;
  scalar_accesses(*upd->value, acc, f, d);
  bool unit = false;
  for (auto& a : acc) if (get_stride(strides_of(r, a.node, *a.idcs), loops.back()->sym) == 1) unit = true;
  auto pow2_floor = [](int64_t x) { int64_t p2 = 1; while (p2 * 2 <= x) p2 *= 2; return p2; };
  int lanes = 1;
  if (unit && rext >= 16) lanes = (int)std::min<int64_t>(64, pow2_floor(rext));
  else if (P < 16384 && R >= 256 && rext >= 2) lanes = (int)std::min<int64_t>(64, pow2_floor(rext));
  // a handful of long reductions (a loss summed over all tokens): a whole workgroup each
  if (lanes == 64 && P <= 16 && rext >= 256 && R >= 2048) lanes = 256;
  if (lanes > 1) { ph.coop_lanes = lanes; ph.coop_scope = found[0]; ph.coop_accum = accum; }
}

// Does the innermost sequential symbol walk one of the phase's big operands with unit stride?  Only
// the operands that every other one is small against count: a per-row scalar inlined into the
// addend (the mean and deviation of a layer norm) is contiguous along the rows and says nothing
// about how the tensors that carry the traffic lie.
static bool reduction_walks_unit_stride(const Routine& r, const Phase& ph, const Stmt& set) {
  std::map<int, int64_t> ext;
  for (size_t i = 0; i < ph.par_syms.size(); ++i) ext[ph.par_syms[i]] = ph.par_ext[i];
  for (size_t i = 0; i < ph.seq_syms.size(); ++i) ext[ph.seq_syms[i]] = ph.seq_to[i] - ph.seq_from[i] + 1;
  std::vector<Access> acc; bool f = false; std::set<ScopeId> d;
  scalar_accesses(*set.value, acc, f, d);
  std::vector<int64_t> foot(acc.size(), 0);
  int64_t biggest = 0;
  for (size_t i = 0; i < acc.size(); ++i) {
    if (acc[i].node == set.node) continue;
    int64_t n = 1;
    for (auto& kv : ext) {
      bool m = false;
      for (auto& ix : *acc[i].idcs) m = m || ix.mentions(kv.first);
      if (m) n *= kv.second;
    }
    foot[i] = n;
    biggest = std::max(biggest, n);
  }
  for (size_t i = 0; i < acc.size(); ++i) {
    if (acc[i].node == set.node || foot[i] * 16 < biggest) continue;
    if (get_stride(strides_of(r, acc[i].node, *acc[i].idcs), ph.seq_syms.back()) == 1) return true;
  }
  return false;
}

void choose_coop(const Routine& r, Phase& ph, const PlanOptions& opt) {
  ph.coop_lanes = 1;
  if (!opt.enable_coop) return;
  if (ph.seq_syms.empty()) { choose_scope_coop(r, ph); return; }
  Binop accum;
  if (!reduction_shape(r, ph, &accum)) return;
  const Stmt& set = *ph.inner[0];
  const Prec p = r.node(set.node).prec;
  if (!(p == Prec::Single || p == Prec::Double || p == Prec::Bfloat16 || p == Prec::Half)) return;
  const int64_t rext = ph.seq_to.back() - ph.seq_from.back() + 1;
  int64_t P = 1, R = 1;
  for (auto e : ph.par_ext) P *= e;
  for (size_t i = 0; i < ph.seq_syms.size(); ++i) R *= ph.seq_to[i] - ph.seq_from[i] + 1;
  auto pow2_floor = [](int64_t x) { int64_t p2 = 1; while (p2 * 2 <= x) p2 *= 2; return p2; };
  if (ph.sums_partials) {
    // One thread per output would walk all the slices alone: a few thousand threads, each waiting on
    // a long run of loads, and the launch lasts as long as that wait.  Lanes that share an output take
    // slices next to one another, so one load of a wavefront stays inside lanes x (one slice) of
    // memory and adjacent outputs fill the sectors it touches; 8 to 32 lanes, for at most about 16
    // loads per lane where that is enough.
    if (R >= 16) {
      int64_t lanes = 8;
      while (lanes < 32 && R / lanes > 16) lanes *= 2;
      ph.coop_lanes = (int)std::min<int64_t>(lanes, pow2_floor(rext));
    }
    return;
  }
  const bool unit = reduction_walks_unit_stride(r, ph, set);
  if (unit && rext >= 16) ph.coop_lanes = (int)std::min<int64_t>(64, pow2_floor(rext));
  else if (P < 16384 && R >= 256 && rext >= 2) ph.coop_lanes = (int)std::min<int64_t>(64, pow2_floor(rext));
  if (ph.coop_lanes == 64 && P <= 16 && rext >= 256 && R >= 2048) ph.coop_lanes = 256;
}

// Algorithmic bytes of a generic phase: every distinct (node, index tuple) read once, every
// written element once; extents taken from the chain loops (inner loops count for reads).
void account_bytes(const Routine& r, Phase& ph) {
  std::map<int, int64_t> ext;
  for (size_t i = 0; i < ph.par_syms.size(); ++i) ext[ph.par_syms[i]] = ph.par_ext[i];
  for (size_t i = 0; i < ph.seq_syms.size(); ++i) ext[ph.seq_syms[i]] = ph.seq_to[i] - ph.seq_from[i] + 1;
  std::function<void(const Block&)> inner_loops = [&](const Block& b) {
    for (auto& s : b) {
      if (s->kind == Stmt::For) { ext[s->sym] = s->to - s->from + 1; inner_loops(s->body); }
      std::function<void(const Scalar&)> sc = [&](const Scalar& x) {
        if (x.kind == Scalar::LocalScope) inner_loops(x.body);
        if (x.a) sc(*x.a); if (x.b) sc(*x.b); if (x.c) sc(*x.c);
      };
      if (s->value) sc(*s->value);
    }
  };
  inner_loops(ph.inner);
  std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
  block_accesses(ph.inner, acc, w, f, d);
  std::set<std::pair<int, std::string>> seen;
  double bytes = 0;
  // an accumulation whose zero fill was folded in starts from zero: its target is not read
  const int unread = ph.fused_zero_init && ph.inner.size() == 1 && ph.inner[0]->kind == Stmt::Set ? ph.inner[0]->node : -1;
  for (auto& a : acc) {
    if (!a.write && a.node == unread) continue;
    std::set<int> syms;
    std::string key = a.write ? "w" : "r";
    for (auto& ix : *a.idcs) {
      if (ix.kind == AxisIndex::Iter) { syms.insert(ix.sym); key += "i" + std::to_string(ix.sym); }
      else if (ix.kind == AxisIndex::Affine) { for (auto& t : ix.terms) { syms.insert(t.second); key += "a" + std::to_string(t.second); } }
      else key += "f" + std::to_string(ix.fixed);
      key += ",";
    }
    if (!seen.insert({a.node, key}).second) continue;
    double n = 1;
    for (int s : syms) { auto it = ext.find(s); if (it != ext.end()) n *= (double)it->second; }
    const Node& nd = r.node(a.node);
    n = std::min(n, (double)nd.num_elems());
    if (a.vec_len > 0) n *= a.vec_len;
    bytes += n * prec_in_bytes(nd.prec);
  }
  ph.bytes = bytes;
}

// Does the phase read or write `node`?
bool phase_touches(const Phase& ph, int node) {
  if (ph.kind == Phase::Fill) return ph.fill_node == node;
  if (ph.kind == Phase::Contraction) {
    for (auto& m : ph.gemm.group) if (m.a.node == node || m.b.node == node || m.c.node == node || m.c_copy == node) return true;
    if (ph.gemm.c_copy == node || ph.gemm.epi_bias == node || ph.gemm.epi_relu == node) return true;
    for (auto& pr : ph.gemm.more) if (pr.first.node == node || pr.second.node == node) return true;
    return ph.gemm.a.node == node || ph.gemm.b.node == node || ph.gemm.c.node == node;
  }
  if (!ph.parallel_members.empty()) { for (auto& m : ph.parallel_members) if (phase_touches(m, node)) return true; return false; }
  if (ph.fused_x >= 0 && (ph.fused_x == node || ph.fused_a.node == node || ph.fused_b.node == node)) return true;
  if (ph.proj_y >= 0 && (ph.proj_b.node == node || ph.proj_c.node == node || ph.proj_c_copy == node)) return true;
  if (!ph.members.empty()) { for (auto& m : ph.members) if (phase_touches(m, node)) return true; return false; }
  if (!ph.serial_members.empty()) { for (auto& m : ph.serial_members) if (phase_touches(m, node)) return true; return false; }
  std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
  block_accesses(ph.inner, acc, w, f, d);
  if (w) return true;   // a Zero_out inside the nest: not tracked per node, assume the worst
  for (auto& a : acc) if (a.node == node) return true;
  return false;
}

Block strip_comments(const Block& b, std::string* last_comment) {
  Block out;
  for (auto& s : b) {
    if (s->kind == Stmt::Comment) { if (last_comment) *last_comment = s->text; }
    else out.push_back(s);
  }
  return out;
}

}  // namespace

// debug logging: every loop of a statement stays inside one thread, in program order
static thread_local bool g_all_sequential = false;

// Chain/inner split and parallel classification of one top-level statement.
// Returns false when the statement runs nothing (a zero-trip loop).
static bool analyze_nest(const Routine& r, const StmtP& sp, Phase& ph) {
  (void)r;
  std::vector<const Stmt*> chain;
  Block inner;
  if (sp->kind == Stmt::For) {
    const Stmt* cur = sp.get();
    for (;;) {
      chain.push_back(cur);
      Block body = strip_comments(cur->body, nullptr);
      if (body.size() == 1 && body[0]->kind == Stmt::For) { cur = body[0].get(); continue; }
      inner = body;
      break;
    }
  } else {
    inner = {sp};
  }
  for (const Stmt* l : chain)
    if (l->to - l->from + 1 <= 0) return false;
  std::vector<Access> acc;
  bool whole = false, foreign = false;
  std::set<ScopeId> declared;
  block_accesses(inner, acc, whole, foreign, declared);
  std::map<int, int64_t> extents;   // of every loop symbol in the nest
  for (const Stmt* l : chain) extents[l->sym] = l->to - l->from + 1;
  std::function<void(const Block&)> inner_loops = [&](const Block& b) {
    for (auto& s : b) {
      // (sibling loops may share a symbol, low_level.ml:2741-2775: keep the longer range)
      if (s->kind == Stmt::For) { extents[s->sym] = std::max(extents[s->sym], s->to - s->from + 1); inner_loops(s->body); }
      std::function<void(const Scalar&)> sc = [&](const Scalar& x) {
        if (x.kind == Scalar::LocalScope) inner_loops(x.body);
        if (x.a) sc(*x.a); if (x.b) sc(*x.b); if (x.c) sc(*x.c);
      };
      if (s->value) sc(*s->value);
    }
  };
  inner_loops(inner);
  for (const Stmt* l : chain) {
    const int64_t ext = l->to - l->from + 1;
    const bool par = !g_all_sequential && !whole && !foreign && symbol_is_parallel(l->sym, acc, extents);
    if (par) { ph.par_syms.push_back(l->sym); ph.par_from.push_back(l->from); ph.par_ext.push_back(ext); }
    else { ph.seq_syms.push_back(l->sym); ph.seq_from.push_back(l->from); ph.seq_to.push_back(l->to); }
  }
  ph.inner = inner;
  return true;
}

static void set_contraction_bytes(Phase& ph) {
  const GemmDesc& g = ph.gemm;
  auto op_bytes = [&](const GemmOperand& o, double rows, double cols) {
    double n = rows * cols;
    for (int i = 0; i < g.nbatch; ++i) if (o.s_batch[i]) n *= (double)g.batch_ext[i];
    return n * prec_in_bytes(o.prec);
  };
  ph.bytes = op_bytes(g.a, (double)g.M, (double)g.K) + op_bytes(g.b, (double)g.N, (double)g.K) +
             op_bytes(g.c, (double)g.M, (double)g.N) * (g.accumulate ? 2 : 1);
  if (g.c_copy >= 0) ph.bytes += op_bytes(g.c, (double)g.M, (double)g.N) / prec_in_bytes(g.c.prec) * 2.0;
}

// De-virtualisation.  The optimiser inlines a contraction that is read once into its consumer as
//   v { v := 0; for k.. { v := fma(a[..], b[..], v) } }
// (arrayjit/lib/low_level.ml:1165-1316; test/einsum/inline_permuted_view-c_fwd.ll.expected).  When
// such a reduction is large enough for the MFMA kernels it is given a scratch tensor indexed by the
// enclosing loop symbols it depends on, computed by a contraction phase of its own, and the
// consumer reads the scratch element instead.
static void devirtualise(Routine& r, const StmtP& sp, const PlanOptions& opt, Plan& plan, const std::string& label) {
  if (!opt.enable_mfma) return;
  // enclosing perfect chain
  std::vector<const Stmt*> chain;
  Block inner;
  if (sp->kind == Stmt::For) {
    const Stmt* cur = sp.get();
    for (;;) {
      chain.push_back(cur);
      Block body = strip_comments(cur->body, nullptr);
      if (body.size() == 1 && body[0]->kind == Stmt::For) { cur = body[0].get(); continue; }
      inner = body;
      break;
    }
  } else inner = {sp};
  if (inner.size() != 1 || inner[0]->kind != Stmt::Set) return;
  for (const Stmt* l : chain) if (l->from != 0 || l->to < l->from) return;

  std::vector<Scalar*> found;
  std::function<void(Scalar&)> walk = [&](Scalar& s) {
    if (s.kind == Scalar::LocalScope) { found.push_back(&s); return; }
    if (s.a) walk(*s.a);
    if (s.b) walk(*s.b);
    if (s.c) walk(*s.c);
  };
  walk(*inner[0]->value);
  for (Scalar* ls : found) {
    Block body = strip_comments(ls->body, nullptr);
    if (body.size() != 2 || body[0]->kind != Stmt::SetLocal || !(body[0]->scope == ls->scope)) continue;
    if (body[0]->value->kind != Scalar::Const || body[0]->value->cst != 0.0) continue;
    if (body[1]->kind != Stmt::For) continue;
    std::vector<const Stmt*> red;
    const Stmt* cur = body[1].get();
    const Stmt* upd = nullptr;
    for (;;) {
      red.push_back(cur);
      Block b2 = strip_comments(cur->body, nullptr);
      if (b2.size() != 1) break;
      if (b2[0]->kind == Stmt::For) { cur = b2[0].get(); continue; }
      if (b2[0]->kind == Stmt::SetLocal && b2[0]->scope == ls->scope) upd = b2[0].get();
      break;
    }
    if (!upd) continue;
    const Scalar& v = *upd->value;
    if (!(v.kind == Scalar::Tern && v.tern == Ternop::Fma && v.c->kind == Scalar::GetLocal && v.c->scope == ls->scope)) continue;
    if (v.a->kind != Scalar::Get || v.b->kind != Scalar::Get) continue;
    // enclosing symbols the operands depend on
    std::vector<const Stmt*> dep;
    double flops = 2.0;
    for (const Stmt* l : chain) {
      bool used = false;
      for (auto& ix : v.a->idcs) used |= ix.mentions(l->sym);
      for (auto& ix : v.b->idcs) used |= ix.mentions(l->sym);
      if (used) { dep.push_back(l); flops *= (double)(l->to + 1); }
    }
    bool ok = true;
    for (const Stmt* l : red) { if (l->from != 0 || l->to < 0) ok = false; flops *= (double)(l->to - l->from + 1); }
    if (!ok || flops < (double)opt.min_mfma_flops) continue;

    // scratch node + candidate nest
    int new_id = 1;
    for (auto& kv : r.nodes) new_id = std::max(new_id, kv.first + 1);
    Node t;
    t.id = new_id;
    t.ident = "ctr" + std::to_string(new_id) + "_" + r.node(ls->scope.node).ident;
    // a bf16 scalar is rounded by the serial code after every step; the scratch tensor keeps that
    // precision (rounded once, from the fp32 accumulator) and half the traffic
    t.prec = r.node(ls->scope.node).prec == Prec::Bfloat16 ? Prec::Bfloat16 : Prec::Single;
    t.mode = Mode::Local;
    for (const Stmt* l : dep) t.dims.push_back(l->to + 1);
    if (t.dims.empty()) t.dims.push_back(1);
    Indices tix;
    for (const Stmt* l : dep) { AxisIndex a; a.kind = AxisIndex::Iter; a.sym = l->sym; tix.push_back(a); }
    if (dep.empty()) { AxisIndex a; a.kind = AxisIndex::Fixed; a.fixed = 0; tix.push_back(a); }

    auto self = std::make_shared<Scalar>();
    self->kind = Scalar::Get; self->node = t.id; self->idcs = tix;
    auto fma = std::make_shared<Scalar>();
    fma->kind = Scalar::Tern; fma->tern = Ternop::Fma; fma->arg_prec = v.arg_prec;
    fma->a = v.a; fma->b = v.b; fma->c = self;
    auto set = std::make_shared<Stmt>();
    set->kind = Stmt::Set; set->node = t.id; set->idcs = tix; set->value = fma;
    StmtP nest = set;
    auto wrap = [&](const Stmt* l) {
      auto f = std::make_shared<Stmt>();
      f->kind = Stmt::For; f->sym = l->sym; f->from = l->from; f->to = l->to; f->body = {nest};
      nest = f;
    };
    for (auto it = red.rbegin(); it != red.rend(); ++it) wrap(*it);
    for (auto it = dep.rbegin(); it != dep.rend(); ++it) wrap(*it);

    r.nodes.emplace(t.id, t);
    Phase ph;
    ph.label = label + " (contraction of " + r.node(ls->scope.node).ident + ")";
    ph.stmt = nest;
    ph.fused_zero_init = true;
    if (!analyze_nest(r, nest, ph) || !match_contraction(r, ph, opt)) { r.nodes.erase(t.id); continue; }
    set_contraction_bytes(ph);
    plan.phases.push_back(std::move(ph));
    plan.scratch.push_back(t);
    // the consumer now reads the scratch element
    Scalar repl;
    repl.kind = Scalar::Get; repl.node = t.id; repl.idcs = tix;
    *ls = repl;
  }
}

// ---- split reductions ---------------------------------------------------------------------------
// `out[p] := out[p] + e(p, k1..kn)` where the output is small and the reduction runs over the slow
// axes of its operands (bias / gain gradients: a column sum over all rows).  One thread per output
// would leave most of the chip idle, and lanes sharing a column read a whole row apart.  Instead
// the outer part of the reduction range becomes parallel: phase 1 sums slice s into a scratch
// tensor partial[s, p] (threads adjacent along p: coalesced), phase 2 adds the slices to `out` in
// index order (deterministic).

static int fresh_symbol(const Routine& r, int* next) {
  if (*next == 0) {
    int mx = 0;
    std::function<void(const Block&)> scan = [&](const Block& b) {
      for (auto& s : b) {
        if (s->kind == Stmt::For) { mx = std::max(mx, s->sym); scan(s->body); }
        std::function<void(const Scalar&)> sc = [&](const Scalar& x) {
          if (x.kind == Scalar::LocalScope) scan(x.body);
          if (x.a) sc(*x.a); if (x.b) sc(*x.b); if (x.c) sc(*x.c);
        };
        if (s->value) sc(*s->value);
      }
    };
    scan(r.body);
    for (auto& st : r.statics) mx = std::max(mx, st.sym);
    *next = mx + 1;
  }
  return (*next)++;
}

// index with `sym` replaced by from + len * hi + lo
static AxisIndex subst_index(const AxisIndex& a, int sym, int64_t from, int64_t len, int hi, int lo) {
  if (!a.mentions(sym)) return a;
  AxisIndex o;
  o.kind = AxisIndex::Affine;
  if (a.kind == AxisIndex::Iter) {
    o.terms = {{len, hi}, {1, lo}};
    o.offset = from;
  } else {
    o.offset = a.offset;
    for (auto& t : a.terms) {
      if (t.second != sym) { o.terms.push_back(t); continue; }
      o.terms.push_back({t.first * len, hi});
      o.terms.push_back({t.first, lo});
      o.offset += t.first * from;
    }
  }
  return o;
}

static ScalarP subst_scalar(const ScalarP& sp, int sym, int64_t from, int64_t len, int hi, int lo, bool* ok);

// statements of a scope body with `sym` rewritten; a loop that rebinds `sym` cannot be handled
static Block subst_block(const Block& b, int sym, int64_t from, int64_t len, int hi, int lo, bool* ok) {
  Block out;
  for (auto& s : b) {
    auto o = std::make_shared<Stmt>(*s);
    if (s->kind == Stmt::For && s->sym == sym) *ok = false;
    for (auto& ix : o->idcs) ix = subst_index(ix, sym, from, len, hi, lo);
    o->value = subst_scalar(s->value, sym, from, len, hi, lo, ok);
    o->body = subst_block(s->body, sym, from, len, hi, lo, ok);
    out.push_back(o);
  }
  return out;
}

static ScalarP subst_scalar(const ScalarP& sp, int sym, int64_t from, int64_t len, int hi, int lo, bool* ok) {
  if (!sp) return sp;
  auto o = std::make_shared<Scalar>(*sp);
  if (sp->kind == Scalar::LocalScope) o->body = subst_block(sp->body, sym, from, len, hi, lo, ok);
  for (auto& ix : o->idcs) ix = subst_index(ix, sym, from, len, hi, lo);
  if (o->kind == Scalar::Index) o->index = subst_index(o->index, sym, from, len, hi, lo);
  o->a = subst_scalar(sp->a, sym, from, len, hi, lo, ok);
  o->b = subst_scalar(sp->b, sym, from, len, hi, lo, ok);
  o->c = subst_scalar(sp->c, sym, from, len, hi, lo, ok);
  return o;
}

static StmtP make_for(int sym, int64_t from, int64_t to, StmtP body) {
  auto f = std::make_shared<Stmt>();
  f->kind = Stmt::For; f->sym = sym; f->from = from; f->to = to; f->body = {std::move(body)};
  return f;
}

// On success pushes phase 1 onto the plan and rewrites `ph` into phase 2.
static bool split_reduction(Routine& r, Phase& ph, const PlanOptions& opt, Plan& plan, int* next_sym) {
  if (!opt.enable_coop || ph.seq_syms.empty()) return false;
  Binop accum;
  if (!reduction_shape(r, ph, &accum) || accum != Binop::Add) return false;
  const Stmt& set = *ph.inner[0];
  const Node& out = r.node(set.node);
  if (!(out.prec == Prec::Single || out.prec == Prec::Double || out.prec == Prec::Bfloat16 || out.prec == Prec::Half))
    return false;
  int64_t P = 1, R = 1;
  for (auto e : ph.par_ext) P *= e;
  for (size_t i = 0; i < ph.seq_syms.size(); ++i) R *= ph.seq_to[i] - ph.seq_from[i] + 1;
  if (P >= 32768 || R < 128 || P * R < (1 << 20)) return false;
  for (auto f : ph.par_from) if (f != 0) return false;
  // lanes sharing the innermost loop already read contiguously: leave those to the lane groups
  if (reduction_walks_unit_stride(r, ph, set)) return false;
  // threads wanted: enough to keep the loads of a streaming sum in flight; twice that where every term
  // costs a division or a transcendental (the visit rule inlines a layer norm's normalisation into its
  // gain gradient), whose threads are bound by their own arithmetic and gain from more of them
  //   measured, the eight gain-gradient launches of the visit-rule transformer step: 14.6 -> 11.6 us each,
  //   while the streaming sums of the other form do not change and their combine only grows
  std::function<bool(const Scalar&)> costly = [&](const Scalar& x) -> bool {
    if (x.kind == Scalar::Bin && (x.bin == Binop::Div || x.bin == Binop::Pow || x.bin == Binop::Mod)) return true;
    if (x.kind == Scalar::Un && (x.un == Unop::Exp || x.un == Unop::Log || x.un == Unop::Exp2 || x.un == Unop::Log2 || x.un == Unop::Sin ||
                                 x.un == Unop::Cos || x.un == Unop::Sqrt || x.un == Unop::Recip || x.un == Unop::RecipSqrt || x.un == Unop::Tanh))
      return true;
    if (x.kind == Scalar::LocalScope) {
      bool any = false;
      std::function<void(const Block&)> walk = [&](const Block& b) {
        for (auto& st : b) { if (st->value && costly(*st->value)) any = true; walk(st->body); }
      };
      walk(x.body);
      if (any) return true;
    }
    return (x.a && costly(*x.a)) || (x.b && costly(*x.b)) || (x.c && costly(*x.c));
  };
  const int64_t threads_wanted = costly(*set.value) ? 262144 : 131072;
  const int64_t s_target = std::min<int64_t>(std::max<int64_t>((threads_wanted + P - 1) / P, 2), R / 8);
  // whole outer loops first, then a divisor of the next one
  size_t whole = 0;
  int64_t S = 1;
  while (whole < ph.seq_syms.size() && S * (ph.seq_to[whole] - ph.seq_from[whole] + 1) <= s_target) {
    S *= ph.seq_to[whole] - ph.seq_from[whole] + 1;
    ++whole;
  }
  int64_t hi_ext = 1, lo_ext = 0;
  if (whole < ph.seq_syms.size()) {
    const int64_t E = ph.seq_to[whole] - ph.seq_from[whole] + 1;
    for (int64_t h = std::min(E, s_target / S); h > 1; --h)
      if (E % h == 0) { hi_ext = h; break; }
    lo_ext = E / hi_ext;
  }
  if (S * hi_ext < 2) return false;

  // value with the split symbol rewritten
  ScalarP value = set.value;
  int hi = -1, lo = -1;
  if (hi_ext > 1) {
    hi = fresh_symbol(r, next_sym);
    lo = fresh_symbol(r, next_sym);
    bool ok = true;
    value = subst_scalar(value, ph.seq_syms[whole], ph.seq_from[whole], lo_ext, hi, lo, &ok);
    if (!ok) return false;
  }
  // scratch tensor partial[slice, p..]: output symbols ordered as the output stores them.  The slice
  // axes (the whole outer loops, then the upper part of the divided one) share ONE axis, as the
  // digits of a mixed-radix number: the combine below walks it with a single loop.
  std::vector<size_t> order(ph.par_syms.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = i;
  Strides so = strides_of(r, set.node, set.idcs);
  std::stable_sort(order.begin(), order.end(), [&](size_t x, size_t y) {
    return get_stride(so, ph.par_syms[x]) > get_stride(so, ph.par_syms[y]); });
  int new_id = 1;
  for (auto& kv : r.nodes) new_id = std::max(new_id, kv.first + 1);
  Node t;
  t.id = new_id;
  t.ident = "part" + std::to_string(new_id) + "_" + out.ident;
  t.prec = out.prec == Prec::Double ? Prec::Double : Prec::Single;
  t.mode = Mode::Local;
  Indices tix, tix2;
  auto iter = [](int sym) { AxisIndex a; a.kind = AxisIndex::Iter; a.sym = sym; return a; };
  const int64_t n_slices = S * hi_ext;
  const int slice = fresh_symbol(r, next_sym);
  {
    AxisIndex a;
    a.kind = AxisIndex::Affine;
    int64_t mult = n_slices;
    for (size_t i = 0; i < whole; ++i) {
      mult /= ph.seq_to[i] - ph.seq_from[i] + 1;
      a.terms.push_back({mult, ph.seq_syms[i]});
      a.offset -= mult * ph.seq_from[i];
    }
    if (hi_ext > 1) a.terms.push_back({1, hi});
    if (a.terms.size() == 1 && a.terms[0].first == 1 && a.offset == 0) a = iter(a.terms[0].second);
    t.dims.push_back(n_slices);
    tix.push_back(a);
    tix2.push_back(iter(slice));
  }
  for (size_t k : order) { t.dims.push_back(ph.par_ext[k]); tix.push_back(iter(ph.par_syms[k])); tix2.push_back(iter(ph.par_syms[k])); }

  // the same accumulation with the scratch element in place of the output element
  auto self = std::make_shared<Scalar>();
  self->kind = Scalar::Get; self->node = t.id; self->idcs = tix;
  auto is_self = [&](const Scalar& x) { return x.kind == Scalar::Get && x.node == set.node && same_indices(x.idcs, set.idcs); };
  auto v1 = std::make_shared<Scalar>(*value);
  if (v1->kind == Scalar::Tern) v1->c = self;
  else if (is_self(*set.value->a)) v1->a = self;
  else v1->b = self;
  auto set1 = std::make_shared<Stmt>();
  set1->kind = Stmt::Set; set1->node = t.id; set1->idcs = tix; set1->value = v1;
  StmtP nest1 = set1;
  for (size_t i = ph.seq_syms.size(); i-- > whole + (hi_ext > 1 ? 1 : 0);)
    nest1 = make_for(ph.seq_syms[i], ph.seq_from[i], ph.seq_to[i], nest1);
  if (hi_ext > 1) {
    nest1 = make_for(lo, 0, lo_ext - 1, nest1);
    nest1 = make_for(hi, 0, hi_ext - 1, nest1);
  }
  for (size_t i = whole; i-- > 0;) nest1 = make_for(ph.seq_syms[i], ph.seq_from[i], ph.seq_to[i], nest1);
  for (size_t k = order.size(); k-- > 0;)
    nest1 = make_for(ph.par_syms[order[k]], 0, ph.par_ext[order[k]] - 1, nest1);

  // phase 2: out[p] := out[p] + partial[slice, p..] over the slices
  auto get_t = std::make_shared<Scalar>();
  get_t->kind = Scalar::Get; get_t->node = t.id; get_t->idcs = tix2;
  auto lhs = std::make_shared<Scalar>();
  lhs->kind = Scalar::Get; lhs->node = set.node; lhs->idcs = set.idcs;
  auto v2 = std::make_shared<Scalar>();
  v2->kind = Scalar::Bin; v2->bin = Binop::Add; v2->a = lhs; v2->b = get_t;
  auto set2 = std::make_shared<Stmt>();
  set2->kind = Stmt::Set; set2->node = set.node; set2->idcs = set.idcs; set2->value = v2;
  StmtP nest2 = make_for(slice, 0, n_slices - 1, set2);
  for (size_t k = order.size(); k-- > 0;)
    nest2 = make_for(ph.par_syms[order[k]], 0, ph.par_ext[order[k]] - 1, nest2);

  r.nodes.emplace(t.id, t);
  Phase p1;
  p1.label = ph.label + " (partial sums)";
  p1.stmt = nest1;
  p1.fused_zero_init = true;
  Phase p2;
  p2.label = ph.label;
  p2.stmt = nest2;
  p2.fused_zero_init = ph.fused_zero_init;
  p2.sums_partials = true;
  Binop a1, a2;
  if (!analyze_nest(r, nest1, p1) || !analyze_nest(r, nest2, p2) || !reduction_shape(r, p1, &a1) ||
      !reduction_shape(r, p2, &a2) || p1.par_syms.size() != order.size() + whole + (hi_ext > 1 ? 1 : 0) ||
      p2.par_syms.size() != order.size()) {
    r.nodes.erase(t.id);
    return false;
  }
  p1.kind = Phase::Generic;
  choose_coop(r, p1, opt);
  account_bytes(r, p1);
  plan.phases.push_back(std::move(p1));
  plan.scratch.push_back(t);
  ph = std::move(p2);
  return true;
}

std::vector<size_t> store_order(const Routine& r, const Phase& ph) {
  std::vector<size_t> order(ph.par_syms.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = i;
  const Stmt* first_set = nullptr;
  std::function<void(const Block&)> find_set = [&](const Block& b) {
    for (auto& s : b) {
      if (first_set) return;
      if (s->kind == Stmt::Set || s->kind == Stmt::SetVec) first_set = s.get();
      else if (s->kind == Stmt::For) find_set(s->body);
    }
  };
  find_set(ph.inner);
  auto lhs_stride = [&](int sym) -> int64_t {
    if (!first_set) return 0;
    const Node& n = r.node(first_set->node);
    int64_t st = 0, rs = 1;
    for (int p = (int)first_set->idcs.size() - 1; p >= 0; --p) {
      const AxisIndex& a = first_set->idcs[p];
      if (a.kind == AxisIndex::Iter && a.sym == sym) st += rs;
      if (a.kind == AxisIndex::Affine) for (auto& t : a.terms) if (t.second == sym) st += t.first * rs;
      rs *= n.dims[p];
    }
    return st;
  };
  std::stable_sort(order.begin(), order.end(), [&](size_t x, size_t y) {
    return lhs_stride(ph.par_syms[x]) > lhs_stride(ph.par_syms[y]); });
  return order;
}

// ---- row groups ---------------------------------------------------------------------------------

namespace {

struct RowShape { std::vector<int64_t> outer; int64_t len = -1; };

// Classifies `ph` as a member of a row group over `shape` (filling in what the shape leaves open).
bool row_member(const Routine& r, Phase& ph, RowShape& shape, bool first) {
  if (ph.kind != Phase::Generic || !ph.members.empty()) return false;
  if (ph.inner.size() != 1 || ph.inner[0]->kind != Stmt::Set) return false;
  for (auto f : ph.par_from) if (f != 0) return false;
  for (auto f : ph.seq_from) if (f != 0) return false;
  std::vector<size_t> order = store_order(r, ph);
  std::vector<int64_t> ext;
  std::vector<int> syms;
  for (size_t k : order) { ext.push_back(ph.par_ext[k]); syms.push_back(ph.par_syms[k]); }
  const size_t n = first ? 0 : shape.outer.size();
  auto outer_matches = [&](size_t count) {
    if (first) return true;
    if (count != n) return false;
    for (size_t i = 0; i < n; ++i) if (ext[i] != shape.outer[i]) return false;
    return true;
  };
  Binop accum;
  if (ph.seq_syms.size() == 1 && reduction_shape(r, ph, &accum)) {          // a row reduction
    const int64_t T = ph.seq_to[0] + 1;
    if (!outer_matches(ext.size()) || (shape.len >= 0 && shape.len != T) || T < 16) return false;
    // lanes share a row through a float (or double) accumulator: integer rows stay sequential and exact
    const Prec rp = r.node(ph.inner[0]->node).prec;
    if (!(rp == Prec::Single || rp == Prec::Double || rp == Prec::Bfloat16 || rp == Prec::Half)) return false;
    // the reduced operand must be walked contiguously
    std::vector<Access> acc; bool fl = false; std::set<ScopeId> d;
    scalar_accesses(*ph.inner[0]->value, acc, fl, d);
    bool unit = false;
    for (auto& a : acc) if (a.node != ph.inner[0]->node && get_stride(strides_of(r, a.node, *a.idcs), ph.seq_syms[0]) == 1) unit = true;
    if (!unit) return false;
    ph.row_role = Phase::RowReduce; ph.row_outer_syms = syms; ph.row_sym = ph.seq_syms[0];
    if (first) shape.outer = ext;
    shape.len = T;
    return true;
  }
  if (!ph.seq_syms.empty()) return false;
  if (ph.coop_scope) {                                                        // per-row scalar holding a reduction
    std::vector<const Stmt*> loops; const Stmt* init = nullptr; const Stmt* upd = nullptr;
    if (!scope_reduction(*ph.coop_scope, loops, init, upd, &accum) || loops.size() != 1 || loops[0]->from != 0) return false;
    const int64_t T = loops[0]->to + 1;
    if (!outer_matches(ext.size()) || (shape.len >= 0 && shape.len != T) || T < 16) return false;
    ph.row_role = Phase::RowScalar; ph.row_outer_syms = syms; ph.row_sym = loops[0]->sym;
    if (first) shape.outer = ext;
    shape.len = T;
    return true;
  }
  if (ph.coop_lanes != 1) return false;
  if (!first && ext.size() == n) {                                            // per-row scalar
    if (!outer_matches(ext.size())) return false;
    ph.row_role = Phase::RowScalar; ph.row_outer_syms = syms; ph.row_sym = -1;
    return true;
  }
  if (first && ext.empty()) {                                                 // a chain of plain scalars
    ph.row_role = Phase::RowScalar; ph.row_outer_syms = syms; ph.row_sym = -1;
    shape.outer.clear();
    return true;
  }
  if (ext.empty()) return false;                                              // pointwise over rows x T
  const int64_t T = ext.back();
  // (short rows leave lanes idle: the caller takes such a group only when it is launch-bound anyway)
  if (!outer_matches(ext.size() - 1) || (shape.len >= 0 && shape.len != T) || T < 2) return false;
  // the row position must be the unit-stride axis of the store
  if (get_stride(strides_of(r, ph.inner[0]->node, ph.inner[0]->idcs), syms.back()) != 1) return false;
  ph.row_role = Phase::RowPointwise;
  ph.row_outer_syms.assign(syms.begin(), syms.end() - 1);
  ph.row_sym = syms.back();
  if (first) shape.outer.assign(ext.begin(), ext.end() - 1);
  shape.len = T;
  return true;
}

// Signature of an access relative to the member's row symbols: which outer axis / row position /
// constant drives each axis.  Empty when an index is of another form.
std::string row_signature(const Phase& ph, const Indices& idcs) {
  std::string sig;
  for (auto& ix : idcs) {
    if (ix.kind == AxisIndex::Fixed) sig += "f" + std::to_string(ix.fixed);
    else if (ix.kind == AxisIndex::Iter) {
      if (ix.sym == ph.row_sym) sig += "r";
      else {
        int pos = -1;
        for (size_t j = 0; j < ph.row_outer_syms.size(); ++j) if (ph.row_outer_syms[j] == ix.sym) pos = (int)j;
        if (pos < 0) return "";
        sig += "o" + std::to_string(pos);
      }
    } else return "";
    sig += ",";
  }
  return sig.empty() ? "scalar" : sig;
}

struct RowDeps {
  std::map<int, std::set<std::string>> sigs;   // node -> signatures seen (empty string: irregular)
  std::set<int> written;
  bool add(const Phase& ph) {
    std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
    block_accesses(ph.inner, acc, w, f, d);
    if (w || f) return false;
    for (auto& a : acc) {
      sigs[a.node].insert(row_signature(ph, *a.idcs));
      if (a.write) written.insert(a.node);
    }
    for (int node : written) {
      const auto& s = sigs[node];
      if (s.size() != 1 || s.begin()->empty()) return false;
    }
    return true;
  }
};

void group_rows(const Routine& r, Plan& plan) {
  double routine_bytes = 0;
  for (auto& ph : plan.phases) routine_bytes += ph.bytes;
  const bool launch_bound = routine_bytes < 8e6;
  std::vector<Phase> out;
  size_t i = 0;
  while (i < plan.phases.size()) {
    RowShape shape;
    std::vector<Phase> run;
    RowDeps deps;
    size_t j = i;
    while (j < plan.phases.size()) {
      Phase cand = plan.phases[j];
      RowShape trial = shape;
      if (!row_member(r, cand, trial, run.empty())) break;
      RowDeps d2 = deps;
      if (!d2.add(cand)) break;
      shape = trial; deps = d2;
      run.push_back(std::move(cand));
      ++j;
    }
    // a group must know its row length and be worth a launch of its own
    int64_t rows = 1;
    for (auto e : shape.outer) rows *= e;
    // ... or sit in a routine so small that launches are all there is to save (in a large routine
    // such a group was measured slower than its members as separate, overlapping launches)
    if (shape.len < 0 && shape.outer.empty() && run.size() >= 2) shape.len = 1;   // scalars only
    const int64_t points = rows * std::max<int64_t>(shape.len, 1);
    // ... or be a chain of tiny phases over the same few points (the steps between the loss and the
    // gradient of the logits: 8192 points, 6 us of launch latency each, four launches less in the
    // transformer step)
    bool tiny_chain = run.size() >= 2 && points <= 16384;
    for (auto& m : run) tiny_chain = tiny_chain && m.bytes <= (double)(1 << 20);
    if (run.size() >= 2 && shape.len >= 1 && ((shape.len >= 16 && points >= (1 << 16)) || (launch_bound && points < 8192) || tiny_chain)) {
      Phase g;
      g.kind = Phase::Generic;
      g.label = run.front().label + " .. " + run.back().label;
      g.row_outer_ext = shape.outer;
      g.row_len = shape.len;
      int lanes = 1;
      while (lanes * 2 <= 64 && lanes * 2 <= shape.len) lanes *= 2;
      // a long row (more than 16 elements per lane of a wave) goes to a whole workgroup when that
      // brings it down to <= 16 per thread: everything the group produces then fits in registers
      if (shape.len / lanes > 16 && shape.len % 256 == 0 && shape.len / 256 <= 16) lanes = 256;
      g.coop_lanes = lanes;
      // algorithmic bytes: every array the group writes, once, plus every array it reads without
      // having produced it, once; an array indexed by the row position counts rows x T elements,
      // a per-row one counts rows, anything else (broadcast operands) its own size at most
      std::set<int> produced, counted_r, counted_w;
      double bytes = 0;
      auto touched = [&](const Phase& m, const Access& a) {
        const Node& nd = r.node(a.node);
        const std::string sig = row_signature(m, *a.idcs);
        double n = sig.empty() ? (double)nd.num_elems()
                               : (double)rows * (sig.find('r') != std::string::npos ? (double)shape.len : 1.0);
        return std::min(n, (double)nd.num_elems()) * prec_in_bytes(nd.prec);
      };
      for (auto& m : run) {
        std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
        block_accesses(m.inner, acc, w, f, d);
        const int unread = m.fused_zero_init && m.inner.size() == 1 && m.inner[0]->kind == Stmt::Set ? m.inner[0]->node : -1;
        for (auto& a : acc)
          if (!a.write && a.node != unread && !produced.count(a.node) && counted_r.insert(a.node).second) bytes += touched(m, a);
        for (auto& a : acc)
          if (a.write) { produced.insert(a.node); if (counted_w.insert(a.node).second) bytes += touched(m, a); }
      }
      g.bytes = bytes;
      g.members = std::move(run);
      out.push_back(std::move(g));
      i = j;
    } else {
      out.push_back(plan.phases[i]);
      ++i;
    }
  }
  plan.phases = std::move(out);
}

}  // namespace

// ---- contractions that share a launch ---------------------------------------------------------------
// Two ways in which contractions of identical shapes, strides and precisions share a launch:
//   * a group of independent ones (the q / k / v projections of one input; the weight gradients of
//     those projections): the grid's z axis runs over the members.  A small contraction alone puts at
//     most one workgroup on a compute unit; several together let workgroups hide each other's memory
//     latency;
//   * a chain `c =+ a1 * b1; c =+ a2 * b2; ...` into one result (the input gradient of a tensor that
//     feeds several projections): K runs over every operand pair, C is read and written once.
// The statements need not be adjacent.  A later one is hoisted to the earlier one's position when
// nothing in between touches its result or writes its operands; otherwise the earlier ones are sunk
// to the later position under the same condition on them.
namespace {

bool phase_writes(const Phase& ph, int node);

bool same_layout(const GemmOperand& x, const GemmOperand& y) {
  if (x.prec != y.prec || x.s_row != y.s_row || x.s_k != y.s_k) return false;
  for (int i = 0; i < 3; ++i) if (x.s_batch[i] != y.s_batch[i]) return false;
  return true;
}

void merge_contractions(Plan& plan, bool chain, int window = 1 << 30) {
  std::map<int, int> mirror_source;   // bf16 copy -> the tensor whose stores keep it in step
  for (auto& kv : plan.mirrors) mirror_source[kv.second] = kv.first;
  auto source_of = [&](int node) { auto m = mirror_source.find(node); return m == mirror_source.end() ? node : m->second; };
  auto writes_operand = [&](const Phase& q, const GemmOperand& op) {
    return phase_writes(q, op.node) || phase_writes(q, source_of(op.node));
  };
  auto touches_result = [&](const Phase& q, const GemmOperand& c) {
    if (phase_touches(q, c.node)) return true;
    auto m = plan.mirrors.find(c.node);
    return m != plan.mirrors.end() && phase_touches(q, m->second);
  };
  using Member = GemmDesc::Member;
  auto members_of = [](const GemmDesc& g) {
    std::vector<Member> v{{g.a, g.b, g.c, g.c_copy}};
    for (auto& pr : g.more) v.push_back({pr.first, pr.second, g.c, g.c_copy});
    for (auto& m : g.group) v.push_back(m);
    return v;
  };
  // may the contraction `x` run at another place of phases (lo, hi), i.e. does nothing there touch
  // its result or write its operands?
  auto free_between = [&](const Member& x, size_t lo, size_t hi) {
    for (size_t k = lo + 1; k < hi; ++k) {
      const Phase& mid = plan.phases[k];
      if (touches_result(mid, x.c) || writes_operand(mid, x.a) || writes_operand(mid, x.b)) return false;
      if (x.c_copy >= 0 && phase_touches(mid, x.c_copy)) return false;
    }
    return true;
  };
  for (size_t i = 0; i < plan.phases.size(); ++i) {
    if (plan.phases[i].kind != Phase::Contraction) continue;
    {
      const GemmDesc& g = plan.phases[i].gemm;
      if (chain ? !g.group.empty() : !g.more.empty()) continue;
      if (chain) {
        // the kernels built for operand-pair lists: bf16 operands, fp32 result
        if (g.a.prec != Prec::Bfloat16 || g.b.prec != Prec::Bfloat16 || g.c.prec != Prec::Single) continue;
      } else {
        // grouping pays where a launch alone leaves compute units idle or with one workgroup each
        double tiles = (double)((g.M + 127) / 128) * (double)((g.N + 127) / 128);
        for (int b = 0; b < g.nbatch; ++b) tiles *= (double)g.batch_ext[b];
        if (tiles > 256) continue;
      }
    }
    bool sunk = false;
    for (size_t j = i + 1; j < plan.phases.size() && !sunk; ++j) {
      Phase& p = plan.phases[i];
      GemmDesc& g = p.gemm;
      if (g.group.size() + g.more.size() >= 3) break;
      if (!chain && (long)j - (long)i > (long)window) break;
      Phase& q = plan.phases[j];
      const GemmDesc& h = q.gemm;
      bool candidate = q.kind == Phase::Contraction && h.group.empty() && h.more.empty() && h.epi_bias < 0 && h.epi_relu < 0 &&
                       g.epi_bias < 0 && g.epi_relu < 0 && h.M == g.M && h.N == g.N &&
                       h.K == g.K && h.nbatch == g.nbatch && same_layout(h.a, g.a) && same_layout(h.b, g.b) && same_layout(h.c, g.c);
      for (int b = 0; b < g.nbatch && candidate; ++b) candidate = h.batch_ext[b] == g.batch_ext[b];
      const std::vector<Member> mine = members_of(g);
      if (candidate && chain)
        candidate = h.accumulate && h.c_copy < 0 && h.c.node == g.c.node && h.c.offset == g.c.offset &&
                    h.c.static_terms == g.c.static_terms && source_of(h.a.node) != g.c.node && source_of(h.b.node) != g.c.node &&
                    (g.c_copy < 0 || (h.a.node != g.c_copy && h.b.node != g.c_copy));
      if (candidate && !chain) {
        candidate = h.accumulate == g.accumulate && (h.c_copy >= 0) == (g.c_copy >= 0);
        for (auto& x : mine) {
          const int xc = x.c.node, hc = h.c.node;
          if (x.c_copy >= 0) candidate = candidate && h.a.node != x.c_copy && h.b.node != x.c_copy;
          if (h.c_copy >= 0) candidate = candidate && x.a.node != h.c_copy && x.b.node != h.c_copy;
          candidate = candidate && hc != xc && source_of(h.a.node) != xc && source_of(h.b.node) != xc && h.a.node != xc && h.b.node != xc &&
                      source_of(x.a.node) != hc && source_of(x.b.node) != hc && x.a.node != hc && x.b.node != hc;
        }
      }
      if (!candidate) {
        // someone else reads or writes C: the chain cannot reach past it
        if (chain && (phase_touches(q, g.c.node) || (g.c_copy >= 0 && phase_touches(q, g.c_copy)))) break;
        continue;
      }
      const Member joiner{h.a, h.b, h.c, h.c_copy};
      bool hoist = free_between(joiner, i, j), sink = false;
      if (!hoist) {
        sink = true;
        for (auto& x : mine) sink = sink && free_between(x, i, j);
      }
      if (!hoist && !sink) {
        if (chain) break;
        continue;
      }
      if (chain) {
        double c_bytes = (double)g.M * (double)g.N * prec_in_bytes(g.c.prec);
        for (int b = 0; b < g.nbatch; ++b) c_bytes *= (double)g.batch_ext[b];
        g.more.push_back({h.a, h.b});
        p.bytes += q.bytes - 2.0 * c_bytes;   // C is read and written once less
      } else {
        g.group.push_back(joiner);
        p.bytes += q.bytes;
      }
      p.flops = g.flops();
      p.label += (chain ? " + " : " | ") + q.label;
      if (hoist) {
        plan.phases.erase(plan.phases.begin() + j);
        --j;
      } else {
        // the merged launch takes the later statement's place; position i now holds what followed
        // and is looked at again
        plan.phases[j] = std::move(plan.phases[i]);
        plan.phases.erase(plan.phases.begin() + i);
        sunk = true;
        --i;
      }
    }
  }
}

}  // namespace

// ---- tiny routines ---------------------------------------------------------------------------------
namespace {

bool writes_whole_node(const Routine& r, const Phase& ph, int node);

// LDS shadows for a serial group (see Phase::serial_shadows).
void choose_shadows(const Routine& r, Phase& g) {
  struct Flat { const Phase* ph; int member; };
  std::vector<Flat> flat;
  for (size_t q = 0; q < g.serial_members.size(); ++q) {
    const Phase& m = g.serial_members[q];
    if (m.members.empty()) flat.push_back({&m, (int)q});
    else for (auto& sub : m.members) flat.push_back({&sub, (int)q});
  }
  int64_t budget = 48 * 1024;
  for (auto& kv : r.nodes) {
    const Node& n = kv.second;
    if (n.mode == Mode::Virtual || n.prec == Prec::Uint4x32 || n.prec == Prec::Void) continue;
    const int64_t bytes = (int64_t)n.size_in_bytes();
    if (bytes > budget || bytes > 16 * 1024) continue;
    int valid_after = -1;
    bool ok = true;
    for (auto& f : flat) {
      const Phase& ph = *f.ph;
      if (ph.kind == Phase::Fill) {
        if (ph.fill_node == n.id && valid_after < 0) valid_after = f.member;
        continue;
      }
      std::vector<Access> acc; bool w = false, fo = false; std::set<ScopeId> d;
      block_accesses(ph.inner, acc, w, fo, d);
      if (w) { ok = false; break; }   // a Zero_out inside a nest: stores the printer does not route
      bool touches = false, writes = false, reads = false, vec = false;
      for (auto& a : acc) if (a.node == n.id) {
        touches = true;
        if (a.write) { writes = true; vec |= a.vec_len > 0; }
        else if (!(ph.fused_zero_init && ph.inner.size() == 1 && ph.inner[0]->kind == Stmt::Set && ph.inner[0]->node == n.id)) reads = true;
      }
      if (!touches) continue;
      if (vec) { ok = false; break; }
      if (valid_after < 0) {
        // the first touch has to store the whole tensor without reading it
        if (!writes || reads || !writes_whole_node(r, ph, n.id)) { ok = false; break; }
        valid_after = f.member;
      }
    }
    if (ok && valid_after >= 0 && valid_after + 1 < (int)g.serial_members.size()) {
      g.serial_shadows[n.id] = valid_after;
      budget -= bytes;
    }
  }
}

void serialise_tiny(const Routine& r, Plan& plan) {
  if (plan.phases.size() < 4) return;
  double bytes = 0;
  // the workgroup's 256 threads loop over each phase's points, and with four waves nothing hides
  // the memory latency of a trip (about a microsecond each, measured): worth it only while the
  // trips per phase stay below what a launch costs
  int64_t iterations = 0;
  for (auto& ph : plan.phases) {
    if (ph.kind == Phase::Fill) {
      iterations += r.node(ph.fill_node).num_elems() / 256 + 1;
    } else if (ph.kind == Phase::Generic && !ph.members.empty()) {
      int64_t threads = ph.coop_lanes;
      for (auto e : ph.row_outer_ext) threads *= e;
      if (threads > 131072) return;
      iterations += (threads / 256 + 1) * (int64_t)ph.members.size();
    } else if (ph.kind == Phase::Generic) {
      int64_t threads = ph.coop_lanes;
      for (auto e : ph.par_ext) threads *= e;
      int64_t work = 1;
      for (size_t i = 0; i < ph.seq_syms.size(); ++i) work *= ph.seq_to[i] - ph.seq_from[i] + 1;
      if (threads > 131072 || work > 4096) return;
      iterations += threads / 256 + 1;
    } else return;
    bytes += ph.bytes;
  }
  int64_t statements = 0;   // a row group counts as the statements it fuses
  for (auto& ph : plan.phases) statements += ph.members.empty() ? 1 : (int64_t)ph.members.size();
  if (iterations > 8 * statements) return;
  Phase g;
  g.kind = Phase::Generic;
  g.label = "whole routine, one workgroup";
  g.bytes = bytes;
  g.serial_members = std::move(plan.phases);
  choose_shadows(r, g);
  plan.phases.clear();
  plan.phases.push_back(std::move(g));
}

}  // namespace

// ---- independent small phases ------------------------------------------------------------------------
// A run of consecutive small generated phases none of which touches what another writes (the updates
// of the many small parameters of a model, the finishing touches of bias gradients) becomes one
// kernel: each member owns a range of workgroups, so they run side by side instead of as launches of
// a few microseconds each in a row.
namespace {

bool phase_writes(const Phase& ph, int node);

void group_independent(const Routine& r, Plan& plan) {
  (void)r;
  if (plan.phases.size() < 2) return;
  struct Sets { std::set<int> reads, writes; bool ok = false; };
  auto add_accesses = [&](const Phase& ph, Sets& s) {
    std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
    block_accesses(ph.inner, acc, w, f, d);
    if (w || f) return false;
    for (auto& a : acc) {
      (a.write ? s.writes : s.reads).insert(a.node);
      if (a.write) { auto m = plan.mirrors.find(a.node); if (m != plan.mirrors.end()) s.writes.insert(m->second); }
    }
    return true;
  };
  auto sets_of = [&](const Phase& ph) {
    Sets s;
    if (ph.kind != Phase::Generic || !ph.serial_members.empty() || !ph.parallel_members.empty() || ph.fused_x >= 0) return s;
    if (ph.bytes > (double)(32 << 20)) return s;
    bool ok = true;
    if (ph.members.empty()) ok = add_accesses(ph, s);
    else for (auto& m : ph.members) ok = ok && add_accesses(m, s);
    s.ok = ok;
    return s;
  };
  auto disjoint = [](const std::set<int>& x, const std::set<int>& y) {
    for (int v : x) if (y.count(v)) return false;
    return true;
  };
  // A small phase that stands at the end of its window (a phase that cannot join follows it) waits
  // for the first later phase that conflicts with it and runs right before that one -- the second
  // half of a split bias-gradient sum, say, joins the window of the optimiser's updates, the first
  // thing that reads it.  (From the last phase backwards, so that positions ahead stay valid.)
  for (size_t i = plan.phases.size(); i-- > 0;) {
    const Sets mine = sets_of(plan.phases[i]);
    if (!mine.ok || plan.phases[i].bytes > (double)(2 << 20) || i + 1 >= plan.phases.size()) continue;
    if (sets_of(plan.phases[i + 1]).ok) continue;
    size_t t = i + 1;
    for (; t < plan.phases.size(); ++t) {
      const Phase& q = plan.phases[t];
      bool conflict = false;
      for (int n : mine.writes) conflict = conflict || phase_touches(q, n);
      for (int n : mine.reads) conflict = conflict || phase_writes(q, n);
      if (conflict) break;
    }
    if (t == i + 1) continue;
    // worth it only next to a phase it can share a launch with
    const bool joins = (t < plan.phases.size() && sets_of(plan.phases[t]).ok) || sets_of(plan.phases[t - 1]).ok;
    if (!joins) continue;
    std::rotate(plan.phases.begin() + i, plan.phases.begin() + i + 1, plan.phases.begin() + t);
  }
  std::vector<Sets> sets;
  for (auto& ph : plan.phases) sets.push_back(sets_of(ph));
  std::vector<Phase> out;
  size_t i = 0;
  while (i < plan.phases.size()) {
    if (!sets[i].ok) { out.push_back(std::move(plan.phases[i])); ++i; continue; }
    size_t j = i;
    while (j < plan.phases.size() && sets[j].ok) ++j;
    // [i, j): a window of eligible phases.  A phase's level is one more than the highest level among
    // the earlier phases of the window it conflicts with, so phases of one level are independent and
    // conflicting phases keep their order when the levels run one after the other.
    std::vector<int> level(j - i, 0);
    int top = 0;
    for (size_t k = i; k < j; ++k) {
      for (size_t e = i; e < k; ++e) {
        const bool conflict = !disjoint(sets[k].writes, sets[e].reads) || !disjoint(sets[k].writes, sets[e].writes) ||
                              !disjoint(sets[e].writes, sets[k].reads);
        if (conflict) level[k - i] = std::max(level[k - i], level[e - i] + 1);
      }
      top = std::max(top, level[k - i]);
    }
    for (int lv = 0; lv <= top; ++lv) {
      std::vector<size_t> same;
      for (size_t k = i; k < j; ++k) if (level[k - i] == lv) same.push_back(k);
      // reductions first: few threads that each wait on a run of dependent loads; started at the head of
      // the grid they wait while the streaming members run, at its tail the launch would wait for them
      std::stable_sort(same.begin(), same.end(), [&](size_t x, size_t y) {
        return !plan.phases[x].seq_syms.empty() && plan.phases[y].seq_syms.empty(); });
      for (size_t c = 0; c < same.size(); c += 32) {
        const size_t n = std::min<size_t>(32, same.size() - c);
        if (n == 1) { out.push_back(std::move(plan.phases[same[c]])); continue; }
        Phase g;
        g.kind = Phase::Generic;
        g.label = std::to_string(n) + " independent phases side by side";
        for (size_t q = c; q < c + n; ++q) {
          g.bytes += plan.phases[same[q]].bytes;
          g.flops += plan.phases[same[q]].flops;
          g.parallel_members.push_back(std::move(plan.phases[same[q]]));
        }
        out.push_back(std::move(g));
      }
    }
    i = j;
  }
  plan.phases = std::move(out);
}

}  // namespace

// ---- bf16 copies of fp32 contraction operands -----------------------------------------------------
// A contraction with one fp32 and one bf16 operand runs on the bf16 matrix cores: the fp32
// operand is rounded to bf16 on the way in.  Doing that rounding once, in a pass of its own into a
// scratch tensor, gives the same bits, lets every contraction that reads the tensor (a gradient
// feeds both the input-gradient and the weight-gradient contraction) take the all-bf16 kernel, and
// halves what they read.

namespace {

bool phase_writes(const Phase& ph, int node) {
  if (ph.kind == Phase::Fill) return ph.fill_node == node;
  if (ph.kind == Phase::Contraction) {
    for (auto& m : ph.gemm.group) if (m.c.node == node || m.c_copy == node) return true;
    return ph.gemm.c.node == node || ph.gemm.c_copy == node || ph.gemm.epi_relu == node;
  }
  auto writes = [&](const Phase& q) {
    std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
    block_accesses(q.inner, acc, w, f, d);
    if (w) return true;
    for (auto& a : acc) if (a.write && a.node == node) return true;
    return false;
  };
  if (ph.fused_x == node && ph.fused_x_store) return true;
  if (ph.proj_y >= 0 && (ph.proj_c.node == node || ph.proj_c_copy == node)) return true;
  if (!ph.members.empty()) { for (auto& m : ph.members) if (writes(m)) return true; return false; }
  if (!ph.parallel_members.empty()) { for (auto& m : ph.parallel_members) if (phase_writes(m, node)) return true; return false; }
  if (!ph.serial_members.empty()) { for (auto& m : ph.serial_members) if (phase_writes(m, node)) return true; return false; }
  return writes(ph);
}

// Does the generated phase store to every element of `node`?  (Every axis of its store is a
// full-range parallel iterator or has extent 1.)
bool writes_whole_node(const Routine& r, const Phase& ph, int node) {
  if (ph.inner.size() != 1 || ph.inner[0]->kind != Stmt::Set || ph.inner[0]->node != node) return false;
  const Stmt& set = *ph.inner[0];
  const Node& n = r.node(node);
  for (size_t p = 0; p < set.idcs.size(); ++p) {
    const AxisIndex& a = set.idcs[p];
    if (a.kind == AxisIndex::Fixed) { if (n.dims[p] != 1) return false; }
    else if (a.kind == AxisIndex::Iter) {
      bool ok = false;
      for (size_t i = 0; i < ph.par_syms.size(); ++i)
        if (ph.par_syms[i] == a.sym) ok = ph.par_from[i] == 0 && ph.par_ext[i] == n.dims[p];
      if (!ok) return false;
    } else return false;
  }
  return true;
}

struct Bf16Copies {
  std::map<int, int> copy_of;       // fp32 node -> its bf16 scratch copy
  std::map<int, size_t> made_at;    // fp32 node -> position in plan.phases from which writers make the copy stale
  // positions move when the planner erases a folded fill or inserts a fill for a copy
  void erased(size_t at) { for (auto& kv : made_at) if (kv.second > at) --kv.second; }
  void inserted(size_t at) { for (auto& kv : made_at) if (kv.second >= at) ++kv.second; }
};

void use_bf16_copies(Routine& r, Plan& plan, Phase& ph, Bf16Copies& copies, int* next_sym) {
  GemmDesc& g = ph.gemm;
  if ((g.a.prec == Prec::Single) == (g.b.prec == Prec::Single)) return;   // all-fp32 stays exact fp32
  GemmOperand& op = g.a.prec == Prec::Single ? g.a : g.b;
  const Node src = r.node(op.node);
  int copy = -1;
  auto it = copies.copy_of.find(src.id);
  if (it != copies.copy_of.end()) {
    bool stale = false;
    for (size_t q = copies.made_at[src.id]; q < plan.phases.size(); ++q) stale |= phase_writes(plan.phases[q], src.id);
    if (!stale) copy = it->second;
  }
  if (copy < 0) {
    // a mirror is kept in step by generated stores and zero fills only: once a contraction has
    // written the tensor it no longer stands for it
    auto m = plan.mirrors.find(src.id);
    if (m != plan.mirrors.end()) {
      bool in_step = true;
      for (auto& q : plan.phases) in_step &= !(q.kind == Phase::Contraction && q.gemm.c.node == src.id);
      if (in_step) copy = m->second;
    }
  }
  // Can the kernels that produce the tensor keep the copy themselves?  Yes when everything that
  // writes it in this routine is a generated kernel (or a zero fill), and some writer covers the
  // whole tensor before this contraction reads it.
  bool mirror = false;
  std::vector<size_t> fills;
  if (copy < 0) {
    bool all_generated = true, whole = false, any = false;
    for (size_t q = 0; q < plan.phases.size(); ++q) {
      const Phase& w = plan.phases[q];
      if (!phase_writes(w, src.id)) continue;
      any = true;
      if (w.kind == Phase::Fill) { fills.push_back(q); whole = true; }
      else if (w.kind == Phase::Generic && w.members.empty() && w.serial_members.empty()) whole |= writes_whole_node(r, w, src.id);
      else all_generated = false;
    }
    mirror = any && all_generated && whole && src.mode != Mode::Virtual && !src.read_only;
  }
  if (copy < 0) {
    int new_id = 1;
    for (auto& kv : r.nodes) new_id = std::max(new_id, kv.first + 1);
    Node t;
    t.id = new_id;
    t.ident = "bf" + std::to_string(new_id) + "_" + src.ident;
    t.prec = Prec::Bfloat16;
    t.mode = Mode::Local;
    t.dims = src.dims;
    if (mirror) {
      r.nodes.emplace(t.id, t);
      plan.scratch.push_back(t);
      plan.mirrors[src.id] = t.id;
      // a remaining zero fill of the tensor zeroes the copy too (bf16 zero is all-zero bits)
      for (size_t k = fills.size(); k-- > 0;) {
        Phase f;
        f.kind = Phase::Fill; f.label = "zero bf16 copy of " + src.ident; f.fill_node = t.id;
        f.bytes = (double)t.size_in_bytes();
        plan.phases.insert(plan.phases.begin() + fills[k] + 1, std::move(f));
        copies.inserted(fills[k] + 1);
      }
      op.node = t.id;
      op.prec = Prec::Bfloat16;
      set_contraction_bytes(ph);
      return;
    }
    // The tensor's last writer is a matrix-core contraction that stores all of it in fp32: its
    // epilogue writes the rounded copy as well, instead of a conversion pass over the tensor.
    for (int q = (int)plan.phases.size() - 1; q >= 0; --q) {
      Phase& producer = plan.phases[q];
      if (!phase_writes(producer, src.id)) continue;
      GemmDesc& pg = producer.gemm;
      int64_t written = pg.M * pg.N, total = 1;
      for (int b = 0; b < pg.nbatch; ++b) written *= pg.batch_ext[b];
      for (int64_t d : src.dims) total *= d;
      if (producer.kind == Phase::Contraction && pg.c.node == src.id && pg.c_copy < 0 && pg.c.prec == Prec::Single &&
          pg.c.offset == 0 && pg.c.static_terms.empty() && written == total) {
        r.nodes.emplace(t.id, t);
        plan.scratch.push_back(t);
        pg.c_copy = t.id;
        set_contraction_bytes(producer);
        copies.copy_of[src.id] = t.id;
        copies.made_at[src.id] = plan.phases.size();
        op.node = t.id;
        op.prec = Prec::Bfloat16;
        set_contraction_bytes(ph);
        return;
      }
      break;   // only the last writer can stand for the tensor's contents
    }
    Indices ix;
    std::vector<int> syms;
    for (size_t p = 0; p < src.dims.size(); ++p) {
      AxisIndex a; a.kind = AxisIndex::Iter; a.sym = fresh_symbol(r, next_sym);
      syms.push_back(a.sym); ix.push_back(a);
    }
    auto get = std::make_shared<Scalar>();
    get->kind = Scalar::Get; get->node = src.id; get->idcs = ix;
    auto set = std::make_shared<Stmt>();
    set->kind = Stmt::Set; set->node = t.id; set->idcs = ix; set->value = get;
    StmtP nest = set;
    for (size_t p = src.dims.size(); p-- > 0;) nest = make_for(syms[p], 0, src.dims[p] - 1, nest);
    r.nodes.emplace(t.id, t);
    Phase cv;
    cv.label = "bf16 copy of " + src.ident;
    cv.stmt = nest;
    if (!analyze_nest(r, nest, cv)) { r.nodes.erase(t.id); return; }
    cv.kind = Phase::Generic;
    account_bytes(r, cv);
    plan.phases.push_back(std::move(cv));
    plan.scratch.push_back(t);
    copies.copy_of[src.id] = t.id;
    copies.made_at[src.id] = plan.phases.size();
    copy = t.id;
  }
  op.node = copy;
  op.prec = Prec::Bfloat16;
  set_contraction_bytes(ph);
}

}  // namespace

// ---- scalar locals at routine scope ------------------------------------------------------------
// `Declare_local` / `Set_local` outside any `Local_scope` (low_level.mli:22-51) declare a scalar
// that lives across top-level statements.  The serial C code keeps it in a variable; here the
// statements become different kernels, so the scalar gets a one-element scratch tensor: the
// declaration disappears (a zero fill if it asked for initialisation), `Set_local` becomes a store
// and every read of the scalar a load.
namespace {

void lift_routine_locals(Routine& r, Plan& plan) {
  std::map<ScopeId, int> lifted;
  for (auto& sp : r.body)
    if (sp->kind == Stmt::DeclareLocal) lifted[sp->scope] = -1;
  if (lifted.empty()) return;
  int new_id = 1;
  for (auto& kv : r.nodes) new_id = std::max(new_id, kv.first + 1);
  for (auto& kv : lifted) {
    Node t;
    t.id = new_id++;
    t.ident = "v" + std::to_string(kv.first.scope) + "_" + r.node(kv.first.node).ident;
    t.prec = r.node(kv.first.node).prec;
    t.mode = Mode::Local;
    t.dims = {1};
    r.nodes.emplace(t.id, t);
    plan.scratch.push_back(t);
    kv.second = t.id;
  }
  Indices zero(1);
  zero[0].kind = AxisIndex::Fixed; zero[0].fixed = 0;
  std::function<ScalarP(const ScalarP&)> sc;
  std::function<Block(const Block&)> blk;
  sc = [&](const ScalarP& s) -> ScalarP {
    if (!s) return s;
    if (s->kind == Scalar::GetLocal) {
      auto it = lifted.find(s->scope);
      if (it == lifted.end()) return s;
      auto g = std::make_shared<Scalar>();
      g->kind = Scalar::Get; g->node = it->second; g->idcs = zero;
      return g;
    }
    auto o = std::make_shared<Scalar>(*s);
    if (s->kind == Scalar::LocalScope) o->body = blk(s->body);
    o->a = sc(s->a); o->b = sc(s->b); o->c = sc(s->c);
    return o;
  };
  blk = [&](const Block& b) -> Block {
    Block out;
    for (auto& sp : b) {
      auto o = std::make_shared<Stmt>(*sp);
      if (sp->kind == Stmt::For) o->body = blk(sp->body);
      if (sp->value) o->value = sc(sp->value);
      if (sp->kind == Stmt::SetLocal) {
        auto it = lifted.find(sp->scope);
        if (it != lifted.end()) { o->kind = Stmt::Set; o->node = it->second; o->idcs = zero; }
      }
      if (sp->kind == Stmt::DeclareLocal && lifted.count(sp->scope)) {
        if (!sp->needs_init) continue;
        o->kind = Stmt::ZeroOut; o->node = lifted.at(sp->scope);
      }
      out.push_back(o);
    }
    return out;
  };
  r.body = blk(r.body);
}

}  // namespace

// ---- a contraction as the prologue of the row group that consumes it ------------------------------------
// `x[o.., t] = sum_k a[..] * b[..]` with a short K (both operands unit-stride along it) whose only
// reader is the row group that follows -- Q K^T ahead of the soft-max chain, dOut V^T ahead of its
// backward chain -- is taken out of the plan: the group's kernel computes 32 rows of x at a time on
// the matrix cores into LDS and its members read them there.  Saves a launch, the write of x when it
// is planner scratch, and its read in either case.
namespace {

void fuse_row_contractions(Routine& r, Plan& plan, bool also_stored, int waves) {
  std::map<int, int> mirror_source;
  for (auto& kv : plan.mirrors) mirror_source[kv.second] = kv.first;
  for (size_t j = 0; j < plan.phases.size(); ++j) {
    Phase& G = plan.phases[j];
    if (G.kind != Phase::Generic || G.members.empty() || G.fused_x >= 0) continue;
    if (G.coop_lanes != 64 || G.row_len % 128 != 0 || G.row_len / 64 > 16 || G.row_outer_ext.empty()) continue;
    // tensors the members read without having written them, through the identity signature only
    std::set<int> written, bad;
    std::vector<int> cands;
    const size_t n_outer = G.row_outer_ext.size();
    std::string identity;
    for (size_t k = 0; k < n_outer; ++k) identity += "o" + std::to_string(k) + ",";
    identity += "r,";
    for (auto& m : G.members) {
      std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
      block_accesses(m.inner, acc, w, f, d);
      for (auto& a : acc) {
        if (a.write) { written.insert(a.node); continue; }
        if (written.count(a.node)) continue;
        if (row_signature(m, *a.idcs) != identity) { bad.insert(a.node); continue; }
        if (std::find(cands.begin(), cands.end(), a.node) == cands.end()) cands.push_back(a.node);
      }
    }
    for (int X : cands) {
      if (bad.count(X) || written.count(X)) continue;
      const Node& xn = r.node(X);
      if (xn.dims.size() != n_outer + 1 || xn.dims.back() != G.row_len) continue;
      bool dims_ok = true;
      for (size_t k = 0; k < n_outer; ++k) dims_ok = dims_ok && xn.dims[k] == G.row_outer_ext[k];
      if (!dims_ok || !(xn.prec == Prec::Bfloat16 || xn.prec == Prec::Single)) continue;
      if ((int64_t)32 * G.row_len * prec_in_bytes(xn.prec) > 65536) continue;   // the rows live in static LDS
      // the producer: the latest earlier phase that writes x
      int i = -1;
      for (int q = (int)j - 1; q >= 0; --q) if (phase_writes(plan.phases[q], X)) { i = q; break; }
      if (i < 0) continue;
      const Phase& P = plan.phases[i];
      const GemmDesc& g = P.gemm;
      if (P.kind != Phase::Contraction || g.c.node != X || g.accumulate || !g.group.empty() || !g.more.empty() || g.c_copy >= 0) continue;
      if (g.a.prec != Prec::Bfloat16 || g.b.prec != Prec::Bfloat16 || g.a.s_k != 1 || g.b.s_k != 1) continue;
      if (g.K % 16 != 0 || g.K > 128 || g.N != G.row_len) continue;
      if (!g.a.static_terms.empty() || !g.b.static_terms.empty() || !g.c.static_terms.empty() || g.c.offset != 0) continue;
      if (P.inner.size() != 1 || P.inner[0]->kind != Stmt::Set) continue;
      const Stmt& set = *P.inner[0];
      const Scalar& v = *set.value;
      if (!(v.kind == Scalar::Tern && v.tern == Ternop::Fma && v.a->kind == Scalar::Get && v.b->kind == Scalar::Get)) continue;
      // x must be written through plain iterators, one per axis
      std::vector<int> xsym;   // (-1: an axis of extent 1 written at position 0)
      bool plain = set.idcs.size() == xn.dims.size();
      std::set<int> distinct;
      for (size_t p = 0; p < set.idcs.size() && plain; ++p) {
        const AxisIndex& ix = set.idcs[p];
        if (ix.kind == AxisIndex::Fixed && ix.fixed == 0 && xn.dims[p] == 1) { xsym.push_back(-1); continue; }
        plain = ix.kind == AxisIndex::Iter && !r.is_static(ix.sym) && distinct.insert(ix.sym).second;
        xsym.push_back(ix.sym);
      }
      if (!plain || xsym.back() < 0) continue;
      Strides s1 = strides_of(r, v.a->node, v.a->idcs), s2 = strides_of(r, v.b->node, v.b->idcs);
      const int nsym = xsym.back();
      const bool first_is_a = get_stride(s1, nsym) == 0 && get_stride(s2, nsym) != 0;
      const bool second_is_a = get_stride(s2, nsym) == 0 && get_stride(s1, nsym) != 0;
      if (!first_is_a && !second_is_a) continue;
      const Strides& sa = first_is_a ? s1 : s2;
      const Strides& sb = first_is_a ? s2 : s1;
      // the one remaining loop symbol is K: unit stride in both operands
      std::vector<int> ksyms;
      auto all_syms = P.par_syms; all_syms.insert(all_syms.end(), P.seq_syms.begin(), P.seq_syms.end());
      for (int sy : all_syms) if (std::find(xsym.begin(), xsym.end(), sy) == xsym.end()) ksyms.push_back(sy);
      if (ksyms.size() != 1 || get_stride(sa, ksyms[0]) != 1 || get_stride(sb, ksyms[0]) != 1) continue;
      if (!sa.statics.empty() || !sb.statics.empty()) continue;
      Phase F;   // the fields, filled in before G is touched
      F.fused_a = g.a; F.fused_b = g.b;
      F.fused_a.offset = sa.offset; F.fused_b.offset = sb.offset;
      F.fused_k = g.K;
      F.fused_b_row = get_stride(sb, nsym);
      bool aligned = F.fused_b_row % 8 == 0 && sa.offset % 8 == 0 && sb.offset % 8 == 0;
      int m_axis = -1;
      for (size_t k = 0; k < n_outer; ++k) {
        const int64_t ak = xsym[k] < 0 ? 0 : get_stride(sa, xsym[k]), bk = xsym[k] < 0 ? 0 : get_stride(sb, xsym[k]);
        F.fused_a_stride.push_back(ak); F.fused_b_stride.push_back(bk);
        aligned = aligned && ak % 8 == 0 && bk % 8 == 0 && ak >= 0 && bk >= 0;
        if (bk == 0 && ak != 0 && G.row_outer_ext[k] % 32 == 0 && (m_axis < 0 || G.row_outer_ext[k] > G.row_outer_ext[m_axis])) m_axis = (int)k;
      }
      if (!aligned || m_axis < 0) continue;
      // nothing between the contraction and the group may touch x or write the operands; nothing else
      // before the group may read x; a later reader means the rows have to be stored
      auto source_of = [&](int node) { auto m = mirror_source.find(node); return m == mirror_source.end() ? node : m->second; };
      bool free_to_move = true;
      for (size_t q = (size_t)i + 1; q < j && free_to_move; ++q) {
        const Phase& mid = plan.phases[q];
        free_to_move = !phase_touches(mid, X) && !phase_writes(mid, g.a.node) && !phase_writes(mid, g.b.node) &&
                       !phase_writes(mid, source_of(g.a.node)) && !phase_writes(mid, source_of(g.b.node));
      }
      if (!free_to_move) continue;
      // ... nor may the group itself: a member's stores in one workgroup would race with another
      // workgroup's prologue loads, which a kernel boundary used to order
      if (phase_writes(G, g.a.node) || phase_writes(G, g.b.node) || phase_writes(G, source_of(g.a.node)) ||
          phase_writes(G, source_of(g.b.node)))
        continue;
      bool later_reader = false;
      for (size_t q = j + 1; q < plan.phases.size(); ++q) later_reader = later_reader || phase_touches(plan.phases[q], X);
      // When the rows have to be stored anyway the separate launches were measured faster (the
      // transformer step's backward soft-max chain: 112 us apart, 150 us as one kernel).
      if ((xn.mode == Mode::Ctx || later_reader) && !also_stored) continue;
      G.fused_x = X;
      G.fused_x_store = xn.mode == Mode::Ctx || later_reader;
      G.fused_a = F.fused_a; G.fused_b = F.fused_b;
      G.fused_a_stride = F.fused_a_stride; G.fused_b_stride = F.fused_b_stride;
      G.fused_b_row = F.fused_b_row; G.fused_k = F.fused_k; G.fused_m_axis = m_axis;
      G.fused_waves = waves == 4 || waves == 8 || waves == 16 ? waves : G.row_len <= 512 ? 16 : 8;
      G.flops = P.flops;
      const double x_bytes = (double)xn.size_in_bytes();
      G.bytes += P.bytes - 2.0 * x_bytes + (G.fused_x_store ? x_bytes : 0.0);   // x is neither written (unless stored) nor read
      G.label = P.label + " -> " + G.label;
      if (!G.fused_x_store) r.nodes.at(X).mode = Mode::Virtual;   // no memory behind it any more
      plan.phases.erase(plan.phases.begin() + i);
      --j;
      break;
    }
  }
}


// ---- ... and a contraction as the epilogue of the row group that produces its operand -------------------
// `c[o.., n] (=) sum_t y[o.., t] * b[.., t, n]` right behind a row group with a prologue, y being what one
// of its members stores per row position (attention weights times V: lib/nn_blocks.ml:233-236): the
// group's workgroup, which holds 32 finished rows of y, multiplies them with b itself.  Saves a launch
// and the read of y; y is still stored (it is a context node).
void fuse_row_projections(Routine& r, Plan& plan) {
  std::map<int, int> mirror_source;
  for (auto& kv : plan.mirrors) mirror_source[kv.second] = kv.first;
  auto source_of = [&](int node) { auto m = mirror_source.find(node); return m == mirror_source.end() ? node : m->second; };
  for (size_t j = 0; j < plan.phases.size(); ++j) {
    Phase& G = plan.phases[j];
    if (G.kind != Phase::Generic || G.members.empty() || G.fused_x < 0 || G.proj_y >= 0) continue;
    const size_t n_outer = G.row_outer_ext.size();
    const int ma = G.fused_m_axis;
    std::string identity;
    for (size_t k = 0; k < n_outer; ++k) identity += "o" + std::to_string(k) + ",";
    identity += "r,";
    // per-position results of the group: node -> index of the last member that stores it
    std::map<int, size_t> stored_by;
    for (size_t mi = 0; mi < G.members.size(); ++mi) {
      const Phase& m = G.members[mi];
      if (m.inner.size() != 1 || m.inner[0]->kind != Stmt::Set) continue;
      const Stmt& st = *m.inner[0];
      if (m.row_role == Phase::RowPointwise && row_signature(m, st.idcs) == identity) stored_by[st.node] = mi;
      else stored_by.erase(st.node);
    }
    for (size_t i = j + 1; i < plan.phases.size() && G.proj_y < 0; ++i) {
      const Phase& P = plan.phases[i];
      if (P.kind != Phase::Contraction) continue;
      const GemmDesc& g = P.gemm;
      if (g.accumulate || !g.group.empty() || !g.more.empty() || g.epi_bias >= 0 || g.epi_relu >= 0) continue;
      if (P.inner.size() != 1 || P.inner[0]->kind != Stmt::Set) continue;
      const Stmt& set = *P.inner[0];
      const Scalar& v = *set.value;
      const Scalar *pa = nullptr, *pb = nullptr;
      if (v.kind == Scalar::Tern && v.tern == Ternop::Fma) { pa = v.a.get(); pb = v.b.get(); }
      else if (v.kind == Scalar::Bin && v.bin == Binop::Add) {
        const Scalar* mul = v.b->kind == Scalar::Bin && v.b->bin == Binop::Mul ? v.b.get() : v.a->kind == Scalar::Bin && v.a->bin == Binop::Mul ? v.a.get() : nullptr;
        if (mul) { pa = mul->a.get(); pb = mul->b.get(); }
      }
      if (!pa || !pb || pa->kind != Scalar::Get || pb->kind != Scalar::Get) continue;
      const Scalar* yget = stored_by.count(pa->node) ? pa : stored_by.count(pb->node) ? pb : nullptr;
      if (!yget) continue;
      const Scalar* bget = yget == pa ? pb : pa;
      const int Y = yget->node;
      if (stored_by.count(bget->node) || bget->node == G.fused_x) continue;
      const Node& yn = r.node(Y);
      if (!(yn.prec == Prec::Bfloat16 || yn.prec == Prec::Single) || yn.dims.size() != n_outer + 1 || yn.dims.back() != G.row_len) continue;
      // which operand of the planned contraction stands for y (itself, or the bf16 copy its stores keep in step)
      auto is_y = [&](const GemmOperand& o) { return o.node == Y || source_of(o.node) == Y; };
      if (is_y(g.a) == is_y(g.b)) continue;
      const GemmOperand& yop = is_y(g.a) ? g.a : g.b;
      const GemmOperand& bop = is_y(g.a) ? g.b : g.a;
      if (yop.prec != Prec::Bfloat16 || bop.prec != Prec::Bfloat16) continue;
      if (r.node(bop.node).dims != r.node(bget->node).dims) continue;   // (a bf16 copy has its source's layout)
      if (g.c.prec != Prec::Bfloat16 || g.c_copy >= 0) continue;   // (what the attention blocks produce; fp32 results and copies stay launches)
      // y read through plain iterators, one per axis; those loops run over the group's rows
      std::map<int, std::pair<int64_t, int64_t>> range;   // symbol -> (from, extent)
      for (size_t q = 0; q < P.par_syms.size(); ++q) range[P.par_syms[q]] = {P.par_from[q], P.par_ext[q]};
      for (size_t q = 0; q < P.seq_syms.size(); ++q) range[P.seq_syms[q]] = {P.seq_from[q], P.seq_to[q] - P.seq_from[q] + 1};
      std::vector<int> ysym;
      bool plain = yget->idcs.size() == yn.dims.size();
      std::set<int> distinct;
      for (size_t p = 0; p < yget->idcs.size() && plain; ++p) {
        const AxisIndex& ix = yget->idcs[p];
        const int64_t want = p < n_outer ? G.row_outer_ext[p] : G.row_len;
        if (ix.kind == AxisIndex::Fixed && ix.fixed == 0 && want == 1) { ysym.push_back(-1); continue; }
        plain = ix.kind == AxisIndex::Iter && !r.is_static(ix.sym) && distinct.insert(ix.sym).second && range.count(ix.sym) &&
                range[ix.sym].first == 0 && range[ix.sym].second == want && yn.dims[p] == want;
        ysym.push_back(ix.sym);
      }
      if (!plain || ysym.back() < 0) continue;
      const int tsym = ysym.back();
      std::vector<int> others;
      for (auto& kv : range) if (!distinct.count(kv.first) && kv.second.second != 1) others.push_back(kv.first);
      if (others.size() != 1 || range[others[0]].first != 0) continue;
      const int nsym = others[0];
      const int64_t N = range[nsym].second;
      if (N % 32 != 0 || N > 128) continue;
      const Strides sb = strides_of(r, bget->node, bget->idcs), sc = strides_of(r, set.node, set.idcs);
      if (!sb.statics.empty() || !sc.statics.empty()) continue;
      if (get_stride(sb, nsym) != 1 || get_stride(sc, nsym) != 1 || get_stride(sc, tsym) != 0 || get_stride(sb, tsym) <= 0) continue;
      Phase F;
      bool ok = sb.offset % 4 == 0 && sc.offset % 4 == 0 && sb.offset >= 0 && sc.offset >= 0;
      for (size_t k = 0; k < n_outer; ++k) {
        const int64_t bk = ysym[k] < 0 ? 0 : get_stride(sb, ysym[k]), ck = ysym[k] < 0 ? 0 : get_stride(sc, ysym[k]);
        F.proj_b_stride.push_back(bk); F.proj_c_stride.push_back(ck);
        ok = ok && bk >= 0 && ck >= 0 && ck % 4 == 0 && ((int)k != ma || (bk == 0 && ck > 0));
      }
      if (!ok) continue;
      // c must keep its rows apart: one (outer.., n) cell per (rows, n)
      {
        std::vector<std::pair<int64_t, int64_t>> ax{{1, N}};   // (stride, extent)
        for (size_t k = 0; k < n_outer; ++k) if (G.row_outer_ext[k] > 1) ax.push_back({F.proj_c_stride[k], G.row_outer_ext[k]});
        std::sort(ax.begin(), ax.end());
        for (size_t q = 1; q < ax.size(); ++q) ok = ok && ax[q].first >= ax[q - 1].first * ax[q - 1].second;
      }
      if (!ok) continue;
      // the contraction moves up to the group: nothing in between may write y or b, or touch c
      bool free_to_move = true;
      for (size_t q = j + 1; q < i && free_to_move; ++q) {
        const Phase& mid = plan.phases[q];
        free_to_move = !phase_writes(mid, Y) && !phase_writes(mid, yop.node) &&
                       !phase_writes(mid, bop.node) && !phase_writes(mid, source_of(bop.node)) && !phase_touches(mid, g.c.node) &&
                       (g.c_copy < 0 || !phase_touches(mid, g.c_copy));
        auto cm = plan.mirrors.find(g.c.node);
        if (cm != plan.mirrors.end()) free_to_move = free_to_move && !phase_touches(mid, cm->second);
      }
      if (!free_to_move || plan.mirrors.count(g.c.node)) continue;
      // ... and the group itself must not touch c or write b
      if (phase_touches(G, g.c.node) || phase_writes(G, bop.node) || phase_writes(G, source_of(bop.node))) continue;
      // the sum over t is split over the waves that the static LDS budget lets hold a partial result;
      // with fewer than four waves at work the separate launch is faster (measured: 1024-long rows,
      // whose bf16 tile fills the 64 KiB: 2.78 against 2.69 ms for the attention step)
      const int NW = G.fused_waves, NB = (int)(N / 32);
      int KP = 1;
      while (KP * 2 * NB <= NW && KP < 4 && (G.row_len / 16) % (KP * 2) == 0 &&
             32 * G.row_len * (int64_t)prec_in_bytes(r.node(G.fused_x).prec) + (int64_t)(KP * 2) * 32 * N * 4 <= 60 * 1024) KP *= 2;
      if (KP * NB < 4) continue;
      G.proj_kp = KP;
      G.proj_y = Y;
      G.proj_b = bop; G.proj_b.offset = sb.offset;
      G.proj_c = g.c; G.proj_c.offset = sc.offset;
      G.proj_b_stride = F.proj_b_stride; G.proj_c_stride = F.proj_c_stride;
      G.proj_b_row = get_stride(sb, tsym);
      G.proj_n = N;
      G.proj_c_copy = g.c_copy;
      G.flops += P.flops;
      G.bytes += P.bytes - (double)yn.num_elems() * 2.0;   // y is not read back
      G.label += " -> " + P.label;
      plan.phases.erase(plan.phases.begin() + i);
      break;
    }
  }
}

}  // namespace

// ---- contractions off the critical path ---------------------------------------------------------------
// A weight gradient `dW += dY^T X` is needed only when the optimiser runs, dozens of phases later, while
// the kernels that follow it form a chain in which each waits for the one before and few fill the
// chip.  Such a contraction is put on the device's second queue: it starts once the main queue has
// reached its position and runs beside the phases that follow; the first phase that touches its result
// or rewrites one of its operands waits for it.  Same kernels, same operands, same bits.
namespace {

void assign_side_queue(Plan& plan, bool also_generated) {
  std::map<int, int> mirror_source;
  for (auto& kv : plan.mirrors) mirror_source[kv.second] = kv.first;
  auto source_of = [&](int node) { auto m = mirror_source.find(node); return m == mirror_source.end() ? node : m->second; };
  struct Sets { std::vector<int> outs, ins; bool ok = true; };
  // what a generated phase reads and writes (false: something in it is not tracked per tensor)
  std::function<bool(const Phase&, Sets&)> generic_sets = [&](const Phase& ph, Sets& s) -> bool {
    if (!ph.serial_members.empty() || ph.fused_x >= 0 || ph.proj_y >= 0) return false;
    if (!ph.parallel_members.empty()) { for (auto& m : ph.parallel_members) if (!generic_sets(m, s)) return false; return true; }
    if (!ph.members.empty()) { for (auto& m : ph.members) if (!generic_sets(m, s)) return false; return true; }
    std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
    block_accesses(ph.inner, acc, w, f, d);
    if (w || f) return false;
    for (auto& a : acc) (a.write ? s.outs : s.ins).push_back(a.node);
    return true;
  };
  auto sets_of = [&](const Phase& ph) {
    Sets s;
    if (ph.kind == Phase::Generic) {
      s.ok = generic_sets(ph, s);
    } else {
      const GemmDesc& g = ph.gemm;
      s.outs = {g.c.node}; s.ins = {g.a.node, g.b.node};
      if (g.c_copy >= 0) s.outs.push_back(g.c_copy);
      if (g.epi_relu >= 0) s.outs.push_back(g.epi_relu);
      if (g.epi_bias >= 0) s.ins.push_back(g.epi_bias);
      for (auto& m : g.group) { s.outs.push_back(m.c.node); if (m.c_copy >= 0) s.outs.push_back(m.c_copy); s.ins.push_back(m.a.node); s.ins.push_back(m.b.node); }
      for (auto& pr : g.more) { s.ins.push_back(pr.first.node); s.ins.push_back(pr.second.node); }
    }
    for (int o : std::vector<int>(s.outs)) { auto m = plan.mirrors.find(o); if (m != plan.mirrors.end()) s.outs.push_back(m->second); }
    return s;
  };
  auto conflicts = [&](const Sets& s, const Phase& later) {
    for (int o : s.outs) if (phase_touches(later, o)) return true;
    for (int i : s.ins) if (phase_writes(later, i) || phase_writes(later, source_of(i))) return true;
    return false;
  };
  constexpr size_t kMinSlack = 4;   // phases that must lie between the phase and its first dependant
  for (size_t p = 0; p < plan.phases.size(); ++p) {
    Phase& ph = plan.phases[p];
    // a contraction of some size, or a generated kernel that moves a few MB (the partial sums of bias and
    // gain gradients: column sums over all rows, wanted by the optimiser only)
    const bool contraction = ph.kind == Phase::Contraction && ph.flops >= 4e9;
    const bool generated = also_generated && ph.kind == Phase::Generic && ph.bytes >= (double)(4 << 20);
    if (!contraction && !generated) continue;
    const Sets s = sets_of(ph);
    if (!s.ok) continue;
    size_t q = p + 1;
    while (q < plan.phases.size() && !conflicts(s, plan.phases[q])) ++q;
    if (q - p > kMinSlack && q < plan.phases.size()) ph.stream = 1;
    else if (q - p > kMinSlack && contraction) ph.stream = 1;
  }
  // every phase of the main queue waits for the side-queue phases before it that it conflicts with
  // (side-queue phases among themselves run in order)
  for (size_t p = 0; p < plan.phases.size(); ++p) {
    if (plan.phases[p].stream != 1) continue;
    const Sets s = sets_of(plan.phases[p]);
    for (size_t q = p + 1; q < plan.phases.size(); ++q)
      if (plan.phases[q].stream == 0 && conflicts(s, plan.phases[q])) plan.phases[q].wait_for.push_back((int)p);
  }
}

}  // namespace

// ---- pointwise consumers folded into a contraction's epilogue ----------------------------------------
// `y[..] := x + bias[n]` (either order) right after the contraction that produces the inlined product
// x, optionally followed by `z[..] := relu(y[..])`: an mlp layer (lib/nn_blocks.ml:108-135).  The
// contraction then stores y (and z) itself; x, which was planner scratch, is never written.
namespace {

void fold_epilogues(Routine& r, Plan& plan) {
  std::set<int> scratch;
  for (auto& n : plan.scratch) scratch.insert(n.id);
  auto identity_set = [&](const Phase& q, int64_t rank) -> const Stmt* {   // Set through plain full-range iterators, no loops left inside a thread
    if (q.kind != Phase::Generic || !q.members.empty() || !q.seq_syms.empty() || q.coop_lanes != 1) return nullptr;
    if (q.inner.size() != 1 || q.inner[0]->kind != Stmt::Set) return nullptr;
    const Stmt& st = *q.inner[0];
    if ((int64_t)st.idcs.size() != rank || !writes_whole_node(r, q, st.node)) return nullptr;
    for (auto& ix : st.idcs) if (ix.kind != AxisIndex::Iter) return nullptr;
    return &st;
  };
  for (size_t i = 0; i + 1 < plan.phases.size(); ++i) {
    Phase& P = plan.phases[i];
    GemmDesc& g = P.gemm;
    if (P.kind != Phase::Contraction || !scratch.count(g.c.node) || g.accumulate || g.c_copy >= 0 || !g.group.empty() || !g.more.empty()) continue;
    const int X = g.c.node;
    const Node xn = r.node(X);
    if (xn.prec != Prec::Bfloat16 || g.c.offset != 0 || !g.c.static_terms.empty()) continue;
    int64_t written = g.M * g.N;
    for (int b = 0; b < g.nbatch; ++b) written *= g.batch_ext[b];
    if (written != xn.num_elems() || g.N != xn.dims.back()) continue;
    const Stmt* ys = identity_set(plan.phases[i + 1], (int64_t)xn.dims.size());
    if (!ys) continue;
    const Node& yn = r.node(ys->node);
    // (the visit rule inlines y as well when z is its only reader: one statement z := relu(x + bias))
    const bool relu_of_sum = ys->value->kind == Scalar::Un && ys->value->un == Unop::Relu && ys->value->a->kind == Scalar::Bin;
    const Scalar& v = relu_of_sum ? *ys->value->a : *ys->value;
    if (yn.prec != Prec::Bfloat16 || yn.dims != xn.dims || !(v.kind == Scalar::Bin && v.bin == Binop::Add)) continue;
    const Scalar* xg = nullptr; const Scalar* bg = nullptr;
    for (const Scalar* s : {v.a.get(), v.b.get()}) {
      if (s->kind == Scalar::Get && s->node == X && s->idcs == ys->idcs) xg = s;
      else if (s->kind == Scalar::Get && s->idcs.size() == 1 && s->idcs[0] == ys->idcs.back()) bg = s;
    }
    if (!xg || !bg) continue;
    const Node& bn = r.node(bg->node);
    if (bn.prec != Prec::Bfloat16 || bn.dims.size() != 1 || bn.dims[0] != g.N || bn.mode == Mode::Virtual) continue;
    // an optional relu of y right behind
    int Z = relu_of_sum ? ys->node : -1;   // C itself receives the relu
    if (!relu_of_sum && i + 2 < plan.phases.size()) {
      const Stmt* zs = identity_set(plan.phases[i + 2], (int64_t)xn.dims.size());
      if (zs && zs->node != ys->node) {
        const Node& zn = r.node(zs->node);
        const Scalar& zv = *zs->value;
        if (zn.prec == Prec::Bfloat16 && zn.dims == xn.dims && zv.kind == Scalar::Un && zv.un == Unop::Relu && zv.a->kind == Scalar::Get &&
            zv.a->node == ys->node && zv.a->idcs == zs->idcs)
          Z = zs->node;
      }
    }
    // x must have no other reader
    bool alone = true;
    for (size_t q = 0; q < plan.phases.size(); ++q) if (q != i && q != i + 1 && phase_touches(plan.phases[q], X)) alone = false;
    if (!alone) continue;
    const double tensor_bytes = (double)xn.size_in_bytes();
    g.c.node = ys->node;
    g.epi_bias = bg->node;
    g.epi_relu = Z;
    P.bytes += (double)bn.size_in_bytes() + (Z >= 0 && !relu_of_sum ? tensor_bytes : 0.0);
    P.label += " + bias" + std::string(Z >= 0 ? " + relu" : "");
    r.nodes.at(X).mode = Mode::Virtual;   // never stored
    plan.phases.erase(plan.phases.begin() + i + 1, plan.phases.begin() + i + (Z >= 0 && !relu_of_sum ? 3 : 2));
  }
}

}  // namespace

Plan make_plan(Routine& r, const PlanOptions& requested) {
  PlanOptions opt = requested;
  if (r.merge_node >= 0) {
    // routines that read the merge buffer are short pointwise accumulations (cuda_backend.ml:1009-1011
    // binds the buffer at launch): plain one-kernel-per-statement plans, no fusing rewrites
    opt.enable_mfma = opt.enable_row_groups = opt.enable_serial_group = opt.enable_bf16_copies = opt.fuse_row_contractions = false;
  }
  if (opt.debug_log) {
    opt.enable_mfma = opt.enable_coop = opt.enable_row_groups = opt.enable_serial_group = opt.enable_parallel_groups = false;
    opt.enable_bf16_copies = opt.fuse_row_contractions = opt.side_queue = opt.fuse_epilogues = false;
  }
  if (opt.reuse_stored && !opt.debug_log && r.merge_node < 0) reuse_stored_values(r);
  struct SeqGuard { bool old; SeqGuard(bool v) : old(g_all_sequential) { g_all_sequential = v; } ~SeqGuard() { g_all_sequential = old; } } seq_guard(opt.debug_log);
  Plan plan;
  plan.debug_log = opt.debug_log;
  plan.row_vec4 = opt.row_vec4;
  plan.use_graphs = opt.use_graphs;
  plan.large_index = opt.large_models;
  for (auto& kv : r.nodes) if (kv.second.num_elems() > (int64_t)0x7FFFFFFF) plan.large_index = true;
  std::string label;
  int next_sym = 0;
  Bf16Copies copies;
  std::set<int> debug_zeroed;      // nodes whose first Zero_out has been seen (logging only)
  lift_routine_locals(r, plan);
  std::vector<std::string> pending_comments;
  Block top = r.body;
  for (size_t ti = 0; ti < top.size(); ++ti) {
    StmtP sp = top[ti];
    if (sp->kind == Stmt::Comment) { label = sp->text; if (opt.debug_log) pending_comments.push_back(sp->text); continue; }
    Phase ph;
    ph.label = label;
    ph.stmt = sp;
    if (sp->kind == Stmt::ZeroOut && opt.debug_log) {
      // With logging a Zero_out is the loop nest of `tn[..] := 0` statements that the reference prints,
      // each logging its element under the text `<ident> := 0` (c_syntax.ml:468-479) -- except the
      // first function-scope Zero_out of a local node that its declaration already zeroes
      // (c_syntax.ml:424-432), which prints nothing.
      const Node& n = r.node(sp->node);
      if (n.mode == Mode::Virtual) continue;
      const bool first = debug_zeroed.insert(sp->node).second;
      if (first && n.zero_initialized_by_code && n.mode == Mode::Local) {
        // (the node still needs its zeros: a fill without log lines)
        ph.kind = Phase::Fill;
        ph.fill_node = sp->node;
        ph.bytes = (double)n.size_in_bytes();
        plan.phases.push_back(std::move(ph));
        continue;
      }
      auto set = std::make_shared<Stmt>();
      set->kind = Stmt::Set; set->node = sp->node; set->text = n.ident + " := 0";
      auto zero = std::make_shared<Scalar>();
      zero->kind = Scalar::Const; zero->cst = 0.0;
      set->value = zero;
      StmtP nest = set;
      std::vector<int> syms;
      for (size_t ax = 0; ax < n.dims.size(); ++ax) syms.push_back(fresh_symbol(r, &next_sym));
      for (size_t ax = 0; ax < n.dims.size(); ++ax) { AxisIndex a; a.kind = AxisIndex::Iter; a.sym = syms[ax]; set->idcs.push_back(a); }
      for (size_t ax = n.dims.size(); ax-- > 0;) {
        auto loop = std::make_shared<Stmt>();
        loop->kind = Stmt::For; loop->sym = syms[ax]; loop->from = 0; loop->to = n.dims[ax] - 1;
        loop->body.push_back(nest);
        nest = loop;
      }
      sp = nest;
      ph.stmt = sp;
    }
    if (sp->kind == Stmt::ZeroOut) {
      const Node& n = r.node(sp->node);
      if (n.mode == Mode::Virtual) continue;
      ph.kind = Phase::Fill;
      ph.fill_node = sp->node;
      ph.bytes = (double)n.size_in_bytes();
      plan.phases.push_back(std::move(ph));
      auto mirror = plan.mirrors.find(sp->node);
      if (mirror != plan.mirrors.end()) {   // the bf16 copy follows (bf16 zero is all-zero bits)
        Phase f;
        f.kind = Phase::Fill; f.label = "zero bf16 copy of " + n.ident; f.fill_node = mirror->second;
        f.bytes = (double)r.node(mirror->second).size_in_bytes();
        plan.phases.push_back(std::move(f));
      }
      continue;
    }
    if (sp->kind == Stmt::DeclareLocal || sp->kind == Stmt::SetLocal)
      throw InvalidArgument("hip backend: Set_local of an undeclared scalar at routine scope (routine " + r.name + ")");
    devirtualise(r, sp, opt, plan, label);
    if (!analyze_nest(r, sp, ph)) continue;

    // fold the preceding Zero_out of the accumulation target into this phase (the accumulation then
    // starts from zero instead of reading the array) when no phase in between touches the array and
    // the nest overwrites all of it: every axis is a full-range parallel iterator or has extent 1.
    Binop accum;
    int fill_at = -1;
    if (!opt.debug_log && reduction_shape(r, ph, &accum) && accum == Binop::Add) {
      // the latest Zero_out of the target with nothing touching the target in between
      const int target = ph.inner[0]->node;
      for (int q = (int)plan.phases.size() - 1; q >= 0; --q) {
        const Phase& prev = plan.phases[q];
        if (prev.kind == Phase::Fill && prev.fill_node == target) { fill_at = q; break; }
        if (phase_touches(prev, target)) break;
      }
    }
    if (fill_at >= 0) {
      const Stmt& set = *ph.inner[0];
      const Node& n = r.node(set.node);
      bool full = true;
      for (size_t p = 0; p < set.idcs.size() && full; ++p) {
        const AxisIndex& a = set.idcs[p];
        if (a.kind == AxisIndex::Fixed) full = n.dims[p] == 1;
        else if (a.kind == AxisIndex::Iter) {
          full = false;
          for (size_t i = 0; i < ph.par_syms.size(); ++i)
            if (ph.par_syms[i] == a.sym) full = ph.par_from[i] == 0 && ph.par_ext[i] == n.dims[p];
        } else full = false;
      }
      if (full) { ph.fused_zero_init = true; plan.phases.erase(plan.phases.begin() + fill_at); copies.erased((size_t)fill_at); }
    }
    // a dead fill: the nest stores to every element of a tensor without reading it, and nothing has
    // touched the tensor since its Zero_out
    if (!opt.debug_log && fill_at < 0 && ph.seq_syms.empty() && ph.inner.size() == 1 && ph.inner[0]->kind == Stmt::Set) {
      const int target = ph.inner[0]->node;
      std::vector<Access> acc; bool w = false, f = false; std::set<ScopeId> d;
      block_accesses(ph.inner, acc, w, f, d);
      bool reads_target = w || f;
      for (auto& a : acc) if (!a.write && a.node == target) reads_target = true;
      if (!reads_target && writes_whole_node(r, ph, target)) {
        for (int q = (int)plan.phases.size() - 1; q >= 0; --q) {
          const Phase& prev = plan.phases[q];
          if (prev.kind == Phase::Fill && prev.fill_node == target) { plan.phases.erase(plan.phases.begin() + q); copies.erased((size_t)q); break; }
          if (phase_touches(prev, target)) break;
        }
      }
    }

    if (!match_contraction(r, ph, opt)) {
      ph.kind = Phase::Generic;
      split_reduction(r, ph, opt, plan, &next_sym);
      choose_coop(r, ph, opt);
      account_bytes(r, ph);
    } else {
      set_contraction_bytes(ph);
      if (opt.enable_bf16_copies) use_bf16_copies(r, plan, ph, copies, &next_sym);
    }
    ph.comments_before.swap(pending_comments);
    plan.phases.push_back(std::move(ph));
  }
  plan.trailing_comments.swap(pending_comments);
  if (opt.enable_mfma && opt.fuse_epilogues) fold_epilogues(r, plan);
  if (opt.enable_mfma && opt.merge_chains) merge_contractions(plan, true);
  if (opt.enable_mfma && opt.group_contractions) merge_contractions(plan, false, opt.group_window);
  if (opt.enable_coop && opt.enable_row_groups) group_rows(r, plan);
  if (opt.enable_mfma && opt.enable_coop && opt.enable_row_groups && opt.fuse_row_contractions) fuse_row_contractions(r, plan, opt.fuse_stored_rows, opt.row_tile_waves);
  if (opt.enable_mfma && opt.enable_coop && opt.enable_row_groups && opt.fuse_row_contractions && opt.fuse_row_projections) fuse_row_projections(r, plan);
  if (opt.enable_serial_group) serialise_tiny(r, plan);
  if (opt.enable_coop && opt.enable_parallel_groups) group_independent(r, plan);
  if (opt.enable_mfma && opt.side_queue && r.merge_node < 0) assign_side_queue(plan, opt.side_queue_generated);
  return plan;
}

}  // namespace ocannl
