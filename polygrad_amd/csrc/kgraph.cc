#include "kgraph.h"

#include <algorithm>
#include <climits>
#include <cstdint>
#include <cstdlib>
#include <cstring>

namespace polyhip {

static const char *const kOpNames[] = {
  "?", "DEFINE_VAR", "BIND", "SPECIAL", "DEFINE_LOCAL", "DEFINE_REG", "NOOP", "REWRITE_ERROR", "PARAM",
  "CALL", "PROGRAM", "LINEAR", "SOURCE", "BINARY", "SINK", "AFTER", "GROUP", "GEP", "VECTORIZE", "INDEX",
  "LOAD", "STORE", "WMMA", "CAST", "BITCAST", "EXP2", "LOG2", "SIN", "SQRT", "RECIPROCAL", "NEG", "TRUNC",
  "ADD", "MUL", "SHL", "SHR", "IDIV", "MAX", "MOD", "CMPLT", "CMPNE", "CMPEQ", "XOR", "OR", "AND",
  "THREEFRY", "SUB", "FDIV", "POW", "WHERE", "MULACC", "BARRIER", "RANGE", "IF", "END", "ENDIF", "VCONST",
  "CONST", "CUSTOM", "CUSTOMI", "INS", "UNIQUE", "DEVICE", "ASSIGN", "LUNIQUE", "CONTIGUOUS",
  "CONTIGUOUS_BACKWARD", "DETACH", "BUFFERIZE", "COPY", "BUFFER", "BUFFER_VIEW", "MSELECT", "MSTACK",
  "ENCDEC", "RESHAPE", "PERMUTE", "EXPAND", "PAD", "SHRINK", "FLIP", "MULTI", "REDUCE_AXIS", "REDUCE",
  "ALLREDUCE", "UNROLL", "CONTRACT", "VCAT", "PTRCAT"};

const char *op_name(PolyOps op) {
  int i = (int)op;
  if (i < 1 || i >= (int)(sizeof(kOpNames) / sizeof(kOpNames[0]))) return "?";
  return kOpNames[i];
}

static const int64_t kBig = (int64_t)1 << 60;
static int64_t clampb(__int128 v) {
  if (v > kBig) return kBig;
  if (v < -kBig) return -kBig;
  return (int64_t)v;
}

// ── Lin arithmetic ────────────────────────────────────────────────────────

static std::string lin_key(const Lin &l) {
  std::string k = strf("%lld", (long long)l.c0);
  for (const Term &t : l.terms) k += strf("|%lld*%d", (long long)t.coef, t.atom);
  return k;
}

// a * b and a + b in 64 bits; on overflow *flag is set and the result is harmless
static int64_t ck_mul(int64_t a, int64_t b, bool *flag) {
  int64_t r;
  if (__builtin_mul_overflow(a, b, &r)) { *flag = true; return 0; }
  return r;
}
static int64_t ck_add(int64_t a, int64_t b, bool *flag) {
  int64_t r;
  if (__builtin_add_overflow(a, b, &r)) { *flag = true; return 0; }
  return r;
}

Lin KernelGraph::lin_add(const Lin &a, const Lin &b, int64_t sb) const {
  Lin r;
  bool *of = &lin_overflow;
  r.c0 = ck_add(a.c0, ck_mul(sb, b.c0, of), of);
  size_t i = 0, j = 0;
  while (i < a.terms.size() || j < b.terms.size()) {
    if (j >= b.terms.size() || (i < a.terms.size() && a.terms[i].atom < b.terms[j].atom)) {
      r.terms.push_back(a.terms[i++]);
    } else if (i >= a.terms.size() || b.terms[j].atom < a.terms[i].atom) {
      r.terms.push_back({ck_mul(sb, b.terms[j].coef, of), b.terms[j].atom});
      j++;
    } else {
      int64_t c = ck_add(a.terms[i].coef, ck_mul(sb, b.terms[j].coef, of), of);
      if (c != 0) r.terms.push_back({c, a.terms[i].atom});
      i++; j++;
    }
  }
  return r;
}

// c*(X/c) + (X%c) == X for X >= 0: recombine a DIV atom with its MOD twin.
Lin KernelGraph::lin_recombine(const Lin &a) const {
  for (size_t i = 0; i < a.terms.size(); i++) {
    const Atom &m = atoms[(size_t)a.terms[i].atom];
    if (m.kind != Atom::MOD) continue;
    for (size_t j = 0; j < a.terms.size(); j++) {
      const Atom &d = atoms[(size_t)a.terms[j].atom];
      if (d.kind != Atom::DIV) continue;
      if (a.terms[j].coef != a.terms[i].coef * m.c) continue;
      if (d.c != m.c || lin_key(d.inner) != lin_key(m.inner)) {
        // nested form: c*(Y/(p*c)) + (Y/p)%c == Y/p
        if (m.inner.c0 != 0 || m.inner.terms.size() != 1 || m.inner.terms[0].coef != 1) continue;
        const Atom &in = atoms[(size_t)m.inner.terms[0].atom];
        if (in.kind != Atom::DIV || d.c != in.c * m.c || lin_key(d.inner) != lin_key(in.inner)) continue;
        int64_t lo2, hi2;
        lin_bounds(in.inner, &lo2, &hi2);
        if (lo2 < 0) continue;
        Lin rest2;
        rest2.c0 = a.c0;
        for (size_t t = 0; t < a.terms.size(); t++)
          if (t != i && t != j) rest2.terms.push_back(a.terms[t]);
        return lin_recombine(lin_add(rest2, lin_scale(m.inner, a.terms[i].coef)));
      }
      int64_t lo, hi;
      lin_bounds(d.inner, &lo, &hi);
      if (lo < 0) continue;
      Lin rest;
      rest.c0 = a.c0;
      for (size_t t = 0; t < a.terms.size(); t++)
        if (t != i && t != j) rest.terms.push_back(a.terms[t]);
      return lin_recombine(lin_add(rest, lin_scale(d.inner, a.terms[i].coef)));
    }
  }
  return a;
}

Lin KernelGraph::lin_scale(const Lin &a, int64_t s) const {
  Lin r;
  if (s == 0) return r;
  r.c0 = ck_mul(a.c0, s, &lin_overflow);
  for (const Term &t : a.terms) {
    const int64_t c = ck_mul(t.coef, s, &lin_overflow);
    if (c != 0) r.terms.push_back({c, t.atom});
  }
  return r;
}

void KernelGraph::lin_bounds(const Lin &a, int64_t *lo, int64_t *hi) const {
  __int128 l = a.c0, h = a.c0;
  for (const Term &t : a.terms) {
    const Atom &at = atoms[(size_t)t.atom];
    if (t.coef > 0) { l += (__int128)t.coef * at.lo; h += (__int128)t.coef * at.hi; }
    else            { l += (__int128)t.coef * at.hi; h += (__int128)t.coef * at.lo; }
  }
  *lo = clampb(l);
  *hi = clampb(h);
}


int KernelGraph::intern_atom(const Atom &a) {
  for (size_t i = 0; i < atoms.size(); i++) {
    const Atom &b = atoms[i];
    if (a.kind != b.kind) continue;
    if (a.kind == Atom::DIV || a.kind == Atom::MOD) {
      if (a.c == b.c && lin_key(a.inner) == lin_key(b.inner)) return (int)i;
    } else if (a.node == b.node) {
      return (int)i;
    }
  }
  atoms.push_back(a);
  return (int)atoms.size() - 1;
}

int KernelGraph::atom_for_node(int node, Atom::Kind kind, int64_t lo, int64_t hi) {
  Atom a;
  a.kind = kind; a.node = node; a.lo = lo; a.hi = hi;
  return intern_atom(a);
}

static int64_t floordiv(int64_t a, int64_t b) {
  int64_t q = a / b, r = a % b;
  return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q;
}

static int64_t gcd64(int64_t a, int64_t b) {
  if (a < 0) a = -a;
  if (b < 0) b = -b;
  while (b) { int64_t t = a % b; a = b; b = t; }
  return a;
}

// Split a = c*Q + R with every term of Q an exact multiple and 0 <= const(R) < c.
static void split_multiple(const Lin &a, int64_t c, Lin *Q, Lin *R) {
  Q->terms.clear(); R->terms.clear();
  int64_t q0 = floordiv(a.c0, c);
  Q->c0 = q0;
  R->c0 = a.c0 - q0 * c;
  for (const Term &t : a.terms) {
    if (t.coef % c == 0) Q->terms.push_back({t.coef / c, t.atom});
    else R->terms.push_back(t);
  }
}

Lin KernelGraph::lin_div(const Lin &a, int64_t c) {
  if (c == 1) return a;
  if (a.is_const()) return lin_const(a.c0 / c);  // C semantics: truncation
  int64_t lo, hi;
  lin_bounds(a, &lo, &hi);
  if (c > 0 && lo >= 0) {
    // (x / p) / c == x / (p*c) for x >= 0
    if (a.c0 == 0 && a.terms.size() == 1 && a.terms[0].coef == 1 &&
        atoms[(size_t)a.terms[0].atom].kind == Atom::DIV) {
      const Atom at = atoms[(size_t)a.terms[0].atom];
      if (at.c < ((int64_t)1 << 31) / c) return lin_div(at.inner, at.c * c);
    }
    Lin Q, R;
    split_multiple(a, c, &Q, &R);
    int64_t rlo, rhi;
    lin_bounds(R, &rlo, &rhi);
    if (rlo >= 0) {
      if (rhi < c) return Q;
      // floor((g*X + S) / (g*c')) == floor(X / c') when 0 <= S < g: split R into
      // the terms whose coefficients share a factor g with c and a small rest S.
      // Candidates for g: gcd of c with the coefficients not smaller than each term's.
      int64_t cc = c;
      for (size_t pick = 0; pick <= R.terms.size(); pick++) {
        int64_t thresh = pick < R.terms.size() ? std::llabs(R.terms[pick].coef) : 0;
        if (pick == R.terms.size() && !R.terms.empty()) break;
        int64_t g = c;
        for (const Term &t : R.terms) if (std::llabs(t.coef) >= thresh) g = gcd64(g, t.coef);
        if (g <= 1) continue;
        Lin X, S;
        for (const Term &t : R.terms) {
          if (t.coef % g == 0) X.terms.push_back({t.coef / g, t.atom});
          else S.terms.push_back(t);
        }
        int64_t r0 = R.c0 % g;
        X.c0 = (R.c0 - r0) / g;
        S.c0 = r0;
        int64_t slo, shi;
        lin_bounds(S, &slo, &shi);
        if (slo < 0 || shi >= g) continue;
        int64_t xlo, xhi;
        lin_bounds(X, &xlo, &xhi);
        if (xlo < 0) continue;
        // X / c' may simplify further (e.g. a quotient of a quotient)
        return lin_add(Q, lin_div(X, c / g));
      }
      Atom d;
      d.kind = Atom::DIV; d.inner = R; d.c = cc;
      int64_t l2, h2;
      lin_bounds(R, &l2, &h2);
      d.lo = l2 / cc; d.hi = h2 / cc;
      return lin_add(Q, lin_atom(intern_atom(d)));
    }
  }
  Atom d;
  d.kind = Atom::DIV; d.inner = a; d.c = c;
  if (c > 0) { d.lo = lo / c; d.hi = hi / c; if (d.lo > d.hi) std::swap(d.lo, d.hi); }
  else { d.lo = -kBig; d.hi = kBig; }
  return lin_atom(intern_atom(d));
}

Lin KernelGraph::lin_mod(const Lin &a, int64_t c) {
  if (c == 1) return lin_const(0);
  if (a.is_const()) return lin_const(a.c0 % c);
  int64_t lo, hi;
  lin_bounds(a, &lo, &hi);
  if (c > 0 && lo >= 0) {
    if (hi < c) return a;
    Lin Q, R;
    split_multiple(a, c, &Q, &R);
    int64_t rlo, rhi;
    lin_bounds(R, &rlo, &rhi);
    if (rlo >= 0) {
      if (rhi < c) return R;
      // (x % (p*c)) % c == x % c; also x % p with p a multiple of c
      if (R.c0 == 0 && R.terms.size() == 1 && R.terms[0].coef == 1 &&
          atoms[(size_t)R.terms[0].atom].kind == Atom::MOD &&
          atoms[(size_t)R.terms[0].atom].c % c == 0) {
        const Atom at = atoms[(size_t)R.terms[0].atom];
        return lin_mod(at.inner, c);
      }
      // (g*X + S) % (g*c') == g*(X % c') + S when 0 <= S < g
      for (size_t pick = 0; pick < R.terms.size(); pick++) {
        int64_t thresh = std::llabs(R.terms[pick].coef);
        int64_t g = c;
        for (const Term &t : R.terms) if (std::llabs(t.coef) >= thresh) g = gcd64(g, t.coef);
        if (g <= 1 || g == c) continue;
        Lin X, S;
        for (const Term &t : R.terms) {
          if (t.coef % g == 0) X.terms.push_back({t.coef / g, t.atom});
          else S.terms.push_back(t);
        }
        int64_t r0 = R.c0 % g;
        X.c0 = (R.c0 - r0) / g;
        S.c0 = r0;
        int64_t slo, shi, xlo, xhi;
        lin_bounds(S, &slo, &shi);
        lin_bounds(X, &xlo, &xhi);
        if (slo < 0 || shi >= g || xlo < 0) continue;
        return lin_add(lin_scale(lin_mod(X, c / g), g), S);
      }
      Atom m;
      m.kind = Atom::MOD; m.inner = R; m.c = c;
      m.lo = 0; m.hi = std::min(c - 1, rhi);
      return lin_atom(intern_atom(m));
    }
  }
  Atom m;
  m.kind = Atom::MOD; m.inner = a; m.c = c;
  int64_t ac = c < 0 ? -c : c;
  m.lo = lo >= 0 ? 0 : -(ac - 1);
  m.hi = hi <= 0 ? 0 : (ac - 1);
  return lin_atom(intern_atom(m));
}

uint64_t KernelGraph::atom_deps(int atom) const {
  const Atom &a = atoms[(size_t)atom];
  if (a.kind == Atom::DIV || a.kind == Atom::MOD) return lin_deps(a.inner);
  return nodes[(size_t)a.node].deps;
}

uint64_t KernelGraph::lin_deps(const Lin &l) const {
  uint64_t d = 0;
  for (const Term &t : l.terms) d |= atom_deps(t.atom);
  return d;
}

bool KernelGraph::lin_is_affine(const Lin &l) const {
  for (const Term &t : l.terms) {
    Atom::Kind k = atoms[(size_t)t.atom].kind;
    if (k != Atom::RANGE && k != Atom::VAR) return false;
  }
  return true;
}

int64_t KernelGraph::lin_range_coef(const Lin &l, int ord, bool *affine) const {
  int64_t coef = 0;
  *affine = true;
  for (const Term &t : l.terms) {
    const Atom &a = atoms[(size_t)t.atom];
    if (a.kind == Atom::RANGE) {
      auto it = range_ord.find(a.node);
      if (it != range_ord.end() && it->second == ord) coef += t.coef;
    } else if (a.kind != Atom::VAR) {
      if (atom_deps(t.atom) & ((uint64_t)1 << ord)) *affine = false;
    }
  }
  return coef;
}

int KernelGraph::param_slot(int param_node) const {
  for (size_t i = 0; i < params.size(); i++)
    if (params[i].node == param_node) return (int)i;
  return -1;
}

// ── graph construction ────────────────────────────────────────────────────

static bool is_index_int(DT t) { return t == DT_I32 || t == DT_INDEX; }

bool KernelGraph::build(const PolyUOp *root) {
  if (!root || root->op != POLY_OP_SINK) { error = "kernel root is not a SINK"; return false; }

  // iterative post-order DFS
  auto src_of = [&](const PolyUOp *u, int i) -> const PolyUOp * {
    return slab_value && u->op == POLY_OP_STORE && i == 1 ? slab_value : u->src[i];
  };
  struct Frame { const PolyUOp *u; int next; };
  std::vector<Frame> stack;
  std::unordered_map<const PolyUOp *, char> state;  // 1 = on stack, 2 = done
  for (const PolyUOp *p : slab_params) {
    if (p->op != POLY_OP_PARAM || p->n_src != 0) { error = "slab parameter is not a plain PARAM"; return false; }
    if (!state.count(p)) { state[p] = 1; stack.push_back({p, 0}); }
  }
  std::reverse(stack.begin(), stack.end());
  stack.insert(stack.begin(), {root, 0});
  state[root] = 1;
  while (!stack.empty()) {
    Frame &f = stack.back();
    if (f.next < (int)f.u->n_src) {
      const PolyUOp *s = src_of(f.u, f.next);
      f.next++;
      if (!s) { error = "null source pointer"; return false; }
      auto it = state.find(s);
      if (it == state.end()) { state[s] = 1; stack.push_back({s, 0}); }
      else if (it->second == 1) { error = "cycle in kernel graph"; return false; }
    } else {
      const PolyUOp *u = f.u;
      KNode kn;
      kn.u = u; kn.op = u->op; kn.dt = classify_dtype(u->dtype); kn.is_ptr = u->dtype.is_ptr;
      if (kn.dt == DT_BAD) { error = strf("unsupported dtype on %s", op_name(u->op)); return false; }
      if (u->dtype.count > 1 || (u->dtype.is_ptr && u->dtype.vcount > 1)) {
        error = strf("vector dtype on %s in a scheduled kernel", op_name(u->op));
        return false;
      }
      for (int i = 0; i < (int)u->n_src; i++) kn.src.push_back(ids[src_of(u, i)]);
      ids[u] = (int)nodes.size();
      nodes.push_back(std::move(kn));
      state[u] = 2;
      stack.pop_back();
    }
  }
  for (KNode &k : nodes)
    for (int s : k.src) nodes[(size_t)s].n_uses++;

  // loads predicated by the WHERE that selects them
  for (KNode &w : nodes) {
    if (w.op != POLY_OP_WHERE || w.src.size() != 3) continue;
    for (int b = 1; b <= 2; b++) {
      int n = w.src[(size_t)b];
      if (nodes[(size_t)n].op == POLY_OP_CAST && nodes[(size_t)n].n_uses == 1) n = nodes[(size_t)n].src[0];
      KNode &ld = nodes[(size_t)n];
      if (ld.op == POLY_OP_LOAD && ld.n_uses == 1 && ld.guard < 0) { ld.guard = w.src[0]; ld.guard_neg = (b == 2); }
      // a reduction that only this branch uses need not run where the branch is not taken
      // (the derivative of a concatenation: each output position takes one of several sums)
      if (ld.op == POLY_OP_REDUCE && ld.n_uses == 1 && ld.guard < 0) { ld.guard = w.src[0]; ld.guard_neg = (b == 2); }
    }
  }

  // ranges, params, vars
  for (int i = 0; i < (int)nodes.size(); i++) {
    KNode &k = nodes[(size_t)i];
    if (k.op == POLY_OP_RANGE) {
      if (k.src.empty()) { error = "RANGE without bound"; return false; }
      RangeInfo r;
      r.node = i; r.bound_node = k.src[0]; r.is_reduce = false; r.extent = -1;
      const PolyUOp *b = nodes[(size_t)k.src[0]].u;
      if (b->op == POLY_OP_CONST) r.extent = b->arg.i;
      if (r.extent > ((int64_t)1 << 40)) { error = "RANGE with an extent beyond 2^40"; return false; }
      if (k.u == slab_range) {
        if (r.extent < 0 || slab_lo < 0 || slab_extent <= 0 || slab_lo + slab_extent > r.extent) { error = "slab outside its range"; return false; }
        r.extent = slab_extent;
      }
      r.axis_id = k.u->arg.kind == POLY_ARG_RANGE ? k.u->arg.range.axis_id
                  : (k.u->arg.kind == POLY_ARG_INT ? k.u->arg.i : -1);
      if (ranges.size() >= 64) { error = "more than 64 ranges in one kernel"; return false; }
      range_ord[i] = (int)ranges.size();
      ranges.push_back(r);
    } else if (k.op == POLY_OP_PARAM) {
      ParamInfo p;
      p.node = i; p.index = (int)k.u->arg.i; p.dt = k.dt; p.numel = k.u->dtype.ptr_size;
      params.push_back(p);
    } else if (k.op == POLY_OP_DEFINE_VAR) {
      VarInfo v;
      v.node = i;
      if (k.u->arg.kind == POLY_ARG_DEFINE_VAR) {
        v.name = k.u->arg.define_var.name ? k.u->arg.define_var.name : "var";
        v.lo = k.u->arg.define_var.min_val; v.hi = k.u->arg.define_var.max_val;
      } else { v.name = "var"; v.lo = 0; v.hi = INT_MAX; }
      vars.push_back(v);
    }
  }
  std::sort(params.begin(), params.end(),
            [](const ParamInfo &a, const ParamInfo &b) { return a.index < b.index; });
  for (size_t i = 0; i < params.size(); i++)
    if (params[i].index != (int)i) { error = "PARAM indices are not dense"; return false; }

  // reduce ranges + REDUCE validation
  for (int i = 0; i < (int)nodes.size(); i++) {
    KNode &k = nodes[(size_t)i];
    if (k.op != POLY_OP_REDUCE) continue;
    if (k.src.empty()) { error = "REDUCE without a value"; return false; }
    if (k.u->arg.kind != POLY_ARG_INT && k.u->arg.kind != POLY_ARG_OPS) {
      error = "REDUCE without an op argument"; return false;
    }
    {
      // read as an integer: the value is checked before anything treats it as a PolyOps
      const int64_t rop = k.u->arg.kind == POLY_ARG_OPS ? (int64_t)(int)k.u->arg.ops : k.u->arg.i;
      if (rop != POLY_OP_ADD && rop != POLY_OP_MUL && rop != POLY_OP_MAX) { error = "REDUCE with an op other than ADD, MUL, MAX"; return false; }
    }
    // Axes of extent 1 arrive as constants in place of ranges (or as no source at all); only
    // real RANGEs make a loop, as in the reference's lowering (src/codegen.c:1431-1439).
    std::vector<int> kept{k.src[0]};
    for (size_t s = 1; s < k.src.size(); s++) {
      auto it = range_ord.find(k.src[s]);
      if (it == range_ord.end()) {
        if (nodes[(size_t)k.src[s]].op == POLY_OP_CONST) continue;
        error = "REDUCE source is neither a RANGE nor a constant";
        return false;
      }
      ranges[(size_t)it->second].is_reduce = true;
      kept.push_back(k.src[s]);
    }
    k.src = kept;
    if (k.src.size() == 1) {
      // nothing to loop over: the value itself, not identity-op-value (src/codegen.c:1444-1450)
      k.op = POLY_OP_CAST;
      continue;
    }
    reduces.push_back(i);
  }

  // dependencies on ranges
  for (int i = 0; i < (int)nodes.size(); i++) {
    KNode &k = nodes[(size_t)i];
    uint64_t d = 0;
    if (k.op == POLY_OP_RANGE) {
      d = (uint64_t)1 << range_ord[i];
      d |= nodes[(size_t)k.src[0]].deps;
    } else {
      for (int s : k.src) d |= nodes[(size_t)s].deps;
      if (k.op == POLY_OP_REDUCE || k.op == POLY_OP_END)
        for (size_t s = 1; s < k.src.size(); s++) {
          auto it = range_ord.find(k.src[s]);
          if (it != range_ord.end()) d &= ~((uint64_t)1 << it->second);
        }
    }
    k.deps = d;
  }

  // stores: peel END chains below the SINK
  {
    struct Item { int node; std::vector<int> rng; };
    std::vector<Item> work;
    for (int s : nodes.back().src) work.push_back({s, {}});
    while (!work.empty()) {
      Item it = work.back();
      work.pop_back();
      const KNode &k = nodes[(size_t)it.node];
      if (k.op == POLY_OP_END) {
        Item nx{k.src[0], it.rng};
        for (size_t s = 1; s < k.src.size(); s++) {
          auto r = range_ord.find(k.src[s]);
          if (r == range_ord.end()) { error = "END source is not a RANGE"; return false; }
          if (ranges[(size_t)r->second].is_reduce) { error = "range closed by both END and REDUCE"; return false; }
          nx.rng.push_back(r->second);
        }
        work.push_back(nx);
      } else if (k.op == POLY_OP_STORE) {
        StoreInfo st;
        st.store = it.node;
        st.index = k.src[0];
        const KNode &ix = nodes[(size_t)st.index];
        if (ix.op != POLY_OP_INDEX || ix.src.size() < 2) { error = "STORE target is not INDEX(PARAM, idx)"; return false; }
        st.param = ix.src[0];
        if (nodes[(size_t)st.param].op != POLY_OP_PARAM) { error = "STORE target buffer is not a PARAM"; return false; }
        if (ix.src.size() >= 3) st.gate = ix.src[2];
        st.value = k.src[1];
        st.ranges = it.rng;
        // every range the store depends on must be one of its END ranges
        uint64_t have = 0;
        for (int r : st.ranges) have |= (uint64_t)1 << r;
        if (k.deps & ~have) { error = "STORE depends on a range that no END closes"; return false; }
        stores.push_back(st);
      } else if (k.op == POLY_OP_GROUP || k.op == POLY_OP_NOOP || k.op == POLY_OP_SINK) {
        for (int s : k.src) work.push_back({s, it.rng});
      } else {
        error = strf("unexpected %s under SINK", op_name(k.op));
        return false;
      }
    }
    if (stores.empty()) { error = "kernel has no STORE"; return false; }
    std::reverse(stores.begin(), stores.end());
    for (const StoreInfo &st : stores) params[(size_t)param_slot(st.param)].written = true;
  }
  for (const KNode &k : nodes)
    if (k.op == POLY_OP_LOAD) {
      const KNode &ix = nodes[(size_t)k.src[0]];
      if (ix.op != POLY_OP_INDEX || nodes[(size_t)ix.src[0]].op != POLY_OP_PARAM) {
        error = "LOAD source is not INDEX(PARAM, idx)"; return false;
      }
      params[(size_t)param_slot(ix.src[0])].read = true;
    }

  // canonical forms for index-typed integer nodes
  for (int i = 0; i < (int)nodes.size(); i++) {
    KNode &k = nodes[(size_t)i];
    if (k.is_ptr || !is_index_int(k.dt)) continue;
    auto L = [&](int s) -> const Lin * {
      int li = nodes[(size_t)k.src[(size_t)s]].lin;
      return li >= 0 ? &lins[(size_t)li] : nullptr;
    };
    Lin out;
    bool ok = false;
    switch (k.op) {
      case POLY_OP_CONST: out = lin_const(k.u->arg.i); ok = true; break;
      case POLY_OP_RANGE: {
        const RangeInfo &r = ranges[(size_t)range_ord[i]];
        int64_t hi = INT_MAX;
        if (r.extent >= 0) hi = r.extent - 1;
        else if (nodes[(size_t)r.bound_node].lin >= 0) {
          int64_t bl, bh;
          lin_bounds(lins[(size_t)nodes[(size_t)r.bound_node].lin], &bl, &bh);
          hi = bh - 1;
        }
        out = lin_atom(atom_for_node(i, Atom::RANGE, 0, hi < 0 ? 0 : hi));
        if (k.u == slab_range) out.c0 = slab_lo;
        ok = true;
        break;
      }
      case POLY_OP_DEFINE_VAR: {
        int64_t lo = 0, hi = INT_MAX;
        if (k.u->arg.kind == POLY_ARG_DEFINE_VAR) { lo = k.u->arg.define_var.min_val; hi = k.u->arg.define_var.max_val; }
        out = lin_atom(atom_for_node(i, Atom::VAR, lo, hi));
        ok = true;
        break;
      }
      case POLY_OP_ADD: if (L(0) && L(1)) { out = lin_recombine(lin_add(*L(0), *L(1))); ok = true; } break;
      case POLY_OP_SUB: if (L(0) && L(1)) { out = lin_recombine(lin_add(*L(0), *L(1), -1)); ok = true; } break;
      case POLY_OP_NEG: if (L(0)) { out = lin_scale(*L(0), -1); ok = true; } break;
      case POLY_OP_MUL:
        if (L(0) && L(1)) {
          if (L(1)->is_const()) { out = lin_scale(*L(0), L(1)->c0); ok = true; }
          else if (L(0)->is_const()) { out = lin_scale(*L(1), L(0)->c0); ok = true; }
        }
        break;
      case POLY_OP_SHL:
        if (L(0) && L(1) && L(1)->is_const() && L(1)->c0 >= 0 && L(1)->c0 < 31) {
          out = lin_scale(*L(0), (int64_t)1 << L(1)->c0); ok = true;
        }
        break;
      case POLY_OP_SHR:
        if (L(0) && L(1) && L(1)->is_const() && L(1)->c0 >= 0 && L(1)->c0 < 31) {
          int64_t lo, hi;
          lin_bounds(*L(0), &lo, &hi);
          if (lo >= 0) { out = lin_div(*L(0), (int64_t)1 << L(1)->c0); ok = true; }
        }
        break;
      case POLY_OP_IDIV:
        if (L(0) && L(1) && L(1)->is_const() && L(1)->c0 > 0) { out = lin_div(*L(0), L(1)->c0); ok = true; }
        break;
      case POLY_OP_MOD:
        if (L(0) && L(1) && L(1)->is_const() && L(1)->c0 > 0) { out = lin_mod(*L(0), L(1)->c0); ok = true; }
        break;
      case POLY_OP_CAST:
        if (!k.src.empty() && is_index_int(nodes[(size_t)k.src[0]].dt) && L(0)) { out = *L(0); ok = true; }
        break;
      default: break;
    }
    if (!ok) {
      bool has_value = !(k.op == POLY_OP_INDEX || k.op == POLY_OP_STORE || k.op == POLY_OP_END ||
                         k.op == POLY_OP_SINK);
      if (!has_value) continue;
      int64_t lo = INT_MIN, hi = INT_MAX;
      if (k.op == POLY_OP_CAST && !k.src.empty() && nodes[(size_t)k.src[0]].dt == DT_BOOL) { lo = 0; hi = 1; }
      out = lin_atom(atom_for_node(i, Atom::OPAQUE, lo, hi));
    }
    k.lin = (int)lins.size();
    lins.push_back(out);
  }

  // Tighten the range dependencies with the simplified forms: an index that
  // mentions a range only in terms that cancelled no longer depends on it.
  for (int i = 0; i < (int)nodes.size(); i++) {
    KNode &k = nodes[(size_t)i];
    if (k.op == POLY_OP_RANGE) continue;
    if (k.lin >= 0) {
      const Lin &l = lins[(size_t)k.lin];
      bool self = l.c0 == 0 && l.terms.size() == 1 && atoms[(size_t)l.terms[0].atom].kind == Atom::OPAQUE &&
                  atoms[(size_t)l.terms[0].atom].node == i;
      if (!self) { k.deps = lin_deps(l); continue; }
    }
    uint64_t d = 0;
    for (int s : k.src) d |= nodes[(size_t)s].deps;
    if (k.op == POLY_OP_REDUCE || k.op == POLY_OP_END)
      for (size_t s = 1; s < k.src.size(); s++) {
        auto it = range_ord.find(k.src[s]);
        if (it != range_ord.end()) d &= ~((uint64_t)1 << it->second);
      }
    k.deps = d;
  }
  if (lin_overflow) { error = "index arithmetic leaves the 64-bit range"; return false; }
  return true;
}


// ── self-check of the index simplifier ────────────────────────────────────

namespace {
struct RawEval {
  const KernelGraph &g;
  const std::vector<int64_t> &rv;   // value per range ordinal
  bool ok = true;
  int64_t node(int id) {
    const KNode &k = g.n(id);
    auto S = [&](size_t i) { return node(k.src[i]); };
    switch (k.op) {
      case POLY_OP_CONST: return k.u->arg.i;
      case POLY_OP_RANGE: return rv[(size_t)g.range_ord.at(id)] + (g.slab_range && k.u == g.slab_range ? g.slab_lo : 0);
      // (wrapping arithmetic: the check compares two evaluations, it must not trip over
      // what a damaged graph makes them compute)
      case POLY_OP_ADD: return (int64_t)((uint64_t)S(0) + (uint64_t)S(1));
      case POLY_OP_SUB: return (int64_t)((uint64_t)S(0) - (uint64_t)S(1));
      case POLY_OP_MUL: return (int64_t)((uint64_t)S(0) * (uint64_t)S(1));
      case POLY_OP_NEG: return (int64_t)(0 - (uint64_t)S(0));
      case POLY_OP_IDIV: { const int32_t a = (int32_t)S(0), b = (int32_t)S(1); if (b == 0 || (a == INT32_MIN && b == -1)) { ok = false; return 0; } return (int64_t)(a / b); }
      case POLY_OP_MOD: { const int32_t a = (int32_t)S(0), b = (int32_t)S(1); if (b == 0 || (a == INT32_MIN && b == -1)) { ok = false; return 0; } return (int64_t)(a % b); }
      case POLY_OP_SHL: return (int64_t)((uint64_t)S(0) << (S(1) & 31));
      case POLY_OP_SHR: return S(0) >> (S(1) & 31);
      case POLY_OP_CAST:
        if (g.n(k.src[0]).dt == DT_I32 || g.n(k.src[0]).dt == DT_INDEX) return S(0);
        ok = false; return 0;
      default: ok = false; return 0;
    }
  }
  int64_t atom(int a) {
    const Atom &at = g.atoms[(size_t)a];
    switch (at.kind) {
      case Atom::RANGE: return rv[(size_t)g.range_ord.at(at.node)];
      case Atom::DIV: { const int64_t v = lin(at.inner); if (at.c == 0 || (v == INT64_MIN && at.c == -1)) { ok = false; return 0; } return v / at.c; }
      case Atom::MOD: { const int64_t v = lin(at.inner); if (at.c == 0 || (v == INT64_MIN && at.c == -1)) { ok = false; return 0; } return v % at.c; }
      case Atom::OPAQUE: return node_raw_opaque(at.node);
      default: ok = false; return 0;
    }
  }
  int64_t node_raw_opaque(int id) { return node(id); }
  int64_t lin(const Lin &l) {
    uint64_t v = (uint64_t)l.c0;
    for (const Term &t : l.terms) v += (uint64_t)t.coef * (uint64_t)atom(t.atom);
    return (int64_t)v;
  }
};
}  // namespace

int KernelGraph::check_lins(int samples, std::string *first_bad) const {
  std::vector<int64_t> ext;
  double space = 1;
  for (const RangeInfo &r : ranges) { ext.push_back(r.extent > 0 ? r.extent : 1); space *= (double)ext.back(); }
  std::vector<int64_t> rv(ranges.size(), 0);
  int bad = 0;
  uint64_t rng = 0x9E3779B97F4A7C15ull;
  bool exhaustive = space <= (double)samples;
  int64_t total = exhaustive ? (int64_t)space : samples;
  for (int64_t it = 0; it < total; it++) {
    if (exhaustive) {
      int64_t t = it;
      for (size_t r = 0; r < ext.size(); r++) { rv[r] = t % ext[r]; t /= ext[r]; }
    } else {
      for (size_t r = 0; r < ext.size(); r++) {
        rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17;
        uint64_t pick = rng % 8;
        rv[r] = pick == 0 ? 0 : pick == 1 ? ext[r] - 1 : (int64_t)((rng >> 8) % (uint64_t)ext[r]);
      }
    }
    for (int i = 0; i < (int)nodes.size(); i++) {
      const KNode &k = nodes[(size_t)i];
      if (k.lin < 0 || k.op == POLY_OP_RANGE || k.op == POLY_OP_CONST) continue;
      RawEval e{*this, rv};
      int64_t raw = e.node(i);
      if (!e.ok) continue;
      int64_t viaLin = e.lin(lins[(size_t)k.lin]);
      if (!e.ok) continue;
      if (raw != viaLin) {
        if (bad == 0 && first_bad)
          *first_bad = strf("node %d (%s): raw %lld, simplified %lld", i, op_name(k.op), (long long)raw, (long long)viaLin);
        bad++;
      }
    }
  }
  return bad;
}

}  // namespace polyhip
