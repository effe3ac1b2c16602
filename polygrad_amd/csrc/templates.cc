// Hand-written kernel templates selected by pattern match on the scheduled
// root (where the structure is still explicit: one REDUCE over a product of
// two loads is a matmul, a REDUCE over WHERE(idx == arange, table, 0) is an
// embedding lookup).  Anything that does not match falls through to the
// generic lowering in render_hip.cc; nothing here changes results beyond the
// order of the fp32 accumulation.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>

#include "templates.h"

namespace polyhip {

namespace {

const char *const kMatmulTemplate =
#include "matmul_mfma.hip.inc"
    ;
const char *const kMatmulDmaTemplate =
#include "matmul_dma.hip.inc"
    ;
const char *const kMatmulF32Template =
#include "matmul_f32_mfma.hip.inc"
    ;
const char *const kOperandSplitTemplate =
#include "operand_split.hip.inc"
    ;

thread_local uint64_t g_input_params = 0;
// What the plan knows about the kernel's fp32 buffer parameters; see matmul_hint_param_kinds.
thread_local std::vector<int> g_param_kinds;

PolyOps reduce_op(const KNode &k) {
  return k.u->arg.kind == POLY_ARG_OPS ? k.u->arg.ops : (PolyOps)k.u->arg.i;
}

typedef MmOperand Operand;
typedef MmDim Dim;

bool match_operand(const KernelGraph &g, int node, Operand *o) {
  const KNode *k = &g.n(node);
  if (k->op == POLY_OP_CAST && k->dt == DT_F32) { node = k->src[0]; k = &g.n(node); }
  if (k->op != POLY_OP_LOAD || k->guard >= 0) return false;
  const KNode &ix = g.n(k->src[0]);
  if (ix.src.size() != 2) return false;  // gated
  o->load = node;
  o->param = g.param_slot(ix.src[0]);
  o->lin = g.n(ix.src[1]).lin;
  o->dt = k->dt;
  return o->lin >= 0 && o->param >= 0;
}

// Extracts the dependence of `l` on reduce range `kr` (extent K).
bool k_dependence(const KernelGraph &g, const Lin &l, int kr, int64_t K, KSplit *ks) {
  bool have_plain = false, have_div = false, have_mod = false;
  int64_t s = 0, s_hi = 0, s_lo = 0, c_div = 0, c_mod = 0;
  for (const Term &t : l.terms) {
    const Atom &a = g.atoms[(size_t)t.atom];
    if (!(g.atom_deps(t.atom) & ((uint64_t)1 << kr))) continue;
    if (a.kind == Atom::RANGE) { have_plain = true; s = t.coef; continue; }
    if (a.kind != Atom::DIV && a.kind != Atom::MOD) return false;
    // inner must be exactly the range k
    if (a.inner.c0 != 0 || a.inner.terms.size() != 1 || a.inner.terms[0].coef != 1) return false;
    const Atom &in = g.atoms[(size_t)a.inner.terms[0].atom];
    if (in.kind != Atom::RANGE || g.range_ord.at(in.node) != kr) return false;
    if (a.kind == Atom::DIV) { if (have_div) return false; have_div = true; s_hi = t.coef; c_div = a.c; }
    else { if (have_mod) return false; have_mod = true; s_lo = t.coef; c_mod = a.c; }
  }
  if (have_plain) {
    if (have_div || have_mod) return false;
    *ks = {K, 0, s};
    return true;
  }
  if (have_div && have_mod && c_div == c_mod) { *ks = {c_div, s_hi, s_lo}; return true; }
  if (have_div && !have_mod) { *ks = {c_div, s_hi, 0}; return true; }
  if (have_mod && !have_div) { *ks = {c_mod, 0, s_lo}; return true; }
  return false;  // no dependence on k at all
}

struct DigitUse { int64_t coef, a, b; };  // coef * ((r / a) % b), b = 0: no modulus

// Collects how `l` uses global range `ord`; false when some use is not of the
// digit form above.
bool digit_uses(const KernelGraph &g, const Lin &l, int ord, std::vector<DigitUse> *uses) {
  auto is_range = [&](const Lin &in) {
    if (in.c0 != 0 || in.terms.size() != 1 || in.terms[0].coef != 1) return false;
    const Atom &a = g.atoms[(size_t)in.terms[0].atom];
    return a.kind == Atom::RANGE && g.range_ord.at(a.node) == ord;
  };
  for (const Term &t : l.terms) {
    const Atom &a = g.atoms[(size_t)t.atom];
    if (!(g.atom_deps(t.atom) & ((uint64_t)1 << ord))) continue;
    if (a.kind == Atom::RANGE) { uses->push_back({t.coef, 1, 0}); continue; }
    if (a.kind == Atom::DIV && is_range(a.inner)) { uses->push_back({t.coef, a.c, 0}); continue; }
    if (a.kind == Atom::MOD && is_range(a.inner)) { uses->push_back({t.coef, 1, a.c}); continue; }
    if (a.kind == Atom::MOD && a.inner.c0 == 0 && a.inner.terms.size() == 1 && a.inner.terms[0].coef == 1) {
      const Atom &d = g.atoms[(size_t)a.inner.terms[0].atom];
      if (d.kind == Atom::DIV && is_range(d.inner)) { uses->push_back({t.coef, d.c, a.c}); continue; }
    }
    // (r / c1) / c2 = r / (c1 c2) for a non-negative r
    if (a.kind == Atom::DIV && a.inner.c0 == 0 && a.inner.terms.size() == 1 && a.inner.terms[0].coef == 1) {
      const Atom &d = g.atoms[(size_t)a.inner.terms[0].atom];
      if (d.kind == Atom::DIV && is_range(d.inner)) { uses->push_back({t.coef, d.c * a.c, 0}); continue; }
    }
    return false;
  }
  return true;
}

// Splits range `ord` (extent E) into digits consistent with every use in la / lb
// and returns them outermost first with their coefficients in both operands.
bool factor_range(const KernelGraph &g, const Lin &la, const Lin &lb, int ord, int64_t E, std::vector<Dim> *out) {
  std::vector<DigitUse> ua, ub;
  if (!digit_uses(g, la, ord, &ua) || !digit_uses(g, lb, ord, &ub)) return false;
  std::vector<int64_t> cuts{1, E};
  for (const std::vector<DigitUse> *u : {&ua, &ub})
    for (const DigitUse &d : *u) {
      cuts.push_back(d.a);
      if (d.b > 0) cuts.push_back(d.a * d.b);
    }
  std::sort(cuts.begin(), cuts.end());
  cuts.erase(std::unique(cuts.begin(), cuts.end()), cuts.end());
  while (!cuts.empty() && cuts.back() > E) cuts.pop_back();
  for (size_t i = 0; i + 1 < cuts.size(); i++) if (cuts[i + 1] % cuts[i] != 0) return false;
  if (cuts.back() != E) return false;
  auto coef = [&](const std::vector<DigitUse> &u, int64_t cut) {
    int64_t c = 0;
    for (const DigitUse &d : u)
      if (cut >= d.a && (d.b == 0 || cut < d.a * d.b)) c += d.coef * (cut / d.a);
    return c;
  };
  for (size_t i = cuts.size() - 1; i-- > 0;) {
    Dim d{ord, cuts[i + 1] / cuts[i], coef(ua, cuts[i]), coef(ub, cuts[i]), cuts[i]};
    out->push_back(d);
  }
  return true;
}

std::string offset_fn(const char *name, const std::vector<Dim> &dims, bool use_a, int64_t c0) {
  // dims are outermost first; the flattened coordinate has the last one fastest
  std::string s = strf("__device__ __forceinline__ int %s(int x) {\n", name);
  s += strf("  int off = %lld;\n", (long long)c0);
  for (size_t i = dims.size(); i-- > 0;) {
    int64_t c = use_a ? dims[i].ca : dims[i].cb;
    if (i == 0) s += strf("  off += x * %lld;\n", (long long)c);
    else s += strf("  off += (x %% %lld) * %lld; x /= %lld;\n", (long long)dims[i].extent, (long long)c, (long long)dims[i].extent);
  }
  s += "  return off;\n}\n";
  return s;
}

// Merges adjacent dims whose strides nest exactly for both operands.
void collapse(std::vector<Dim> &dims) {
  for (size_t i = 0; i + 1 < dims.size();) {
    Dim &o = dims[i], &in = dims[i + 1];
    if (o.ca == in.ca * in.extent && o.cb == in.cb * in.extent) {
      in.extent *= o.extent;
      dims.erase(dims.begin() + (long)i);
    } else i++;
  }
}

static bool reject(int line) {
  if (getenv("POLY_HIP_DEBUG")) fprintf(stderr, "polygrad: render_hip: matmul template rejected at templates.cc:%d\n", line);
  return false;
}

}  // namespace

bool match_matmul(const KernelGraph &g, MatmulMatch *mm, int *reject_line) {
#define MM_REJECT() do { if (reject_line) *reject_line = __LINE__; return false; } while (0)
  if (g.stores.size() != 1 || g.reduces.size() != 1 || !g.vars.empty()) MM_REJECT();
  const StoreInfo &st = g.stores[0];
  if (st.gate >= 0) MM_REJECT();
  const int red = g.reduces[0];
  const KNode &R = g.n(red);
  if (reduce_op(R) != POLY_OP_ADD || R.dt != DT_F32 || (R.src.size() != 2 && R.src.size() != 3)) MM_REJECT();
  const bool two_k = R.src.size() == 3;
  if (two_k && getenv("POLY_HIP_MM_ONE_K_RANGE")) MM_REJECT();
  const int kr = two_k ? -1 : g.range_ord.at(R.src[1]);
  int64_t K = 1;
  for (size_t i = 1; i < R.src.size(); i++) {
    const int64_t e = g.ranges[(size_t)g.range_ord.at(R.src[i])].extent;
    if (e <= 0 || K > 2147483647LL / e) MM_REJECT();
    K *= e;
  }
  if (K < 16) MM_REJECT();
  const KNode &mul = g.n(R.src[0]);
  if (mul.op != POLY_OP_MUL || mul.dt != DT_F32) MM_REJECT();
  Operand A, B;
  if (!match_operand(g, mul.src[0], &A) || !match_operand(g, mul.src[1], &B)) MM_REJECT();
  if (A.dt != B.dt || (A.dt != DT_BF16 && A.dt != DT_F16 && A.dt != DT_F32)) MM_REJECT();
  for (const ParamInfo &p : g.params) if (p.numel >= ((int64_t)1 << 31)) MM_REJECT();
  const Lin &la = g.lins[(size_t)A.lin], &lb = g.lins[(size_t)B.lin];
  KSplit ka, kb;
  if (!two_k) {
    if (!k_dependence(g, la, kr, K, &ka) || !k_dependence(g, lb, kr, K, &kb)) MM_REJECT();
  } else {
    // Two reduce ranges p, q that both operands index plainly: k = p * |q| + q walks them as
    // one depth of two levels (one level where the strides nest).  The sum runs over the
    // same products in either nesting; the one whose inner stride in A is smaller is taken.
    const int r1 = g.range_ord.at(R.src[1]), r2 = g.range_ord.at(R.src[2]);
    const int64_t e1 = g.ranges[(size_t)r1].extent, e2 = g.ranges[(size_t)r2].extent;
    KSplit a1, a2, b1, b2;
    if (!k_dependence(g, la, r1, e1, &a1) || !k_dependence(g, la, r2, e2, &a2)) MM_REJECT();
    if (!k_dependence(g, lb, r1, e1, &b1) || !k_dependence(g, lb, r2, e2, &b2)) MM_REJECT();
    if (a1.kb != e1 || a2.kb != e2 || b1.kb != e1 || b2.kb != e2) MM_REJECT();   // plain uses only
    const bool q_inner = std::llabs(a2.s_lo) <= std::llabs(a1.s_lo);
    const int64_t ei = q_inner ? e2 : e1;
    auto level = [&](const KSplit &p, const KSplit &q) {
      const int64_t hi = q_inner ? p.s_lo : q.s_lo, lo = q_inner ? q.s_lo : p.s_lo;
      return KSplit{ei, hi, lo};
    };
    ka = level(a1, a2);
    kb = level(b1, b2);
    if (ka.s_hi == ka.s_lo * ei && kb.s_hi == kb.s_lo * ei) { ka = {K, 0, ka.s_lo}; kb = {K, 0, kb.s_lo}; }
  }

  // classify the END ranges of the store
  std::vector<Dim> md, nd, zd;
  auto place_dim = [&](const Dim &d) {
    if (d.ca != 0 && d.cb == 0) md.push_back(d);
    else if (d.ca == 0 && d.cb != 0) nd.push_back(d);
    else zd.push_back(d);
  };
  for (int r : st.ranges) {
    const int64_t e = g.ranges[(size_t)r].extent;
    if (e < 0) MM_REJECT();
    std::vector<Dim> digits;
    if (!factor_range(g, la, lb, r, e, &digits)) MM_REJECT();
    for (const Dim &d : digits) place_dim(d);
  }
  if (md.empty() || nd.empty()) MM_REJECT();
#undef MM_REJECT

  // N and Z digits keep END order (outermost first); the innermost one is the fast
  // coordinate.  The M digits are put in the order of their strides in A, largest first, so
  // that consecutive rows of a tile are neighbours in memory whatever order the kernel's
  // ranges came in (a [B, T, d] activation whose ranges arrive as (t, b) would otherwise
  // deal the rows of a tile to B distant streams); the epilogue finds every range value
  // from the digits, so the order is free.
  std::stable_sort(md.begin(), md.end(), [](const Dim &x, const Dim &y) { return std::llabs(x.ca) > std::llabs(y.ca); });
  mm->md_full = md; mm->nd_full = nd; mm->zd_full = zd;
  collapse(md); collapse(nd); collapse(zd);
  mm->md = md; mm->nd = nd; mm->zd = zd;
  mm->M = mm->N = mm->Z = 1;
  for (const Dim &d : md) mm->M *= d.extent;
  for (const Dim &d : nd) mm->N *= d.extent;
  for (const Dim &d : zd) mm->Z *= d.extent;
  mm->red = red; mm->kr = kr; mm->K = K;
  mm->A = A; mm->B = B; mm->ka = ka; mm->kb = kb;
  mm->a_c0 = la.c0; mm->b_c0 = lb.c0;
  return true;
}

std::string matmul_decompose(const MatmulMatch &mm, Emitter *em) {
  std::string decomp;
  std::vector<std::pair<int, std::string>> range_sum;   // ordinal -> sum of digit * cut
  auto decompose = [&](const std::vector<Dim> &dims, const char *var) {
    if (dims.empty()) return;
    decomp += strf("  int t_%s = %s;\n", var, var);
    for (size_t i = dims.size(); i-- > 0;) {
      const Dim &d = dims[i];
      std::string dv = strf("d%d_%lld", d.ord, (long long)d.cut);
      if (i == 0) decomp += strf("  const int %s = t_%s;\n", dv.c_str(), var);
      else decomp += strf("  const int %s = t_%s %% %lld; t_%s /= %lld;\n", dv.c_str(), var, (long long)d.extent, var, (long long)d.extent);
      std::string term = d.cut == 1 ? dv : strf("%s * %lld", dv.c_str(), (long long)d.cut);
      bool found = false;
      for (auto &rs : range_sum) if (rs.first == d.ord) { rs.second += " + " + term; found = true; }
      if (!found) range_sum.push_back({d.ord, term});
    }
  };
  decompose(mm.md_full, "m");
  decompose(mm.nd_full, "n");
  decompose(mm.zd_full, "z");
  for (auto &rs : range_sum) {
    decomp += strf("  const int r%d = %s;\n", rs.first, rs.second.c_str());
    if (em) em->bind_range(rs.first, strf("r%d", rs.first));
  }
  return decomp;
}

std::string matmul_offset_fn(const char *name, const std::vector<MmDim> &dims, bool use_a, int64_t c0) {
  return offset_fn(name, dims, use_a, c0);
}

std::string matmul_k_fn(const char *name, const KSplit &ks, int64_t K) {
  if (ks.kb >= K) return strf("__device__ __forceinline__ int %s(int k) { return k * %lld; }\n", name, (long long)ks.s_lo);
  return strf("__device__ __forceinline__ int %s(int k) { return (k / %lld) * %lld + (k %% %lld) * %lld; }\n", name,
              (long long)ks.kb, (long long)ks.s_hi, (long long)ks.kb, (long long)ks.s_lo);
}

int64_t matmul_eval_offset(const std::vector<MmDim> &dims, bool use_a, int64_t x) {
  int64_t off = 0;
  for (size_t i = dims.size(); i-- > 0;) {
    const int64_t c = use_a ? dims[i].ca : dims[i].cb;
    if (i == 0) off += x * c;
    else { off += (x % dims[i].extent) * c; x /= dims[i].extent; }
  }
  return off;
}

int64_t matmul_range_value(const MatmulMatch &mm, int ord, int64_t m, int64_t n, int64_t z) {
  int64_t v = 0;
  auto walk = [&](const std::vector<MmDim> &dims, int64_t x) {
    for (size_t i = dims.size(); i-- > 0;) {
      int64_t digit = i == 0 ? x : x % dims[i].extent;
      if (i != 0) x /= dims[i].extent;
      if (dims[i].ord == ord) v += digit * dims[i].cut;
    }
  };
  walk(mm.md_full, m);
  walk(mm.nd_full, n);
  walk(mm.zd_full, z);
  return v;
}

bool matmul_store_contiguous(const KernelGraph &g, const MatmulMatch &mm, const Lin &l) {
  if (mm.nd_full.empty()) return false;
  const MmDim &inner = mm.nd_full.back();
  if (inner.cut != 1) return false;
  if (mm.nd_full.size() > 1 && inner.extent % 8 != 0) return false;
  bool aff;
  const int64_t c = g.lin_range_coef(l, inner.ord, &aff);
  if (!aff || c != 1) return false;
  // a range split into several digits contributes through / and % atoms: not affine
  for (const Term &t : l.terms) {
    const Atom &a = g.atoms[(size_t)t.atom];
    if (a.kind != Atom::RANGE && (g.atom_deps(t.atom) & ((uint64_t)1 << inner.ord))) return false;
  }
  return true;
}

// The kernel's epilogue from its own graph: everything outside the REDUCE, per output
// element (signature, device functions, the statement that stores one element, and the
// value/address split when rows are contiguous along n).
static bool epilogue_from_graph(const KernelGraph &g, const MatmulMatch &mm, MatmulEpilogue *epo) {
  const StoreInfo &st = g.stores[0];
  // Parts of the epilogue that are functions of ONE 16-bit value it loads (the derivative of
  // GELU at the saved pre-activation, in bf16 arithmetic: an exponential and three divisions
  // among some twenty operations, each rounded to bf16) have 65 536 possible values: a table
  // filled once by the same expression replaces the arithmetic, bit for bit.  Taken are the
  // largest such parts of six operations or more, four tables at most.
  struct Part { int node, load; };
  std::vector<Part> parts;
  if (!getenv("POLY_HIP_NO_LUT")) {
    struct Info { bool known = false, impure = false; int load = -1, n_alu = 0; };
    std::vector<Info> info(g.nodes.size());
    std::function<const Info &(int)> look = [&](int id) -> const Info & {
      Info &f = info[(size_t)id];
      if (f.known) return f;
      f.known = true;
      const KNode &k = g.n(id);
      if (k.op == POLY_OP_CONST) return f;
      if (k.op == POLY_OP_LOAD) {
        const KNode &ix = g.n(k.src[0]);
        if ((k.dt == DT_BF16 || k.dt == DT_F16) && k.guard < 0 && ix.op == POLY_OP_INDEX && ix.src.size() == 2) f.load = id;
        else f.impure = true;
        return f;
      }
      if (id == mm.red || k.src.empty() || k.op == POLY_OP_RANGE || k.op == POLY_OP_INDEX || k.op == POLY_OP_PARAM || k.op == POLY_OP_DEFINE_VAR ||
          k.op == POLY_OP_REDUCE || k.op == POLY_OP_SPECIAL || k.op == POLY_OP_BIND) { f.impure = true; return f; }
      f.n_alu = 1;
      for (int c : k.src) {
        const Info ci = look(c);
        if (ci.impure) f.impure = true;
        if (ci.load >= 0) { if (f.load >= 0 && f.load != ci.load) f.impure = true; f.load = ci.load; }
        f.n_alu += ci.n_alu;
      }
      return f;
    };
    std::vector<char> seen(g.nodes.size(), 0);
    std::function<void(int)> visit = [&](int id) {
      if (seen[(size_t)id]) return;
      seen[(size_t)id] = 1;
      const Info f = look(id);
      const KNode &k = g.n(id);
      if (!f.impure && f.load >= 0 && f.n_alu >= 6 && dt_is_float(k.dt) && dt_size(k.dt) <= 4) {
        if (parts.size() < 4) parts.push_back({id, f.load});
        return;
      }
      if (id == mm.red || k.op == POLY_OP_LOAD) return;
      for (int c : k.src) visit(c);
    };
    visit(st.value);
  }
  MatmulEpilogue &ep0 = *epo;
  // Parts of one load share a table: an entry holds the values of all of them (padded to a
  // power of two), so an element costs one gather however many parts it has -- the address
  // path serves two or three lanes a cycle, and three gathers per element of a 4096 x 4096
  // output were 45 us of an 82 us launch.
  struct Tab { int load; std::vector<int> nodes; std::string type; };
  std::vector<Tab> tabs;
  std::string lut_types;        // declarations of the packed entries
  {
    std::vector<Tab> wanted;
    for (const Part &pt : parts) {
      Tab *t = nullptr;
      if (!getenv("POLY_HIP_NO_LUT_PACK"))
        for (Tab &w : wanted) if (w.load == pt.load) t = &w;
      if (!t) { wanted.push_back({pt.load, {}, ""}); t = &wanted.back(); }
      t->nodes.push_back(pt.node);
    }
    for (Tab &t : wanted) {
      // (fields by size, largest first: every one naturally aligned)
      std::stable_sort(t.nodes.begin(), t.nodes.end(), [&](int x, int y) { return dt_size(g.n(x).dt) > dt_size(g.n(y).dt); });
      Emitter et(g);
      Scope St;
      St.indent = 1;
      et.preset(t.load, "x");
      std::vector<std::string> vals;
      size_t bytes = 0;
      for (int node : t.nodes) { vals.push_back(et.emit(node, &St)); bytes += (size_t)dt_size(g.n(node).dt); }
      if (et.failed() || et.uses_threefry) continue;
      const DT idt = g.n(t.load).dt;
      size_t entry = 2;
      while (entry < bytes) entry *= 2;
      std::string decl, stores;
      if (t.nodes.size() == 1) {
        t.type = dt_cname(g.n(t.nodes[0]).dt);
        stores = strf("  out[i] = %s;\n", vals[0].c_str());
      } else {
        t.type = strf("poly_lutpack%zu_t", tabs.size());
        decl = strf("struct __attribute__((aligned(%zu))) %s {", entry, t.type.c_str());
        for (size_t j = 0; j < t.nodes.size(); j++) decl += strf(" %s v%zu;", dt_cname(g.n(t.nodes[j]).dt), j);
        decl += " };\n";
        // (the kernels take the table as a plain pointer: first stages share the signature without these declarations)
        decl += strf("__device__ __forceinline__ %s poly_lutpack%zu_get(const void* __restrict__ t, unsigned short code) { return ((const %s*)t)[code]; }\n",
                     t.type.c_str(), tabs.size(), t.type.c_str());
        stores = strf("  %s e = {};\n", t.type.c_str());
        for (size_t j = 0; j < t.nodes.size(); j++) stores += strf("  e.v%zu = %s;\n", j, vals[j].c_str());
        stores += "  out[i] = e;\n";
      }
      RenderedKernel::Table rt;
      rt.source = std::string(hip_prelude()) + decl +
                  strf("extern \"C\" __global__ void __launch_bounds__(256) poly_lut_fill(%s* out) {\n"
                       "  const unsigned int i = blockIdx.x * 256u + threadIdx.x;\n"
                       "  const %s x = __builtin_bit_cast(%s, (unsigned short)i);\n",
                       t.type.c_str(), dt_cname(idt), dt_cname(idt)) +
                  St.code + stores + "}\n";
      rt.entry = "poly_lut_fill";
      rt.bytes = (size_t)65536 * (t.nodes.size() == 1 ? (size_t)dt_size(g.n(t.nodes[0]).dt) : entry);
      rt.launch.grid[0] = 256;
      rt.launch.block[0] = 256;
      ep0.tables.push_back(rt);
      lut_types += decl;
      ep0.table_parts += (int)t.nodes.size();
      tabs.push_back(t);
    }
  }
  // (an emitter reads a table entry in place of the part: the load first, then the lookup)
  auto use_tables = [&](Emitter &e, Scope *S) {
    for (size_t i = 0; i < tabs.size(); i++) {
      const std::string x = e.emit(tabs[i].load, S);
      if (tabs[i].nodes.size() == 1) e.preset(tabs[i].nodes[0], strf("poly_lut%zu[__builtin_bit_cast(unsigned short, %s)]", i, x.c_str()));
      else
        for (size_t j = 0; j < tabs[i].nodes.size(); j++)
          e.preset(tabs[i].nodes[j], strf("poly_lutpack%zu_get(poly_lut%zu, __builtin_bit_cast(unsigned short, %s)).v%zu", i, i, x.c_str(), j));
    }
  };
  Emitter em(g);
  Scope S0;
  S0.indent = 1;
  for (int r : st.ranges) S0.avail |= (uint64_t)1 << r;
  std::string decomp = matmul_decompose(mm, &em);
  em.preset(mm.red, "acc");
  use_tables(em, &S0);
  std::string val = em.emit(st.value, &S0);
  std::string idx = em.emit(g.n(st.index).src[1], &S0);
  if (em.failed()) return reject(__LINE__);
  const int pout = g.param_slot(st.param);
  MatmulEpilogue &ep = *epo;
  std::string params_call;
  for (size_t i = 0; i < g.params.size(); i++) {
    const ParamInfo &p = g.params[i];
    if (i) { ep.signature += ", "; params_call += ", "; }
    if (p.written) ep.signature += strf("%s* data%zu", dt_cname(p.dt), i);
    else ep.signature += strf("const %s* __restrict__ data%zu", dt_cname(p.dt), i);
    params_call += strf("data%zu", i);
  }
  for (size_t i = 0; i < ep.tables.size(); i++) {
    ep.signature += strf(", const %s* __restrict__ poly_lut%zu", tabs[i].nodes.size() == 1 ? tabs[i].type.c_str() : "void", i);
    params_call += strf(", poly_lut%zu", i);
  }
  ep.params_call = params_call;
  ep.code = lut_types + strf("__device__ __forceinline__ void poly_epilogue(float acc, int m, int n, int z, %s) {\n", ep.signature.c_str());
  ep.code += decomp + S0.code;
  ep.code += strf("  data%d[%s] = %s;\n}\n", pout, idx.c_str(), val.c_str());
  ep.call = strf("poly_epilogue(acc, m, n, z, %s)", params_call.c_str());
  {
    const int li = g.n(g.n(st.index).src[1]).lin;
    const DT odt = g.n(st.param).dt;
    ep.out_16bit = odt == DT_BF16 || odt == DT_F16;
    if (li >= 0 && g.n(st.value).dt == odt && matmul_store_contiguous(g, mm, g.lins[(size_t)li])) {
      // the same code once more, split into the value and the address of an element
      Emitter ev(g), ea(g);
      Scope Sv, Sa;
      Sv.indent = Sa.indent = 1;
      Sv.avail = Sa.avail = S0.avail;
      matmul_decompose(mm, &ev);
      matmul_decompose(mm, &ea);
      ev.preset(mm.red, "acc");
      use_tables(ev, &Sv);
      std::string v2 = ev.emit(st.value, &Sv);
      std::string i2 = ea.emit(g.n(st.index).src[1], &Sa);
      if (!ev.failed() && !ea.failed()) {
        ep.out_type = dt_cname(odt);
        ep.code += strf("__device__ __forceinline__ %s poly_ep_value(float acc, int m, int n, int z, %s) {\n", ep.out_type.c_str(), ep.signature.c_str());
        ep.code += decomp + Sv.code + strf("  return %s;\n}\n", v2.c_str());
        ep.code += strf("__device__ __forceinline__ %s* poly_ep_ptr(int m, int n, int z, %s) {\n", ep.out_type.c_str(), ep.signature.c_str());
        ep.code += decomp + Sa.code + strf("  return data%d + %s;\n}\n", pout, i2.c_str());
        ep.value_call = strf("poly_ep_value(acc, m, n, z, %s)", params_call.c_str());
        ep.ptr_call = strf("poly_ep_ptr(m, n, z, %s)", params_call.c_str());
        ep.contiguous_n = true;
      }
    }
  }
  ep.n_params = (int)g.params.size();
  // distinct elements: A, B once each (broadcast operands counted once), output once,
  // plus whatever the epilogue reads per output row/column
  for (size_t i = 0; i < g.params.size(); i++) {
    const ParamInfo &p = g.params[i];
    double n = (double)std::max<int64_t>(p.numel, 0);
    if ((int)i == pout) n = (double)mm.M * mm.N * mm.Z;
    ep.bytes += n * dt_size(p.dt);
  }
  return true;
}

static thread_local MatmulEpilogue::BlockMaxima g_block_maxima;
static thread_local int64_t g_block_maxima_rows = 0, g_block_maxima_pitch = 0;
void matmul_hint_block_maxima(const MatmulEpilogue *e, int64_t rows, int64_t pitch) {
  g_block_maxima = e ? e->block_maxima : MatmulEpilogue::BlockMaxima();
  g_block_maxima_rows = rows;
  g_block_maxima_pitch = pitch;
}
// Does the kernel store element (m, n) at m * pitch + n, for the blocks of 64 x 64 of the
// columns [lo, hi)?  (checked at the corners and one inner point of every block)
static bool store_is_row_major(const KernelGraph &g, const MatmulMatch &mm, int64_t pitch, int64_t lo, int64_t hi) {
  const StoreInfo &st = g.stores[0];
  const int li = g.n(g.n(st.index).src[1]).lin;
  if (li < 0) return false;
  const Lin &lin = g.lins[(size_t)li];
  std::vector<std::pair<int, int64_t>> terms;
  for (const auto &t : lin.terms) {
    const Atom &a = g.atoms[(size_t)t.atom];
    if (a.kind != Atom::RANGE) return false;
    terms.push_back({g.range_ord.at(a.node), t.coef});
  }
  auto flat = [&](int64_t m, int64_t n) {
    int64_t v = lin.c0;
    for (auto &t : terms) v += t.second * matmul_range_value(mm, t.first, m, n, 0);
    return v;
  };
  for (int64_t m = 0; m + 63 < mm.M; m += 64)
    for (int64_t n = lo; n < hi; n += 64)
      if (flat(m, n) != m * pitch + n || flat(m, n + 63) != m * pitch + n + 63 || flat(m + 63, n) != (m + 63) * pitch + n ||
          flat(m + 31, n + 17) != (m + 31) * pitch + n + 17)
        return false;
  return true;
}

bool try_render_matmul(const KernelGraph &g, const std::string &fn, const RenderOptions &opt, RenderedKernel *out) {
  (void)fn; (void)opt;
  MatmulMatch mm;
  int line = 0;
  if (!match_matmul(g, &mm, &line)) return reject(line);
  MatmulEpilogue ep;
  if (!epilogue_from_graph(g, mm, &ep)) return false;
  if (g_block_maxima.wanted && mm.Z == 1 && mm.M == g_block_maxima_rows && mm.N == g_block_maxima_pitch && mm.M % 64 == 0 &&
      store_is_row_major(g, mm, g_block_maxima_pitch, g_block_maxima.lo, g_block_maxima.hi))
    ep.block_maxima = g_block_maxima;
  ep.a_ptr = strf("data%d", mm.A.param);
  ep.b_ptr = strf("data%d", mm.B.param);
  ep.b_from_hbm = mm.B.param >= 0 && mm.B.param < 64 && ((g_input_params >> mm.B.param) & 1);
  if (!render_matmul(mm, ep, out)) return false;
  out->tables = ep.tables;
  if (!ep.tables.empty()) {
    const std::string note = strf(", %d parts of the epilogue as 16-bit lookup tables (%zu, one per load)", ep.table_parts, ep.tables.size());
    out->strategy += note;
    for (RenderedKernel::Variant &v : out->variants) v.strategy += note;
  }
  return true;
}

// Second stage of a split-K product: adds the S partial accumulators of an output element
// in split order and finishes the element with the kernel's epilogue.
static const char *const kSplitKCombine = R"HIP(
extern "C" __global__ void __launch_bounds__(256) poly_k(POLY_SIGNATURE) {
  const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= (long long)POLY_Z * POLY_M * POLY_N) return;
  const int n = (int)(gid % POLY_N), m = (int)((gid / POLY_N) % POLY_M), z = (int)(gid / ((long long)POLY_N * POLY_M));
  const float *__restrict__ part = POLY_PARTIALS;
  float acc = part[gid];
#pragma unroll
  for (int s = 1; s < POLY_KSPLIT; s++) acc += part[(size_t)s * POLY_Z * POLY_M * POLY_N + gid];
  POLY_EPILOGUE(acc, m, n, z);
}
)HIP";

// How many workgroups should share the K tiles of one output tile: enough to give every CU
// work when the product has few tiles and a deep K; 1 = no split.  S divides `k_tiles`.
static int ksplit_for(int64_t tiles, int64_t k_tiles, int64_t min_tiles_per_split) {
  if (getenv("POLY_HIP_NO_SPLIT_K") || tiles >= 128) return 1;
  int best = 1;
  for (int s = 2; s <= 16; s++) {
    if (k_tiles % s != 0 || k_tiles / s < min_tiles_per_split) continue;
    if (tiles * s > 640) break;
    best = s;
  }
  return best;
}

// Tile of the fp32 template: 4 waves; narrow outputs get a narrow tile.
static void f32_tile(int64_t M, int64_t N, int64_t Z, int *bm, int *bn, int *wvm, int *wvn) {
  int BM = 128, BN = 128, WVM = 2, WVN = 2;
  if (N <= 32) { BN = 32; BM = 256; WVM = 4; WVN = 1; }
  else if (N <= 64) { BN = 64; BM = 128; WVM = 4; WVN = 1; }
  else if (M <= 32) { BM = 32; BN = 256; WVM = 1; WVN = 4; }
  else if (M <= 64) { BM = 64; BN = 128; WVM = 1; WVN = 4; }
  else if (((M + 127) / 128) * ((N + 127) / 128) * Z < 256) {
    BM = 64; BN = 64; WVM = 2; WVN = 2;
    // still fewer workgroups than CUs: two-wave workgroups on 32x64 tiles
    if (((M + 63) / 64) * ((N + 63) / 64) * Z < 192) { BM = 32; BN = 64; WVM = 1; WVN = 2; }
  }
  *bm = BM; *bn = BN; *wvm = WVM; *wvn = WVN;
}

// The other tile shapes of the fp32 template as tuning candidates (same sums in the same
// order: a tile's shape does not change the order of the terms of an output).  `build`
// renders one shape; the default shape comes first, as the kernel itself.
struct F32Shape { int bm, bn, wvm, wvn; };
static void f32_variants(int64_t M, int64_t N, const F32Shape &chosen, const std::function<void(const F32Shape &, RenderedKernel *)> &build,
                         RenderedKernel *out) {
  if (!matmul_tuning_enabled()) return;
  static const F32Shape shapes[] = {{128, 128, 2, 2}, {128, 128, 4, 2}, {64, 64, 2, 2}, {128, 64, 2, 2}, {64, 128, 2, 2}, {256, 128, 4, 2}, {128, 256, 2, 4},
                                    {32, 64, 1, 2}, {256, 32, 4, 1}, {128, 64, 4, 1}, {32, 256, 1, 4}, {64, 128, 1, 4}};
  out->variants.clear();
  out->variants.push_back({"default", out->source, out->strategy, out->launch});
  for (const F32Shape &sh : shapes) {
    if (sh.bm == chosen.bm && sh.bn == chosen.bn && sh.wvm == chosen.wvm && sh.wvn == chosen.wvn) continue;
    if ((sh.bm > 64 && M <= sh.bm / 2) || (sh.bn > 64 && N <= sh.bn / 2)) continue;       // (mostly padding)
    RenderedKernel v;
    build(sh, &v);
    if (v.source.empty()) continue;
    out->variants.push_back({strf("f32_%dx%dw%dx%d", sh.bm, sh.bn, sh.wvm, sh.wvn), v.source, v.strategy, v.launch});
  }
  if (out->variants.size() < 2) out->variants.clear();
}

// fp32 operands: kernels/matmul_f32_mfma.hip (v_mfma_f32_32x32x2_f32, exact fp32 products).
static bool render_matmul_f32(const MatmulMatch &mm, const MatmulEpilogue &ep, RenderedKernel *out) {
  const int64_t K = mm.K, M = mm.M, N = mm.N, Z = mm.Z;
  if (getenv("POLY_HIP_NO_F32_MFMA")) return reject(__LINE__);
  // operand layout: 16-byte pieces along K, or along the operand's row axis
  auto layout = [&](const KSplit &ks, const std::vector<Dim> &dims, bool is_a, int64_t rows, bool *kc) {
    const int64_t inner_c = is_a ? dims.back().ca : dims.back().cb;
    if (K % 16 != 0) return reject(__LINE__);
    if (ks.s_lo == 1 && ks.kb % 16 == 0) { *kc = true; return true; }
    if (inner_c == 1 && dims.back().extent % 4 == 0 && rows % 4 == 0) { *kc = false; return true; }
    return reject(__LINE__);
  };
  bool a_kc, b_kc;
  if (!layout(mm.ka, mm.md, true, M, &a_kc) || !layout(mm.kb, mm.nd, false, N, &b_kc)) return reject(__LINE__);
  int BM, BN, WVM, WVN;
  f32_tile(M, N, Z, &BM, &BN, &WVM, &WVN);
  // deep product on few tiles: larger tiles, K dealt to several workgroups each
  int S = 1;
  if (M > 64 && N > 64 && K >= 2048) {
    const int64_t t128 = ((M + 127) / 128) * ((N + 127) / 128) * Z, t64 = ((M + 63) / 64) * ((N + 63) / 64) * Z;
    const int s128 = ksplit_for(t128, K / 16, 32), s64 = ksplit_for(t64, K / 16, 32);
    if (s128 > 1 && t128 * s128 >= 128) { BM = BN = 128; WVM = WVN = 2; S = s128; }
    else if (s64 > 1) { BM = BN = 64; WVM = WVN = 2; S = s64; }
  }
  if (((M + BM - 1) / BM) * ((N + BN - 1) / BN) > 2147483647LL / 2) return reject(__LINE__);
  std::string cfg;     // (all but the shape of the tile)
  cfg += strf("#define POLY_M %lld\n#define POLY_N %lld\n#define POLY_K %lld\n#define POLY_Z %lld\n", (long long)M, (long long)N, (long long)K, (long long)Z);
  cfg += strf("#define POLY_A_KC %d\n#define POLY_B_KC %d\n", a_kc ? 1 : 0, b_kc ? 1 : 0);
  cfg += strf("#define POLY_A_PTR %s\n#define POLY_B_PTR %s\n", ep.a_ptr.c_str(), ep.b_ptr.c_str());
  cfg += offset_fn("poly_a_row", mm.md, true, 0);
  cfg += offset_fn("poly_b_row", mm.nd, false, 0);
  if (mm.zd.empty()) {
    cfg += strf("__device__ __forceinline__ int poly_a_z(int) { return %lld; }\n", (long long)mm.a_c0);
    cfg += strf("__device__ __forceinline__ int poly_b_z(int) { return %lld; }\n", (long long)mm.b_c0);
  } else {
    cfg += offset_fn("poly_a_z", mm.zd, true, mm.a_c0);
    cfg += offset_fn("poly_b_z", mm.zd, false, mm.b_c0);
  }
  cfg += matmul_k_fn("poly_a_k", mm.ka, K);
  cfg += matmul_k_fn("poly_b_k", mm.kb, K);
  cfg += strf("#define POLY_SIGNATURE %s%s\n", ep.signature.c_str(), S > 1 ? ", float* poly_scratch" : "");
  cfg += strf("#define POLY_KSPLIT %d\n#define POLY_PARTIALS poly_scratch\n", S);
  cfg += ep.code;
  cfg += strf("#define POLY_EPILOGUE(acc, m, n, z) %s\n", ep.call.c_str());
  const auto build = [&](const F32Shape &sh, RenderedKernel *rk) {
    const int64_t tiles = ((M + sh.bm - 1) / sh.bm) * ((N + sh.bn - 1) / sh.bn);
    *rk = RenderedKernel();
    rk->source = std::string(hip_prelude()) +
                 strf("#define POLY_BM %d\n#define POLY_BN %d\n#define POLY_WAVES_M %d\n#define POLY_WAVES_N %d\n#define POLY_GROUP_M 8\n", sh.bm, sh.bn, sh.wvm, sh.wvn) +
                 cfg + kMatmulF32Template;
    rk->entry = "poly_k";
    rk->launch.grid[0] = (unsigned)tiles;
    rk->launch.grid[1] = (unsigned)(Z * S);
    rk->launch.block[0] = (unsigned)(64 * sh.wvm * sh.wvn);
    rk->klass = KernelClass::MATMUL_MFMA;
    rk->strategy = strf("mfma 32x32x2 f32 M=%lld N=%lld K=%lld Z=%lld tile %dx%dx16 A:%s B:%s", (long long)M, (long long)N, (long long)K,
                        (long long)Z, sh.bm, sh.bn, a_kc ? "k-major" : "m-major", b_kc ? "k-major" : "n-major");
    rk->n_params = ep.n_params;
    rk->n_vars = 0;
    rk->flops = 2.0 * (double)M * (double)N * (double)K * (double)Z;
    rk->bytes = ep.bytes;
  };
  build(F32Shape{BM, BN, WVM, WVN}, out);
  if (S == 1) f32_variants(M, N, F32Shape{BM, BN, WVM, WVN}, build, out);
  if (S > 1) {
    // the template becomes the first stage; the kernel proper adds the partial results up
    RenderedKernel::Pre pre{out->source, out->entry, out->launch};
    out->pres.push_back(pre);
    out->scratch_bytes = (size_t)S * (size_t)Z * (size_t)M * (size_t)N * sizeof(float);
    out->source = std::string(hip_prelude()) + strf("#define POLY_BM %d\n#define POLY_BN %d\n", BM, BN) + cfg + kSplitKCombine;
    out->launch = LaunchSpec();
    out->launch.grid[0] = (unsigned)(((double)Z * M * N + 255) / 256);
    out->launch.block[0] = 256;
    out->strategy += strf(", K dealt to %d workgroups per tile, partial results added by a second kernel", S);
  }
  return true;
}

void matmul_hint_input_params(uint64_t mask) { g_input_params = mask; }
void matmul_hint_param_kinds(const std::vector<int> &kinds) { g_param_kinds = kinds; }
int matmul_param_kind(int param) {
  return param >= 0 && (size_t)param < g_param_kinds.size() ? g_param_kinds[(size_t)param] : 0;
}

bool matmul_tuning_enabled() {
  const char *e = getenv("POLY_BEAM");
  return e && atoi(e) > 0;
}

bool render_matmul(const MatmulMatch &mm, const MatmulEpilogue &ep, RenderedKernel *out) {
  const int64_t K = mm.K, M = mm.M, N = mm.N, Z = mm.Z;
  const Operand &A = mm.A;
  const KSplit &ka = mm.ka, &kb = mm.kb;
  const std::vector<Dim> &md = mm.md, &nd = mm.nd, &zd = mm.zd;
  if (M > 2147483647LL || N > 2147483647LL || Z > 65535) return reject(__LINE__);
  if (A.dt == DT_F32) return ep.mid_value_call.empty() ? render_matmul_f32(mm, ep, out) : false;     // (no second output in the fp32 template)
  int BK = 64;
  if (const char *e = measurement_env("POLY_HIP_MM_BK")) BK = atoi(e) == 32 ? 32 : 64;
  // operand layout: contiguous along K, or along its row axis
  auto layout = [&](const KSplit &ks, const std::vector<Dim> &dims, bool is_a, int64_t rows, bool *kc) {
    int64_t inner_c = is_a ? dims.back().ca : dims.back().cb;
    if (ks.s_lo == 1 && K % BK == 0 && ks.kb % BK == 0) { *kc = true; return true; }
    if (inner_c == 1 && dims.back().extent % 8 == 0 && rows % 8 == 0 && K % BK == 0) { *kc = false; return true; }
    return reject(__LINE__);
  };
  bool a_kc, b_kc;
  if (!layout(ka, md, true, M, &a_kc) || !layout(kb, nd, false, N, &b_kc)) return reject(__LINE__);

  // tile shape: 4 waves; narrow outputs get a narrow tile
  // Candidates: (BM, BN, waves M x N, workgroups resident per CU, throughput of one CU
  // relative to the 256x256 tile as measured on 8192^3).  Pick the smallest estimated
  // time = rounds over the chip * time of one tile.
  int BM = 128, BN = 128, WVM = 2, WVN = 2;
  // (`alone`: the same with one workgroup on the CU, which is all a launch of at most 256
  // tiles gives it: 4096x1024x4096 took 65 us on 256 tiles of 128x128 and 78 us on 128
  // tiles of 128x256.)
  auto pick_tile = [&](bool count_alone) {
    struct Cand { int bm, bn, wm, wn, per_cu; double thr, alone; };
    // (128x256 before 256x128: equal by the estimate, 1-4 % faster when timed on the device)
    static const Cand cands[] = {{256, 256, 4, 2, 1, 1.00, 1.00}, {128, 256, 2, 4, 1, 0.84, 0.84}, {256, 128, 4, 2, 1, 0.84, 0.84}, {128, 128, 2, 2, 2, 0.80, 0.52}};
    double best = 0;
    for (const Cand &c : cands) {
      if (!a_kc && M % 8) continue;
      double t = (double)((M + c.bm - 1) / c.bm) * (double)((N + c.bn - 1) / c.bn) * (double)Z;
      double rounds = std::ceil(t / (256.0 * c.per_cu));
      double est = rounds * (double)c.bm * c.bn / (c.thr / c.per_cu);
      if (count_alone && t <= 256.0) est = (double)c.bm * c.bn / c.alone;
      if (best == 0 || est < best) { best = est; BM = c.bm; BN = c.bn; WVM = c.wm; WVN = c.wn; }
    }
  };
  const bool fixed_tile = N <= 64 || M <= 64;
  if (N <= 64) { BN = 64; BM = 256; WVM = 4; WVN = 1; }
  else if (M <= 64) { BM = 64; BN = 256; WVM = 1; WVN = 4; }
  else pick_tile(false);
  if (const char *ov = getenv("POLY_HIP_MM_TILE")) {   // "BM,BN,WVM,WVN": tuning experiments
    int a, b2, c2, d2;
    if (sscanf(ov, "%d,%d,%d,%d", &a, &b2, &c2, &d2) == 4) { BM = a; BN = b2; WVM = c2; WVN = d2; }
  }
  // a 256x256 tile holds 128 accumulator registers per lane: no room for the second
  // staging register set of the three-deep pipeline
  int pipe = (BM * BN >= 256 * 256) ? 2 : 3;
  if (const char *e = measurement_env("POLY_HIP_MM_PIPE")) pipe = atoi(e) == 2 ? 2 : 3;

  // A deep product on so few tiles that half the chip would idle: the K tiles of a tile are
  // dealt to S workgroups, which leave fp32 partial results in scratch memory, and a second
  // kernel adds them in split order and runs the epilogue.  S minimises rounds over the
  // chip / S among the divisors of the K tile count that leave every part 64 tiles or more.
  // A product of few tiles and moderate depth (no split by that rule) runs on the tile that is
  // fastest with a CU to itself, and may then be split down to parts of 32 K tiles.
  int S = 1;
  size_t part_off = 0;
  auto pick_split = [&](int64_t min_part) {
    const int64_t t = ((M + BM - 1) / BM) * ((N + BN - 1) / BN) * Z, kt = K / BK;
    double best = 0.75;      // worth a second kernel only from a quarter of the time saved
    S = 1;
    for (int s = 2; s <= 16 && t <= 128; s++) {
      if (kt % s != 0 || kt / s < min_part || Z * s > 65535) continue;
      const double r = std::ceil((double)(t * s) / 256.0) / (double)s;
      if (r < best) { best = r; S = s; }
    }
    if ((double)S * (double)Z * (double)M * (double)N * 4.0 > 1073741824.0) S = 1;
  };
  const bool may_split = !getenv("POLY_HIP_NO_SPLIT_K") && !measurement_env("POLY_HIP_MM_NOEPI") && M > 64 && N > 64;
  if (may_split) pick_split(64);
  if (S == 1 && !fixed_tile && !getenv("POLY_HIP_MM_TILE") && !measurement_env("POLY_HIP_MM_OLD_ESTIMATE")) {
    pick_tile(true);
    pipe = (BM * BN >= 256 * 256) ? 2 : 3;
    if (const char *e = measurement_env("POLY_HIP_MM_PIPE")) pipe = atoi(e) == 2 ? 2 : 3;
    if (may_split) pick_split(32);
  }
  if (may_split) {
    const int64_t kt = K / BK;
    if (const char *e = measurement_env("POLY_HIP_MM_KSPLIT")) {   // tuning experiments: a given split
      const int s = atoi(e);
      if (s >= 1 && s <= 64 && kt % s == 0 && Z * s <= 65535) S = s;
    }
    part_off = (ep.scratch_used + 255) / 256 * 256;
  }
  const std::string partials = ep.scratch_type.empty() ? std::string("poly_scratch") : strf("((float*)((char*)poly_scratch + %zuull))", part_off);
  const std::string signature = ep.signature + (S > 1 && ep.scratch_type.empty() ? ", float* poly_scratch" : "");

  // (n_lo, n_hi: the columns this launch covers; n_lo and, unless it is N, n_hi are
  // multiples of bn)
  // The template whose operand tiles go from memory straight into LDS (matmul_dma.hip)
  // takes a tile shape with its own wave layout, K tile, number of LDS stages and
  // workgroups per CU: 256x256 as 8 waves on four stages of 32; 128x256 and 256x128 as 4
  // waves on three stages of 32, two workgroups to a CU, so that one's epilogue runs
  // under the other's K loop; 128x128 as 4 waves on two stages of 64; narrow tiles as 4
  // waves in a row.  `dma_for` says whether a shape has such a form.
  struct Dma { int bk, stages, wg, wvm, wvn; };
  auto dma_for = [&](int bm, int bn, Dma *d) {
    if (getenv("POLY_HIP_NO_DMA")) return false;
    Dma c;
    if (bm * bn >= 256 * 256) c = Dma{32, 4, 1, 4, 2};
    else if (bm * bn >= 128 * 192) c = Dma{32, 3, 2, 2, 2};
    else if (bm * bn >= 128 * 128) c = Dma{64, 2, 2, 2, 2};
    else c = Dma{32, 4, 2, bm >= bn ? 4 : 1, bm >= bn ? 1 : 4};
    if (d->bk) c = *d;      // the caller's own choice
    if (const char *ov = bm * bn < 256 * 256 ? measurement_env("POLY_HIP_MM_DMA") : measurement_env("POLY_HIP_MM_DMA_256")) {   // "BK,STAGES,WG,WVM,WVN": tuning experiments
      int v[5];
      if (sscanf(ov, "%d,%d,%d,%d,%d", &v[0], &v[1], &v[2], &v[3], &v[4]) == 5) c = Dma{v[0], v[1], v[2], v[3], v[4]};
    }
    const int nw = c.wvm * c.wvn;
    if ((c.bk != 32 && c.bk != 64) || c.stages < 2 || c.wg < 1 || nw < 1 || nw > 16) return false;
    if (bm % (32 * c.wvm) || bn % (32 * c.wvn) || K % c.bk) return false;
    if ((a_kc && ka.kb % c.bk) || (b_kc && kb.kb % c.bk)) return false;
    if ((bm * c.bk * 2) % (1024 * nw) || (bn * c.bk * 2) % (1024 * nw)) return false;      // whole LDS loads per wave
    if ((!a_kc && bm < 64) || (!b_kc && bn < 64)) return false;                            // 8 chunks per k-row for the swizzle
    const int stage_bytes = (bm + bn) * c.bk * 2;
    if (c.stages * stage_bytes > 163840 / c.wg || nw * 32 * 36 * 4 > c.stages * stage_bytes) return false;
    *d = c;
    return true;
  };
  auto emit = [&](int bm, int bn, int wvm, int wvn, int pp, RenderedKernel *rk, int64_t n_lo = 0, int64_t n_hi = -1, bool may_dma = true,
                  Dma dma = Dma{0, 0, 0, 0, 0}) {
    if (n_hi < 0) n_hi = N;
    const bool use_dma = may_dma && dma_for(bm, bn, &dma);
    const int bk = use_dma ? dma.bk : BK;
    if (use_dma) { wvm = dma.wvm; wvn = dma.wvn; }
    const int64_t tiles = ((M + bm - 1) / bm) * ((n_hi - n_lo + bn - 1) / bn);
    if (tiles > 2147483647LL / 2) return reject(__LINE__);
    // ── configuration block ─────────────────────────────────────────────────
    std::string cfg;
    cfg += strf("#define POLY_TIN %s\n", dt_cname(A.dt));
    cfg += strf("#define POLY_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_%s(a, b, c, 0, 0, 0)\n", A.dt == DT_BF16 ? "bf16" : "f16");
    cfg += strf("#define POLY_M %lld\n#define POLY_N %lld\n#define POLY_K %lld\n#define POLY_Z %lld\n", (long long)M, (long long)N, (long long)K, (long long)Z);
    cfg += strf("#define POLY_BM %d\n#define POLY_BN %d\n#define POLY_BK %d\n#define POLY_WAVES_M %d\n#define POLY_WAVES_N %d\n", bm, bn, bk, wvm, wvn);
    if (use_dma) cfg += strf("#define POLY_STAGES %d\n#define POLY_WG_PER_CU %d\n", dma.stages, dma.wg);
    // B in HBM as one dense block of K x N elements: extra workgroups at the front of the
    // grid run ahead through it, so that the others wait for HBM once and not at every K tile
    int touch_wgs = 0;
    if (use_dma && ep.b_from_hbm && S == 1 && Z == 1 && zd.empty() && nd.size() == 1 && kb.kb >= K && !getenv("POLY_HIP_NO_PREFETCH") &&
        ((b_kc && kb.s_lo == 1 && nd[0].cb == K) || (!b_kc && nd[0].cb == 1 && kb.s_lo == N)) && K * N * 2 >= (128 << 10) && tiles >= 64) {
      touch_wgs = K * N * 2 >= (2 << 20) ? 64 : 32;
      cfg += strf("#define POLY_TOUCH_WGS %d\n#define POLY_TOUCH_FIRST %lld\n#define POLY_TOUCH_LINES %lldll\n", touch_wgs,
                  (long long)(mm.b_c0 & ~1ll), (long long)((K * N * 2 - 64) / 64));
    }
    if (n_lo != 0 || n_hi != N) cfg += strf("#define POLY_N_LO %lld\n#define POLY_N_HI %lld\n", (long long)n_lo, (long long)n_hi);
    // each XCD (own L2) works on a contiguous run of tiles: let it re-read the smaller operand
    const bool along_n = N > 2 * M && !measurement_env("POLY_HIP_MM_GROUP_M");
    // (bands of 8 tile columns for the wide product: the 50257-wide head 727 -> 710 us against bands of 4)
    cfg += strf("#define POLY_GROUP_M %d\n", bm >= 256 && !(along_n && use_dma) ? 4 : 8);
    cfg += strf("#define POLY_GROUP_ALONG_N %d\n", along_n ? 1 : 0);
    cfg += strf("#define POLY_PIPE %d\n", pp);
    // timing experiments only (wrong results): walk just the first n K tiles
    if (const char *e = measurement_env("POLY_HIP_MM_KT")) if (atoi(e) > 0 && atoi(e) <= K / bk) cfg += strf("#define POLY_KT %d\n", atoi(e));
    cfg += strf("#define POLY_A_KC %d\n#define POLY_B_KC %d\n", a_kc ? 1 : 0, b_kc ? 1 : 0);
    cfg += strf("#define POLY_A_PTR %s\n#define POLY_B_PTR %s\n", ep.a_ptr.c_str(), ep.b_ptr.c_str());
    cfg += offset_fn("poly_a_row", md, true, 0);
    cfg += offset_fn("poly_b_row", nd, false, 0);
    if (zd.empty()) {
      cfg += strf("__device__ __forceinline__ int poly_a_z(int) { return %lld; }\n", (long long)mm.a_c0);
      cfg += strf("__device__ __forceinline__ int poly_b_z(int) { return %lld; }\n", (long long)mm.b_c0);
    } else {
      cfg += offset_fn("poly_a_z", zd, true, mm.a_c0);
      cfg += offset_fn("poly_b_z", zd, false, mm.b_c0);
    }
    cfg += matmul_k_fn("poly_a_k", ka, K);
    cfg += matmul_k_fn("poly_b_k", kb, K);
    // block maxima for a later launch (MatmulEpilogue::block_maxima): this template, one z, tiles of whole blocks
    const bool block_maxima = ep.block_maxima.wanted && use_dma && S == 1 && Z == 1 && zd.empty() && bm % 64 == 0 && bn % 64 == 0 && M % 64 == 0 &&
                              ep.contiguous_n && (ep.out_type == "__bf16" || ep.out_type == "_Float16") && ep.scratch_type.empty() &&
                              ep.block_maxima.lo % 64 == 0 && ep.block_maxima.hi % 64 == 0 && ep.block_maxima.hi <= N &&
                              !measurement_env("POLY_HIP_MM_NOEPI");
    if (block_maxima)
      cfg += strf("#define POLY_EP_BLOCKMAX_LO %lld\n#define POLY_EP_BLOCKMAX_HI %lld\n#define POLY_EP_BLOCKMAX_IDX(m, n) (%s)\n#define POLY_EP_BLOCKMAX_PTR poly_scratch\n",
                  (long long)ep.block_maxima.lo, (long long)ep.block_maxima.hi, ep.block_maxima.index.c_str());
    cfg += strf("#define POLY_SIGNATURE %s%s\n", signature.c_str(), block_maxima ? ", unsigned int* poly_scratch" : "");
    // LDS beside the operand tiles that an epilogue may use for the middle of its lookup tables
    if (S == 1 && !getenv("POLY_HIP_NO_LUT_WINDOW")) {
      if (!use_dma) cfg += strf("#define POLY_EP_WIN_ROOM %d\n", 163840 - 2 * (bm + bn) * BK * 2);
      else {
        // the window moves into the stage that tile KT - STAGES leaves; the output staging
        // must fit before or behind that stage
        const int kt = (int)(K / bk), stage_bytes = (bm + bn) * bk * 2, out_bytes = wvm * wvn * 32 * 36 * 4;
        const int win_stage = kt >= dma.stages ? (kt - dma.stages) % dma.stages : 0;
        const bool fits = kt >= dma.stages && (out_bytes <= win_stage * stage_bytes || out_bytes <= (dma.stages - 1 - win_stage) * stage_bytes);
        cfg += strf("#define POLY_EP_WIN_ROOM %d\n", fits ? stage_bytes / 1024 * 1024 : 0);
      }
    }
    cfg += ep.code;
    if (S > 1) {
      cfg += strf("#define POLY_KSPLIT %d\n#define POLY_PARTIALS %s\n", S, partials.c_str());
      cfg += "#define POLY_EP_CONTIG 1\n#define POLY_EP_TYPE float\n#define POLY_EP_VALUE(acc, m, n, z) (acc)\n";
      cfg += "#define POLY_EP_PTR(m, n, z) (POLY_PARTIALS + (((size_t)poly_ks * POLY_Z + (z)) * POLY_M + (m)) * POLY_N + (n))\n";
      cfg += "#define POLY_EPILOGUE(acc, m, n, z) *POLY_EP_PTR(m, n, z) = (acc)\n";
    } else
    if (measurement_env("POLY_HIP_MM_NOEPI")) cfg += strf("#define POLY_EPILOGUE(acc, m, n, z) do { if (((m) | (n)) == -1) { %s; } } while (0)\n", ep.call.c_str());
    else
    cfg += strf("#define POLY_EPILOGUE(acc, m, n, z) %s\n", ep.call.c_str());
    const bool split = S == 1 && ep.contiguous_n && !measurement_env("POLY_HIP_MM_NOEPI") && (ep.out_type == "__bf16" || ep.out_type == "_Float16" || ep.out_type == "float");
    if (S == 1) cfg += strf("#define POLY_EP_CONTIG %d\n", split ? 1 : 0);
    if (!ep.mid_value_call.empty() && !split) return false;      // (a second output only in the contiguous form)
    if (split && !ep.mid_value_call.empty())
      cfg += strf("#define POLY_EP_MID_TYPE %s\n#define POLY_EP_MID_VALUE(acc, m, n, z) %s\n#define POLY_EP_MID_PTR(m, n, z) %s\n", ep.mid_type.c_str(),
                  ep.mid_value_call.c_str(), ep.mid_ptr_call.c_str());
    if (split) {
      cfg += strf("#define POLY_EP_TYPE %s\n", ep.out_type.c_str());
      cfg += strf("#define POLY_EP_VALUE(acc, m, n, z) %s\n", ep.value_call.c_str());
      if (!ep.value_call_win.empty()) cfg += strf("#define POLY_EP_VALUE_WIN(acc, m, n, z) %s\n", ep.value_call_win.c_str());
      cfg += strf("#define POLY_EP_PTR(m, n, z) %s\n", ep.ptr_call.c_str());
    }

    *rk = RenderedKernel();
    rk->source = std::string(hip_prelude()) + cfg + (use_dma ? kMatmulDmaTemplate : kMatmulTemplate);
    rk->entry = "poly_k";
    rk->launch.grid[0] = (unsigned)(tiles + touch_wgs);
    rk->launch.grid[1] = (unsigned)(Z * S);
    rk->launch.block[0] = (unsigned)(64 * wvm * wvn);
    rk->klass = KernelClass::MATMUL_MFMA;
    rk->reads_b_ahead = touch_wgs > 0;
    rk->writes_block_maxima = block_maxima;
    if (block_maxima) rk->scratch_bytes = ep.block_maxima.bytes;
    rk->strategy = strf("mfma 32x32x16 %s M=%lld N=%lld K=%lld Z=%lld tile %dx%dx%d A:%s B:%s", A.dt == DT_BF16 ? "bf16" : "f16",
                        (long long)M, (long long)N, (long long)K, (long long)Z, bm, bn, bk, a_kc ? "k-major" : "m-major",
                        b_kc ? "k-major" : "n-major");
    if (use_dma) rk->strategy += strf(", operands straight into LDS: %d waves, %d stages, %d per CU", wvm * wvn, dma.stages, dma.wg);
    if (touch_wgs) rk->strategy += strf(", %d workgroups read B ahead", touch_wgs);
    if (block_maxima) rk->strategy += strf(", leaves the largest magnitude of every 64x64 block of columns [%lld, %lld) for the launch that reads them",
                                           (long long)ep.block_maxima.lo, (long long)ep.block_maxima.hi);
    rk->n_params = ep.n_params;
    rk->n_vars = 0;
    rk->flops = 2.0 * (double)M * (double)N * (double)K * (double)Z;
    rk->bytes = ep.bytes;
    return true;
  };
  // Tile shapes of the straight-into-LDS template, from timings inside the GPT-2 forward
  // plan (M = 8192, K = 768 or 3072) and the GPT-2 medium training step (M = 4096, N = 1024,
  // K = 4096).  A launch of at most 256 tiles of 128x256 leaves a CU one workgroup of four
  // waves, too little to hide anything: 128x128 tiles -- two workgroups to a CU on two
  // stages of 64 when there are more than 256 of them (N = 768: 21.7 -> 19.6 us at K = 768,
  // 47.8 -> 46.2 us at K = 3072), one to a CU on four stages otherwise (4096x1024x4096: 32 us
  // against 48 us on two stages and 44 us for the template that stages through registers).
  // Between one and one and a quarter rounds of 512 workgroups, 128x192 tiles when they
  // divide N and give a round and a half (N = 2304: 43.6 -> 39.9 us).  Narrow outputs (one
  // tile of 64 across) stay with the template that stages through registers.
  Dma chosen{0, 0, 0, 0, 0};
  bool dma_ok = !fixed_tile;
  if (!fixed_tile && !getenv("POLY_HIP_MM_TILE") && BM * BN <= 128 * 256) {
    Dma probe{0, 0, 0, 0, 0};
    auto count = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn) * Z * S; };   // workgroups of the launch
    const int64_t t = count(BM, BN);
    if (dma_for(BM, BN, &probe)) {
      Dma p2{0, 0, 0, 0, 0}, p3{0, 0, 0, 0, 0}, wide{64, 3, 1, 2, 4};
      // Three quarters of a round of 128x256 tiles and more on a deep K, A along k and B along
      // n (8192 x 768 x 3072 of the GPT-2 layer, 192 tiles): the tile stays, on 8 waves of
      // 64x64 and three stages of 64, one workgroup per CU -- found by the tuner, inside the
      // plan 43.5 -> 41.8 us against the 128x128 tiles below (step 3.22 -> 3.20 ms); at
      // K = 768 the two are equal, with 128 tiles (4096 x 1024 x 4096) it loses by a third.
      if (S == 1 && Z == 1 && BM == 128 && BN == 256 && t >= 192 && t <= 256 && a_kc && !b_kc && K >= 1536 && !getenv("POLY_HIP_NO_WIDE_SMALL_LAUNCH") &&
          dma_for(128, 256, &wide)) { WVM = 2; WVN = 4; chosen = wide; }
      else
      if (S == 1 && BM * BN == 128 * 256 && t <= 256 && M % 128 == 0 && dma_for(128, 128, &p2)) { BM = BN = 128; WVM = WVN = 2; }
      else if (S == 1 && BM * BN == 128 * 256 && t > 512 && t < 640 && N % 192 == 0 && count(128, 192) >= 768 && dma_for(128, 192, &p3)) { BM = 128; BN = 192; WVM = WVN = 2; }
      if (BM == 128 && BN == 128 && count(128, 128) <= 256) {
        Dma deep{64, 4, 1, 2, 2};
        if (dma_for(128, 128, &deep)) chosen = deep;
      }
    }
  }
  // Many rounds of a short K loop with both operands contiguous along k (the 50 257-wide
  // head: K = 768 or 1024, 6000 and 3000 tiles of 256x256; from two rounds up: the head for
  // one sequence, 788 tiles, 1.405 -> 1.362 ms for its plan; at 256 tiles a product with a
  // table epilogue was 88 against 98 us the other way round): 192x128 tiles on 64-deep stages,
  // two workgroups to a CU, so that one's stores run under the other's K loop -- the head of
  // GPT-2 small 682 -> 608 us, of GPT-2 medium 565 -> 509 us inside their plans (128x192:
  // 621 and 520; 128x128: 664; on 32-deep stages the same tiles are slower than 256x256, and
  // so is this one for K = 4096 and up or with a row-contiguous B).
  if (!fixed_tile && !getenv("POLY_HIP_MM_TILE") && !getenv("POLY_HIP_NO_HEAD_TILE") && S == 1 && a_kc && b_kc && K >= 512 && K <= 1536 && K % 64 == 0 && BM == 256 &&
      BN == 256 && ((M + 255) / 256) * ((N + 255) / 256) * Z >= 512) {
    Dma d{64, 2, 2, 2, 2};
    if (dma_for(192, 128, &d)) { BM = 192; BN = 128; WVM = WVN = 2; chosen = d; }
  }
  // A K loop of a few tiles (K = 64: the scores of attention and the derivative of its
  // probabilities in a training step, 1024 tiles of 256x256 each) is all prologue and
  // epilogue: one workgroup of 256x256 per CU loads, multiplies and stores in turn, two of
  // 128x256 overlap one's stores with the other's loads -- stand-alone on 8192 x 8192 x 64,
  // 134 MB of bf16 out: 29.5 -> 26.4 us; 268 MB of fp32 out: 70.1 -> 49.1 us.
  if (!fixed_tile && !getenv("POLY_HIP_MM_TILE") && !getenv("POLY_HIP_NO_SHORT_K_TILE") && S == 1 && K <= 128 && BM == 256 && BN == 256) {
    Dma d{0, 0, 0, 0, 0};
    if (dma_for(128, 256, &d)) { BM = 128; BN = 256; WVM = WVN = 2; chosen = d; pipe = 3; }
  }
  if (!emit(BM, BN, WVM, WVN, pipe, out, 0, -1, dma_ok, chosen)) return false;
  if (S > 1) {
    // the template becomes a first stage; the kernel proper adds the partial results up
    RenderedKernel::Pre pre{out->source, out->entry, out->launch};
    out->pres.push_back(pre);
    out->scratch_bytes = part_off + (size_t)S * (size_t)Z * (size_t)M * (size_t)N * sizeof(float);
    std::string cfg;
    cfg += strf("#define POLY_M %lld\n#define POLY_N %lld\n#define POLY_Z %lld\n#define POLY_KSPLIT %d\n", (long long)M, (long long)N, (long long)Z, S);
    cfg += strf("#define POLY_PARTIALS %s\n#define POLY_SIGNATURE %s\n", partials.c_str(), signature.c_str());
    cfg += ep.code;
    cfg += strf("#define POLY_EPILOGUE(acc, m, n, z) %s\n", ep.call.c_str());
    out->source = std::string(hip_prelude()) + cfg + kSplitKCombine;
    out->launch = LaunchSpec();
    out->launch.grid[0] = (unsigned)(((double)Z * M * N + 255) / 256);
    out->launch.block[0] = 256;
    out->strategy += strf(", K dealt to %d workgroups per tile, partial results added by a second kernel", S);
    return true;
  }
  // A last round over the chip that is at most half full (8192 x 2304 in 128 x 256 tiles:
  // 576 tiles, two rounds and a quarter) costs a whole round.  The launch then keeps the
  // columns whose tiles make whole rounds, and the columns left over go to a launch of
  // their own ahead of it, in tiles a quarter or half the size, so that they fill the chip
  // once with short workgroups.  Taken when the estimate (rounds, a small tile's round
  // weighted by its area and by what its narrower wave tiles cost, plus a launch) saves
  // a quarter of a round or more.
  if (Z == 1 && M > 64 && N > 64 && !matmul_tuning_enabled() && !getenv("POLY_HIP_NO_TAIL_LAUNCH") && !measurement_env("POLY_HIP_MM_NOEPI")) {
    const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN, T = tm * tn;
    const int64_t whole = T / 256, rest = T % 256;
    const int64_t keep = std::min<int64_t>(whole * 256 / tm, tn - 1);     // column tiles of the main launch
    if (whole >= 1 && rest > 0 && keep >= 1 && (!a_kc ? M % 8 == 0 : true)) {
      struct Small { int bm, bn, wm, wn; double cost; };
      // cost of a launch of one round of such tiles relative to a round of 128 x 256 tiles
      // (measured at K = 768: 12.6 and 10.5 us against 18.6; most of it does not depend on
      // the tile: the launch, the first loads, the epilogue)
      static const Small smalls[] = {{128, 128, 2, 2, 0.68}, {128, 64, 4, 1, 0.56}};
      const int64_t n_lo = keep * BN;
      const double before = std::ceil((double)T / 256.0);
      double best = before - 0.25;
      const Small *pick = nullptr;
      for (const Small &c : smalls) {
        if (c.bm > BM || c.bn > BN) continue;
        const double scale = (128.0 * 256.0) / ((double)BM * BN);
        const int64_t tt = ((M + c.bm - 1) / c.bm) * ((N - n_lo + c.bn - 1) / c.bn);
        const double after = std::ceil((double)(tm * keep) / 256.0) + std::ceil((double)tt / 256.0) * c.cost * scale + 0.1;
        if (after < best) { best = after; pick = &c; }
      }
      Small forced{0, 0, 0, 0, 0};
      if (const char *ov = measurement_env("POLY_HIP_MM_TAIL_TILE"))    // "BM,BN,WVM,WVN": tuning experiments
        if (sscanf(ov, "%d,%d,%d,%d", &forced.bm, &forced.bn, &forced.wm, &forced.wn) == 4 && BN % forced.bn == 0) pick = &forced;
      RenderedKernel main, tail;
      if (pick && emit(BM, BN, WVM, WVN, pipe, &main, 0, n_lo) && emit(pick->bm, pick->bn, pick->wm, pick->wn, 3, &tail, n_lo, N) &&
          main.writes_block_maxima == out->writes_block_maxima && tail.writes_block_maxima == out->writes_block_maxima) {
        const std::string strategy = out->strategy;
        *out = main;
        out->pres.push_back({tail.source, tail.entry, tail.launch});
        out->scratch_bytes = std::max<size_t>(256, main.scratch_bytes);      // (a kernel with a first stage owns scratch memory)
        out->strategy = strategy + strf(", columns from %lld on by a launch of %dx%d tiles ahead of it", (long long)n_lo, pick->bm, pick->bn);
        return true;
      }
    }
  }
  // Candidates for on-device tuning: the same kernel in the other tile shapes and
  // pipeline depths; the plan times them on its first run when POLY_BEAM is set.
  if (matmul_tuning_enabled() && M > 64 && N > 64 && !(!a_kc && M % 8)) {
    struct Shape { int bm, bn, wm, wn, pp; };
    static const Shape shapes[] = {{256, 256, 4, 2, 2}, {256, 128, 4, 2, 3}, {256, 128, 4, 2, 2}, {128, 256, 2, 4, 3},
                                   {128, 256, 2, 4, 2}, {128, 128, 2, 2, 3}, {128, 128, 2, 2, 2}};
    out->variants.push_back({"default", out->source, out->strategy, out->launch});
    // the template with register staging
    for (const Shape &c : shapes) {
      RenderedKernel v;
      if (emit(c.bm, c.bn, c.wm, c.wn, c.pp, &v, 0, -1, false) && v.source != out->source && v.writes_block_maxima == out->writes_block_maxima)
        out->variants.push_back({strf("%dx%dw%dx%dp%d", c.bm, c.bn, c.wm, c.wn, c.pp), v.source, v.strategy, v.launch});
    }
    // the template that loads straight into LDS: tile, K tile, stages, workgroups per CU, waves
    struct DShape { int bm, bn; Dma d; };
    static const DShape dshapes[] = {{256, 256, {32, 4, 1, 4, 2}}, {256, 256, {64, 2, 1, 4, 2}}, {128, 256, {32, 3, 2, 2, 2}}, {256, 128, {32, 3, 2, 2, 2}},
                                     {128, 256, {64, 3, 1, 2, 4}}, {256, 128, {64, 3, 1, 4, 2}}, {128, 192, {32, 3, 2, 2, 2}}, {128, 128, {64, 2, 2, 2, 2}},
                                     {128, 128, {32, 4, 2, 2, 2}}};
    // (measured and left out: 256x192 and 192x256 on 8 waves; three or four workgroups per CU
    // on two or three stages -- 128x256, 128x192, 128x128 -- all slower than the rules' choice
    // on every product of the GPT-2 step)
    for (const DShape &c : dshapes) {
      RenderedKernel v;
      if (emit(c.bm, c.bn, c.d.wvm, c.d.wvn, 3, &v, 0, -1, true, c.d) && v.source != out->source && v.strategy.find("straight into LDS") != std::string::npos &&
          v.writes_block_maxima == out->writes_block_maxima)
        out->variants.push_back({strf("%dx%dx%dw%dx%ds%dg%d", c.bm, c.bn, c.d.bk, c.d.wvm, c.d.wvn, c.d.stages, c.d.wg), v.source, v.strategy, v.launch});
    }
  }
  return true;
}

// ── matmul-shaped reductions whose operands are expressions ─────────────────
//
// Reverse-mode graphs multiply whatever the scheduler fused into the reduction: an fp32
// gradient with a bf16 activation, a LayerNorm or softmax derivative evaluated in place,
// sums over two ranges (batch and position), extents like 50257.  Any kernel of the form
//     STORE(f(REDUCE(ADD, a * b, k...)))      a, b fp32-valued
// in which some END range feeds only `a` and another only `b` is a matrix product
// C[z][m][n] = sum_k A(z,m,k) B(z,k,n) of two computed operands.  The fp32 MFMA template
// runs it with the operands evaluated on the way into LDS: the loads of an element are
// issued K tiles ahead (phase 1, raw bits kept in registers), the arithmetic on them runs
// when the tile is stored to LDS (phase 2).  Products are exact fp32, accumulation fp32.
// Value of canonical index expression `l` at range values `rv` (false: not a function of
// ranges alone).
static bool eval_lin(const KernelGraph &g, const Lin &l, const std::vector<int64_t> &rv, int64_t *out) {
  int64_t v = l.c0;
  for (const Term &t : l.terms) {
    const Atom &a = g.atoms[(size_t)t.atom];
    int64_t x;
    if (a.kind == Atom::RANGE) x = rv[(size_t)g.range_ord.at(a.node)];
    else if (a.kind == Atom::DIV || a.kind == Atom::MOD) {
      int64_t in;
      if (!eval_lin(g, a.inner, rv, &in) || in < 0 || a.c <= 0) return false;
      x = a.kind == Atom::DIV ? in / a.c : in % a.c;
    } else return false;
    v += t.coef * x;
  }
  *out = v;
  return true;
}

// Does every atom of index `l` depend on ranges of only one of the three groups (bit masks
// of range ordinals), and on no other range?  Then the index is a sum of a part per group.
// A DIV or MOD atom whose inner expression mixes ranges of two groups fails here whatever
// values a sampled comparison would happen to hit.  (An atom over a single range is fine
// even when two groups own digits of that range: its uses are taken apart digit by digit.)
static bool lin_separates(const KernelGraph &g, const Lin &l, uint64_t rows_mask, uint64_t k_mask, uint64_t z_mask) {
  for (const Term &t : l.terms) {
    const uint64_t deps = g.atom_deps(t.atom);
    if (deps & ~(rows_mask | k_mask | z_mask)) return false;
    if ((deps & (deps - 1)) == 0) continue;
    const int groups = ((deps & rows_mask) != 0) + ((deps & k_mask) != 0) + ((deps & z_mask) != 0);
    if (groups > 1) return false;
  }
  return true;
}
static uint64_t ord_mask(const std::vector<Dim> &dims) {
  uint64_t m = 0;
  for (const Dim &d : dims) if (d.ord >= 0 && d.ord < 64) m |= (uint64_t)1 << d.ord;
  return m;
}

// Describes operand `node` of a product without naming ranges (RenderedKernel::OperandPlanes):
// `loads` are its LOADs, `rows` / `kd` / `zd` the digits that make up its row, depth and
// batch coordinates.
static void describe_operand(const KernelGraph &g, int node, const std::vector<int> &loads, const std::vector<Dim> &rows,
                             const std::vector<Dim> &kd, const std::vector<Dim> &zd, int64_t M, int64_t K, int64_t Z,
                             RenderedKernel::OperandPlanes *out) {
  out->valid = false;
  out->rows = M; out->k = K; out->z = Z;
  if (loads.empty() || M + K + Z > 1048576) return;
  // the arithmetic, nodes numbered in the order they are met
  std::map<int, int> seen;
  std::vector<int> load_order;
  bool ok = true;
  std::string text;
  std::function<void(int)> walk = [&](int id) {
    if (!ok) return;
    auto it = seen.find(id);
    if (it != seen.end()) { text += strf("@%d ", it->second); return; }
    const int my = (int)seen.size();
    seen[id] = my;
    const KNode &k = g.n(id);
    if (k.op == POLY_OP_LOAD) {
      const KNode &ix = g.n(k.src[0]);
      if (k.guard >= 0 || ix.op != POLY_OP_INDEX || ix.src.size() != 2 || g.n(ix.src[1]).lin < 0) { ok = false; return; }
      text += strf("L%zu ", load_order.size());
      load_order.push_back(id);
      return;
    }
    if (k.op == POLY_OP_CONST) {
      const PolyArg &a = k.u->arg;
      long long bits = 0;
      if (a.kind == POLY_ARG_FLOAT) memcpy(&bits, &a.f, sizeof bits);
      else if (a.kind == POLY_ARG_INT) bits = (long long)a.i;
      else if (a.kind == POLY_ARG_BOOL) bits = a.b ? 1 : 0;
      else { ok = false; return; }
      text += strf("C%d:%d:%llx ", (int)k.dt, (int)a.kind, bits);
      return;
    }
    if (k.op == POLY_OP_RANGE || k.op == POLY_OP_INDEX || k.op == POLY_OP_PARAM || k.op == POLY_OP_DEFINE_VAR || k.op == POLY_OP_REDUCE ||
        k.op == POLY_OP_SPECIAL || k.op == POLY_OP_BIND || k.op == POLY_OP_STORE || k.u->arg.kind != POLY_ARG_NONE || k.src.empty()) { ok = false; return; }
    text += strf("(%d:%d ", (int)k.op, (int)k.dt);
    for (int c : k.src) walk(c);
    text += ") ";
  };
  walk(node);
  if (!ok || load_order.size() != loads.size()) return;
  // the addresses
  std::vector<int64_t> rv(g.ranges.size());
  auto address = [&](const Lin &l, int64_t m, int64_t k, int64_t z, int64_t *a) {
    std::fill(rv.begin(), rv.end(), 0);
    auto put = [&](const std::vector<Dim> &dims, int64_t x) {
      for (size_t i = dims.size(); i-- > 0;) {
        const int64_t digit = i == 0 ? x : x % dims[i].extent;
        if (i) x /= dims[i].extent;
        rv[(size_t)dims[i].ord] += digit * dims[i].cut;
      }
    };
    put(rows, m); put(kd, k); put(zd, z);
    return eval_lin(g, l, rv, a);
  };
  out->loads.clear();
  for (int id : load_order) {
    const KNode &ld = g.n(id);
    const KNode &ix = g.n(ld.src[0]);
    const Lin &l = g.lins[(size_t)g.n(ix.src[1]).lin];
    RenderedKernel::OperandPlanes::Load d;
    d.param = g.param_slot(ix.src[0]);
    d.dt = (int)ld.dt;
    if (d.param < 0 || !address(l, 0, 0, 0, &d.base)) return;
    if (!lin_separates(g, l, ord_mask(rows), ord_mask(kd), ord_mask(zd))) return;
    d.by_row.resize((size_t)M); d.by_k.resize((size_t)K); d.by_z.resize((size_t)Z);
    int64_t a;
    for (int64_t m = 0; m < M; m++) { if (!address(l, m, 0, 0, &a)) return; d.by_row[(size_t)m] = a - d.base; }
    for (int64_t k = 0; k < K; k++) { if (!address(l, 0, k, 0, &a)) return; d.by_k[(size_t)k] = a - d.base; }
    for (int64_t z = 0; z < Z; z++) { if (!address(l, 0, 0, z, &a)) return; d.by_z[(size_t)z] = a - d.base; }
    // the address is the sum of the three parts (no atom mixes two of them: checked above by
    // structure); compared at scattered points and the far corner all the same
    uint64_t rnd = 0x9e3779b97f4a7c15ull;
    for (int t = 0; t < 256; t++) {
      rnd = rnd * 6364136223846793005ull + 1442695040888963407ull;
      int64_t m = (int64_t)((rnd >> 33) % (uint64_t)M), k = (int64_t)((rnd >> 13) % (uint64_t)K), z = (int64_t)((rnd >> 3) % (uint64_t)Z);
      if (t == 0) { m = M - 1; k = K - 1; z = Z - 1; }
      if (!address(l, m, k, z, &a) || a != d.base + d.by_row[(size_t)m] + d.by_k[(size_t)k] + d.by_z[(size_t)z]) return;
    }
    out->loads.push_back(std::move(d));
  }
  out->dag = text;
  out->valid = true;
}

// Is operand `mine` the operand behind `theirs` with rows and depth exchanged?
static bool exchanged(const RenderedKernel::OperandPlanes &mine, const RenderedKernel::OperandPlanes &theirs) {
  if (!mine.valid || !theirs.valid || mine.parts != theirs.parts || mine.rows != theirs.k || mine.k != theirs.rows || mine.z != theirs.z ||
      mine.dag != theirs.dag || mine.loads.size() != theirs.loads.size())
    return false;
  for (size_t j = 0; j < mine.loads.size(); j++) {
    const auto &a = mine.loads[j], &b = theirs.loads[j];
    if (a.param != b.param || a.dt != b.dt || a.base != b.base || a.by_row != b.by_k || a.by_k != b.by_row || a.by_z != b.by_z) return false;
  }
  return true;
}

bool try_render_matmul_generic(const KernelGraph &g, const std::string &fn, const RenderOptions &opt, RenderedKernel *out) {
  (void)fn;
  if (getenv("POLY_HIP_NO_F32_MFMA") || getenv("POLY_HIP_NO_GENERIC_MM")) return reject(__LINE__);
  if (g.stores.size() != 1 || g.reduces.size() != 1 || !g.vars.empty()) return reject(__LINE__);
  const StoreInfo &st = g.stores[0];
  if (st.gate >= 0) return reject(__LINE__);
  const int red = g.reduces[0];
  const KNode &R = g.n(red);
  if (reduce_op(R) != POLY_OP_ADD || R.dt != DT_F32 || R.src.size() < 2) return reject(__LINE__);
  const KNode &mul = g.n(R.src[0]);
  if (mul.op != POLY_OP_MUL || mul.dt != DT_F32) return reject(__LINE__);
  const int opnd[2] = {mul.src[0], mul.src[1]};
  std::vector<int> kr;
  int64_t K = 1;
  uint64_t kmask = 0;
  for (size_t i = 1; i < R.src.size(); i++) {
    const int o = g.range_ord.at(R.src[i]);
    const int64_t e = g.ranges[(size_t)o].extent;
    if (e <= 0) return reject(__LINE__);
    kr.push_back(o);
    K *= e;
    kmask |= (uint64_t)1 << o;
  }
  const uint64_t dep[2] = {g.n(opnd[0]).deps, g.n(opnd[1]).deps};
  if (!(dep[0] & kmask) || !(dep[1] & kmask)) return reject(__LINE__);
  // How each operand uses the END ranges.  A flat output range may carry the row of one
  // operand in its upper digits and the column of the other in its lower ones (r / c and
  // r % c in the load indices); such a range is cut into digits as in match_matmul.  That
  // needs every use of the range inside the operand to be a load index: `direct` marks
  // ranges an operand also reaches outside INDEX nodes (then the operand owns all of it).
  std::vector<const Lin *> lins[2];
  uint64_t direct[2] = {0, 0};
  for (int side = 0; side < 2; side++) {
    std::vector<int> stack{opnd[side]};
    std::vector<char> seen(g.nodes.size(), 0);
    while (!stack.empty()) {
      const int id = stack.back();
      stack.pop_back();
      if (seen[(size_t)id]) continue;
      seen[(size_t)id] = 1;
      const KNode &k = g.n(id);
      if (k.op == POLY_OP_RANGE) { direct[side] |= (uint64_t)1 << g.range_ord.at(id); continue; }
      if (k.op == POLY_OP_INDEX) {
        for (size_t i = 1; i < k.src.size(); i++) {
          const int li = g.n(k.src[i]).lin;
          if (li >= 0) lins[side].push_back(&g.lins[(size_t)li]);
          else direct[side] |= g.n(k.src[i]).deps;      // an index or gate that is no canonical expression
        }
        continue;
      }
      for (int c : k.src) stack.push_back(c);
    }
  }
  MatmulMatch mm;
  for (int r : st.ranges) {
    const int64_t e = g.ranges[(size_t)r].extent;
    if (e <= 0) return reject(__LINE__);
    const uint64_t bit = (uint64_t)1 << r;
    std::vector<DigitUse> uses[2];
    bool digits_ok = !((direct[0] | direct[1]) & bit);
    for (int side = 0; side < 2 && digits_ok; side++)
      for (const Lin *l : lins[side]) if (!digit_uses(g, *l, r, &uses[side])) { digits_ok = false; break; }
    std::vector<int64_t> cuts{1, e};
    if (digits_ok) {
      for (int side = 0; side < 2; side++)
        for (const DigitUse &d : uses[side]) {
          cuts.push_back(d.a);
          if (d.b > 0) cuts.push_back(d.a * d.b);
        }
      std::sort(cuts.begin(), cuts.end());
      cuts.erase(std::unique(cuts.begin(), cuts.end()), cuts.end());
      while (!cuts.empty() && cuts.back() > e) cuts.pop_back();
      for (size_t i = 0; i + 1 < cuts.size(); i++) if (cuts[i + 1] % cuts[i] != 0) digits_ok = false;
      if (cuts.empty() || cuts.back() != e) digits_ok = false;
    }
    if (!digits_ok) {
      const bool in_a = (dep[0] & bit) != 0, in_b = (dep[1] & bit) != 0;
      Dim d{r, e, 0, 0, 1};
      if (in_a && !in_b) mm.md_full.push_back(d);
      else if (in_b && !in_a) mm.nd_full.push_back(d);
      else mm.zd_full.push_back(d);
      continue;
    }
    auto used = [&](const std::vector<DigitUse> &u, int64_t cut) {
      for (const DigitUse &d : u)
        if (cut >= d.a && (d.b == 0 || cut < d.a * d.b) && d.coef != 0) return true;
      return false;
    };
    for (size_t i = cuts.size() - 1; i-- > 0;) {
      Dim d{r, cuts[i + 1] / cuts[i], 0, 0, cuts[i]};
      const bool in_a = used(uses[0], cuts[i]), in_b = used(uses[1], cuts[i]);
      if (in_a && !in_b) mm.md_full.push_back(d);
      else if (in_b && !in_a) mm.nd_full.push_back(d);
      else mm.zd_full.push_back(d);
    }
  }
  if (mm.md_full.empty() || mm.nd_full.empty()) return reject(__LINE__);
  mm.M = mm.N = mm.Z = 1;
  for (const Dim &d : mm.md_full) mm.M *= d.extent;
  for (const Dim &d : mm.nd_full) mm.N *= d.extent;
  for (const Dim &d : mm.zd_full) mm.Z *= d.extent;
  mm.md = mm.md_full; mm.nd = mm.nd_full; mm.zd = mm.zd_full;
  mm.red = red; mm.K = K;
  const int64_t M = mm.M, N = mm.N, Z = mm.Z;
  // worth a tile pipeline: enough rows, columns and depth
  if (M < 32 || N < 32 || K < 32 || Z > 65535 || M > 2147483647LL || N > 2147483647LL || K > 2147483647LL) return reject(__LINE__);
  if ((double)M * (double)N * (double)K * (double)Z < 1048576.0) return reject(__LINE__);
  for (const ParamInfo &p : g.params) if (p.numel >= ((int64_t)1 << 31)) return reject(__LINE__);

  MatmulEpilogue ep;
  if (!epilogue_from_graph(g, mm, &ep)) return reject(__LINE__);
  const std::string params_call = ep.params_call;

  // C text that splits flattened coordinate `var` into digits (last one fastest); the
  // value of a range is the sum of its digits times their cuts over the coordinates a
  // function has (an operand never looks at the digits it does not get: they count as 0)
  struct Bound { std::string code; std::map<int, std::string> range_sum; };
  auto split_digits = [&](const std::vector<Dim> &dims, const char *var, Bound *b) {
    if (dims.empty()) return;
    b->code += strf("  int t_%s = %s;\n", var, var);
    for (size_t i = dims.size(); i-- > 0;) {
      const Dim &d = dims[i];
      const std::string dv = strf("d%d_%lld", d.ord, (long long)d.cut);
      if (i == 0) b->code += strf("  const int %s = t_%s;\n", dv.c_str(), var);
      else b->code += strf("  const int %s = t_%s %% %lld; t_%s /= %lld;\n", dv.c_str(), var, (long long)d.extent, var, (long long)d.extent);
      const std::string term = d.cut == 1 ? dv : strf("%s * %lld", dv.c_str(), (long long)d.cut);
      std::string &sum = b->range_sum[d.ord];
      sum = sum.empty() ? term : sum + " + " + term;
    }
  };
  std::vector<Dim> k_dims;
  for (int o : kr) k_dims.push_back(Dim{o, g.ranges[(size_t)o].extent, 0, 0, 1});
  auto bind_all = [&](const std::vector<Dim> &rows, const char *rowvar, Emitter &em, Scope &S) {
    Bound b;
    split_digits(rows, rowvar, &b);
    split_digits(k_dims, "k", &b);
    split_digits(mm.zd_full, "z", &b);
    for (auto &rs : b.range_sum) {
      b.code += strf("  const int r%d = %s;\n", rs.first, rs.second.c_str());
      em.bind_range(rs.first, strf("r%d", rs.first));
      S.avail |= (uint64_t)1 << rs.first;
    }
    return b.code;
  };
  int n_loads[2] = {0, 0};
  bool walk_k[2] = {true, true};
  std::vector<int> a_loads;
  std::string code;
  for (int side = 0; side < 2; side++) {
    const char *nm = side == 0 ? "a" : "b";
    const char *rowvar = side == 0 ? "m" : "n";
    const std::vector<Dim> &row_dims = side == 0 ? mm.md_full : mm.nd_full;
    // the loads under this operand, in topological order
    std::vector<char> mark(g.nodes.size(), 0);
    mark_reachable(g, opnd[side], mark);
    std::vector<int> loads;
    for (size_t id = 0; id < g.nodes.size(); id++)
      if (mark[id] && g.n((int)id).op == POLY_OP_LOAD) {
        const int sz = dt_size(g.n((int)id).dt);
        if (sz != 1 && sz != 2 && sz != 4) return reject(__LINE__);
        loads.push_back((int)id);
      }
    if (loads.size() > 6) return reject(__LINE__);
    n_loads[side] = (int)loads.size();
    if (side == 0) a_loads = loads;
    // which way memory runs: along k when the first load has unit stride in the innermost
    // reduce range, along the rows when it has unit stride in the innermost row range
    if (!loads.empty()) {
      const int li = g.n(g.n(g.n(loads[0]).src[0]).src[1]).lin;
      if (li >= 0) {
        const Lin &l = g.lins[(size_t)li];
        bool aff_k;
        const int64_t ck = g.lin_range_coef(l, kr.back(), &aff_k);
        // stride of the innermost row digit
        const Dim &rd = row_dims.back();
        std::vector<DigitUse> u;
        int64_t cr = 0;
        if (digit_uses(g, l, rd.ord, &u))
          for (const DigitUse &d : u)
            if (rd.cut >= d.a && (d.b == 0 || rd.cut < d.a * d.b)) cr += d.coef * (rd.cut / d.a);
        if (!(aff_k && (ck == 1 || ck == -1)) && (cr == 1 || cr == -1)) walk_k[side] = false;
      }
    }
    const int nraw = std::max(1, n_loads[side]);
    auto raw_of = [&](int j, DT dt) {
      const int sz = dt_size(dt);
      if (dt == DT_BOOL) return strf("(raw[%d] != 0u)", j);
      if (sz == 4) return strf("__builtin_bit_cast(%s, raw[%d])", dt_cname(dt), j);
      if (sz == 2) return strf("__builtin_bit_cast(%s, (unsigned short)raw[%d])", dt_cname(dt), j);
      return strf("__builtin_bit_cast(%s, (unsigned char)raw[%d])", dt_cname(dt), j);
    };
    auto to_raw = [&](const std::string &v, DT dt) {
      const int sz = dt_size(dt);
      if (dt == DT_BOOL) return strf("((%s) ? 1u : 0u)", v.c_str());
      if (sz == 4) return strf("__builtin_bit_cast(unsigned int, (%s)(%s))", dt_cname(dt), v.c_str());
      if (sz == 2) return strf("(unsigned int)__builtin_bit_cast(unsigned short, (%s)(%s))", dt_cname(dt), v.c_str());
      return strf("(unsigned int)__builtin_bit_cast(unsigned char, (%s)(%s))", dt_cname(dt), v.c_str());
    };
    // phase 1: the loads
    {
      Emitter em(g);
      Scope S;
      S.indent = 1;
      std::string head = bind_all(row_dims, rowvar, em, S);
      std::string body;
      for (size_t j = 0; j < loads.size(); j++) {
        const std::string v = em.emit(loads[j], &S);
        body += strf("  raw[%zu] = %s;\n", j, to_raw(v, g.n(loads[j]).dt).c_str());
      }
      if (em.failed()) return reject(__LINE__);
      code += strf("__device__ __forceinline__ void poly_%s_load(int %s, int k, int z, unsigned int (&raw)[%d], %s) {\n", nm, rowvar, nraw,
                   ep.signature.c_str());
      code += head + S.code + body + "}\n";
    }
    // phase 2: the arithmetic
    {
      Emitter em(g);
      Scope S;
      S.indent = 1;
      std::string head = bind_all(row_dims, rowvar, em, S);
      for (size_t j = 0; j < loads.size(); j++) em.preset(loads[j], raw_of((int)j, g.n(loads[j]).dt));
      const std::string v = em.emit(opnd[side], &S);
      if (em.failed()) return reject(__LINE__);
      code += strf("__device__ __forceinline__ float poly_%s_math(int %s, int k, int z, const unsigned int (&raw)[%d], %s) {\n", nm, rowvar, nraw,
                   ep.signature.c_str());
      code += head + S.code + strf("  return %s;\n}\n", v.c_str());
    }
  }

  // ── on the bf16 MFMA when the products allow it ───────────────────────────────
  // An operand that is a bf16 value cast to fp32 is exact in bf16; an fp32-valued one is the
  // sum of three bf16 pieces (kernels/operand_split.hip).  With at least one exact side,
  // a first stage writes both operands as k-contiguous bf16 planes into scratch memory and
  // the 16-bit template multiplies them (K' = planes x K rounded up to its K tile).
  {
    // (a plain load from an fp32 buffer that only ever receives bf16 values, or holds them
    // as bf16 in the first place: matmul_hint_param_kinds)
    int kind[2] = {0, 0};
    for (int side = 0; side < 2; side++) {
      Operand o;
      if (g.n(opnd[side]).op == POLY_OP_LOAD && g.n(opnd[side]).dt == DT_F32 && match_operand(g, opnd[side], &o)) kind[side] = matmul_param_kind(o.param);
    }
    auto exact16 = [&](int side) {
      const KNode &k = g.n(opnd[side]);
      return kind[side] != 0 || (k.op == POLY_OP_CAST && k.dt == DT_F32 && g.n(k.src[0]).dt == DT_BF16);
    };
    // (two pieces, hi + lo, leave an error below 2^-17 |x|: enough where the result is
    // stored as a 16-bit float, whose own rounding is 2^-9 or 2^-12 of it)
    const int pieces = ep.out_16bit && !getenv("POLY_HIP_SPLIT_THREE") ? 2 : 3;
    const int parts[2] = {exact16(0) ? 1 : pieces, exact16(1) ? 1 : pieces};
    const int P = std::max(parts[0], parts[1]);
    const int64_t KP = (K + 63) / 64 * 64;
    const double elems_a = (double)Z * (double)M * parts[0] * (double)KP, elems_b = (double)Z * (double)N * parts[1] * (double)KP;
    // (int offsets inside the template; and the planes should stay a small part of the card's memory)
    const bool fits = elems_a < 2147483647.0 && elems_b < 2147483647.0 && (elems_a + elems_b) * 2.0 <= 8.0 * 1073741824.0;
    // worth the extra pass over the operands only for deep or large products
    double min_work = 1073741824.0;
    if (const char *e = getenv("POLY_HIP_BF16_SPLIT_MIN")) min_work = std::max(1.0, atof(e));   // tests: small products through this path
    const bool large = (double)M * (double)N * (double)K * (double)Z >= min_work;
    // (planes meet plane by plane along K: one side has to be a single plane)
    if (!getenv("POLY_HIP_NO_BF16_SPLIT") && (parts[0] == 1 || parts[1] == 1) && fits && large) {
      const size_t off_b = ((size_t)elems_a * 2 + 255) / 256 * 256;       // bytes
      const size_t scratch_bytes = off_b + (size_t)elems_b * 2;
      // Operand A may already lie in the scratch memory with rows and depth exchanged (an
      // earlier kernel of the same launch wrote it): read row m, plane p, depth k at
      // [z][k][p][m] then, and write no planes.  Sizes in whole K tiles, so that both
      // kernels put operand B behind the same number of bytes and no padding is read.
      RenderedKernel::OperandPlanes mine;
      if (!getenv("POLY_HIP_NO_SHARED_PLANES")) describe_operand(g, opnd[0], a_loads, mm.md_full, k_dims, mm.zd_full, M, K, Z, &mine);
      mine.parts = parts[0];
      const bool shared = opt.planes_before && M % 64 == 0 && K % 64 == 0 && exchanged(mine, *opt.planes_before);
      // An operand that is a bf16 buffer read at an index of the plain template's kind needs
      // no plane: the template reads it where it lies (the probabilities P in dv = P^T dO
      // are 134 MB per layer that a copy would read and write again).  Needs whole K tiles
      // (a padded depth would be read outside the buffer) and one reduce range.
      struct InPlace { bool ok = false; Operand op; KSplit ks{0, 0, 0}; std::vector<Dim> rows, z; int64_t c0 = 0; };
      InPlace in_place[2];
      for (int side = 0; side < 2 && !getenv("POLY_HIP_NO_IN_PLACE_OPERAND"); side++) {
        InPlace &ip = in_place[side];
        // (a buffer that holds bf16 values where the schedule has fp32 ones is read as the
        // 16-bit buffer it is, at the same element indices)
        const bool narrow = kind[side] == 2;
        if (parts[side] != 1 || K % 64 != 0 || kr.size() > 2 || (side == 0 && shared)) continue;
        if (!match_operand(g, opnd[side], &ip.op) || ip.op.dt != (narrow ? DT_F32 : DT_BF16)) continue;
        if (!narrow && kind[side] != 0) continue;
        const Lin &l = g.lins[(size_t)ip.op.lin];
        if (kr.size() == 1) {
          if (!k_dependence(g, l, kr[0], K, &ip.ks) || ip.ks.kb < K) continue;
        } else {
          // two reduce ranges whose strides nest are one depth
          const int64_t e0 = g.ranges[(size_t)kr[0]].extent, e1 = g.ranges[(size_t)kr[1]].extent;
          KSplit k0, k1;
          if (!k_dependence(g, l, kr[0], e0, &k0) || !k_dependence(g, l, kr[1], e1, &k1) || k0.kb != e0 || k1.kb != e1 || k0.s_lo != k1.s_lo * e1) continue;
          ip.ks = KSplit{K, 0, k1.s_lo};
        }
        bool ok = true;
        auto coefs = [&](const std::vector<Dim> &dims, std::vector<Dim> *out) {
          for (const Dim &d : dims) {
            std::vector<DigitUse> u;
            if (!digit_uses(g, l, d.ord, &u)) { ok = false; return; }
            int64_t c = 0;
            for (const DigitUse &x : u)
              if (d.cut >= x.a && (x.b == 0 || d.cut < x.a * x.b)) c += x.coef * (d.cut / x.a);
            Dim e = d;
            e.ca = side == 0 ? c : 0;
            e.cb = side == 0 ? 0 : c;
            out->push_back(e);
          }
        };
        coefs(side == 0 ? mm.md_full : mm.nd_full, &ip.rows);
        coefs(mm.zd_full, &ip.z);
        {
          uint64_t k_mask = 0;
          for (int r : kr) if (r >= 0 && r < 64) k_mask |= (uint64_t)1 << r;
          if (!lin_separates(g, l, ord_mask(ip.rows), k_mask, ord_mask(ip.z))) ok = false;
        }
        // (the digits must be all there is to the index: checked against the canonical form
        // at the far corner and at scattered points)
        std::vector<int64_t> rv(g.ranges.size());
        uint64_t rnd = 0x2545f4914f6cdd1dull;
        for (int t = 0; t < 64 && ok; t++) {
          std::fill(rv.begin(), rv.end(), 0);
          int64_t want = l.c0, got = 0;
          auto put = [&](const std::vector<Dim> &dims) {
            for (const Dim &d : dims) {
              rnd = rnd * 6364136223846793005ull + 1442695040888963407ull;
              const int64_t digit = t == 0 ? d.extent - 1 : (int64_t)((rnd >> 33) % (uint64_t)d.extent);
              rv[(size_t)d.ord] += digit * d.cut;
              want += digit * (side == 0 ? d.ca : d.cb);
            }
          };
          put(ip.rows); put(ip.z);
          rnd = rnd * 6364136223846793005ull + 1442695040888963407ull;
          const int64_t kk = t == 0 ? K - 1 : (int64_t)((rnd >> 33) % (uint64_t)K);
          if (kr.size() == 1) rv[(size_t)kr[0]] = kk;
          else { const int64_t e1 = g.ranges[(size_t)kr[1]].extent; rv[(size_t)kr[0]] = kk / e1; rv[(size_t)kr[1]] = kk % e1; }
          want += kk * ip.ks.s_lo;
          if (!eval_lin(g, l, rv, &got) || got != want) ok = false;
        }
        ip.c0 = l.c0;
        if (narrow) ip.op.dt = DT_BF16;
        ip.ok = ok;
      }
      RenderedKernel::Pre pre[2];
      for (int side = 0; side < 2; side++) {
        const char *nm = side == 0 ? "a" : "b";
        const int64_t rows = side == 0 ? M : N;
        std::string c2;
        c2 += strf("#define POLY_SP_ROWS %lld\n#define POLY_SP_K %lld\n#define POLY_SP_KP %lld\n#define POLY_SP_Z %lld\n", (long long)rows, (long long)K,
                   (long long)KP, (long long)Z);
        c2 += strf("#define POLY_SP_PARTS %d\n#define POLY_SP_WALK_K %d\n#define POLY_SP_NRAW %d\n", parts[side], walk_k[side] ? 1 : 0, std::max(1, n_loads[side]));
        c2 += strf("#define POLY_SIGNATURE %s, __bf16* poly_scratch\n", ep.signature.c_str());
        c2 += code;
        c2 += strf("#define POLY_SP_LOAD(row, k, z, raw) poly_%s_load(row, k, z, raw, %s)\n#define POLY_SP_MATH(row, k, z, raw) poly_%s_math(row, k, z, raw, %s)\n",
                   nm, params_call.c_str(), nm, params_call.c_str());
        c2 += strf("#define POLY_SP_OUT ((__bf16*)((char*)poly_scratch + %zuull))\n", side == 0 ? (size_t)0 : off_b);
        pre[side].source = std::string(hip_prelude()) + c2 + kOperandSplitTemplate;
        pre[side].entry = "poly_k";
        pre[side].launch.grid[0] = (unsigned)((KP / 64) * ((rows + 63) / 64));
        pre[side].launch.grid[1] = (unsigned)Z;
        pre[side].launch.block[0] = 256;
      }
      // the product of the planes, as the 16-bit template sees it (a second time with every
      // operand as planes if the template does not take an operand where it lies)
      for (int attempt = 0; attempt < 2; attempt++) {
      if (attempt == 1) {
        if (!in_place[0].ok && !in_place[1].ok) break;
        in_place[0].ok = in_place[1].ok = false;
      }
      MatmulMatch m2;
      m2.red = red; m2.K = P * KP; m2.M = M; m2.N = N; m2.Z = Z;
      m2.A.dt = m2.B.dt = DT_BF16;
      m2.ka = parts[0] == P ? KSplit{P * KP, 0, 1} : KSplit{KP, 0, 1};
      m2.kb = parts[1] == P ? KSplit{P * KP, 0, 1} : KSplit{KP, 0, 1};
      m2.md.push_back(Dim{-1, M, parts[0] * KP, 0, 1});
      m2.nd.push_back(Dim{-1, N, 0, parts[1] * KP, 1});
      if (Z > 1) m2.zd.push_back(Dim{-1, Z, M * parts[0] * KP, N * parts[1] * KP, 1});
      if (shared) {
        // (the planes were written for K rows of M: M is the padded depth there)
        m2.ka = KSplit{KP, parts[0] == P ? M : 0, parts[0] * M};
        m2.md[0].ca = 1;
      }
      if (in_place[0].ok || in_place[1].ok) {
        // batch digits one by one: a plane operand's stride of a digit is the plane stride
        // times the extents of the digits inside it
        m2.zd.clear();
        int64_t inner = 1;
        std::vector<Dim> zs(mm.zd_full.size());
        for (size_t i = mm.zd_full.size(); i-- > 0;) {
          Dim d = mm.zd_full[i];
          d.ca = in_place[0].ok ? in_place[0].z[i].ca : M * parts[0] * KP * inner;
          d.cb = in_place[1].ok ? in_place[1].z[i].cb : N * parts[1] * KP * inner;
          inner *= d.extent;
          zs[i] = d;
        }
        m2.zd = zs;
        if (in_place[0].ok) {
          m2.md = in_place[0].rows;
          collapse(m2.md);
          m2.ka = KSplit{KP, 0, in_place[0].ks.s_lo};
          m2.a_c0 = in_place[0].c0;
          m2.A = in_place[0].op;
        }
        if (in_place[1].ok) {
          m2.nd = in_place[1].rows;
          collapse(m2.nd);
          m2.kb = KSplit{KP, 0, in_place[1].ks.s_lo};
          m2.b_c0 = in_place[1].c0;
        }
      }
      m2.md_full = mm.md_full; m2.nd_full = mm.nd_full; m2.zd_full = mm.zd_full;
      MatmulEpilogue ep2 = ep;
      ep2.signature += ", __bf16* poly_scratch";
      ep2.scratch_type = "__bf16";
      const size_t planes_bytes = in_place[1].ok ? (in_place[0].ok ? (size_t)256 : std::max<size_t>(off_b, 256)) : scratch_bytes;
      ep2.scratch_used = planes_bytes;
      ep2.a_ptr = "((const __bf16*)poly_scratch)";
      ep2.b_ptr = strf("((const __bf16*)((const char*)poly_scratch + %zuull))", off_b);
      if (in_place[0].ok) ep2.a_ptr = strf(kind[0] == 2 ? "((const __bf16*)data%d)" : "data%d", in_place[0].op.param);
      if (in_place[1].ok) ep2.b_ptr = strf(kind[1] == 2 ? "((const __bf16*)data%d)" : "data%d", in_place[1].op.param);
      RenderedKernel main;
      if (render_matmul(m2, ep2, &main)) {
        *out = main;
        // planes first, then a split product's first stage
        if (!in_place[1].ok) out->pres.insert(out->pres.begin(), pre[1]);
        if (!shared && !in_place[0].ok) out->pres.insert(out->pres.begin(), pre[0]);
        out->scratch_bytes = std::max(planes_bytes, main.scratch_bytes);
        out->flops = 2.0 * (double)M * (double)N * (double)K * (double)Z;
        out->strategy = strf("operands as expressions, written as bf16 planes first (%d + %d planes of K=%lld, %.0f MB%s): ", parts[0], parts[1],
                             (long long)KP, (double)planes_bytes / 1e6,
                             shared ? "; A is what the kernel before left as its A, rows and depth exchanged, and is not written again"
                             : in_place[0].ok && in_place[1].ok ? "; both read in place" : in_place[0].ok ? "; A read in place" : in_place[1].ok ? "; B read in place" : "") + out->strategy;
        out->narrow_loads = (in_place[0].ok && kind[0] == 2 ? 1 : 0) + (in_place[1].ok && kind[1] == 2 ? 1 : 0);
        out->tables = ep.tables;
        if (!ep.tables.empty()) out->strategy += strf(", %d parts of the epilogue as 16-bit lookup tables (%zu, one per load)", ep.table_parts, ep.tables.size());
        out->reads_planes_before = shared;
        if (!shared && !in_place[0].ok) out->a_planes = mine;
        for (RenderedKernel::Variant &v : out->variants) v.strategy = out->strategy;
        return true;
      }
      }
    }
  }

  int BM, BN, WVM, WVN;
  f32_tile(M, N, Z, &BM, &BN, &WVM, &WVN);
  if (((M + BM - 1) / BM) * ((N + BN - 1) / BN) > 2147483647LL / 2) return reject(__LINE__);
  const int depth = n_loads[0] + n_loads[1] <= 2 ? 4 : n_loads[0] + n_loads[1] <= 4 ? 2 : 1;
  std::string cfg;     // (all but the shape of the tile)
  cfg += strf("#define POLY_M %lld\n#define POLY_N %lld\n#define POLY_K %lld\n#define POLY_Z %lld\n", (long long)M, (long long)N, (long long)K, (long long)Z);
  cfg += strf("#define POLY_GEN 1\n#define POLY_PF_DEPTH %d\n#define POLY_A_KC %d\n#define POLY_B_KC %d\n", depth, walk_k[0] ? 1 : 0, walk_k[1] ? 1 : 0);
  cfg += strf("#define POLY_A_NLOADS %d\n#define POLY_B_NLOADS %d\n", std::max(1, n_loads[0]), std::max(1, n_loads[1]));
  cfg += strf("#define POLY_SIGNATURE %s\n", ep.signature.c_str());
  cfg += ep.code + code;
  cfg += strf("#define POLY_A_LOAD(m, k, z, raw) poly_a_load(m, k, z, raw, %s)\n#define POLY_A_MATH(m, k, z, raw) poly_a_math(m, k, z, raw, %s)\n",
              params_call.c_str(), params_call.c_str());
  cfg += strf("#define POLY_B_LOAD(n, k, z, raw) poly_b_load(n, k, z, raw, %s)\n#define POLY_B_MATH(n, k, z, raw) poly_b_math(n, k, z, raw, %s)\n",
              params_call.c_str(), params_call.c_str());
  cfg += strf("#define POLY_EPILOGUE(acc, m, n, z) %s\n", ep.call.c_str());
  const auto build = [&](const F32Shape &sh, RenderedKernel *rk) {
    *rk = RenderedKernel();
    rk->source = std::string(hip_prelude()) +
                 strf("#define POLY_BM %d\n#define POLY_BN %d\n#define POLY_WAVES_M %d\n#define POLY_WAVES_N %d\n#define POLY_GROUP_M 8\n", sh.bm, sh.bn, sh.wvm, sh.wvn) +
                 cfg + kMatmulF32Template;
    rk->entry = "poly_k";
    rk->launch.grid[0] = (unsigned)(((M + sh.bm - 1) / sh.bm) * ((N + sh.bn - 1) / sh.bn));
    rk->launch.grid[1] = (unsigned)Z;
    rk->launch.block[0] = (unsigned)(64 * sh.wvm * sh.wvn);
    rk->klass = KernelClass::MATMUL_MFMA;
    rk->strategy = strf("mfma 32x32x2 f32, operands as expressions (%d + %d loads per element pair, %d tiles ahead) M=%lld N=%lld K=%lld Z=%lld tile %dx%dx16 A:%s B:%s",
                        n_loads[0], n_loads[1], depth, (long long)M, (long long)N, (long long)K, (long long)Z, sh.bm, sh.bn,
                        walk_k[0] ? "k-major" : "m-major", walk_k[1] ? "k-major" : "n-major");
    rk->n_params = ep.n_params;
    rk->n_vars = 0;
    rk->flops = 2.0 * (double)M * (double)N * (double)K * (double)Z;
    rk->bytes = ep.bytes;
    rk->tables = ep.tables;
    if (!ep.tables.empty()) rk->strategy += strf(", %d parts of the epilogue as 16-bit lookup tables (%zu, one per load)", ep.table_parts, ep.tables.size());
  };
  build(F32Shape{BM, BN, WVM, WVN}, out);
  f32_variants(M, N, F32Shape{BM, BN, WVM, WVN}, build, out);
  return true;
}

// ── guarded embedding gather ──────────────────────────────────────────────
//
// The frontend expresses an embedding lookup as a masked sum over the whole
// table (src/frontend.c:3494-3583, src/modelzoo/models/gpt2.c:93-153):
//     out[..., j] = sum_v where(ids[...] == arange[v], table[v, j], 0)
// When arange[v] == v for every v, at most one term is non-zero and the sum is
// table[ids, j] (or 0 for an id that is not an integer in range).  The fast
// kernel does that one load; a one-workgroup guard kernel checks the arange
// buffer on every run, and the generic lowering runs instead when it fails.

namespace {

// cond is "a == b" in one of the forms the frontend produces.
bool match_equal(const KernelGraph &g, int node, int *a, int *b) {
  const KNode *k = &g.n(node);
  if (k->op == POLY_OP_CAST && k->src.size() == 1) { node = k->src[0]; k = &g.n(node); }
  if (k->op == POLY_OP_CMPEQ) { *a = k->src[0]; *b = k->src[1]; return true; }
  if (k->op == POLY_OP_WHERE) {
    const KNode &c = g.n(k->src[0]), &t = g.n(k->src[1]), &f = g.n(k->src[2]);
    if (c.op != POLY_OP_CMPNE || t.op != POLY_OP_CONST || f.op != POLY_OP_CONST) return false;
    auto cval = [](const KNode &n) { return n.u->arg.kind == POLY_ARG_FLOAT ? n.u->arg.f : (double)n.u->arg.i; };
    if (cval(t) != 0.0 || cval(f) == 0.0) return false;
    *a = c.src[0]; *b = c.src[1];
    return true;
  }
  if (k->op == POLY_OP_NEG && k->dt == DT_BOOL && g.n(k->src[0]).op == POLY_OP_CMPNE) {
    *a = g.n(k->src[0]).src[0]; *b = g.n(k->src[0]).src[1];
    return true;
  }
  return false;
}

bool is_zero_const(const KNode &n) {
  if (n.op != POLY_OP_CONST) return false;
  return n.u->arg.kind == POLY_ARG_FLOAT ? n.u->arg.f == 0.0 : n.u->arg.i == 0;
}

}  // namespace

bool try_render_gather(const KernelGraph &g, const std::string &fn, const RenderOptions &opt, RenderedKernel *out) {
  if (g.reduces.size() != 1 || !g.vars.empty() || opt.exit_if_flag || opt.exit_unless_flag) return reject(__LINE__);
  const int red = g.reduces[0];
  const KNode &R = g.n(red);
  if (reduce_op(R) != POLY_OP_ADD || !dt_is_float(R.dt) || R.src.size() != 2) return reject(__LINE__);
  const int vr = g.range_ord.at(R.src[1]);
  const int64_t V = g.ranges[(size_t)vr].extent;
  if (V < 64) return reject(__LINE__);
  const KNode &W = g.n(R.src[0]);
  if (W.op != POLY_OP_WHERE || !is_zero_const(g.n(W.src[2]))) return reject(__LINE__);
  int ea, eb;
  if (!match_equal(g, W.src[0], &ea, &eb)) return reject(__LINE__);
  const uint64_t vbit = (uint64_t)1 << vr;
  // one side of the comparison is arange[v], the other does not depend on v
  int ids = -1, ar = -1;
  if (!(g.n(ea).deps & vbit) && (g.n(eb).deps & vbit)) { ids = ea; ar = eb; }
  else if (!(g.n(eb).deps & vbit) && (g.n(ea).deps & vbit)) { ids = eb; ar = ea; }
  else return reject(__LINE__);
  const KNode &AR = g.n(ar);
  if (AR.op != POLY_OP_LOAD || AR.guard >= 0) return reject(__LINE__);
  const KNode &arix = g.n(AR.src[0]);
  if (arix.src.size() != 2) return reject(__LINE__);
  const int ar_lin = g.n(arix.src[1]).lin;
  if (ar_lin < 0) return reject(__LINE__);
  {
    const Lin &l = g.lins[(size_t)ar_lin];
    if (l.c0 != 0 || l.terms.size() != 1 || l.terms[0].coef != 1) return reject(__LINE__);
    const Atom &a = g.atoms[(size_t)l.terms[0].atom];
    if (a.kind != Atom::RANGE || g.range_ord.at(a.node) != vr) return reject(__LINE__);
  }
  const int ar_param = g.param_slot(arix.src[0]);
  if (g.params[(size_t)ar_param].written || g.params[(size_t)ar_param].numel < V) return reject(__LINE__);
  const DT ids_dt = g.n(ids).dt;
  if (ids_dt != AR.dt || !(dt_is_float(ids_dt) || dt_is_int(ids_dt))) return reject(__LINE__);
  // the selected value: [CAST](LOAD(table[affine in v]))
  int val = W.src[1];
  if (g.n(val).dt != R.dt) return reject(__LINE__);
  int tl = val;
  if (g.n(tl).op == POLY_OP_CAST) tl = g.n(tl).src[0];
  const KNode &TL = g.n(tl);
  if (TL.op != POLY_OP_LOAD) return reject(__LINE__);
  const KNode &tix = g.n(TL.src[0]);
  if (tix.src.size() != 2) return reject(__LINE__);
  const int t_lin = g.n(tix.src[1]).lin;
  if (t_lin < 0) return reject(__LINE__);
  bool aff;
  const int64_t cv = g.lin_range_coef(g.lins[(size_t)t_lin], vr, &aff);
  if (!aff || cv <= 0) return reject(__LINE__);
  const int t_param = g.param_slot(tix.src[0]);
  if (g.params[(size_t)t_param].written) return reject(__LINE__);
  // nothing else under the REDUCE may depend on v
  // (ids side was checked; the table index is affine in v; the comparison is consumed)

  const DT rdt = R.dt, tdt = TL.dt;
  RenderOptions fast = opt;
  fast.allow_templates = false;
  fast.exit_unless_flag = true;
  fast.reduce_override[red] = [=, &g](Emitter &em, Scope *t) -> std::string {
    std::string idv = em.emit(ids, t);
    std::string gi = strf("gi%d", red), gh = strf("gh%d", red), acc = strf("acc%d", red);
    em.stmt(t, strf("const int %s = (int)(%s);", gi.c_str(), idv.c_str()));
    em.stmt(t, strf("const bool %s = ((%s)%s == %s) && %s >= 0 && %s < %lld;", gh.c_str(), dt_cname(ids_dt), gi.c_str(),
                    idv.c_str(), gi.c_str(), gi.c_str(), (long long)V));
    em.bind_range(vr, gi);
    std::string addr = em.emit_lin(g.lins[(size_t)t_lin], t);
    // 0 + x: the sum starts from +0, so a selected -0 comes out as +0
    em.stmt(t, strf("const %s %s = %s ? (%s)0 + (%s)((%s)data%d[%s]) : (%s)0;", dt_cname(rdt), acc.c_str(), gh.c_str(),
                    dt_cname(rdt), dt_cname(rdt), dt_cname(tdt), t_param, addr.c_str(), dt_cname(rdt)));
    return acc;
  };
  std::string err;
  RenderedKernel fk;
  if (!render_kernel(g, fn, fast, &fk, &err)) return reject(__LINE__);
  RenderOptions slow = opt;
  slow.allow_templates = false;
  slow.allow_coop_reduce = false;   // one thread per output: a small grid that exits at once when unused
  slow.exit_if_flag = true;
  RenderedKernel sk;
  if (!render_kernel(g, fn, slow, &sk, &err)) return reject(__LINE__);

  RenderedKernel::Guard gd;
  gd.entry = "poly_guard";
  // one workgroup of 1024 threads, four consecutive elements per thread and step
  gd.source = strf(R"HIP(
extern "C" __global__ void __launch_bounds__(1024) poly_guard(int* flag, const %s* __restrict__ ar) {
  __shared__ int bad;
  if (threadIdx.x == 0) bad = 0;
  __syncthreads();
  int mine = 0;
  // (unrolled: the loads of all steps are in flight together -- one memory latency for the
  // whole check instead of one per step)
#pragma unroll 16
  for (long long i = (long long)threadIdx.x * 4; i < %lldll; i += 4096) {
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (i + j < %lldll && ar[i + j] != (%s)(i + j)) mine = 1;
  }
  if (mine) bad = 1;
  __syncthreads();
  if (threadIdx.x == 0) *flag = bad ? 0 : 1;
}
)HIP", dt_cname(AR.dt), (long long)V, (long long)V, dt_cname(AR.dt));
  gd.launch.grid[0] = 1;
  gd.launch.block[0] = 1024;
  gd.arg_params.push_back(ar_param);

  *out = fk;
  out->klass = KernelClass::GATHER;
  out->strategy = "guarded gather (arange check) + " + fk.strategy;
  out->guards.push_back(gd);
  out->fallback_source = sk.source;
  out->fallback_entry = sk.entry;
  out->fallback_launch = sk.launch;
  // algorithmic bytes: ids + gathered rows + output (not the V-long masked sum)
  double outn = 1;
  for (int r : g.stores[0].ranges) outn *= (double)std::max<int64_t>(1, g.ranges[(size_t)r].extent);
  out->bytes = outn * (dt_size(tdt) + dt_size(g.n(g.stores[0].param).dt)) + (double)V * dt_size(AR.dt);
  return true;
}

}  // namespace polyhip
