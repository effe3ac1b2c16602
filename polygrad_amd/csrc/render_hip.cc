// Generic lowering of a scheduled kernel to HIP C for gfx950.
//
// Three shapes of kernel come out of here:
//   ELEMENTWISE   every END-closed range is flattened over the grid, fastest
//                 varying range last in the thread id; when that range is
//                 unit-stride in the store (and in a load) the access becomes one
//                 128-bit (or 64-bit) vector access per thread.
//   ROW_REDUCE    one wave (64 lanes) or one workgroup (256 lanes) per output
//                 element; lanes stride over the flattened reduce ranges with
//                 vector loads, then combine with DPP/ds_swizzle (+LDS across
//                 the four waves of a workgroup).
//   THREAD_REDUCE one thread per output element with serial reduce loops
//                 (short reductions, or reductions this file cannot split).
// Matmul-shaped and gather-shaped kernels are tried first in templates.cc.
#include "render_hip.h"
#include "templates.h"

#include <algorithm>
#include <cmath>
#include <set>

namespace polyhip {

bool lin_vec_ok(const KernelGraph &g_, const Lin &l, int F, int V, bool any_alignment) {
  if (l.c0 % V && !any_alignment) return false;
  bool seenF = false;
  for (const Term &t : l.terms) {
    const Atom &a = g_.atoms[(size_t)t.atom];
    if (a.kind == Atom::RANGE && g_.range_ord.at(a.node) == F) {
      if (t.coef != 1) return false;
      seenF = true;
    } else {
      if (g_.atom_deps(t.atom) & ((uint64_t)1 << F)) return false;
      if (t.coef % V && !any_alignment) return false;
    }
  }
  return seenF;
}

void mark_reachable(const KernelGraph &g_, int root, std::vector<char> &mark) {
  std::vector<int> st{root};
  while (!st.empty()) {
    int n = st.back(); st.pop_back();
    if (mark[(size_t)n]) continue;
    mark[(size_t)n] = 1;
    for (int s : g_.n(n).src) st.push_back(s);
  }
}

std::vector<int> hoist_vector_loads(const KernelGraph &g_, Emitter &em_, const std::vector<int> &roots, int F, int V,
                                    const std::string &f0, Scope *outer,
                                    const std::function<std::string(int, const std::string &)> *wrap, bool any_alignment) {
  std::vector<char> mark(g_.nodes.size(), 0);
  for (int r : roots) mark_reachable(g_, r, mark);
  std::vector<int> done;
  for (int i = 0; i < (int)g_.nodes.size(); i++) {
    if (!mark[(size_t)i]) continue;
    const KNode &k = g_.n(i);
    if (k.op != POLY_OP_LOAD) continue;
    if (em_.is_preset(i)) continue;
    if (!(k.deps & ((uint64_t)1 << F))) continue;
    // loads that also depend on ranges not bound in `outer` (nested serial
    // reduces) stay scalar
    if (k.deps & ~(outer->avail | ((uint64_t)1 << F))) continue;
    const KNode &ix = g_.n(k.src[0]);
    int li = g_.n(ix.src[1]).lin;
    if (li < 0 || !lin_vec_ok(g_, g_.lins[(size_t)li], F, V, any_alignment)) continue;
    if (ix.src.size() >= 3 && (g_.n(ix.src[2]).deps & ((uint64_t)1 << F))) continue;
    if (k.guard >= 0 && (g_.n(k.guard).deps & ((uint64_t)1 << F))) continue;
    if (dt_size(k.dt) * V > 16) continue;
    int p = g_.param_slot(ix.src[0]);
    em_.bind_range(F, f0);
    std::string addr = em_.emit_lin(g_.lins[(size_t)li], outer);
    std::string name = strf("ld%d", i);
    std::string ld = strf("poly_vload<%s,%d>(data%d + %s)", dt_cname(k.dt), V, p, addr.c_str());
    std::string gate;
    if (ix.src.size() >= 3) gate = em_.emit(ix.src[2], outer);
    if (k.guard >= 0) {
      std::string g2 = em_.emit(k.guard, outer);
      if (k.guard_neg) g2 = "(!" + g2 + ")";
      gate = gate.empty() ? g2 : "(" + gate + "&&" + g2 + ")";
    }
    if (!gate.empty()) ld = strf("(%s ? %s : poly_vec<%s,%d>{})", gate.c_str(), ld.c_str(), dt_cname(k.dt), V);
    else if (wrap) ld = (*wrap)(i, ld);
    outer->code.append((size_t)outer->indent * 2, ' ');
    outer->code += strf("const poly_vec<%s,%d> %s = %s;\n", dt_cname(k.dt), V, name.c_str(), ld.c_str());
    em_.preset(i, name + ".v[u]");
    done.push_back(i);
  }
  return done;
}

std::string wave_reduce_call(PolyOps op, DT dt, const std::string &v, int lanes) {
  if (dt == DT_F32) {
    const char *fn = op == POLY_OP_ADD ? "add" : op == POLY_OP_MUL ? "mul" : "max";
    return strf("poly_%s_%s_f32(%s)", lanes == 32 ? "half" : "wave", fn, v.c_str());
  }
  const char *ct = dt_cname(dt);
  std::string comb = Emitter::reduce_combine(op, dt, "a_", "b_");
  if (lanes == 32) {
    // (the lambda's type cannot be named in front of the lane count: the call goes through a variable)
    return strf("[&]() { auto f_ = [](%s a_, %s b_) { return (%s)%s; }; return poly_wave_reduce_any<%s, decltype(f_), 32>(%s, f_); }()", ct, ct, ct, comb.c_str(),
                ct, v.c_str());
  }
  return strf("poly_wave_reduce_any<%s>(%s, [](%s a_, %s b_) { return (%s)%s; })", ct, v.c_str(), ct, ct, ct, comb.c_str());
}

namespace {

struct Group {
  std::vector<int> ranges;     // ordinals, outermost first (END order)
  std::vector<int> stores;     // indices into g.stores
};

PolyOps reduce_op(const KNode &k) {
  return k.u->arg.kind == POLY_ARG_OPS ? k.u->arg.ops : (PolyOps)k.u->arg.i;
}

// Extent of a range as a C expression (constant or symbolic) and as a number.
struct Ext { int64_t n; std::string expr; };

class Generic {
 public:
  Generic(const KernelGraph &g, const std::string &fn, const RenderOptions &opt)
      : g_(g), fn_(fn), opt_(opt), em_(g) {}

  bool run(RenderedKernel *out, std::string *err) {
    if (!prepare(err)) return false;
    for (auto &ov : opt_.reduce_override) {
      auto fn = ov.second;
      em_.custom_reduce(ov.first, [this, fn](Scope *s) { return fn(em_, s); });
    }
    std::string body;
    bool coop = false;
    if (n_loop_reduces() > 0 && opt_.allow_coop_reduce && groups_.size() == 1 && opt_.reduce_override.empty()) coop = plan_coop();
    if (coop && opt_.ordered_stage) {
      // the cooperative form is the better lowering; rendering it under a stage number
      // would hand back the whole kernel as "stage one" and again as "stage two"
      *err = "not an ordered reduction";
      return false;
    }
    if (coop) {
      body = render_coop(out);
    } else if (plan_ordered()) {
      body = opt_.ordered_stage ? render_ordered_stage(out) : render_ordered(out);
    } else if (opt_.ordered_stage) {
      *err = "not an ordered reduction";
      return false;
    } else {
      body = render_flat(out);
    }
    if (em_.failed()) { *err = em_.error(); return false; }
    if (!error_.empty()) { *err = error_; return false; }
    std::string prologue = opt_.exit_if_flag ? "  if (*poly_flag != 0) return;\n"
                           : opt_.exit_unless_flag ? "  if (*poly_flag == 0) return;\n" : "";
    out->source = std::string(hip_prelude()) + signature() + " {\n" + prologue + body + "}\n";
    out->entry = fn_;
    out->n_params = (int)g_.params.size();
    out->n_vars = (int)g_.vars.size();
    for (const VarInfo &v : g_.vars) out->var_uops.push_back(g_.n(v.node).u);
    account(out);
    return true;
  }

 private:
  const KernelGraph &g_;
  std::string fn_;
  RenderOptions opt_;
  Emitter em_;
  std::vector<Group> groups_;
  std::vector<int> top_reduces_;
  std::string error_;
  // coop plan
  int coop_G_ = 0;
  int64_t coop_R_ = 0;
  std::vector<int> coop_ranges_;

  // REDUCE nodes that still need a loop (not replaced by a caller-supplied value)
  int n_loop_reduces() const {
    int n = 0;
    for (int r : g_.reduces) if (!opt_.reduce_override.count(r)) n++;
    return n;
  }

  std::string signature() const {
    std::string s = strf("extern \"C\" __global__ void __launch_bounds__(%d) %s(", opt_.block, fn_.c_str());
    bool first = true;
    for (size_t i = 0; i < g_.params.size(); i++) {
      const ParamInfo &p = g_.params[i];
      if (!first) s += ", ";
      first = false;
      if (p.written) s += strf("%s* data%zu", dt_cname(p.dt), i);
      else s += strf("const %s* __restrict__ data%zu", dt_cname(p.dt), i);
    }
    for (size_t i = 0; i < g_.vars.size(); i++) {
      if (!first) s += ", ";
      first = false;
      s += strf("const int var%zu", i);
    }
    if (opt_.scratch_param) { s += std::string(first ? "" : ", ") + "float* poly_scratch"; first = false; }
    if (opt_.exit_if_flag || opt_.exit_unless_flag) s += std::string(first ? "" : ", ") + "const int* __restrict__ poly_flag";
    return s + ")";
  }

  bool prepare(std::string *err) {
    for (const ParamInfo &p : g_.params)
      if (p.numel >= ((int64_t)1 << 31)) { *err = "buffer with 2^31 or more elements"; return false; }
    for (size_t si = 0; si < g_.stores.size(); si++) {
      const StoreInfo &st = g_.stores[si];
      bool placed = false;
      for (Group &gr : groups_)
        if (gr.ranges == st.ranges) { gr.stores.push_back((int)si); placed = true; break; }
      if (!placed) { Group gr; gr.ranges = st.ranges; gr.stores.push_back((int)si); groups_.push_back(gr); }
    }
    // top-level reduces: not inside the source of another REDUCE
    std::vector<char> inside(g_.nodes.size(), 0);
    for (int i = (int)g_.nodes.size() - 1; i >= 0; i--) {
      const KNode &k = g_.n(i);
      bool in = inside[(size_t)i];
      if (k.op == POLY_OP_REDUCE) inside[(size_t)k.src[0]] = 1;
      if (in) for (int s : k.src) inside[(size_t)s] = 1;
    }
    for (int r : g_.reduces) if (!inside[(size_t)r]) top_reduces_.push_back(r);
    if (opt_.promote_reduce >= 0) {
      // the reductions directly inside the promoted one take its place
      const int T = opt_.promote_reduce;
      std::vector<char> in_t(g_.nodes.size(), 0), deeper(g_.nodes.size(), 0);
      mark_reachable(g_, g_.n(T).src[0], in_t);
      for (int r : g_.reduces) if (r != T && in_t[(size_t)r]) mark_reachable(g_, g_.n(r).src[0], deeper);
      top_reduces_.clear();
      for (int r : g_.reduces) if (r != T && in_t[(size_t)r] && !deeper[(size_t)r]) top_reduces_.push_back(r);
      if (top_reduces_.empty() || groups_.size() != 1) { *err = "nothing to promote"; return false; }
    }
    return true;
  }

  Ext extent(int ord, Scope *s) {
    const RangeInfo &r = g_.ranges[(size_t)ord];
    if (r.extent >= 0) return {r.extent, strf("%lld", (long long)r.extent)};
    return {-1, em_.emit(r.bound_node, s)};
  }

  // Orders a group's ranges fastest-first using the first store's index strides.
  std::vector<int> fastest_first(const Group &gr) const {
    if (opt_.promote_reduce >= 0) {
      RenderOptions plain = opt_;
      plain.promote_reduce = -1;
      std::vector<int> order;
      const KNode &T = g_.n(opt_.promote_reduce);
      for (size_t i = T.src.size(); i-- > 1;) order.push_back(g_.range_ord.at(T.src[i]));
      Generic base(g_, fn_, plain);
      for (int r : base.fastest_first(gr)) order.push_back(r);
      return order;
    }
    const StoreInfo &st = g_.stores[(size_t)gr.stores[0]];
    int li = g_.n(g_.n(st.index).src[1]).lin;
    std::vector<std::pair<int64_t, int>> keyed;
    int pos = 0;
    for (auto it = gr.ranges.rbegin(); it != gr.ranges.rend(); ++it, ++pos) {
      int64_t key = (int64_t)1 << 50;  // unknown stride: keep END order (inner = fast)
      if (li >= 0) {
        bool aff;
        int64_t c = g_.lin_range_coef(g_.lins[(size_t)li], *it, &aff);
        if (aff && c != 0) key = c < 0 ? -c : c;
        else if (aff && c == 0) key = ((int64_t)1 << 55);
      }
      keyed.push_back({key * 64 + pos, *it});
    }
    std::sort(keyed.begin(), keyed.end());
    std::vector<int> order;
    for (auto &k : keyed) order.push_back(k.second);
    return order;
  }

  bool vec_ok(const Lin &l, int F, int V) const { return lin_vec_ok(g_, l, F, V); }

  bool node_under(int root, std::vector<char> &mark) const { mark_reachable(g_, root, mark); return true; }
  std::vector<int> hoist_vector_loads(const std::vector<int> &roots, int F, int V, const std::string &f0,
                                      Scope *outer, bool, bool any_alignment = false) {
    return polyhip::hoist_vector_loads(g_, em_, roots, F, V, f0, outer, nullptr, any_alignment);
  }

  static void line(std::string &code, int indent, const std::string &s) {
    code.append((size_t)indent * 2, ' ');
    code += s;
    code += "\n";
  }

  // ── flat: one thread per (vector of) output element(s) ───────────────────
  std::string render_flat(RenderedKernel *out) {
    std::string body;
    line(body, 1, "const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;");
    double max_threads = 1;
    bool dynamic = false;
    bool any_reduce = n_loop_reduces() > 0;
    std::string strat;
    for (size_t gi = 0; gi < groups_.size(); gi++) {
      const Group &gr = groups_[gi];
      std::vector<int> order = fastest_first(gr);
      Scope S0;
      S0.indent = 2;
      for (int r : gr.ranges) S0.avail |= (uint64_t)1 << r;
      int V = 1;
      int F = order.empty() ? -1 : order[0];
      // choose a vector width from the stores of the group
      if (opt_.allow_vectorize && !any_reduce && F >= 0 && g_.ranges[(size_t)F].extent > 0) {
        int v0 = 8;
        for (int si : gr.stores) {
          const StoreInfo &st = g_.stores[(size_t)si];
          v0 = std::min(v0, 16 / std::max(1, dt_size(g_.n(st.value).dt)));
        }
        for (int v = v0; v >= 2; v /= 2) {
          bool ok = g_.ranges[(size_t)F].extent % v == 0;
          for (int si : gr.stores) {
            const StoreInfo &st = g_.stores[(size_t)si];
            int li = g_.n(g_.n(st.index).src[1]).lin;
            if (li < 0 || !vec_ok(g_.lins[(size_t)li], F, v)) ok = false;
            if (st.gate >= 0 && (g_.n(st.gate).deps & ((uint64_t)1 << F))) ok = false;
            if (dt_size(g_.n(st.value).dt) != dt_size(g_.n(st.param).dt)) ok = false;
          }
          if (ok) { V = v; break; }
        }
      }
      // thread count of this group
      std::string nthreads = "1";
      double nthreads_n = 1;
      std::string decomp;
      line(decomp, 2, "long long t_ = gid;");
      for (size_t oi = 0; oi < order.size(); oi++) {
        int ord = order[oi];
        Ext e = extent(ord, &S0);
        std::string rv = strf("r%d", ord);
        int64_t e_hi = e.n;
        if (e.n < 0) {
          // symbolic extent (a DEFINE_VAR or an expression of some): the grid is sized
          // for its upper bound and the kernel compares against the run-time value
          const int bl = g_.n(g_.ranges[(size_t)ord].bound_node).lin;
          int64_t lo = 0, hi = -1;
          if (bl >= 0) g_.lin_bounds(g_.lins[(size_t)bl], &lo, &hi);
          if (hi <= 0) dynamic = true;
          e_hi = hi;
        }
        if (oi == 0 && V > 1) {
          int64_t nv = e.n / V;
          line(decomp, 2, strf("const int %s_0 = (int)(t_ %% %lld) * %d; t_ /= %lld;", rv.c_str(), (long long)nv, V, (long long)nv));
          nthreads += strf("*%lldll", (long long)nv);
          nthreads_n *= (double)nv;
        } else {
          if (oi + 1 == order.size() && opt_.slice_reduce < 0)
            line(decomp, 2, strf("const int %s = (int)t_;", rv.c_str()));
          else
            line(decomp, 2, strf("const int %s = (int)(t_ %% %s); t_ /= %s;", rv.c_str(), e.expr.c_str(), e.expr.c_str()));
          nthreads += "*(long long)" + e.expr;
          nthreads_n *= (double)std::max<int64_t>(e_hi, 1);
          em_.bind_range(ord, rv);
        }
      }
      std::string sect;
      if (opt_.slice_reduce >= 0) {
        // first stage of a sliced reduction: the digit left in t_ is the part number
        line(decomp, 2, "const int part_ = (int)t_;");
        const std::string n_out = nthreads;
        nthreads += strf("*%dll", opt_.slice_parts);
        nthreads_n *= (double)opt_.slice_parts;
        em_.slice_reduce(opt_.slice_reduce, opt_.slice_range, "part_", opt_.slice_parts);
        const std::string v = em_.emit(opt_.slice_reduce, &S0);
        line(S0.code, 2, strf("poly_scratch[(gid %% (%s)) * %dll + part_] = %s;", n_out.c_str(), opt_.slice_parts, v.c_str()));
        sect = S0.code;
        strat += strf("partial sums, %d per output; ", opt_.slice_parts);
        max_threads = std::max(max_threads, nthreads_n);
        line(body, 1, strf("if (gid < %s) {", nthreads.c_str()));
        body += decomp + sect;
        line(body, 1, "}");
        continue;
      }
      max_threads = std::max(max_threads, nthreads_n);
      if (V > 1) {
        std::string f0 = strf("r%d_0", F);
        std::vector<int> roots;
        for (int si : gr.stores) roots.push_back(g_.stores[(size_t)si].value);
        Scope outer = S0;
        outer.avail &= ~((uint64_t)1 << F);
        outer.code.clear();
        std::vector<int> pres = hoist_vector_loads(roots, F, V, f0, &outer, false);
        Scope inner;
        inner.parent = &outer;
        inner.avail = outer.avail | ((uint64_t)1 << F);
        inner.indent = 3;
        em_.bind_range(F, strf("r%d", F));
        std::string stores_code;
        for (int si : gr.stores) {
          const StoreInfo &st = g_.stores[(size_t)si];
          std::string v = em_.emit(st.value, &inner);
          line(inner.code, 3, strf("out%d.v[u] = %s;", si, v.c_str()));
        }
        std::string pre;
        for (int si : gr.stores) {
          const StoreInfo &st = g_.stores[(size_t)si];
          line(pre, 2, strf("poly_vec<%s,%d> out%d;", dt_cname(g_.n(st.param).dt), V, si));
        }
        std::string post;
        for (int si : gr.stores) {
          const StoreInfo &st = g_.stores[(size_t)si];
          int li = g_.n(g_.n(st.index).src[1]).lin;
          em_.bind_range(F, f0);
          std::string addr = em_.emit_lin(g_.lins[(size_t)li], &outer);
          int p = g_.param_slot(st.param);
          std::string stmt = strf("poly_vstore<%s,%d>(data%d + %s, out%d);", dt_cname(g_.n(st.param).dt), V, p, addr.c_str(), si);
          if (st.gate >= 0) stmt = "if (" + em_.emit(st.gate, &outer) + ") " + stmt;
          line(post, 2, stmt);
        }
        sect = outer.code + pre;
        line(sect, 2, "#pragma unroll");
        line(sect, 2, strf("for (int u = 0; u < %d; u++) {", V));
        line(sect, 3, strf("const int r%d = %s + u;", F, f0.c_str()));
        sect += inner.code;
        line(sect, 2, "}");
        sect += post;
        for (int n : pres) em_.clear_preset(n);
        strat += strf("flat vec%d; ", V);
      } else {
        for (int si : gr.stores) {
          const StoreInfo &st = g_.stores[(size_t)si];
          std::string v = em_.emit(st.value, &S0);
          std::string idx = em_.emit(g_.n(st.index).src[1], &S0);
          int p = g_.param_slot(st.param);
          std::string stmt = strf("data%d[%s] = %s;", p, idx.c_str(), v.c_str());
          if (st.gate >= 0) stmt = "if (" + em_.emit(st.gate, &S0) + ") " + stmt;
          line(S0.code, 2, stmt);
        }
        sect = S0.code;
        strat += any_reduce ? "thread-per-output serial reduce; " : "flat scalar; ";
      }
      line(body, 1, strf("if (gid < %s) {", nthreads.c_str()));
      body += decomp + sect;
      line(body, 1, "}");
    }
    if (dynamic) { error_ = "a symbolic range bound has no known upper limit"; return body; }
    double blocks = std::ceil(max_threads / opt_.block);
    if (blocks > 2147483647.0) { error_ = "grid too large"; return body; }
    out->launch.grid[0] = (unsigned)std::max(1.0, blocks);
    out->launch.block[0] = (unsigned)opt_.block;
    out->klass = any_reduce ? KernelClass::THREAD_REDUCE : KernelClass::ELEMENTWISE;
    out->strategy = strat;
    return body;
  }

  // ── cooperative row reduction ─────────────────────────────────────────────
  bool plan_coop() {
    if (top_reduces_.empty()) return false;
    const KNode &first = g_.n(top_reduces_[0]);
    std::vector<int> rr;
    for (size_t i = 1; i < first.src.size(); i++) rr.push_back(g_.range_ord.at(first.src[i]));
    int64_t R = 1;
    for (int r : rr) {
      if (g_.ranges[(size_t)r].extent < 0) return false;
      R *= g_.ranges[(size_t)r].extent;
    }
    for (int id : top_reduces_) {
      const KNode &k = g_.n(id);
      std::vector<int> r2;
      for (size_t i = 1; i < k.src.size(); i++) r2.push_back(g_.range_ord.at(k.src[i]));
      if (r2 != rr) return false;
      if (dt_size(k.dt) != 4 && dt_size(k.dt) != 8) return false;
      PolyOps op = reduce_op(k);
      if (op != POLY_OP_ADD && op != POLY_OP_MAX && op != POLY_OP_MUL) return false;
    }
    for (int r : groups_[0].ranges) if (g_.ranges[(size_t)r].extent < 0) return false;
    double rows = 1;
    for (int r : groups_[0].ranges) rows *= (double)g_.ranges[(size_t)r].extent;
    if (R < 128) return false;
    // Lanes that walk along the reduce range only pay off when some operand is contiguous
    // along it.  When every load is strided there (X^T W forms: the reduce axis is the
    // outer axis of both operands) but contiguous along an output range, one thread per
    // output with a serial loop is the coalesced mapping: neighbouring lanes read
    // neighbouring addresses at every step.
    {
      const int QF = rr.back();
      bool unit_along_reduce = false, unit_along_output = false;
      std::vector<char> mark(g_.nodes.size(), 0);
      for (int id : top_reduces_) mark_reachable(g_, g_.n(id).src[0], mark);
      for (int i = 0; i < (int)g_.nodes.size(); i++) {
        if (!mark[(size_t)i] || g_.n(i).op != POLY_OP_LOAD) continue;
        const int li = g_.n(g_.n(g_.n(i).src[0]).src[1]).lin;
        if (li < 0) { unit_along_reduce = true; continue; }   // unknown: keep the default
        bool aff;
        if (g_.lin_range_coef(g_.lins[(size_t)li], QF, &aff) == 1 && aff) unit_along_reduce = true;
        // unit stride along an output range, or along the fastest digit (r % c) of a
        // flattened one
        for (const Term &t : g_.lins[(size_t)li].terms) {
          if (t.coef != 1) continue;
          const Atom &a = g_.atoms[(size_t)t.atom];
          const Atom *base = &a;
          if (a.kind == Atom::MOD && a.inner.c0 == 0 && a.inner.terms.size() == 1 && a.inner.terms[0].coef == 1)
            base = &g_.atoms[(size_t)a.inner.terms[0].atom];
          else if (a.kind != Atom::RANGE) continue;
          if (base->kind != Atom::RANGE) continue;
          const int ord = g_.range_ord.at(base->node);
          for (int r : groups_[0].ranges) if (r == ord) unit_along_output = true;
        }
      }
      if (!unit_along_reduce && unit_along_output && (rows >= 65536 || opt_.coop_needs_unit_stride) && opt_.promote_reduce < 0) return false;
    }
    // Long rows, or too few rows to fill the chip with one wave each: a whole
    // workgroup per row.
    if (R >= 4096 || (rows < 2048 && R >= 1024)) coop_G_ = 256; else coop_G_ = 64;
    coop_R_ = R;
    coop_ranges_ = rr;
    return true;
  }

  std::string wave_reduce_call(PolyOps op, DT dt, const std::string &v) const { return polyhip::wave_reduce_call(op, dt, v, 64); }

  std::string render_coop(RenderedKernel *out) {
    const Group &gr = groups_[0];
    const int G = coop_G_;
    const int rows_per_block = opt_.block / G;
    std::vector<int> order = fastest_first(gr);
    double rows = 1;
    std::string body;
    Scope S0;
    S0.indent = 2;
    for (int r : gr.ranges) S0.avail |= (uint64_t)1 << r;
    if (opt_.promote_reduce >= 0) {
      const KNode &T = g_.n(opt_.promote_reduce);
      for (size_t i = 1; i < T.src.size(); i++) S0.avail |= (uint64_t)1 << g_.range_ord.at(T.src[i]);
    }
    if (G == 64) {
      line(body, 1, "const int lane = threadIdx.x & 63;");
      line(body, 1, strf("const long long row = (long long)blockIdx.x * %d + (threadIdx.x >> 6);", rows_per_block));
    } else {
      line(body, 1, "const int lane = threadIdx.x;");
      line(body, 1, "const long long row = blockIdx.x;");
    }
    std::string decomp;
    line(decomp, 2, "long long t_ = row;");
    for (size_t oi = 0; oi < order.size(); oi++) {
      int ord = order[oi];
      int64_t e = g_.ranges[(size_t)ord].extent;
      rows *= (double)e;
      std::string rv = strf("r%d", ord);
      if (oi + 1 == order.size()) line(decomp, 2, strf("const int %s = (int)t_;", rv.c_str()));
      else line(decomp, 2, strf("const int %s = (int)(t_ %% %lld); t_ /= %lld;", rv.c_str(), (long long)e, (long long)e));
      em_.bind_range(ord, rv);
    }
    // vector width along the fastest reduce range
    int QF = coop_ranges_.back();
    int64_t eF = g_.ranges[(size_t)QF].extent;
    int V = 1;
    bool ragged = false;
    if (opt_.allow_vectorize) {
      int maxsz = 1;
      std::vector<char> mark(g_.nodes.size(), 0);
      for (int id : top_reduces_) node_under(g_.n(id).src[0], mark);
      for (int i = 0; i < (int)g_.nodes.size(); i++)
        if (mark[(size_t)i] && g_.n(i).op == POLY_OP_LOAD && (g_.n(i).deps & ((uint64_t)1 << QF)))
          maxsz = std::max(maxsz, dt_size(g_.n(i).dt));
      V = std::max(1, 16 / maxsz);
      while (V > 1 && (eF % V != 0 || coop_R_ < (int64_t)G * V)) V /= 2;
      // A single reduce range whose extent is no multiple of the vector width (a vocabulary
      // of 50257): vectors up to the last full one, wherever the row starts, and the
      // remaining R mod V elements one lane each.
      if (V == 1 && coop_ranges_.size() == 1 && !getenv("POLY_HIP_NO_RAGGED_VEC")) {
        int vr = std::max(1, 16 / maxsz);
        while (vr > 1 && coop_R_ < (int64_t)G * vr * 4) vr /= 2;
        if (vr > 1) { V = vr; ragged = true; }
      }
    }
    // accumulators
    std::string accs;
    for (int id : top_reduces_) {
      const KNode &k = g_.n(id);
      line(accs, 2, strf("%s acc%d = %s;", dt_cname(k.dt), id, Emitter::reduce_identity(reduce_op(k), k.dt).c_str()));
    }
    // loop over the flattened reduce index
    Scope L;
    L.parent = &S0;
    L.avail = S0.avail;
    L.indent = 3;
    std::string qdecomp;
    line(qdecomp, 3, "int q_ = q0;");
    for (size_t i = coop_ranges_.size(); i-- > 0;) {
      int ord = coop_ranges_[i];
      int64_t e = g_.ranges[(size_t)ord].extent;
      std::string rv = strf("r%d", ord);
      bool fastest = (i + 1 == coop_ranges_.size());
      std::string nm = fastest && V > 1 ? rv + "_0" : rv;
      if (i == 0) line(qdecomp, 3, strf("const int %s = q_;", nm.c_str()));
      else line(qdecomp, 3, strf("const int %s = q_ %% %lld; q_ /= %lld;", nm.c_str(), (long long)e, (long long)e));
      em_.bind_range(ord, nm);
      if (!(fastest && V > 1)) L.avail |= (uint64_t)1 << ord;
    }
    std::vector<int> roots;
    for (int id : top_reduces_) roots.push_back(g_.n(id).src[0]);
    std::vector<int> pres;
    std::string loop_body;
    if (V > 1) {
      pres = hoist_vector_loads(roots, QF, V, strf("r%d_0", QF), &L, true, ragged);
      Scope U;
      U.parent = &L;
      U.avail = L.avail | ((uint64_t)1 << QF);
      U.indent = 4;
      em_.bind_range(QF, strf("r%d", QF));
      for (int id : top_reduces_) {
        const KNode &k = g_.n(id);
        std::string v = em_.emit(k.src[0], &U);
        std::string acc = strf("acc%d", id);
        line(U.code, 4, strf("%s = %s;", acc.c_str(), Emitter::reduce_combine(reduce_op(k), k.dt, acc, v).c_str()));
      }
      loop_body = L.code;
      line(loop_body, 3, "#pragma unroll");
      line(loop_body, 3, strf("for (int u = 0; u < %d; u++) {", V));
      line(loop_body, 4, strf("const int r%d = r%d_0 + u;", QF, QF));
      loop_body += U.code;
      line(loop_body, 3, "}");
    } else {
      for (int id : top_reduces_) {
        const KNode &k = g_.n(id);
        std::string v = em_.emit(k.src[0], &L);
        std::string acc = strf("acc%d", id);
        line(L.code, 3, strf("%s = %s;", acc.c_str(), Emitter::reduce_combine(reduce_op(k), k.dt, acc, v).c_str()));
      }
      loop_body = L.code;
    }
    for (int n : pres) em_.clear_preset(n);
    std::string ragged_tail;
    if (ragged) {
      Scope Tl;
      Tl.parent = &S0;
      Tl.avail = S0.avail | ((uint64_t)1 << QF);
      Tl.indent = 3;
      em_.bind_range(QF, strf("r%d", QF));
      for (int id : top_reduces_) {
        const KNode &k = g_.n(id);
        std::string v = em_.emit(k.src[0], &Tl);
        std::string acc = strf("acc%d", id);
        line(Tl.code, 3, strf("%s = %s;", acc.c_str(), Emitter::reduce_combine(reduce_op(k), k.dt, acc, v).c_str()));
      }
      line(ragged_tail, 2, strf("if (lane < %lld) {", (long long)(coop_R_ % V)));
      line(ragged_tail, 3, strf("const int r%d = %lld + lane;", QF, (long long)(coop_R_ - coop_R_ % V)));
      ragged_tail += Tl.code;
      line(ragged_tail, 2, "}");
    }
    // S0.code now holds everything hoisted out of the loop (row-invariant values)
    std::string pre_loop = S0.code;
    S0.code.clear();
    std::string red;
    int nred = (int)top_reduces_.size();
    for (int id : top_reduces_) {
      const KNode &k = g_.n(id);
      line(red, 2, strf("acc%d = %s;", id, wave_reduce_call(reduce_op(k), k.dt, strf("acc%d", id)).c_str()));
    }
    if (G == 256) {
      int ri = 0;
      for (int id : top_reduces_) {
        const KNode &k = g_.n(id);
        line(red, 2, strf("if ((threadIdx.x & 63) == 0) red%d[threadIdx.x >> 6] = acc%d;", ri, id));
        ri++;
        (void)k;
      }
      line(red, 2, "__syncthreads();");
      ri = 0;
      for (int id : top_reduces_) {
        const KNode &k = g_.n(id);
        PolyOps op = reduce_op(k);
        std::string e = strf("red%d[0]", ri);
        for (int w = 1; w < 4; w++) e = Emitter::reduce_combine(op, k.dt, e, strf("red%d[%d]", ri, w));
        line(red, 2, strf("acc%d = %s;", id, e.c_str()));
        ri++;
      }
    }
    for (int id : top_reduces_) em_.preset(id, strf("acc%d", id));
    // tail: value + store by lane 0
    std::string tail_stores;
    if (opt_.promote_reduce >= 0) {
      const std::string term = em_.emit(g_.n(opt_.promote_reduce).src[0], &S0);
      line(tail_stores, 2, strf("if (lane == 0) poly_scratch[row] = %s;", term.c_str()));
    } else
    for (int si : gr.stores) {
      const StoreInfo &st = g_.stores[(size_t)si];
      std::string v = em_.emit(st.value, &S0);
      std::string idx = em_.emit(g_.n(st.index).src[1], &S0);
      int p = g_.param_slot(st.param);
      std::string cond = "lane == 0";
      if (st.gate >= 0) cond += " && " + em_.emit(st.gate, &S0);
      line(tail_stores, 2, strf("if (%s) data%d[%s] = %s;", cond.c_str(), p, idx.c_str(), v.c_str()));
    }
    std::string tail = S0.code + tail_stores;

    if (G == 256) {
      int ri = 0;
      for (int id : top_reduces_) {
        line(body, 1, strf("__shared__ %s red%d[4];", dt_cname(g_.n(id).dt), ri));
        ri++;
      }
      line(body, 1, "{");
    } else {
      line(body, 1, strf("if (row < %lldll) {", (long long)rows));
    }
    body += decomp + accs + pre_loop;
    line(body, 2, strf("for (int q0 = lane * %d; q0 < %lld; q0 += %d) {", V, (long long)(coop_R_ - (ragged ? coop_R_ % V : 0)), G * V));
    body += qdecomp + loop_body;
    line(body, 2, "}");
    body += ragged_tail + red + tail;
    line(body, 1, "}");
    (void)nred;

    double blocks = G == 256 ? rows : std::ceil(rows / rows_per_block);
    if (blocks > 2147483647.0) { error_ = "grid too large"; return body; }
    out->launch.grid[0] = (unsigned)std::max(1.0, blocks);
    out->launch.block[0] = (unsigned)opt_.block;
    out->klass = KernelClass::ROW_REDUCE;
    out->strategy = strf("row-reduce G=%d vec%d%s R=%lld rows=%.0f", G, V, ragged ? " (unaligned, scalar tail)" : "", (long long)coop_R_, rows);
    return body;
  }

  // ── ordered reduction with cooperative loads ─────────────────────────────
  //
  // A long reduction for a few thousand outputs that must keep its order (a sum that
  // accumulates in bf16: every partial sum is rounded, so the order is part of the result)
  // and whose loads are contiguous along the outputs.  One thread per output leaves the
  // chip idle and waits a full memory latency every few terms.  Here a workgroup owns 64
  // outputs: all four waves compute terms (wave w the terms w*8 .. w*8+7 of each block of
  // 32) into LDS, then the first wave adds the 32 terms of its outputs in order.
  bool plan_ordered() const {
    if (!opt_.allow_coop_reduce || opt_.promote_reduce >= 0 || opt_.slice_reduce >= 0 || !opt_.reduce_override.empty() ||
        opt_.exit_if_flag || opt_.exit_unless_flag || getenv("POLY_HIP_NO_ORDERED_REDUCE"))
      return false;
    if (groups_.size() != 1 || g_.reduces.size() != 1 || top_reduces_.size() != 1 || !g_.vars.empty()) return false;
    const KNode &T = g_.n(top_reduces_[0]);
    const int sz = dt_size(T.dt);
    if (sz != 2 && sz != 4) return false;
    if (opt_.ordered_stage && !dt_is_float(T.dt)) return false;    // terms travel as fp32
    int64_t K = 1;
    for (size_t i = 1; i < T.src.size(); i++) {
      const int64_t e = g_.ranges[(size_t)g_.range_ord.at(T.src[i])].extent;
      if (e <= 0) return false;
      K *= e;
    }
    double outs = 1;
    for (int r : groups_[0].ranges) {
      if (g_.ranges[(size_t)r].extent <= 0) return false;
      outs *= (double)g_.ranges[(size_t)r].extent;
    }
    if (K < 512 || K % 32 != 0 || outs < 64 || outs > 16384) return false;
    // the loads must run along the outputs, not along the reduce range
    const std::vector<int> order = fastest_first(groups_[0]);
    const int F = order[0], QF = g_.range_ord.at(T.src.back());
    std::vector<char> mark(g_.nodes.size(), 0);
    mark_reachable(g_, T.src[0], mark);
    bool along_out = false;
    for (int i = 0; i < (int)g_.nodes.size(); i++) {
      if (!mark[(size_t)i] || g_.n(i).op != POLY_OP_LOAD) continue;
      const int li = g_.n(g_.n(g_.n(i).src[0]).src[1]).lin;
      if (li < 0) return false;
      bool aff;
      // (a value per reduce index that no output coordinate enters -- a row statistic --
      // is the same for every lane: it does not decide the mapping)
      uint64_t out_bits = 0;
      for (int r : groups_[0].ranges) out_bits |= (uint64_t)1 << r;
      if (!(g_.n(g_.n(g_.n(i).src[0]).src[1]).deps & out_bits)) continue;
      if (g_.lin_range_coef(g_.lins[(size_t)li], QF, &aff) == 1 && aff) return false;
      if (g_.lin_range_coef(g_.lins[(size_t)li], F, &aff) == 1 && aff) along_out = true;
    }
    return along_out;
  }

  std::string render_ordered(RenderedKernel *out) {
    const Group &gr = groups_[0];
    const int T = top_reduces_[0];
    const KNode &tk = g_.n(T);
    const PolyOps rop = reduce_op(tk);
    const std::vector<int> order = fastest_first(gr);
    double outs = 1;
    for (int r : gr.ranges) outs *= (double)g_.ranges[(size_t)r].extent;
    int64_t K = 1;
    std::vector<int> rr;
    for (size_t i = 1; i < tk.src.size(); i++) { rr.push_back(g_.range_ord.at(tk.src[i])); K *= g_.ranges[(size_t)rr.back()].extent; }
    const char *ct = dt_cname(tk.dt);
    std::string body;
    line(body, 1, strf("__shared__ %s poly_terms[32][64];", ct));
    line(body, 1, "const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;");
    line(body, 1, strf("const long long out_id = (long long)blockIdx.x * 64 + lane;"));
    line(body, 1, strf("const bool live = out_id < %.0fll;", outs));
    line(body, 1, "{");
    Scope S0;
    S0.indent = 2;
    for (int r : gr.ranges) S0.avail |= (uint64_t)1 << r;
    std::string decomp;
    line(decomp, 2, strf("long long t_ = live ? out_id : %.0fll;", outs - 1));   // idle lanes redo the last output, store nothing
    for (size_t oi = 0; oi < order.size(); oi++) {
      const int ord = order[oi];
      const long long e = (long long)g_.ranges[(size_t)ord].extent;
      if (oi + 1 == order.size()) line(decomp, 2, strf("const int r%d = (int)t_;", ord));
      else line(decomp, 2, strf("const int r%d = (int)(t_ %% %lld); t_ /= %lld;", ord, e, e));
      em_.bind_range(ord, strf("r%d", ord));
    }
    Scope L;
    L.parent = &S0;
    L.avail = S0.avail;
    L.indent = 4;
    std::string qdecomp;
    line(qdecomp, 4, "int q_ = k0 + w * 8 + t8;");
    for (size_t i = rr.size(); i-- > 0;) {
      const int ord = rr[i];
      const long long e = (long long)g_.ranges[(size_t)ord].extent;
      if (i == 0) line(qdecomp, 4, strf("const int r%d = q_;", ord));
      else line(qdecomp, 4, strf("const int r%d = q_ %% %lld; q_ /= %lld;", ord, e, e));
      em_.bind_range(ord, strf("r%d", ord));
      L.avail |= (uint64_t)1 << ord;
    }
    const std::string term = em_.emit(tk.src[0], &L);
    line(L.code, 4, strf("poly_terms[w * 8 + t8][lane] = %s;", term.c_str()));
    const std::string acc = strf("acc%d", T);
    std::string loop;
    line(loop, 2, strf("%s %s = %s;", ct, acc.c_str(), Emitter::reduce_identity(rop, tk.dt).c_str()));
    line(loop, 2, strf("for (int k0 = 0; k0 < %lld; k0 += 32) {", (long long)K));
    line(loop, 3, "#pragma unroll");
    line(loop, 3, "for (int t8 = 0; t8 < 8; t8++) {");
    loop += qdecomp + L.code;
    line(loop, 3, "}");
    line(loop, 3, "__syncthreads();");
    line(loop, 3, "if (w == 0) {");
    line(loop, 4, "#pragma unroll");
    line(loop, 4, strf("for (int t = 0; t < 32; t++) %s = %s;", acc.c_str(),
                       Emitter::reduce_combine(rop, tk.dt, acc, "poly_terms[t][lane]").c_str()));
    line(loop, 3, "}");
    line(loop, 3, "__syncthreads();");
    line(loop, 2, "}");
    const std::string pre_loop = S0.code;
    S0.code.clear();
    em_.preset(T, acc);
    std::string tail_stores;
    for (int si : gr.stores) {
      const StoreInfo &st = g_.stores[(size_t)si];
      std::string v = em_.emit(st.value, &S0);
      std::string idx = em_.emit(g_.n(st.index).src[1], &S0);
      int p = g_.param_slot(st.param);
      std::string cond = "w == 0 && live";
      if (st.gate >= 0) cond += " && " + em_.emit(st.gate, &S0);
      line(tail_stores, 2, strf("if (%s) data%d[%s] = %s;", cond.c_str(), p, idx.c_str(), v.c_str()));
    }
    body += decomp + pre_loop + loop + S0.code + tail_stores;
    line(body, 1, "}");
    out->launch.grid[0] = (unsigned)std::ceil(outs / 64.0);
    out->launch.block[0] = 256;
    out->klass = KernelClass::THREAD_REDUCE;
    out->strategy = strf("ordered reduce: 64 outputs per workgroup, terms of K=%lld computed by four waves, added in order by one;", (long long)K);
    return body;
  }

  // The two kernels of the same reduction with the terms passing through memory: a first
  // kernel computes them, four consecutive terms of an output per thread (the whole chip
  // instead of outputs / 64 workgroups), and the adder only walks a column of finished terms.
  std::string render_ordered_stage(RenderedKernel *out) {
    const Group &gr = groups_[0];
    const int T = top_reduces_[0];
    const KNode &tk = g_.n(T);
    const PolyOps rop = reduce_op(tk);
    const std::vector<int> order = fastest_first(gr);
    double outs = 1;
    for (int r : gr.ranges) outs *= (double)g_.ranges[(size_t)r].extent;
    int64_t K = 1;
    std::vector<int> rr;
    for (size_t i = 1; i < tk.src.size(); i++) { rr.push_back(g_.range_ord.at(tk.src[i])); K *= g_.ranges[(size_t)rr.back()].extent; }
    const char *ct = dt_cname(tk.dt);
    const bool first = opt_.ordered_stage == 1;
    std::string body;
    Scope S0;
    S0.indent = 2;
    for (int r : gr.ranges) S0.avail |= (uint64_t)1 << r;
    std::string decomp;
    if (first) {
      line(body, 1, "const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;");
      line(body, 1, strf("if (gid < %.0fll) {", outs * (double)(K / 4)));
      line(decomp, 2, strf("long long t_ = gid %% %.0fll;", outs));
    } else {
      line(body, 1, "const long long out_id = (long long)blockIdx.x * 64 + threadIdx.x;");
      line(body, 1, strf("const bool live = out_id < %.0fll;", outs));
      line(body, 1, "{");
      line(decomp, 2, strf("const long long col_ = live ? out_id : %.0fll;", outs - 1));   // idle lanes redo the last output, store nothing
      line(decomp, 2, "long long t_ = col_;");
    }
    for (size_t oi = 0; oi < order.size(); oi++) {
      const int ord = order[oi];
      const long long e = (long long)g_.ranges[(size_t)ord].extent;
      if (oi + 1 == order.size()) line(decomp, 2, strf("const int r%d = (int)t_;", ord));
      else line(decomp, 2, strf("const int r%d = (int)(t_ %% %lld); t_ /= %lld;", ord, e, e));
      em_.bind_range(ord, strf("r%d", ord));
    }
    if (first) {
      Scope L;
      L.parent = &S0;
      L.avail = S0.avail;
      L.indent = 3;
      std::string qdecomp;
      line(qdecomp, 3, strf("int q_ = (int)(gid / %.0fll) * 4 + e_;", outs));
      for (size_t i = rr.size(); i-- > 0;) {
        const int ord = rr[i];
        const long long e = (long long)g_.ranges[(size_t)ord].extent;
        if (i == 0) line(qdecomp, 3, strf("const int r%d = q_;", ord));
        else line(qdecomp, 3, strf("const int r%d = q_ %% %lld; q_ /= %lld;", ord, e, e));
        em_.bind_range(ord, strf("r%d", ord));
        L.avail |= (uint64_t)1 << ord;
      }
      const std::string term = em_.emit(tk.src[0], &L);
      line(L.code, 3, strf("four_[e_] = (float)(%s);", term.c_str()));
      body += decomp + S0.code;
      line(body, 2, "poly_f32x4 four_;");
      line(body, 2, "#pragma unroll");
      line(body, 2, "for (int e_ = 0; e_ < 4; e_++) {");
      body += qdecomp + L.code;
      line(body, 2, "}");
      line(body, 2, "*(poly_f32x4 *)(poly_scratch + gid * 4) = four_;");
      line(body, 1, "}");
      out->launch.grid[0] = (unsigned)std::ceil(outs * (double)(K / 4) / 256.0);
      out->launch.block[0] = 256;
      out->klass = KernelClass::ELEMENTWISE;
      out->strategy = strf("ordered reduce, stage 1: the %.0f x %lld terms, four of an output per thread;", outs, (long long)K);
      return body;
    }
    const std::string acc = strf("acc%d", T);
    std::string loop;
    line(loop, 2, strf("%s %s = %s;", ct, acc.c_str(), Emitter::reduce_identity(rop, tk.dt).c_str()));
    // The additions form one dependent chain; what can overlap is the memory latency of
    // the terms.  They lie as [k / 4][output][4], so a thread fetches four of its terms
    // with one 16-byte load; two sets of 16 such loads alternate, one in flight while the
    // 64 terms of the other are added (the load after the last pair fetches block 0
    // again, unused, so that no branch separates a load from the waits that count it).
    const long long NP = K / 128;
    line(loop, 2, "const poly_f32x4 *const col4_ = (const poly_f32x4 *)poly_scratch + col_;");
    auto consume = [&](const char *set) {
      line(loop, 3, "#pragma unroll");
      line(loop, 3, "for (int j = 0; j < 16; j++)");
      line(loop, 3, "#pragma unroll");
      line(loop, 4, strf("for (int e = 0; e < 4; e++) %s = %s;", acc.c_str(),
                         Emitter::reduce_combine(rop, tk.dt, acc, strf("(%s)%s[j][e]", ct, set)).c_str()));
    };
    if (NP > 0) {
      line(loop, 2, "poly_f32x4 a_[16], b_[16];");
      line(loop, 2, "#pragma unroll");
      line(loop, 2, strf("for (int j = 0; j < 16; j++) a_[j] = col4_[(long long)j * %.0fll];", outs));
      line(loop, 2, strf("for (int p = 0; p < %lld; p++) {", NP));
      line(loop, 3, "#pragma unroll");
      line(loop, 3, strf("for (int j = 0; j < 16; j++) b_[j] = col4_[(long long)((2 * p + 1) * 16 + j) * %.0fll];", outs));
      // (the compiler would gather all 32 loads at the top of the iteration and wait for
      // them there: the fences keep each set of loads behind the additions before it)
      line(loop, 3, "__builtin_amdgcn_sched_barrier(0);");
      consume("a_");
      line(loop, 3, "__builtin_amdgcn_sched_barrier(0);");
      line(loop, 3, strf("const int nb_ = p + 1 < %lld ? 2 * p + 2 : 0;", NP));
      line(loop, 3, "#pragma unroll");
      line(loop, 3, strf("for (int j = 0; j < 16; j++) a_[j] = col4_[(long long)(nb_ * 16 + j) * %.0fll];", outs));
      line(loop, 3, "__builtin_amdgcn_sched_barrier(0);");
      consume("b_");
      line(loop, 3, "__builtin_amdgcn_sched_barrier(0);");
      line(loop, 2, "}");
    }
    if (K % 128)
      line(loop, 2, strf("for (int k = %lld; k < %lld; k++) %s = %s;", NP * 128, (long long)K, acc.c_str(),
                         Emitter::reduce_combine(rop, tk.dt, acc, strf("(%s)poly_scratch[((long long)(k >> 2) * %.0fll + col_) * 4 + (k & 3)]", ct, outs)).c_str()));
    em_.preset(T, acc);
    std::string tail_stores;
    for (int si : gr.stores) {
      const StoreInfo &st = g_.stores[(size_t)si];
      std::string v = em_.emit(st.value, &S0);
      std::string idx = em_.emit(g_.n(st.index).src[1], &S0);
      int p = g_.param_slot(st.param);
      std::string cond = "live";
      if (st.gate >= 0) cond += " && " + em_.emit(st.gate, &S0);
      line(tail_stores, 2, strf("if (%s) data%d[%s] = %s;", cond.c_str(), p, idx.c_str(), v.c_str()));
    }
    body += decomp + loop + S0.code + tail_stores;
    line(body, 1, "}");
    out->launch.grid[0] = (unsigned)std::ceil(outs / 64.0);
    out->launch.block[0] = 64;
    out->klass = KernelClass::THREAD_REDUCE;
    out->strategy = strf("stage 2: K=%lld terms per output added in index order, one thread per output;", (long long)K);
    return body;
  }

  // Algorithmic bytes: distinct elements each access can touch, capped by the
  // buffer size, summed over buffers.
  void account(RenderedKernel *out) const {
    std::vector<double> touched(g_.params.size(), 0.0);
    auto distinct = [&](int idx_node) {
      uint64_t d = g_.n(idx_node).deps;
      double n = 1;
      for (size_t r = 0; r < g_.ranges.size(); r++)
        if (d & ((uint64_t)1 << r)) n *= (double)std::max<int64_t>(1, g_.ranges[r].extent);
      return n;
    };
    for (const KNode &k : g_.nodes) {
      if (k.op == POLY_OP_LOAD) {
        const KNode &ix = g_.n(k.src[0]);
        touched[(size_t)g_.param_slot(ix.src[0])] += distinct(ix.src[1]);
      }
    }
    for (const StoreInfo &st : g_.stores) touched[(size_t)g_.param_slot(st.param)] += distinct(g_.n(st.index).src[1]);
    double bytes = 0, stored = 0;
    for (size_t i = 0; i < g_.params.size(); i++) {
      double n = touched[i];
      if (g_.params[i].numel > 0) n = std::min(n, (double)g_.params[i].numel * ((g_.params[i].read && g_.params[i].written) ? 2 : 1));
      bytes += n * dt_size(g_.params[i].dt);
      if (g_.params[i].written) stored += (g_.params[i].read ? n / 2 : n) * dt_size(g_.params[i].dt);
    }
    out->bytes = bytes;
    out->bytes_written = stored;
  }
};

}  // namespace

static bool split_in_two(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt, int T, PolyOps top,
                         double rows, double per_output, int slice_range, int parts, RenderedKernel *out);

// A reduction to few outputs whose terms are reductions themselves (a loss: the sum over
// tokens of a sum over the vocabulary) would run on one workgroup per output, each thread
// walking a whole inner row on its own.  It is cut in two kernels instead: the first
// gives every (output, outer index) pair a workgroup that reduces the inner ranges
// cooperatively and leaves the term in scratch memory; the second is the original kernel
// with the outer REDUCE replaced by a sum over those terms, in index order.
static bool try_split_reduce(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt, RenderedKernel *out) {
  if (!opt.allow_coop_reduce || !opt.reduce_override.empty() || opt.exit_if_flag || opt.exit_unless_flag ||
      opt.promote_reduce >= 0 || getenv("POLY_HIP_NO_SPLIT_REDUCE"))
    return false;
  if (g.stores.empty() || g.reduces.size() < 2) return false;
  for (const StoreInfo &st : g.stores) if (st.ranges != g.stores[0].ranges) return false;
  // exactly one REDUCE that is not nested in another: the one to promote
  std::vector<char> inside(g.nodes.size(), 0);
  for (int r : g.reduces) mark_reachable(g, g.n(r).src[0], inside);
  int T = -1;
  for (int r : g.reduces) if (!inside[(size_t)r]) { if (T >= 0) return false; T = r; }
  if (T < 0) return false;
  const KNode &tk = g.n(T);
  const PolyOps top = tk.u->arg.kind == POLY_ARG_OPS ? tk.u->arg.ops : (PolyOps)tk.u->arg.i;
  if (tk.dt != DT_F32 || (top != POLY_OP_ADD && top != POLY_OP_MAX && top != POLY_OP_MUL)) return false;
  double rows = 1, rt = 1, inner = 0;
  for (int r : g.stores[0].ranges) { if (g.ranges[(size_t)r].extent <= 0) return false; rows *= (double)g.ranges[(size_t)r].extent; }
  for (size_t i = 1; i < tk.src.size(); i++) {
    const int64_t e = g.ranges[(size_t)g.range_ord.at(tk.src[i])].extent;
    if (e <= 0) return false;
    rt *= (double)e;
  }
  for (int r : g.reduces) {
    if (r == T) continue;
    double n = 1;
    for (size_t i = 1; i < g.n(r).src.size(); i++) {
      const int64_t e = g.ranges[(size_t)g.range_ord.at(g.n(r).src[i])].extent;
      if (e <= 0) return false;
      n *= (double)e;
    }
    inner = std::max(inner, n);
  }
  // few outputs, many terms, long inner rows
  if (rows > 64 || rt < 64 || inner < 256 || rows * rt > 16777216.0) return false;
  return split_in_two(g, fn_name, opt, T, top, rows, rt, -1, 0, out);
}

// The other shape: one REDUCE over many terms for a modest number of outputs, where lanes
// along the outputs are the coalesced mapping (column sums: bias and LayerNorm-parameter
// gradients) and one thread per output leaves most of the chip idle.  Each output gets
// `parts` threads that walk the longest reduce range in steps of `parts`; the second
// kernel adds the partial results in part order.
static bool try_slice_reduce(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt, RenderedKernel *out) {
  if (!opt.reduce_override.empty() || opt.exit_if_flag || opt.exit_unless_flag || opt.promote_reduce >= 0 ||
      opt.slice_reduce >= 0 || getenv("POLY_HIP_NO_SPLIT_REDUCE"))
    return false;
  if (g.stores.empty() || g.reduces.size() != 1 || !g.vars.empty()) return false;
  for (const StoreInfo &st : g.stores) if (st.ranges != g.stores[0].ranges) return false;
  const int T = g.reduces[0];
  const KNode &tk = g.n(T);
  const PolyOps top = tk.u->arg.kind == POLY_ARG_OPS ? tk.u->arg.ops : (PolyOps)tk.u->arg.i;
  if (tk.dt != DT_F32 || (top != POLY_OP_ADD && top != POLY_OP_MAX && top != POLY_OP_MUL)) return false;
  double rows = 1, rt = 1;
  for (int r : g.stores[0].ranges) { if (g.ranges[(size_t)r].extent <= 0) return false; rows *= (double)g.ranges[(size_t)r].extent; }
  int longest = -1;
  for (size_t i = 1; i < tk.src.size(); i++) {
    const int ord = g.range_ord.at(tk.src[i]);
    const int64_t e = g.ranges[(size_t)ord].extent;
    if (e <= 0) return false;
    rt *= (double)e;
    if (longest < 0 || e > g.ranges[(size_t)longest].extent) longest = ord;
  }
  if (rows > 16384 || rt < 1024) return false;
  // only where the plain lowering is one thread per output
  {
    RenderedKernel plain;
    std::string err;
    RenderOptions strict = opt;
    strict.coop_needs_unit_stride = true;
    Generic gen(g, fn_name, strict);
    if (!gen.run(&plain, &err) || plain.klass != KernelClass::THREAD_REDUCE) return false;
  }
  int parts = 1;
  while (parts < 128 && rows * parts < 65536.0 && (int64_t)parts * 8 <= g.ranges[(size_t)longest].extent) parts *= 2;
  if (parts < 4) return false;
  return split_in_two(g, fn_name, opt, T, top, rows, (double)parts, longest, parts, out);
}

// Renders the two kernels of a split reduction of REDUCE node T: the first stage leaves
// `per_output` terms per output in scratch memory (promoted ranges when slice_range < 0,
// else `parts` strided slices of that range), the second is the kernel itself with T
// replaced by the combination of those terms in index order.
static bool split_in_two(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt, int T, PolyOps top,
                         double rows, double per_output, int slice_range, int parts, RenderedKernel *out) {
  const double rt = per_output;

  RenderOptions o1 = opt;
  o1.scratch_param = true;
  if (slice_range >= 0) { o1.slice_reduce = T; o1.slice_range = slice_range; o1.slice_parts = parts; o1.allow_coop_reduce = false; }
  else o1.promote_reduce = T;
  RenderedKernel pre;
  std::string err;
  {
    Generic gen(g, fn_name, o1);
    if (!gen.run(&pre, &err)) return false;
    if (slice_range < 0 && pre.klass != KernelClass::ROW_REDUCE) return false;
  }
  RenderOptions o2 = opt;
  o2.scratch_param = true;
  o2.allow_vectorize = false;       // thread id == flat output index, which is what the terms are filed under
  const long long RT = (long long)rt;
  o2.reduce_override[T] = [T, RT, top](Emitter &em, Scope *s) {
    (void)em;
    const std::string acc = strf("acc%d", T);
    std::string pad((size_t)s->indent * 2, ' ');
    s->code += pad + strf("float %s = %s;\n", acc.c_str(), Emitter::reduce_identity(top, DT_F32).c_str());
    s->code += pad + strf("for (int q_ = 0; q_ < %lld; q_++) %s = %s;\n", RT, acc.c_str(),
                          Emitter::reduce_combine(top, DT_F32, acc, strf("poly_scratch[gid * %lldll + q_]", RT)).c_str());
    return acc;
  };
  Generic gen2(g, fn_name, o2);
  if (!gen2.run(out, &err) || out->klass == KernelClass::ROW_REDUCE) return false;
  out->pres.push_back({pre.source, pre.entry, pre.launch});
  out->scratch_bytes = (size_t)(rows * rt) * sizeof(float);
  out->klass = KernelClass::ROW_REDUCE;
  out->strategy = "two stages: " + pre.strategy + " into scratch, then " + out->strategy;
  out->bytes = pre.bytes;
  return true;
}

// The order-preserving reduction (a sum that rounds to 16 bits at every step) with its terms
// computed by a first kernel over the whole chip; the second only adds, in index order.
static bool try_ordered_two_stage(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt, RenderedKernel *out) {
  if (opt.ordered_stage || opt.scratch_param || !opt.reduce_override.empty() || opt.exit_if_flag || opt.exit_unless_flag ||
      opt.promote_reduce >= 0 || opt.slice_reduce >= 0 || getenv("POLY_HIP_NO_SPLIT_REDUCE"))
    return false;
  if (g.stores.empty() || g.reduces.size() != 1 || !g.vars.empty()) return false;
  double terms = 1;
  for (const RangeInfo &r : g.ranges) { if (r.extent <= 0) return false; terms *= (double)r.extent; }
  if (terms * 4 > 268435456.0) return false;        // scratch: at most 256 MiB
  RenderOptions o1 = opt, o2 = opt;
  o1.ordered_stage = 1; o1.scratch_param = true;
  o2.ordered_stage = 2; o2.scratch_param = true;
  RenderedKernel pre;
  std::string err;
  Generic g1(g, fn_name, o1);
  if (!g1.run(&pre, &err)) return false;
  Generic g2(g, fn_name, o2);
  if (!g2.run(out, &err)) return false;
  out->pres.push_back({pre.source, pre.entry, pre.launch});
  out->scratch_bytes = (size_t)terms * sizeof(float);
  out->strategy = pre.strategy + " " + out->strategy;
  out->bytes = pre.bytes;
  return true;
}

// For which values of range ordinal R can boolean node `id` (negated when `neg`) hold?
// Narrows [*lo, *hi) and returns true when the answer is that interval exactly: conjunctions
// of comparisons of R with constants, and comparisons that the bounds of their operands decide.
static bool cond_interval(const KernelGraph &g, int id, bool neg, int R, int64_t *lo, int64_t *hi) {
  const KNode &k = g.n(id);
  auto is_true = [&](int n) { return g.n(n).op == POLY_OP_CONST && g.n(n).dt == DT_BOOL && g.n(n).u->arg.b; };
  if (k.op == POLY_OP_CONST && k.dt == DT_BOOL) {
    if (k.u->arg.b == neg) *hi = *lo;
    return true;
  }
  if (k.dt == DT_BOOL && k.op == POLY_OP_NEG) return cond_interval(g, k.src[0], !neg, R, lo, hi);
  if (k.dt == DT_BOOL && (k.op == POLY_OP_CMPNE || k.op == POLY_OP_XOR) && k.src.size() == 2 && g.n(k.src[0]).dt == DT_BOOL) {
    if (is_true(k.src[1])) return cond_interval(g, k.src[0], !neg, R, lo, hi);
    if (is_true(k.src[0])) return cond_interval(g, k.src[1], !neg, R, lo, hi);
    return false;
  }
  if (k.op == POLY_OP_AND && k.dt == DT_BOOL && !neg)
    return cond_interval(g, k.src[0], false, R, lo, hi) && cond_interval(g, k.src[1], false, R, lo, hi);
  if (k.op == POLY_OP_CMPLT && k.src.size() == 2) {
    const int la = g.n(k.src[0]).lin, lb = g.n(k.src[1]).lin;
    if (la < 0 || lb < 0) return false;
    const Lin d = g.lin_add(g.lins[(size_t)la], g.lins[(size_t)lb], -1);      // holds when d < 0
    int64_t dl, dh;
    g.lin_bounds(d, &dl, &dh);
    if (dh < 0) { if (neg) *hi = *lo; return true; }
    if (dl >= 0) { if (!neg) *hi = *lo; return true; }
    if (d.terms.size() != 1) return false;
    const Atom &a = g.atoms[(size_t)d.terms[0].atom];
    if (a.kind != Atom::RANGE || g.range_ord.at(a.node) != R) return false;
    if (d.terms[0].coef == 1) {            // R + c0 < 0  <=>  R < -c0
      if (!neg) *hi = std::min(*hi, -d.c0); else *lo = std::max(*lo, -d.c0);
    } else if (d.terms[0].coef == -1) {    // c0 - R < 0  <=>  R > c0
      if (!neg) *lo = std::max(*lo, d.c0 + 1); else *hi = std::min(*hi, d.c0 + 1);
    } else return false;
    if (*hi < *lo) *hi = *lo;
    return true;
  }
  return false;
}

// A kernel whose stored value is a sum of where(cond_i, X_i, 0) with the conditions cutting
// one output range into adjacent slabs -- the derivative of a concatenation, e.g. of the
// q | k | v columns of an attention block, every X_i its own batched matmul -- computes, as
// one kernel, every sum in every thread.  It is rendered as one kernel per slab instead
// (range restricted, value X_i), run one after the other: each is then a plain kernel that
// the matmul lowerings can take.  x + 0 + 0 is x, so the values are the same (a -0 result
// stays -0 instead of becoming +0).  Done only when every slab lands on the matrix pipe.
static bool fis_reject(int line) {
  if (getenv("POLY_HIP_DEBUG")) fprintf(stderr, "polygrad: render_hip: slab fission rejected at render_hip.cc:%d\n", line);
  return false;
}

static bool try_slab_fission(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt, RenderedKernel *out) {
  if (!opt.allow_templates || !opt.reduce_override.empty() || opt.exit_if_flag || opt.exit_unless_flag || opt.promote_reduce >= 0 ||
      opt.slice_reduce >= 0 || opt.scratch_param || g.slab_range || getenv("POLY_HIP_NO_FISSION"))
    return false;
  if (g.stores.size() != 1 || g.stores[0].gate >= 0 || !g.vars.empty() || g.reduces.size() < 2) return false;
  const StoreInfo &st = g.stores[0];
  // leaves of the sum
  struct Piece { int cond, value; int64_t lo, hi; };
  std::vector<Piece> pieces;
  std::vector<int> stack{st.value};
  while (!stack.empty()) {
    const int id = stack.back();
    stack.pop_back();
    const KNode &k = g.n(id);
    if (k.op == POLY_OP_ADD && dt_is_float(k.dt) && k.dt == g.n(st.value).dt) { stack.push_back(k.src[1]); stack.push_back(k.src[0]); continue; }
    if (k.op != POLY_OP_WHERE || k.src.size() != 3) return fis_reject(__LINE__);
    const KNode &z = g.n(k.src[2]);
    if (z.op != POLY_OP_CONST || !dt_is_float(z.dt) || z.u->arg.f != 0.0 || g.n(k.src[1]).dt != k.dt) return fis_reject(__LINE__);
    pieces.push_back({k.src[0], k.src[1], 0, 0});
  }
  if (pieces.size() < 2 || pieces.size() > 8) return fis_reject(__LINE__);
  for (const int R : st.ranges) {
    const int64_t ext = g.ranges[(size_t)R].extent;
    if (ext <= 0) continue;
    bool ok = true;
    for (Piece &p : pieces) {
      p.lo = 0; p.hi = ext;
      if (!cond_interval(g, p.cond, false, R, &p.lo, &p.hi) || p.hi <= p.lo) { ok = false; break; }
    }
    if (!ok) continue;
    std::vector<Piece> order = pieces;
    std::sort(order.begin(), order.end(), [](const Piece &a, const Piece &b) { return a.lo < b.lo; });
    int64_t at = 0;
    for (const Piece &p : order) { if (p.lo != at) { ok = false; break; } at = p.hi; }
    if (!ok || at != ext) continue;
    // one kernel per slab
    std::vector<RenderedKernel> parts(order.size());
    const PolyUOp *root = g.nodes.back().u;
    // (operand planes that an earlier slab left in the scratch memory and nothing has
    // overwritten since: a later slab may read them)
    const RenderedKernel::OperandPlanes *planes = nullptr;
    for (size_t i = 0; i < order.size() && ok; i++) {
      KernelGraph sub;
      sub.slab_range = g.n(g.ranges[(size_t)R].node).u;
      sub.slab_lo = order[i].lo;
      sub.slab_extent = order[i].hi - order[i].lo;
      sub.slab_value = g.n(order[i].value).u;
      for (const ParamInfo &pi : g.params) sub.slab_params.push_back(g.n(pi.node).u);
      std::string err;
      RenderOptions sopt = opt;
      sopt.planes_before = planes;
      if (!sub.build(root) || !render_kernel(sub, fn_name, sopt, &parts[i], &err)) {
        if (getenv("POLY_HIP_DEBUG")) fprintf(stderr, "polygrad: render_hip: slab %zu: %s%s\n", i, sub.error.c_str(), err.c_str());
        ok = false;
        break;
      }
      const RenderedKernel &pk = parts[i];
      if (pk.klass != KernelClass::MATMUL_MFMA || !pk.guards.empty() || !pk.tables.empty() || !pk.fallback_source.empty() ||
          pk.n_vars != 0 || pk.n_params != parts[0].n_params)
        ok = false;
      if (!pk.reads_planes_before) planes = pk.a_planes.valid ? &parts[i].a_planes : nullptr;
    }
    if (!ok) return fis_reject(__LINE__);
    *out = parts.back();
    out->variants.clear();
    out->pres.clear();
    out->narrow_loads = -1;      // (each slab passed render_kernel's check by itself)
    out->scratch_bytes = 256;
    out->strategy = "";
    out->bytes = 0;
    out->flops = 0;
    for (size_t i = 0; i < parts.size(); i++) {
      const RenderedKernel &pk = parts[i];
      for (const RenderedKernel::Pre &pp : pk.pres) out->pres.push_back(pp);
      if (i + 1 < parts.size()) out->pres.push_back({pk.source, pk.entry, pk.launch});
      out->scratch_bytes = std::max(out->scratch_bytes, pk.scratch_bytes);
      out->strategy += strf("%s[%lld,%lld) %s", i ? "; " : "", (long long)order[i].lo, (long long)order[i].hi, pk.strategy.c_str());
      out->bytes += pk.bytes;
      out->flops += pk.flops;
    }
    out->strategy = strf("%zu slabs of one output range, one kernel each: ", parts.size()) + out->strategy;
    return true;
  }
  return fis_reject(__LINE__);
}

static bool render_kernel_any(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt, RenderedKernel *out, std::string *err);

bool render_kernel(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt,
                   RenderedKernel *out, std::string *err) {
  // loads from fp32 buffers that hold bf16 values at the time of the launch
  // (matmul_hint_param_kinds, kind 2): the lowering has to read every one of them as such
  int narrow_loads = 0;
  for (int id = 0; id < (int)g.nodes.size(); id++) {
    const KNode &k = g.n(id);
    if (k.op != POLY_OP_LOAD) continue;
    const KNode &ix = g.n(k.src[0]);
    if (!ix.src.empty() && matmul_param_kind(g.param_slot(ix.src[0])) == 2) narrow_loads++;
  }
  if (!render_kernel_any(g, fn_name, opt, out, err)) return false;
  if (narrow_loads > 0 && out->narrow_loads != -1 && out->narrow_loads != narrow_loads) {
    if (err) *err = "a buffer of bf16 values would be read as fp32 values";
    return false;
  }
  return true;
}

static bool render_kernel_any(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt,
                   RenderedKernel *out, std::string *err) {
  if (opt.allow_templates) {
    if (try_render_matmul(g, fn_name, opt, out)) return true;
    if (try_render_gather(g, fn_name, opt, out)) return true;
    if (try_render_matmul_generic(g, fn_name, opt, out)) return true;
    *out = RenderedKernel();
    if (try_slab_fission(g, fn_name, opt, out)) return true;
  }
  *out = RenderedKernel();
  if (try_split_reduce(g, fn_name, opt, out)) return true;
  *out = RenderedKernel();
  if (try_slice_reduce(g, fn_name, opt, out)) return true;
  *out = RenderedKernel();
  if (try_ordered_two_stage(g, fn_name, opt, out)) return true;
  *out = RenderedKernel();
  Generic gen(g, fn_name, opt);
  return gen.run(out, err);
}

}  // namespace polyhip
