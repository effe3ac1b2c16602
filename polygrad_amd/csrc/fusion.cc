// Plan-level fusion: kernel groups of a schedule that one launch can execute
// without materialising their intermediates.
//
// The only group recognised so far is attention as a scheduler cuts it
// (reference builder: src/modelzoo/models/gpt2.c:411-441):
//     S   : scores[z,m,n] = f(sum_k Q[z,m,k] K[z,n,k])           (matmul, 16-bit operands)
//     E*  : pointwise kernels on the score tensor (scale, mask)   (0..4 of them)
//     MAX : mx[z,m]  = max_n  cast(x[z,m,n])
//     SUM : sum[z,m] = sum_n  exp2((cast(x[z,m,n]) - mx[z,m]) * c)
//     P   : p[z,m,n] = g(x[z,m,n], mx[z,m], sum[z,m])             (pointwise)
//     PV  : out[z,m,d] = h(sum_n p[z,m,n] V[z,n,d])               (matmul)
// The match is structural: which buffer feeds which kernel, that every consumer
// reads the score tensor at the index the producer wrote (pointwise), that the
// reductions run over the key axis, and that nothing outside the group reads the
// intermediates.  f, the E kernels, g and h are not interpreted; their code is
// generated from their own graphs into the hooks of kernels/attention_mfma.hip.
#include "fusion.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>

namespace polyhip {

namespace {

const char *const kAttentionTemplate =
#include "attention_mfma.hip.inc"
    ;

int fa_item = -1;     // the schedule item a group is being grown from (for the message below)
bool fa_reject(int line) {
  if (getenv("POLY_HIP_DEBUG")) fprintf(stderr, "polygrad: fusion: group from kernel %d rejected at fusion.cc:%d\n", fa_item, line);
  return false;
}
#define FA_REJECT() return fa_reject(__LINE__)

PolyOps reduce_op(const KNode &k) { return k.u->arg.kind == POLY_ARG_OPS ? k.u->arg.ops : (PolyOps)k.u->arg.i; }

// An index expression in the coordinates of the group's first kernel ("master"
// ranges): constant + sum of coef * master range.
struct Aff {
  std::map<int, int64_t> c;
  int64_t c0 = 0;
  bool operator==(const Aff &o) const { return c0 == o.c0 && c == o.c; }
};
typedef std::map<int, int> RangeMap;   // range ordinal of a kernel -> master ordinal

bool lin_to_aff(const KernelGraph &g, const Lin &l, const RangeMap &rm, Aff *out) {
  out->c.clear();
  out->c0 = l.c0;
  for (const Term &t : l.terms) {
    const Atom &a = g.atoms[(size_t)t.atom];
    if (a.kind != Atom::RANGE) return false;
    auto it = rm.find(g.range_ord.at(a.node));
    if (it == rm.end()) return false;
    out->c[it->second] += t.coef;
  }
  for (auto it = out->c.begin(); it != out->c.end();) it = it->second == 0 ? out->c.erase(it) : std::next(it);
  return true;
}

// A consumer reads the producer's buffer at `l` (in its own ranges); the producer
// wrote it at `prod` (master coordinates).  When both are affine with pairwise
// distinct coefficients, equal coefficients identify the consumer's ranges with
// master ranges.  Extends *rm; false when the two cannot describe the same element.
bool derive_map(const KernelGraph &g, const Lin &l, const Aff &prod, const std::vector<int64_t> &master_extent, RangeMap *rm) {
  if (l.c0 != prod.c0 || l.terms.size() != prod.c.size()) return false;
  std::set<int64_t> seen;
  for (auto &kv : prod.c) if (!seen.insert(kv.second).second) return false;
  for (const Term &t : l.terms) {
    const Atom &a = g.atoms[(size_t)t.atom];
    if (a.kind != Atom::RANGE) return false;
    const int ord = g.range_ord.at(a.node);
    int master = -1;
    for (auto &kv : prod.c) if (kv.second == t.coef) master = kv.first;
    if (master < 0) return false;
    if (g.ranges[(size_t)ord].extent != master_extent[(size_t)master]) return false;
    auto it = rm->find(ord);
    if (it != rm->end() && it->second != master) return false;
    for (auto &kv : *rm) if (kv.second == master && kv.first != ord) return false;
    (*rm)[ord] = master;
  }
  return true;
}

struct LoadRef { int node, lin; };

// every LOAD of buffer parameter `param` (position in g.params); false when one is gated
bool loads_of(const KernelGraph &g, int param, std::vector<LoadRef> *out) {
  for (int id = 0; id < (int)g.nodes.size(); id++) {
    const KNode &k = g.n(id);
    if (k.op != POLY_OP_LOAD) continue;
    const KNode &ix = g.n(k.src[0]);
    if (g.param_slot(ix.src[0]) != param) continue;
    if (ix.src.size() != 2 || k.guard >= 0) return false;
    const int lin = g.n(ix.src[1]).lin;
    if (lin < 0) return false;
    out->push_back({id, lin});
  }
  return true;
}

struct Sched {
  const PolySchedule *s;
  const std::vector<KernelGraph> &graphs;
  std::vector<int> step_of;                  // item -> position in exec_order
  std::vector<std::vector<int>> readers, writers;   // per slot: items
  // item -> position at which what it writes exists: its own, or that of the launch of the
  // group that has taken it (groups launch at their last item)
  std::vector<int> launch_step;
  int slot(int item, int param) const { return s->items[item].buf_slot_indices[param]; }
  int param_of(int item, int sl) const {
    const PolyExecItem &it = s->items[item];
    for (int i = 0; i < it.n_buf_slots; i++) if (it.buf_slot_indices[i] == sl) return i;
    return -1;
  }
};

// One kernel of the group with its ranges expressed in master coordinates.
struct Member {
  int item = -1;
  RangeMap rm;
  std::map<int, std::string> preset;   // node -> C expression replacing it
  // ranges bound to an expression of master ranges instead of to one of them (a kernel
  // that walks the buffer with ONE flattened range: the expression is the flat position)
  std::map<int, std::string> range_expr;
};

std::string aff_expr(const Aff &a) {
  std::string e = strf("%lld", (long long)a.c0);
  for (auto &kv : a.c) e += strf(" + %lld * r%d", (long long)kv.second, kv.first);
  return "(" + e + ")";
}

std::string params_decl(const KernelGraph &g) {
  std::string d;
  for (size_t i = 0; i < g.params.size(); i++) {
    const ParamInfo &p = g.params[i];
    if (i) d += ", ";
    if (p.written) d += strf("%s* data%zu", dt_cname(p.dt), i);
    else d += strf("const %s* __restrict__ data%zu", dt_cname(p.dt), i);
  }
  return d;
}

// `item` as a pointwise consumer of buffer `cur` (written at `prod` in master coordinates):
// maps its ranges, replaces its loads of `cur` by `value_name`, and checks that it stores
// its own result at the very same index into a buffer of the same size.
bool pointwise_member(const Sched &sc, int item, int cur, const Aff &prod, const std::vector<int64_t> &mext,
                      const char *value_name, Member *m) {
  const PolySchedule *s = sc.s;
  const KernelGraph &g = sc.graphs[(size_t)item];
  if (!g.reduces.empty() || g.stores.size() != 1 || g.stores[0].gate >= 0 || !g.vars.empty()) return false;
  std::vector<LoadRef> lds;
  const int p = sc.param_of(item, cur);
  if (p < 0 || !loads_of(g, p, &lds) || lds.empty()) return false;
  m->item = item;
  const int li = g.n(g.n(g.stores[0].index).src[1]).lin;
  if (li < 0) return false;
  const int outp = g.param_slot(g.stores[0].param);
  // a kernel over one flattened range p that reads and writes element p
  auto is_flat = [&](const Lin &l, int ord) {
    if (l.c0 != 0 || l.terms.size() != 1 || l.terms[0].coef != 1) return false;
    const Atom &a = g.atoms[(size_t)l.terms[0].atom];
    return a.kind == Atom::RANGE && g.range_ord.at(a.node) == ord;
  };
  if (g.stores[0].ranges.size() == 1 && prod.c0 == 0) {
    const int ord = g.stores[0].ranges[0];
    bool flat = g.ranges[(size_t)ord].extent == s->buf_slots[cur].numel && is_flat(g.lins[(size_t)li], ord);
    for (const LoadRef &l : lds) flat = flat && is_flat(g.lins[(size_t)l.lin], ord);
    // the producer must cover [0, numel) densely for the flat position to be its index
    int64_t span = 1;
    for (auto &kv : prod.c) span += (mext[(size_t)kv.first] - 1) * kv.second;
    if (flat && span == s->buf_slots[cur].numel && prod.c.size() > 1) {
      for (const LoadRef &l : lds) m->preset[l.node] = value_name;
      m->range_expr[ord] = aff_expr(prod);
      if (outp == p || s->buf_slots[sc.slot(item, outp)].numel != s->buf_slots[cur].numel) return false;
      return true;
    }
  }
  for (const LoadRef &l : lds) {
    if (!derive_map(g, g.lins[(size_t)l.lin], prod, mext, &m->rm)) return false;
    m->preset[l.node] = value_name;
  }
  for (int r : g.stores[0].ranges) if (!m->rm.count(r)) return false;
  Aff a;
  if (!lin_to_aff(g, g.lins[(size_t)li], m->rm, &a) || !(a == prod)) return false;
  if (outp == p || s->buf_slots[sc.slot(item, outp)].numel != s->buf_slots[cur].numel) return false;
  return true;
}

// Emits "__device__ ret name(lead_args, int m, int n, int z, <params of the member's kernel>)"
// returning the value of `node`, with the member's ranges bound to the master ranges
// r<ord> that `master_decomp` declares, and its presets applied.  When store_param >= 0
// the function instead stores the value at the kernel's own store index and returns void.
bool emit_member_fn(const Sched &sc, const Member &m, const std::string &master_decomp, const char *name, const char *ret,
                    const std::string &lead_args, int node, const std::map<int, std::string> &extra_preset, bool raw_exp2,
                    bool as_store, std::string *code) {
  const KernelGraph &g = sc.graphs[(size_t)m.item];
  Emitter em(g);
  em.raw_exp2 = raw_exp2;
  Scope S0;
  S0.indent = 1;
  for (auto &kv : m.rm) { em.bind_range(kv.first, strf("r%d", kv.second)); S0.avail |= (uint64_t)1 << kv.first; }
  std::string flat_decl;
  for (auto &kv : m.range_expr) {
    flat_decl += strf("  const int p%d = %s;\n", kv.first, kv.second.c_str());
    em.bind_range(kv.first, strf("p%d", kv.first));
    S0.avail |= (uint64_t)1 << kv.first;
  }
  for (auto &kv : m.preset) em.preset(kv.first, kv.second);
  for (auto &kv : extra_preset) em.preset(kv.first, kv.second);
  std::string v = em.emit(node, &S0);
  std::string idx;
  if (as_store) idx = em.emit(g.n(g.stores[0].index).src[1], &S0);
  if (em.failed() || em.uses_threefry) return false;
  *code += strf("__device__ __forceinline__ %s %s(%s, int m, int n, int z, %s) {\n", as_store ? "void" : ret, name, lead_args.c_str(),
                params_decl(g).c_str());
  *code += master_decomp + flat_decl + S0.code;
  if (as_store) *code += strf("  data%d[%s] = %s;\n}\n", g.param_slot(g.stores[0].param), idx.c_str(), v.c_str());
  else *code += strf("  return %s;\n}\n", v.c_str());
  return true;
}

// Checks that running the group's kernels at the place of its last one changes nothing:
// all members lie between the first and the last in execution order, nobody else writes
// an input after the member that read it, and nobody else touches the output in between.
bool group_is_schedulable(const Sched &sc, const std::vector<int> &items, int first_item, int last_item,
                          const std::set<int> &internal, int out_slot, std::set<int> *inputs) {
  const PolySchedule *s = sc.s;
  const int first_step = sc.step_of[(size_t)first_item], last_step = sc.step_of[(size_t)last_item];
  std::set<int> uniq(items.begin(), items.end());
  if (uniq.size() != items.size()) return false;
  for (int it : items) if (sc.step_of[(size_t)it] < first_step || sc.step_of[(size_t)it] > last_step) return false;
  std::map<int, int> first_read;   // input slot -> earliest original step of a member reading it
  for (int it : items) {
    const PolyExecItem &e = s->items[it];
    for (int i = 0; i < e.n_buf_slots; i++) {
      const int sl = e.buf_slot_indices[i];
      if (internal.count(sl) || sl == out_slot) continue;
      if (sc.graphs[(size_t)it].params[(size_t)i].written) return false;
      inputs->insert(sl);
      const int st = sc.step_of[(size_t)it];
      if (!first_read.count(sl) || st < first_read[sl]) first_read[sl] = st;
    }
  }
  for (int sl : *inputs)
    for (int w : sc.writers[(size_t)sl])
      if (sc.step_of[(size_t)w] >= first_read[sl] && sc.step_of[(size_t)w] <= last_step) return false;
  for (int w : sc.writers[(size_t)out_slot]) if (w != last_item && sc.step_of[(size_t)w] >= first_step && sc.step_of[(size_t)w] <= last_step) return false;
  for (int r : sc.readers[(size_t)out_slot]) if (r != last_item && sc.step_of[(size_t)r] >= first_step && sc.step_of[(size_t)r] <= last_step) return false;
  if (internal.count(out_slot) || inputs->count(out_slot)) return false;
  return true;
}

// Every LOAD of an internal buffer in a member must have been replaced by a value
// (`exempt`: a load the template performs itself).
bool internal_loads_replaced(const Sched &sc, const Member &m, const std::set<int> &internal, int exempt) {
  const KernelGraph &g = sc.graphs[(size_t)m.item];
  for (int id = 0; id < (int)g.nodes.size(); id++) {
    if (g.n(id).op != POLY_OP_LOAD) continue;
    const int p = g.param_slot(g.n(g.n(id).src[0]).src[0]);
    if (!internal.count(sc.slot(m.item, p))) continue;
    if (!m.preset.count(id) && id != exempt) return false;
  }
  return true;
}

}  // namespace

// Does the value of `node` depend on nothing but the member's preset nodes (no other
// load, no range, no variable)?  Counts the arithmetic nodes on the way.
static bool only_depends_on_presets(const KernelGraph &g, const Member &m, int node, int *n_alu) {
  std::vector<int> st{node};
  std::set<int> seen;
  while (!st.empty()) {
    const int id = st.back(); st.pop_back();
    if (!seen.insert(id).second || m.preset.count(id)) continue;
    const KNode &k = g.n(id);
    if (k.op == POLY_OP_LOAD || k.op == POLY_OP_RANGE || k.op == POLY_OP_DEFINE_VAR || k.op == POLY_OP_REDUCE ||
        k.op == POLY_OP_SPECIAL || k.op == POLY_OP_INDEX || k.op == POLY_OP_PARAM || k.op == POLY_OP_BIND) return false;
    if (k.op != POLY_OP_CONST) (*n_alu)++;
    for (int sidx : k.src) st.push_back(sidx);
  }
  return true;
}

// A pointwise kernel whose result is a function of ONE 16-bit value has only 65536
// possible results: a table filled once by the kernel's own expression replaces the
// arithmetic (bit-identical by construction, and a gather instead of dozens of VALU
// instructions per element when the expression rounds to 16 bits after every step).
static bool make_unary_table(const Sched &sc, const Member &m, RenderedKernel::Table *t, std::string *out_type, bool *bf16_in) {
  const KernelGraph &g = sc.graphs[(size_t)m.item];
  const StoreInfo &st = g.stores[0];
  if (m.preset.size() != 1) return false;
  const KNode &in = g.n(m.preset.begin()->first);
  if (in.dt != DT_BF16 && in.dt != DT_F16) return false;
  const DT odt = g.n(st.value).dt;
  if (dt_size(odt) > 4 || odt == DT_BOOL) return false;
  int n_alu = 0;
  if (!only_depends_on_presets(g, m, st.value, &n_alu) || n_alu < 8) return false;
  Emitter em(g);
  Scope S0;
  S0.indent = 1;
  em.preset(m.preset.begin()->first, "x");
  std::string v = em.emit(st.value, &S0);
  if (em.failed() || em.uses_threefry) return false;
  t->source = std::string(hip_prelude()) +
              strf("extern \"C\" __global__ void __launch_bounds__(256) poly_lut_fill(%s* out) {\n"
                   "  const unsigned int i = blockIdx.x * 256u + threadIdx.x;\n"
                   "  const %s x = __builtin_bit_cast(%s, (unsigned short)i);\n",
                   dt_cname(odt), dt_cname(in.dt), dt_cname(in.dt)) +
              S0.code + strf("  out[i] = %s;\n}\n", v.c_str());
  t->entry = "poly_lut_fill";
  t->bytes = (size_t)65536 * (size_t)dt_size(odt);
  t->launch.grid[0] = 256;
  t->launch.block[0] = 256;
  *out_type = dt_cname(odt);
  *bf16_in = in.dt == DT_BF16;
  return true;
}

// Most values that reach such a table are of moderate size, and a gather from memory costs
// the address path a cycle for every cache line a wave instruction touches.  The matmul
// template therefore keeps the entries of 2^-24 <= |x| < 256 (bf16 inputs: 32 binades of 128
// entries per sign) in LDS when it has the room (it says how much in POLY_EP_WIN_ROOM).
// A lookup then comes in two modes: from the window alone, recording in *tmax how far
// outside the window the inputs went (mode 1), or from the table in memory (mode 0); the
// template computes a group of values in mode 1 and, if any input was outside, again in
// mode 0.
static const char *const kNoWindow = "0, (unsigned int*)0";
static const char *const kWindow = "1, &poly_tmax";
static std::string table_window_helpers(const std::vector<RenderedKernel::Table> &tables) {
  size_t bytes = 0;
  std::string src = "(const unsigned char*)0";     // nested ?: from the last table to the first
  std::vector<size_t> offs;
  for (size_t i = 0; i < tables.size(); i++) { offs.push_back(bytes); bytes += tables[i].bytes / 8; }
  for (size_t i = tables.size(); i-- > 0;)
    src = i + 1 == tables.size() ? strf("poly_win_src(poly_lut%zu, (b) - %zu)", i, offs[i])
                                 : strf("((b) < %zu ? poly_win_src(poly_lut%zu, (b) - %zu) : %s)", offs[i + 1], i, offs[i], src.c_str());
  // (the window is read through a pointer that names the LDS address space: with a plain
  // pointer the compiler picks between window and table by address and issues one flat load)
  return strf("#define POLY_LDS __attribute__((address_space(3)))\n"
              "#if defined(POLY_EP_WIN_ROOM) && POLY_EP_WIN_ROOM >= %zu\n#define POLY_EP_WIN_BYTES %zu\n"
              "#define POLY_EP_WIN(off, T) ((POLY_LDS const T*)(poly_win_raw + (off)))\n"
              "#define POLY_EP_WIN_SRC(b) %s   /* where byte b of the windows comes from */\n"
              "#else\n#define POLY_EP_WIN(off, T) ((POLY_LDS const T*)0)\n#endif\n", bytes, bytes, src.c_str()) +
         "#define POLY_WIN_FIRST (103u << 7)   /* code of 2^-24 */\n"
         "#define POLY_WIN_CODES 4096u         /* per sign */\n"
         "template <typename T> __device__ __forceinline__ const unsigned char* poly_win_src(const T* __restrict__ lut, int b) {\n"
         "  constexpr int HALF = (int)POLY_WIN_CODES * (int)sizeof(T);   // bytes per sign\n"
         "  return (const unsigned char*)lut + ((b / HALF) * 0x8000 + (int)POLY_WIN_FIRST) * (int)sizeof(T) + b % HALF;\n"
         "}\n"
         "template <typename T, typename X> __device__ __forceinline__ T poly_lut_get(const T* __restrict__ lut, POLY_LDS const T* win, const int mode, unsigned int* tmax, X x) {\n"
         "  const unsigned int u = __builtin_bit_cast(unsigned short, x);\n"
         "#ifdef POLY_EP_WIN_BYTES\n"
         "  if (mode) {\n"
         "    const unsigned int t = (u & 0x7fffu) - POLY_WIN_FIRST;\n"
         "    *tmax = t > *tmax ? t : *tmax;\n"
         "    return win[(t & (POLY_WIN_CODES - 1u)) | ((u >> 3) & POLY_WIN_CODES)];\n"
         "  }\n"
         "#endif\n"
         "  (void)win; (void)mode; (void)tmax;\n"
         "  return lut[u];\n"
         "}\n";
}

// A matmul whose result only feeds a chain of pointwise kernels (bias/activation/residual
// realised as kernels of their own): the chain becomes the matmul's epilogue.
// Set around a second match of two groups that work together: the product whose output is
// buffer `slot` leaves block maxima there (match_matmul_tail), and the attention group that
// reads its keys from that buffer uses them (match_attention).
static thread_local FusedGroup::KeyBounds g_block_maxima_hint;
static thread_local int g_key_bounds_slot = -1;

static bool match_matmul_tail(const Sched &sc, int s_item, const std::vector<char> &taken, FusedGroup *out) {
  const PolySchedule *s = sc.s;
  const KernelGraph &gS = sc.graphs[(size_t)s_item];
  MatmulMatch mS;
  if (!match_matmul(gS, &mS, nullptr)) return false;
  const StoreInfo &stS = gS.stores[0];
  std::vector<int64_t> mext(gS.ranges.size());
  for (size_t i = 0; i < gS.ranges.size(); i++) mext[i] = gS.ranges[i].extent;
  RangeMap idS;
  for (int r : stS.ranges) idS[r] = r;
  const int lsi = gS.n(gS.n(stS.index).src[1]).lin;
  Aff aS;
  if (lsi < 0 || !lin_to_aff(gS, gS.lins[(size_t)lsi], idS, &aS) || aS.c.size() != stS.ranges.size()) return false;

  std::vector<Member> members;
  { Member m; m.item = s_item; m.rm = idS; members.push_back(m); }
  std::set<int> internal;
  // One buffer on the way may have other readers than the chain (the pre-activation of a
  // layer, which its backward pass reads much later): the launch then stores it as well.
  int mid_slot = -1;
  size_t mid_member = 0;      // the member whose store it is
  int cur = sc.slot(s_item, gS.param_slot(stS.param));
  while (members.size() < 4) {
    if (!s->buf_slots[cur].is_intermediate || sc.writers[(size_t)cur].size() != 1 || sc.readers[(size_t)cur].empty()) break;
    int r = sc.readers[(size_t)cur][0];
    for (int o : sc.readers[(size_t)cur]) if (sc.step_of[(size_t)o] < sc.step_of[(size_t)r]) r = o;      // the first to read it
    const bool shared = sc.readers[(size_t)cur].size() != 1;
    if (shared && (mid_slot >= 0 || getenv("POLY_HIP_NO_STORED_MID"))) break;
    Member m;
    if (taken[(size_t)r] || !pointwise_member(sc, r, cur, aS, mext, "x", &m)) break;
    if (shared) { mid_slot = cur; mid_member = members.size() - 1; }
    else internal.insert(cur);
    members.push_back(m);
    const KernelGraph &g = sc.graphs[(size_t)r];
    cur = sc.slot(r, g.param_slot(g.stores[0].param));
  }
  if (members.size() < 2) return false;
  const int out_slot = cur, last_item = members.back().item;
  std::vector<int> items;
  for (const Member &m : members) items.push_back(m.item);
  std::set<int> inputs;
  // (for the checks below the stored buffer counts as internal: members write and read it;
  // what the others do with it is checked here)
  std::set<int> inside = internal;
  if (mid_slot >= 0) {
    inside.insert(mid_slot);
    if (mid_slot == out_slot) FA_REJECT();
    for (int o : sc.readers[(size_t)mid_slot])
      if (std::find(items.begin(), items.end(), o) == items.end() && sc.step_of[(size_t)o] <= sc.step_of[(size_t)last_item]) FA_REJECT();
  }
  if (!group_is_schedulable(sc, items, s_item, last_item, inside, out_slot, &inputs)) FA_REJECT();
  for (const Member &m : members) if (!internal_loads_replaced(sc, m, inside, -1)) FA_REJECT();

  std::vector<int> arg_slots;
  arg_slots.push_back(out_slot);
  if (mid_slot >= 0) arg_slots.push_back(mid_slot);
  for (int sl : inputs) arg_slots.push_back(sl);
  auto arg_of = [&](int sl) { return (int)(std::find(arg_slots.begin(), arg_slots.end(), sl) - arg_slots.begin()); };
  auto call_args = [&](int item) {
    const KernelGraph &g = sc.graphs[(size_t)item];
    std::string c;
    for (size_t i = 0; i < g.params.size(); i++) {
      const int sl = sc.slot(item, (int)i);
      if (i) c += ", ";
      if (internal.count(sl)) c += strf("(%s%s*)0", g.params[i].written ? "" : "const ", dt_cname(g.params[i].dt));
      else c += strf("fa%d", arg_of(sl));
    }
    return c;
  };
  MatmulEpilogue ep;
  for (size_t j = 0; j < arg_slots.size(); j++) {
    DT dt = DT_VOID;
    for (int it : items) {
      const int p = sc.param_of(it, arg_slots[j]);
      if (p >= 0) dt = sc.graphs[(size_t)it].params[(size_t)p].dt;
    }
    if (j) ep.signature += ", ";
    ep.signature += (j == 0 || arg_slots[j] == mid_slot) ? strf("%s* fa%zu", dt_cname(dt), j) : strf("const %s* __restrict__ fa%zu", dt_cname(dt), j);
    ep.bytes += (double)s->buf_slots[arg_slots[j]].nbytes;
  }
  const std::string master_decomp = matmul_decompose(mS, nullptr);
  if (!emit_member_fn(sc, members[0], master_decomp, "poly_ep_s", dt_cname(gS.n(stS.value).dt), "float acc", stS.value,
                      {{mS.red, "acc"}}, false, false, &ep.code)) FA_REJECT();
  std::string call = strf("poly_ep_s(acc, m, n, z, %s)", call_args(s_item).c_str());
  DT prev_dt = gS.n(stS.value).dt;
  std::vector<RenderedKernel::Table> tables;
  std::map<size_t, int> table_of;     // member -> table index
  std::map<size_t, std::string> lead_of, lut_arg_of, lookup_of;
  size_t win_bytes = 0;               // LDS windows of the tables so far
  bool windowed = false;              // some table takes bf16 codes: its lookups know the window
  std::string mid_call;          // the value of the stored buffer on the way, in terms of acc
  DT mid_dt = DT_VOID;
  for (size_t e = 1; e < members.size(); e++) {
    const Member &m = members[e];
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    const bool last = e + 1 == members.size();
    const std::string fn = strf("poly_ep_e%zu", e);
    if (mid_slot >= 0 && mid_member == e - 1) { mid_call = call; mid_dt = prev_dt; }
    std::string lead = strf("%s x", dt_cname(prev_dt));
    std::map<int, std::string> extra;
    RenderedKernel::Table tab;
    std::string tab_type;
    bool bf16_in = false;
    if (!getenv("POLY_HIP_NO_LUT") && make_unary_table(sc, m, &tab, &tab_type, &bf16_in)) {
      table_of[e] = (int)tables.size();
      lead += strf(", const %s* __restrict__ poly_lut, POLY_LDS const %s* poly_win, const int poly_mode, unsigned int* poly_tmax", tab_type.c_str(), tab_type.c_str());
      lut_arg_of[e] = strf(", poly_lut%zu, POLY_EP_WIN(%zu, %s), %s", tables.size(), win_bytes, tab_type.c_str(), kNoWindow);
      lookup_of[e] = bf16_in ? "poly_lut_get(poly_lut, poly_win, poly_mode, poly_tmax, x)" : "poly_lut[__builtin_bit_cast(unsigned short, x)]";
      if (bf16_in) windowed = true;
      extra[g.stores[0].value] = lookup_of[e];
      ep.signature += strf(", const %s* __restrict__ poly_lut%zu", tab_type.c_str(), tables.size());
      win_bytes += tab.bytes / 8;
      tables.push_back(tab);
    }
    lead_of[e] = lead;
    if (!emit_member_fn(sc, m, master_decomp, fn.c_str(), dt_cname(g.n(g.stores[0].value).dt), lead, g.stores[0].value, extra, false, last,
                        &ep.code)) FA_REJECT();
    call = strf("%s(%s%s, m, n, z, %s)", fn.c_str(), call.c_str(), lut_arg_of.count(e) ? lut_arg_of[e].c_str() : "", call_args(m.item).c_str());
    prev_dt = g.n(g.stores[0].value).dt;
  }
  ep.call = call;
  if (!tables.empty()) ep.code = table_window_helpers(tables) + ep.code;
  {
    // value and address of the last kernel's store, separately, when rows are contiguous
    const Member &m = members.back();
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    const StoreInfo &st = g.stores[0];
    const int li = g.n(g.n(st.index).src[1]).lin;
    Aff a;
    const MmDim &inner = mS.nd_full.back();
    bool have_aff = li >= 0 && lin_to_aff(g, g.lins[(size_t)li], m.rm, &a);
    if (!have_aff && !m.range_expr.empty()) { a = aS; have_aff = true; }   // flat kernel: it stores where the matmul would have
    const bool contiguous = have_aff && inner.cut == 1 && a.c.count(inner.ord) &&
                            a.c[inner.ord] == 1 && (mS.nd_full.size() == 1 || inner.extent % 8 == 0) &&
                            g.n(st.value).dt == g.n(st.param).dt;
    if (contiguous) {
      // `call` is f_last(f_prev(...)): the same chain with the value form of the last link
      const std::string fn = strf("poly_ep_e%zuv", members.size() - 1);
      const size_t open = call.find('(');
      std::string vcall = fn + call.substr(open);
      std::string code2;
      DT before = members.size() >= 3 ? sc.graphs[(size_t)members[members.size() - 2].item].n(sc.graphs[(size_t)members[members.size() - 2].item].stores[0].value).dt
                                      : gS.n(stS.value).dt;
      (void)before;
      const size_t le = members.size() - 1;
      std::map<int, std::string> extra;
      if (table_of.count(le)) extra[st.value] = lookup_of[le];
      bool ok = emit_member_fn(sc, m, master_decomp, fn.c_str(), dt_cname(g.n(st.value).dt), lead_of[le], st.value, extra, false, false, &code2);
      // address: the store index in master coordinates
      Emitter ea(g);
      Scope Sa;
      Sa.indent = 1;
      for (auto &kv : m.rm) { ea.bind_range(kv.first, strf("r%d", kv.second)); Sa.avail |= (uint64_t)1 << kv.first; }
      std::string flat_decl;
      for (auto &kv : m.range_expr) {
        flat_decl += strf("  const int p%d = %s;\n", kv.first, kv.second.c_str());
        ea.bind_range(kv.first, strf("p%d", kv.first));
        Sa.avail |= (uint64_t)1 << kv.first;
      }
      std::string idx = ea.emit(g.n(st.index).src[1], &Sa);
      if (ok && !ea.failed()) {
        ep.out_type = dt_cname(g.n(st.param).dt);
        code2 += strf("__device__ __forceinline__ %s* poly_ep_ptr(int m, int n, int z, %s) {\n", ep.out_type.c_str(), params_decl(g).c_str());
        code2 += master_decomp + flat_decl + Sa.code + strf("  return data%d + %s;\n}\n", g.param_slot(st.param), idx.c_str());
        ep.code += code2;
        ep.value_call = vcall;
        if (windowed) {
          ep.value_call_win = vcall;
          for (size_t at = 0; (at = ep.value_call_win.find(kNoWindow, at)) != std::string::npos; at += strlen(kWindow))
            ep.value_call_win.replace(at, strlen(kNoWindow), kWindow);
        }
        ep.ptr_call = strf("poly_ep_ptr(m, n, z, %s)", call_args(m.item).c_str());
        ep.contiguous_n = true;
        if (mid_slot >= 0) {
          // the buffer stored on the way: same positions as the output (the same affine index
          // in the product's ranges), its own element type
          const Member &mm_ = members[mid_member];
          const KernelGraph &gm = sc.graphs[(size_t)mm_.item];
          const StoreInfo &sm = gm.stores[0];
          const int lm = gm.n(gm.n(sm.index).src[1]).lin;
          Aff am;
          const bool same = mm_.range_expr.empty() && lm >= 0 && lin_to_aff(gm, gm.lins[(size_t)lm], mm_.rm, &am) && am == a &&
                            gm.n(sm.value).dt == gm.n(sm.param).dt && gm.n(sm.value).dt == mid_dt && !mid_call.empty();
          Emitter em2(gm);
          Scope Sm;
          Sm.indent = 1;
          for (auto &kv : mm_.rm) { em2.bind_range(kv.first, strf("r%d", kv.second)); Sm.avail |= (uint64_t)1 << kv.first; }
          const std::string midx = same ? em2.emit(gm.n(sm.index).src[1], &Sm) : std::string();
          if (same && !em2.failed()) {
            ep.mid_type = dt_cname(gm.n(sm.param).dt);
            ep.code += strf("__device__ __forceinline__ %s* poly_ep_mid_ptr(int m, int n, int z, %s) {\n", ep.mid_type.c_str(), params_decl(gm).c_str());
            ep.code += master_decomp + Sm.code + strf("  return data%d + %s;\n}\n", gm.param_slot(sm.param), midx.c_str());
            ep.mid_value_call = mid_call;
            ep.mid_ptr_call = strf("poly_ep_mid_ptr(m, n, z, %s)", call_args(mm_.item).c_str());
          }
        }
      }
    }
  }
  if (mid_slot >= 0 && ep.mid_value_call.empty()) FA_REJECT();
  ep.a_ptr = strf("fa%d", arg_of(sc.slot(s_item, mS.A.param)));
  ep.b_ptr = strf("fa%d", arg_of(sc.slot(s_item, mS.B.param)));
  ep.n_params = (int)arg_slots.size();
  {
    const int bs = sc.slot(s_item, mS.B.param);
    ep.b_from_hbm = !s->buf_slots[bs].is_intermediate && sc.writers[(size_t)bs].empty();
  }
  if (g_block_maxima_hint.slot == out_slot && ep.contiguous_n && mS.Z == 1) {
    // the output as the reader sees it: row-major, `pitch` columns, from element 0 of the buffer
    const FusedGroup::KeyBounds &h = g_block_maxima_hint;
    const Member &m = members.back();
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    const int li = g.n(g.n(g.stores[0].index).src[1]).lin;
    Aff a;
    bool plain = mS.M == h.rows && mS.N == h.pitch && m.range_expr.empty() && li >= 0 && lin_to_aff(g, g.lins[(size_t)li], m.rm, &a);
    auto flat = [&](int64_t mm, int64_t nn) {
      int64_t v = a.c0;
      for (auto &kv : a.c) v += kv.second * matmul_range_value(mS, kv.first, mm, nn, 0);
      return v;
    };
    for (int64_t mm = 0; plain && mm < mS.M; mm += 64)
      for (int64_t nn = h.lo; plain && nn < h.hi; nn += 64)
        plain = flat(mm, nn) == mm * h.pitch + nn && flat(mm, nn + 63) == mm * h.pitch + nn + 63 && flat(mm + 63, nn) == (mm + 63) * h.pitch + nn &&
                flat(mm + 31, nn + 17) == (mm + 31) * h.pitch + nn + 17;
    if (plain) {
      ep.block_maxima.wanted = true;
      ep.block_maxima.lo = h.lo;
      ep.block_maxima.hi = h.hi;
      ep.block_maxima.index = h.index;
      ep.block_maxima.bytes = h.bytes;
    }
  }
  if (!render_matmul(mS, ep, &out->rk)) return false;
  out->rk.tables = tables;
  std::string tail = strf(" + %zu pointwise kernel%s in the epilogue", members.size() - 1, members.size() > 2 ? "s" : "");
  if (!tables.empty()) tail += strf(" (%zu as a 16-bit lookup table)", tables.size());
  if (mid_slot >= 0) tail += ", a value on the way stored as well";
  out->rk.strategy += tail;
  for (RenderedKernel::Variant &v : out->rk.variants) v.strategy += tail;
  out->items = items;
  out->launch_item = last_item;
  out->internal_slots.assign(internal.begin(), internal.end());
  out->arg_slots = arg_slots;
  return true;
}

// ── row chains ──────────────────────────────────────────────────────────────
//
// LayerNorm and softmax reach the backend as three kernels (reference frontend:
// src/frontend.c:3585-3625 and :1131-1159): a row reduction, a second row reduction that
// reads the first one's result, and a pointwise kernel that reads both.  All three walk
// the same rows, so one wave (or one workgroup for long rows) can run the three of them
// back to back for its row: the statistics stay in registers and the row is read from
// HBM once (the second and third reads hit cache).  Each phase is generated from its
// own kernel's graph; only the row structure is matched.

struct RowPhase {
  Member m;
  bool is_map = false;
  bool keeps_row = false;           // a map whose output row only later phases read: kept in registers
  bool is_copy = false;             // a kernel that copies the result before it, one value per row: another name for it
  int red = -1, own_red_ord = -1;   // REDUCE node and its range ordinal (reduce phases)
};

// Value of `l` -- an index expression of a kernel that walks a buffer with ONE flattened
// range `flat_ord` -- in master coordinates, given that the flat position is `pos` there
// (mixed radix: non-negative coefficients).  DIV and MOD by c are exact digit operations
// when every coefficient is either a multiple of c or belongs to a part that stays below c.
static bool flat_lin_to_aff(const KernelGraph &g, const Lin &l, int flat_ord, const Aff &pos, const std::vector<int64_t> &mext, Aff *out) {
  out->c.clear();
  out->c0 = l.c0;
  for (const Term &t : l.terms) {
    const Atom &a = g.atoms[(size_t)t.atom];
    Aff v;
    if (a.kind == Atom::RANGE) {
      if (g.range_ord.at(a.node) != flat_ord) return false;
      v = pos;
    } else if (a.kind == Atom::DIV || a.kind == Atom::MOD) {
      Aff in;
      if (a.c <= 0 || !flat_lin_to_aff(g, a.inner, flat_ord, pos, mext, &in) || in.c0 < 0) return false;
      int64_t low_max = in.c0 % a.c;
      for (auto &kv : in.c) {
        if (kv.second < 0) return false;
        if (kv.second % a.c != 0) low_max += kv.second * (mext[(size_t)kv.first] - 1);
      }
      if (low_max >= a.c) return false;
      v.c0 = a.kind == Atom::DIV ? in.c0 / a.c : in.c0 % a.c;
      for (auto &kv : in.c) {
        if (kv.second % a.c == 0) { if (a.kind == Atom::DIV) v.c[kv.first] = kv.second / a.c; }
        else if (a.kind == Atom::MOD) v.c[kv.first] = kv.second;
      }
    } else {
      return false;
    }
    out->c0 += t.coef * v.c0;
    for (auto &kv : v.c) out->c[kv.first] += t.coef * kv.second;
  }
  for (auto it = out->c.begin(); it != out->c.end();) it = it->second == 0 ? out->c.erase(it) : std::next(it);
  return true;
}

// A pointwise kernel with one flattened range over a buffer of rows x R elements, as the
// last phase of a row chain: its flat position is where the row result `row_at` was stored.
static bool map_phase_flat(const Sched &sc, int item, const std::vector<int64_t> &mext, int red_master,
                           const std::vector<std::pair<int, Aff>> &results, const std::vector<char> &row_result,
                           const std::vector<std::string> &result_names, Member *m) {
  const KernelGraph &g = sc.graphs[(size_t)item];
  if (g.stores.size() != 1 || g.stores[0].ranges.size() != 1) return false;
  const int ord = g.stores[0].ranges[0];
  // the position: the store index of the latest whole-row result, which must be dense
  const Aff *pos = nullptr;
  for (size_t r = results.size(); r-- > 0;) if (row_result[r]) { pos = &results[r].second; break; }
  if (!pos || pos->c0 != 0 || !pos->c.count(red_master) || pos->c.at(red_master) != 1) return false;
  int64_t span = 1;
  for (auto &kv : pos->c) { if (kv.second <= 0) return false; span += (mext[(size_t)kv.first] - 1) * kv.second; }
  int64_t numel = 1;
  for (auto &kv : pos->c) numel *= mext[(size_t)kv.first];
  if (span != numel || g.ranges[(size_t)ord].extent != numel) return false;
  m->item = item;
  for (int id = 0; id < (int)g.nodes.size(); id++) {
    const KNode &k = g.n(id);
    if (k.op != POLY_OP_LOAD) continue;
    const KNode &ix = g.n(k.src[0]);
    const int sl = sc.slot(item, g.param_slot(ix.src[0]));
    const int lin = g.n(ix.src[1]).lin;
    for (size_t r = 0; r < results.size(); r++) {
      if (results[r].first != sl) continue;
      Aff a;
      if (ix.src.size() != 2 || k.guard >= 0 || lin < 0) return false;
      if (!flat_lin_to_aff(g, g.lins[(size_t)lin], ord, *pos, mext, &a) || !(a == results[r].second)) return false;
      m->preset[id] = result_names[r];
    }
  }
  // it must store element p at index p
  const int li = g.n(g.n(g.stores[0].index).src[1]).lin;
  Aff st;
  if (li < 0 || !flat_lin_to_aff(g, g.lins[(size_t)li], ord, *pos, mext, &st) || !(st == *pos)) return false;
  Aff base = *pos;
  base.c.erase(red_master);
  m->range_expr[ord] = aff_expr(base);   // position of the row's first element
  return true;
}

// Maps the ranges of `item` onto master ranges through the buffers it shares with the
// phases before it: results of earlier phases (read at the row they were stored at) and
// inputs that an earlier phase read as well.
static bool map_phase(const Sched &sc, int item, const std::vector<int64_t> &mext,
                      const std::vector<std::pair<int, Aff>> &ref_loads,       // (slot, index) of earlier loads
                      const std::vector<std::pair<int, Aff>> &results,         // (slot, store index) of earlier results
                      const std::vector<std::string> &result_names, Member *m) {
  const KernelGraph &g = sc.graphs[(size_t)item];
  m->item = item;
  for (int id = 0; id < (int)g.nodes.size(); id++) {
    const KNode &k = g.n(id);
    if (k.op != POLY_OP_LOAD) continue;
    const KNode &ix = g.n(k.src[0]);
    const int sl = sc.slot(item, g.param_slot(ix.src[0]));
    const int lin = g.n(ix.src[1]).lin;
    bool is_result = false;
    for (size_t r = 0; r < results.size(); r++) {
      if (results[r].first != sl) continue;
      is_result = true;
      if (ix.src.size() != 2 || k.guard >= 0 || lin < 0) return false;
      if (!derive_map(g, g.lins[(size_t)lin], results[r].second, mext, &m->rm)) return false;
      m->preset[id] = result_names[r];
    }
    if (is_result || lin < 0) continue;
    for (const auto &ref : ref_loads) {
      if (ref.first != sl) continue;
      RangeMap trial = m->rm;
      if (derive_map(g, g.lins[(size_t)lin], ref.second, mext, &trial)) { m->rm = trial; break; }
    }
  }
  return true;
}

static void collect_ref_loads(const Sched &sc, const Member &m, std::vector<std::pair<int, Aff>> *out) {
  const KernelGraph &g = sc.graphs[(size_t)m.item];
  for (int id = 0; id < (int)g.nodes.size(); id++) {
    const KNode &k = g.n(id);
    if (k.op != POLY_OP_LOAD || m.preset.count(id)) continue;
    const KNode &ix = g.n(k.src[0]);
    const int lin = g.n(ix.src[1]).lin;
    Aff a;
    if (lin < 0 || !lin_to_aff(g, g.lins[(size_t)lin], m.rm, &a)) continue;
    out->push_back({sc.slot(m.item, g.param_slot(ix.src[0])), a});
  }
}

// The buffer (slot) whose values the chain being built is to store as the bf16 values they
// are casts of, at the same element indices of the buffer read as a 16-bit one; -1: none.
// (set by find_fused_groups once it knows that the one reader of the buffer takes that)
static thread_local int g_narrow_store_slot = -1;

static bool match_row_chain_impl(const Sched &sc, int a_item, const std::vector<char> &taken, FusedGroup *out, bool allow_rows, bool allow_side = false) {
  const PolySchedule *s = sc.s;
  const KernelGraph &gA = sc.graphs[(size_t)a_item];
  auto reduce_shape = [&](const KernelGraph &g, int *red, int *ord) {
    if (g.reduces.size() != 1 || g.stores.size() != 1 || g.stores[0].gate >= 0 || !g.vars.empty()) return false;
    const KNode &R = g.n(g.reduces[0]);
    if (R.src.size() != 2 || (dt_size(R.dt) != 4 && dt_size(R.dt) != 8)) return false;
    const PolyOps op = reduce_op(R);
    if (op != POLY_OP_ADD && op != POLY_OP_MAX && op != POLY_OP_MUL) return false;
    // the REDUCE must not sit inside another loop of its own kernel
    *red = g.reduces[0];
    *ord = g.range_ord.at(R.src[1]);
    for (int r : g.stores[0].ranges) if (g.ranges[(size_t)r].extent < 0 || r == *ord) return false;
    return g.ranges[(size_t)*ord].extent >= 128;
  };
  RowPhase A;
  if (!reduce_shape(gA, &A.red, &A.own_red_ord)) return false;
  const int64_t R = gA.ranges[(size_t)A.own_red_ord].extent;
  const int red_master = A.own_red_ord;
  std::vector<int64_t> mext(gA.ranges.size());
  for (size_t i = 0; i < gA.ranges.size(); i++) mext[i] = gA.ranges[i].extent;
  A.m.item = a_item;
  for (int r : gA.stores[0].ranges) A.m.rm[r] = r;
  A.m.rm[A.own_red_ord] = A.own_red_ord;
  double rows = 1;
  for (int r : gA.stores[0].ranges) rows *= (double)gA.ranges[(size_t)r].extent;
  if (rows < 1 || rows > 2147483647.0) return false;

  auto store_aff = [&](const Member &m, Aff *a, bool whole_row = false) {
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    const int li = g.n(g.n(g.stores[0].index).src[1]).lin;
    return li >= 0 && lin_to_aff(g, g.lins[(size_t)li], m.rm, a) && (a->c.count(red_master) != 0) == whole_row;
  };
  auto out_slot_of = [&](int item) {
    const KernelGraph &g = sc.graphs[(size_t)item];
    return sc.slot(item, g.param_slot(g.stores[0].param));
  };
  std::vector<RowPhase> phases{A};
  std::vector<std::pair<int, Aff>> results, ref_loads;
  std::vector<std::string> names;
  std::set<int> internal;
  {
    Aff a;
    if (!store_aff(A.m, &a)) return false;
    results.push_back({out_slot_of(a_item), a});
    names.push_back("s1");
  }
  collect_ref_loads(sc, A.m, &ref_loads);
  // grow: the readers of the latest result decide what comes next
  const bool exports_ok = !getenv("POLY_HIP_NO_ROW_CHAIN_EXPORTS");
  std::vector<char> row_result{0};   // per result: a whole row (kept in registers) instead of one value per row
  int n_reduces = 1, n_side = 0;
  for (;;) {
    const int cur = results.back().first;
    if (!s->buf_slots[cur].is_intermediate || sc.writers[(size_t)cur].size() != 1) return false;
    internal.insert(cur);
    int next_reduce = -1, next_map = -1;
    for (int r : sc.readers[(size_t)cur]) {
      // (a reader far down the schedule -- the backward pass reading a statistic of the
      // forward pass -- does not belong to the chain: the value is stored for it, below)
      if (exports_ok && !row_result.back() && sc.step_of[(size_t)r] > sc.step_of[(size_t)a_item] + 16) continue;
      if (taken[(size_t)r]) return false;
      const KernelGraph &g = sc.graphs[(size_t)r];
      if (g.reduces.empty()) { if (next_map >= 0 && next_map != r) return false; next_map = r; }
      else { if (next_reduce >= 0) return false; next_reduce = r; }
    }
    if (next_map < 0) return false;                    // every chain ends in a pointwise kernel
    if (next_reduce >= 0 && n_reduces < 3) {
      RowPhase B;
      const KernelGraph &g = sc.graphs[(size_t)next_reduce];
      if (!reduce_shape(g, &B.red, &B.own_red_ord)) return false;
      if (!map_phase(sc, next_reduce, mext, ref_loads, results, names, &B.m)) FA_REJECT();
      if (!B.m.rm.count(B.own_red_ord) || B.m.rm[B.own_red_ord] != red_master) FA_REJECT();
      for (int r : g.stores[0].ranges) if (!B.m.rm.count(r)) FA_REJECT();
      Aff a;
      if (!store_aff(B.m, &a)) FA_REJECT();
      phases.push_back(B);
      n_reduces++;
      results.push_back({out_slot_of(next_reduce), a});
      row_result.push_back(0);
      names.push_back(strf("s%zu", results.size()));
      collect_ref_loads(sc, B.m, &ref_loads);
      continue;
    }
    if (next_reduce >= 0) return false;
    // Side reductions.  The map may read one value per row that is a copy of the result of
    // another reduction over the same rows, which reads nothing the chain makes (the
    // derivative of a row maximum counts the elements equal to it: a reduction over the
    // scores, whose row the chain holds anyway).  Such a reduction becomes a phase of its
    // own in front of the map, and the copy another name for its result.
    if (allow_side) {
      const KernelGraph &gm = sc.graphs[(size_t)next_map];
      const PolyExecItem &em_ = s->items[next_map];
      for (int p = 0; p < em_.n_buf_slots && p < (int)gm.params.size() && phases.size() < 6; p++) {
        const int sl = em_.buf_slot_indices[p];
        if (gm.params[(size_t)p].written) continue;
        bool known = false;
        for (auto &rs : results) if (rs.first == sl) known = true;
        if (known || !s->buf_slots[sl].is_intermediate || sc.writers[(size_t)sl].size() != 1 || sc.readers[(size_t)sl].size() != 1) continue;
        const int w = sc.writers[(size_t)sl][0];
        if (taken[(size_t)w] || sc.step_of[(size_t)w] <= sc.step_of[(size_t)a_item] || sc.step_of[(size_t)w] >= sc.step_of[(size_t)next_map]) continue;
        // w: out[i] = in[i], nothing else
        const KernelGraph &gw = sc.graphs[(size_t)w];
        if (!gw.reduces.empty() || gw.stores.size() != 1 || gw.stores[0].gate >= 0 || !gw.vars.empty()) continue;
        const KNode &cv = gw.n(gw.stores[0].value);
        if (cv.op != POLY_OP_LOAD || cv.guard >= 0 || cv.dt != gw.n(gw.stores[0].param).dt) continue;
        const KNode &cix = gw.n(cv.src[0]);
        if (cix.src.size() != 2) continue;
        const int l_ld = gw.n(cix.src[1]).lin, l_st = gw.n(gw.n(gw.stores[0].index).src[1]).lin;
        RangeMap idw;
        for (int r : gw.stores[0].ranges) idw[r] = r;
        Aff a_ld, a_st;
        if (l_ld < 0 || l_st < 0 || !lin_to_aff(gw, gw.lins[(size_t)l_ld], idw, &a_ld) || !lin_to_aff(gw, gw.lins[(size_t)l_st], idw, &a_st) || !(a_ld == a_st)) continue;
        const int src = sc.slot(w, gw.param_slot(cix.src[0]));
        if (!s->buf_slots[src].is_intermediate || sc.writers[(size_t)src].size() != 1 || sc.readers[(size_t)src].size() != 1 ||
            s->buf_slots[src].numel != s->buf_slots[sl].numel) continue;
        const int q = sc.writers[(size_t)src][0];
        if (taken[(size_t)q] || sc.step_of[(size_t)q] <= sc.step_of[(size_t)a_item] || sc.step_of[(size_t)q] >= sc.step_of[(size_t)w]) continue;
        RowPhase B;
        const KernelGraph &gq = sc.graphs[(size_t)q];
        if (!reduce_shape(gq, &B.red, &B.own_red_ord) || gq.ranges[(size_t)B.own_red_ord].extent != R) continue;
        // (it reads nothing that a kernel of the chain writes, earlier results aside: map_phase names those)
        bool independent = true;
        for (int pi2 = 0; pi2 < s->items[q].n_buf_slots; pi2++) {
          const int qs = s->items[q].buf_slot_indices[pi2];
          bool is_res = false;
          for (auto &rs : results) if (rs.first == qs) is_res = true;
          if (is_res && qs != results[0].first) independent = false;     // (only the first result, a value per row, may feed it)
        }
        if (!independent) continue;
        if (!map_phase(sc, q, mext, ref_loads, results, names, &B.m)) continue;
        if (!B.m.rm.count(B.own_red_ord) || B.m.rm[B.own_red_ord] != red_master) continue;
        bool mapped = true;
        for (int r : gq.stores[0].ranges) if (!B.m.rm.count(r)) mapped = false;
        Aff qa;
        if (!mapped || !store_aff(B.m, &qa)) continue;
        phases.push_back(B);
        results.push_back({src, qa});
        row_result.push_back(0);
        names.push_back(strf("s%zu", results.size()));
        internal.insert(src);
        collect_ref_loads(sc, B.m, &ref_loads);
        RowPhase Cp;
        Cp.is_copy = true;
        Cp.m.item = w;
        for (int id = 0; id < (int)gw.nodes.size(); id++)
          if (gw.n(id).op == POLY_OP_LOAD) Cp.m.preset[id] = names.back();
        phases.push_back(Cp);
        results.push_back({sl, qa});
        row_result.push_back(0);
        names.push_back(names.back());
        internal.insert(sl);
        n_side++;
      }
    }
    RowPhase C;
    C.is_map = true;
    const KernelGraph &g = sc.graphs[(size_t)next_map];
    if (!g.reduces.empty() || g.stores.size() != 1 || g.stores[0].gate >= 0 || !g.vars.empty()) return false;
    if (!map_phase(sc, next_map, mext, ref_loads, results, names, &C.m)) {
      // one flattened range instead of (rows, position in the row)
      C.m = Member();
      if (!map_phase_flat(sc, next_map, mext, red_master, results, row_result, names, &C.m)) FA_REJECT();
    } else {
      std::set<int> covered;
      for (int r : g.stores[0].ranges) {
        if (!C.m.rm.count(r)) FA_REJECT();
        covered.insert(C.m.rm[r]);
      }
      if (covered.size() != gA.stores[0].ranges.size() + 1 || !covered.count(red_master)) FA_REJECT();
    }
    // A map whose output is an intermediate that one more row reduction (and the map after
    // it) reads -- softmax as max, exp, sum, divide; LayerNorm as mean, centre, variance,
    // scale -- keeps its row in registers and the chain goes on.
    const int c_out = out_slot_of(next_map);
    Aff ca;
    bool row_goes_on = allow_rows && C.m.range_expr.empty() && n_reduces < 3 && !row_result.back() && s->buf_slots[c_out].is_intermediate &&
                       sc.writers[(size_t)c_out].size() == 1 && store_aff(C.m, &ca, true);
    if (row_goes_on) {
      int rr = 0, rm = 0;
      for (int r : sc.readers[(size_t)c_out]) {
        if (taken[(size_t)r]) row_goes_on = false;
        else if (sc.graphs[(size_t)r].reduces.empty()) rm++;
        else {
          rr++;
          // (a reduction of another shape -- a matmul over the rows -- ends the chain here)
          int red, ord;
          if (!reduce_shape(sc.graphs[(size_t)r], &red, &ord) || sc.graphs[(size_t)r].ranges[(size_t)ord].extent != R) row_goes_on = false;
        }
      }
      if (rr != 1 || rm > 1) row_goes_on = false;
    }
    if (row_goes_on) {
      C.keeps_row = true;
      phases.push_back(C);
      results.push_back({c_out, ca});
      row_result.push_back(1);
      names.push_back(strf("t%zu[it].v[u]", results.size()));
      collect_ref_loads(sc, C.m, &ref_loads);
      continue;
    }
    if (allow_side && n_side == 0) return false;      // (this attempt is for chains with side reductions; the plain ones follow)
    phases.push_back(C);
    break;
  }
  // A result is read inside the group only, or it is one value per row that kernels
  // behind the whole group read as well (the row maximum and the sum of a softmax, the mean
  // and the variance of a LayerNorm in a training step, which the backward pass reads): the
  // phase that makes such a value stores it, too.
  std::vector<int> items;
  for (const RowPhase &p : phases) items.push_back(p.m.item);
  std::set<int> exported;
  for (size_t ri = 0; ri < results.size(); ri++)
    for (int r : sc.readers[(size_t)results[ri].first]) {
      if (std::find(items.begin(), items.end(), r) != items.end()) continue;
      if (!exports_ok || row_result[ri] || phases[ri].is_map || sc.step_of[(size_t)r] <= sc.step_of[(size_t)items.back()]) FA_REJECT();
      exported.insert(results[ri].first);
    }
  const int last_item = items.back();
  const int out_slot = out_slot_of(last_item);
  std::set<int> inputs;
  if (!group_is_schedulable(sc, items, a_item, last_item, internal, out_slot, &inputs)) FA_REJECT();
  for (const RowPhase &p : phases) if (!internal_loads_replaced(sc, p.m, internal, -1)) FA_REJECT();
  for (int sl : exported) internal.erase(sl);      // they have memory, and the kernel gets them as arguments

  // ── code generation ────────────────────────────────────────────────────
  int G = (R >= 4096 || (rows < 2048 && R >= 1024)) ? 256 : 64;
  // Rows of 16-bit elements that 64 lanes x 8 elements do not divide but 32 x 8 do (768 =
  // 3 x 32 x 8): half a wave per row, two rows to a wave.  Every load is 16 bytes, a wave
  // has twice the bytes in flight and the launch half the waves.  (Whatever the number of
  // rows: the lanes a row is dealt to decide the order of its sums, and a plan for one
  // sequence must round as the plan for eight does.)
  if (G == 64 && R % 256 == 0 && R % 512 != 0 && R <= 4096 && !getenv("POLY_HIP_NO_HALF_WAVE_ROWS")) {
    int maxsz = 1;
    for (int it : items)
      for (const auto &p : sc.graphs[(size_t)it].params)
        if ((double)s->buf_slots[sc.slot(it, (int)(&p - &sc.graphs[(size_t)it].params[0]))].numel >= rows * (double)R) maxsz = std::max(maxsz, dt_size(p.dt));
    if (maxsz == 2) G = 32;
  }
  std::vector<int> arg_slots;
  arg_slots.push_back(out_slot);
  for (int sl : inputs) arg_slots.push_back(sl);
  for (int sl : exported) arg_slots.push_back(sl);
  auto arg_of = [&](int sl) { return (int)(std::find(arg_slots.begin(), arg_slots.end(), sl) - arg_slots.begin()); };
  auto call_args = [&](int item) {
    const KernelGraph &g = sc.graphs[(size_t)item];
    std::string c;
    for (size_t i = 0; i < g.params.size(); i++) {
      const int sl = sc.slot(item, (int)i);
      if (i) c += ", ";
      if (internal.count(sl)) c += strf("(%s%s*)0", g.params[i].written ? "" : "const ", dt_cname(g.params[i].dt));
      else c += strf("fa%d", arg_of(sl));
    }
    return c;
  };
  std::string sig;
  double bytes = 0, bytes_written = 0;
  for (size_t j = 0; j < arg_slots.size(); j++) {
    DT dt = DT_VOID;
    for (int it : items) {
      const int p = sc.param_of(it, arg_slots[j]);
      if (p >= 0) dt = sc.graphs[(size_t)it].params[(size_t)p].dt;
    }
    if (j) sig += ", ";
    sig += j == 0 || exported.count(arg_slots[j]) ? strf("%s* fa%zu", dt_cname(dt), j) : strf("const %s* __restrict__ fa%zu", dt_cname(dt), j);
    bytes += (double)s->buf_slots[arg_slots[j]].nbytes;
    if (j == 0 || exported.count(arg_slots[j])) bytes_written += (double)s->buf_slots[arg_slots[j]].nbytes;
  }
  // master row decomposition: fastest row range = smallest stride in the first result
  std::string row_decomp;
  {
    std::vector<std::pair<int64_t, int>> keyed;
    for (int r : gA.stores[0].ranges) {
      auto it = results[0].second.c.find(r);
      keyed.push_back({it == results[0].second.c.end() ? ((int64_t)1 << 50) : std::abs(it->second), r});
    }
    std::sort(keyed.begin(), keyed.end());
    row_decomp += "  long long t_ = row;\n";
    for (size_t i = 0; i < keyed.size(); i++) {
      const int ord = keyed[i].second;
      const int64_t e = gA.ranges[(size_t)ord].extent;
      if (i + 1 == keyed.size()) row_decomp += strf("  const int r%d = (int)t_;\n", ord);
      else row_decomp += strf("  const int r%d = (int)(t_ %% %lld); t_ /= %lld;\n", ord, (long long)e, (long long)e);
    }
  }
  std::string code, calls, strat;
  std::string lead;   // results so far, as parameters
  std::string lead_call;
  // Short rows handled by one wave stay in registers between the phases: a vector load
  // that an earlier phase made from the same buffer at the same index is kept instead of
  // being repeated (the row is then read from memory once, not once per phase).
  struct RowCache { std::string key, type; int nit; int V = 0; std::string what; };    // what: the key without the vector width
  std::vector<RowCache> cache;
  int n_cached_uses = 0, n_exported = 0;
  bool narrow_stored = false;
  int n_walked_phases = 0;          // phases that walk their row from memory in a loop (nothing kept for the next one)
  int row_V = 0, row_nit = 0;       // vector width and step count of the rows kept between phases
  std::string row_decls;             // their declarations in the kernel body
  for (size_t pi = 0; pi < phases.size(); pi++) {
    const RowPhase &ph = phases[pi];
    if (ph.is_copy) continue;        // (its value is the result before it, under the same name)
    const KernelGraph &g = sc.graphs[(size_t)ph.m.item];
    Emitter em(g);
    em.recip_div16 = true;
    Scope S0;                        // row-invariant values
    S0.indent = 1;
    int own_f = -1;                  // this kernel's range that walks along the row
    for (auto &kv : ph.m.rm) {
      if (kv.second == red_master) { own_f = kv.first; continue; }
      em.bind_range(kv.first, strf("r%d", kv.second));
      S0.avail |= (uint64_t)1 << kv.first;
    }
    std::string flat_base;           // flat phase: position of the row's first element
    for (auto &kv : ph.m.range_expr) { own_f = kv.first; flat_base = kv.second; }
    if (own_f < 0) FA_REJECT();
    for (auto &kv : ph.m.preset) {
      em.preset(kv.first, kv.second);
      // (the results of earlier phases, s<n>, are one value per row)
      if (kv.second.size() > 1 && kv.second[0] == 's' && kv.second.find_first_not_of("0123456789", 1) == std::string::npos) em.preset_shared(kv.first);
    }
    const std::vector<int> roots{ph.is_map ? g.stores[0].value : g.n(ph.red).src[0]};
    // vector width along the row
    int V = 1;
    bool ragged = false;             // vectors up to the last full one, then R mod V lanes take one element each
    {
      int maxsz = 1;
      std::vector<char> mark(g.nodes.size(), 0);
      mark_reachable(g, roots[0], mark);
      for (int i = 0; i < (int)g.nodes.size(); i++)
        if (mark[(size_t)i] && g.n(i).op == POLY_OP_LOAD && !ph.m.preset.count(i) && (g.n(i).deps & ((uint64_t)1 << own_f)))
          maxsz = std::max(maxsz, dt_size(g.n(i).dt));
      if (ph.is_map) maxsz = std::max(maxsz, dt_size(g.n(g.stores[0].param).dt));
      V = std::max(1, 16 / maxsz);
      bool reads_row = false;
      for (auto &kv : ph.m.preset) if (kv.second.find("[it]") != std::string::npos) reads_row = true;
      if (reads_row) V = row_V;   // positions must line up with the phase that made the row
      while (V > 1 && (R % V != 0 || R < (int64_t)G * V)) V /= 2;
      // a reduction whose row an earlier phase keeps in narrower vectors walks it that way
      // too, and takes the kept registers instead of reading the row again
      if (!reads_row && !ph.is_map && !ph.keeps_row && V > 1) {
        int kept = 0;
        for (int i = 0; i < (int)g.nodes.size() && !kept; i++) {
          if (!mark[(size_t)i] || g.n(i).op != POLY_OP_LOAD || ph.m.preset.count(i) || !(g.n(i).deps & ((uint64_t)1 << own_f))) continue;
          const KNode &ix = g.n(g.n(i).src[0]);
          Aff a;
          if (ix.src.size() != 2 || g.n(ix.src[1]).lin < 0 || !lin_to_aff(g, g.lins[(size_t)g.n(ix.src[1]).lin], ph.m.rm, &a)) continue;
          std::string what = strf("%d:%d:%lld", sc.slot(ph.m.item, g.param_slot(ix.src[0])), (int)g.n(i).dt, (long long)a.c0);
          for (auto &kv : a.c) what += strf(",%d*%lld", kv.first, (long long)kv.second);
          for (const RowCache &c : cache) if (c.what == what && c.V > 1 && c.V < V) kept = c.V;
        }
        if (kept) V = kept;
      }
      // a row that half the vector width deals out evenly (768 = 3 x 64 x 4, against one
      // and a half steps of 64 x 8) is walked that way: no step with half the lanes idle
      // (LayerNorm of 8192 x 768: 12.3 -> 11.2 us)
      if (!reads_row && V >= 8 && G == 64 && R % ((int64_t)G * V) != 0 && R % ((int64_t)G * V / 2) == 0) V /= 2;
      // long rows of an extent that is no multiple of the vector width (a vocabulary of
      // 50257): vector accesses at element alignment and a scalar tail
      if (V == 1 && !reads_row && !ph.keeps_row && !getenv("POLY_HIP_NO_RAGGED_VEC")) {
        int vr = std::max(1, 16 / maxsz);
        while (vr > 1 && R < (int64_t)G * vr * 16) vr /= 2;
        if (vr > 1) { V = vr; ragged = true; }
      }
      if (reads_row && V != row_V) FA_REJECT();
      if (ph.is_map) {
        const int li = g.n(g.n(g.stores[0].index).src[1]).lin;
        while (V > 1 && (li < 0 || !lin_vec_ok(g, g.lins[(size_t)li], own_f, V, ragged) ||
                         dt_size(g.n(g.stores[0].value).dt) != dt_size(g.n(g.stores[0].param).dt))) V /= 2;
      }
      if (V == 1) ragged = false;
    }
    const int64_t R_main = ragged ? R - R % V : R;
    const std::string fv = strf("f%d", own_f);           // C name of the position along the row
    Scope L;                          // loop body, one vector per step
    L.parent = &S0;
    L.avail = S0.avail;
    L.indent = 2;
    std::vector<int> pres;
    const int nit = (int)((R + (int64_t)G * V - 1) / ((int64_t)G * V));
    // iterations as an unrolled loop over `it` (what is kept between phases is indexed by it)
    const bool unrolled = (G <= 64 && nit <= 4) || (G == 256 && nit <= 8);
    if (!unrolled) n_walked_phases++;
    {
      bool reads_row = false;
      for (auto &kv : ph.m.preset) if (kv.second.find("[it]") != std::string::npos) reads_row = true;
      if ((reads_row || ph.keeps_row) && (!unrolled || V <= 1)) FA_REJECT();
      if (reads_row && nit != row_nit) FA_REJECT();
      if (ph.keeps_row) {
        if (row_V && (row_V != V || row_nit != nit)) FA_REJECT();
        row_V = V;
        row_nit = nit;
      }
    }
    const std::function<std::string(int, const std::string &)> keep = [&](int node, const std::string &ld) -> std::string {
      const KNode &ix = g.n(g.n(node).src[0]);
      Aff a;
      if (!lin_to_aff(g, g.lins[(size_t)g.n(ix.src[1]).lin], ph.m.rm, &a)) return ld;
      std::string key = strf("%d:%d:%d:%lld", sc.slot(ph.m.item, g.param_slot(ix.src[0])), V, (int)g.n(node).dt, (long long)a.c0);
      for (auto &kv : a.c) key += strf(",%d*%lld", kv.first, (long long)kv.second);
      for (size_t ci = 0; ci < cache.size(); ci++)
        if (cache[ci].key == key && cache[ci].nit == nit) { n_cached_uses++; return strf("c%zu[it]", ci); }
      if (pi + 1 == phases.size()) return ld;   // nobody comes after the last phase
      {
        std::string what = strf("%d:%d:%lld", sc.slot(ph.m.item, g.param_slot(ix.src[0])), (int)g.n(node).dt, (long long)a.c0);
        for (auto &kv : a.c) what += strf(",%d*%lld", kv.first, (long long)kv.second);
        cache.push_back({key, strf("poly_vec<%s,%d>", dt_cname(g.n(node).dt), V), nit, V, what});
      }
      return strf("(c%zu[it] = %s)", cache.size() - 1, ld.c_str());
    };
    if (ragged && unrolled) FA_REJECT();
    if (V > 1) pres = hoist_vector_loads(g, em, roots, own_f, V, fv + "_0", &L, unrolled ? &keep : nullptr, ragged);
    // the row loop: positions fv_0 = lane * V, + G * V, ...
    // q: position in the row; the phase's own variable starts there (or, for a flat phase,
    // at the row's first element plus q)
    const std::string start = flat_base.empty() ? "q_0" : flat_base + " + q_0";
    const std::string loop_open = unrolled
        ? strf("#pragma unroll\n  for (int it = 0; it < %d; it++) {\n  const int q_0 = lane * %d + it * %d;\n  if (q_0 < %lld) {\n  const int %s_0 = %s;\n", nit, V, G * V,
               (long long)R, fv.c_str(), start.c_str())
        : strf("  for (int q_0 = lane * %d; q_0 < %lld; q_0 += %d) {\n  const int %s_0 = %s;\n", V, (long long)R_main, G * V, fv.c_str(), start.c_str());
    const std::string loop_close = unrolled ? "  }\n  }\n" : "  }\n";
    // the scalar tail of a ragged row: the phase's value emitted once more for one element
    auto ragged_tail = [&](int root, const std::function<std::string(Scope *, const std::string &)> &use) {
      for (int n : pres) em.clear_preset(n);
      pres.clear();
      Scope Tl;
      Tl.parent = &S0;
      Tl.avail = S0.avail | ((uint64_t)1 << own_f);
      Tl.indent = 2;
      em.bind_range(own_f, fv);
      const std::string v = em.emit(root, &Tl);
      const std::string last = use(&Tl, v);
      std::string t = S0.code;       // (row-invariant values the vector form did not need)
      S0.code.clear();
      t += strf("  if (lane < %lld) {\n    const int %s = %s%lld + lane;\n", (long long)(R % V), fv.c_str(), flat_base.empty() ? "" : (flat_base + " + ").c_str(),
                (long long)R_main);
      t += Tl.code + last + "  }\n";
      return t;
    };
    Scope U;                          // one element
    U.parent = &L;
    U.avail = L.avail | ((uint64_t)1 << own_f);
    U.indent = 3;
    em.bind_range(own_f, fv);
    std::string fn = strf("poly_row_p%zu", pi);
    std::string ret = "void", result_expr, tail;
    std::string loop;
    if (!ph.is_map) {
      const KNode &Rn = g.n(ph.red);
      const PolyOps op = reduce_op(Rn);
      std::string v = em.emit(Rn.src[0], &U);
      U.code += strf("      acc = %s;\n", Emitter::reduce_combine(op, Rn.dt, "acc", v).c_str());
      loop += strf("  %s acc = %s;\n", dt_cname(Rn.dt), Emitter::reduce_identity(op, Rn.dt).c_str());
      loop += S0.code;
      S0.code.clear();
      loop += loop_open;
      loop += L.code;
      loop += strf("#pragma unroll\n    for (int u = 0; u < %d; u++) {\n      const int %s = %s_0 + u;\n", V, fv.c_str(), fv.c_str());
      loop += U.code + "    }\n" + loop_close;
      if (ragged)
        loop += ragged_tail(Rn.src[0], [&](Scope *, const std::string &v2) { return strf("    acc = %s;\n", Emitter::reduce_combine(op, Rn.dt, "acc", v2).c_str()); });
      loop += strf("  acc = %s;\n", wave_reduce_call(op, Rn.dt, "acc", G == 32 ? 32 : 64).c_str());
      if (G == 256) {
        loop += strf("  __shared__ %s red[4];\n  __syncthreads();\n  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;\n  __syncthreads();\n",
                     dt_cname(Rn.dt));
        std::string e = "red[0]";
        for (int w = 1; w < 4; w++) e = Emitter::reduce_combine(op, Rn.dt, e, strf("red[%d]", w));
        loop += strf("  acc = %s;\n", e.c_str());
      }
      for (int n : pres) em.clear_preset(n);
      em.preset(ph.red, "acc");
      result_expr = em.emit(g.stores[0].value, &S0);
      ret = dt_cname(g.n(g.stores[0].value).dt);
      if (exported.count(results[pi].first)) {
        // (phase pi makes result pi: every phase before the last map makes one)
        const StoreInfo &st = g.stores[0];
        const std::string idx = em.emit(g.n(st.index).src[1], &S0);
        tail = S0.code + strf("  const %s res_ = %s;\n  if (lane == 0) data%d[%s] = res_;\n  return res_;\n", ret.c_str(), result_expr.c_str(),
                              g.param_slot(st.param), idx.c_str());
        n_exported++;
      } else {
        tail = S0.code + strf("  return %s;\n", result_expr.c_str());
      }
    } else {
      const StoreInfo &st = g.stores[0];
      const int li = g.n(g.n(st.index).src[1]).lin;
      const int p = g.param_slot(st.param);
      // (a buffer whose reader takes bf16 values: what the cast to fp32 is applied to goes
      // there, into the buffer read as a 16-bit one)
      const bool narrow = !ph.keeps_row && g_narrow_store_slot >= 0 && sc.slot(ph.m.item, p) == g_narrow_store_slot;
      if (narrow) {
        const KNode &cv = g.n(st.value);
        if (pi + 1 != phases.size() || cv.op != POLY_OP_CAST || cv.dt != DT_F32 || cv.src.size() != 1 || g.n(cv.src[0]).dt != DT_BF16 ||
            g.n(st.param).dt != DT_F32)
          FA_REJECT();
        narrow_stored = true;
      }
      std::string v = em.emit(narrow ? g.n(st.value).src[0] : st.value, &U);
      const char *odt = narrow ? "__bf16" : dt_cname(g.n(st.param).dt);
      const std::string dst = narrow ? strf("((__bf16*)data%d)", p) : strf("data%d", p);
      if (ph.keeps_row) {
        U.code += strf("      %s = %s;\n", names[pi].c_str(), v.c_str());
      } else if (V > 1) {
        U.code += strf("      out.v[u] = %s;\n", v.c_str());
      } else {
        std::string idx = em.emit(g.n(st.index).src[1], &U);
        U.code += strf("      %s[%s] = %s;\n", dst.c_str(), idx.c_str(), v.c_str());
      }
      std::string addr;
      if (V > 1) { em.bind_range(own_f, fv + "_0"); addr = em.emit_lin(g.lins[(size_t)li], &L); em.bind_range(own_f, fv); }
      loop += S0.code;
      S0.code.clear();
      loop += loop_open;
      loop += L.code;
      if (V > 1 && !ph.keeps_row) loop += strf("    poly_vec<%s,%d> out;\n", odt, V);
      loop += strf("#pragma unroll\n    for (int u = 0; u < %d; u++) {\n      const int %s = %s_0 + u;\n", V, fv.c_str(), fv.c_str());
      loop += U.code + "    }\n";
      if (V > 1 && !ph.keeps_row) loop += strf("    poly_vstore<%s,%d>(%s + %s, out);\n", odt, V, dst.c_str(), addr.c_str());
      loop += loop_close;
      if (ragged)
        loop += ragged_tail(narrow ? g.n(st.value).src[0] : st.value, [&](Scope *tl, const std::string &v2) {
          const std::string idx = em.emit(g.n(st.index).src[1], tl);
          return strf("    %s[%s] = %s;\n", dst.c_str(), idx.c_str(), v2.c_str());
        });
    }
    if (em.failed() || em.uses_threefry) FA_REJECT();
    std::string cache_params, cache_args;
    for (size_t ci = 0; ci < cache.size(); ci++) {
      cache_params += strf(", %s (&c%zu)[%d]", cache[ci].type.c_str(), ci, cache[ci].nit);
      cache_args += strf(", c%zu", ci);
    }
    code += strf("__device__ __forceinline__ %s %s(const long long row, const int lane%s%s, %s) {\n", ret.c_str(), fn.c_str(), lead.c_str(),
                 cache_params.c_str(), params_decl(g).c_str());
    code += row_decomp + loop + tail + "}\n";
    if (ph.keeps_row) {
      // the row it makes: an array the later phases receive by reference
      const std::string base = names[pi].substr(0, names[pi].find('['));
      const std::string type = strf("poly_vec<%s,%d>", dt_cname(g.n(g.stores[0].value).dt), V);
      row_decls += strf("    %s %s[%d];\n", type.c_str(), base.c_str(), nit);
      const std::string param = strf(", %s (&%s)[%d]", type.c_str(), base.c_str(), nit);
      // this phase's own signature needs it too: it was built above without it
      const size_t sig_at = code.rfind(strf("%s(const long long row, const int lane%s", fn.c_str(), lead.c_str()));
      if (sig_at == std::string::npos) FA_REJECT();
      code.insert(sig_at + strf("%s(const long long row, const int lane%s", fn.c_str(), lead.c_str()).size(), param);
      calls += strf("    %s(row, lane%s, %s%s, %s);\n", fn.c_str(), lead_call.c_str(), base.c_str(), cache_args.c_str(), call_args(ph.m.item).c_str());
      lead += param;
      lead_call += ", " + base;
    } else if (!ph.is_map) {
      calls += strf("    const %s %s = %s(row, lane%s%s, %s);\n", ret.c_str(), names[pi].c_str(), fn.c_str(), lead_call.c_str(),
                    cache_args.c_str(), call_args(ph.m.item).c_str());
      lead += strf(", const %s %s", ret.c_str(), names[pi].c_str());
      lead_call += ", " + names[pi];
    } else {
      calls += strf("    %s(row, lane%s%s, %s);\n", fn.c_str(), lead_call.c_str(), cache_args.c_str(), call_args(ph.m.item).c_str());
    }
    strat += strf("%s%s vec%d%s", pi ? ", " : "", ph.is_map ? "map" : "reduce", V, ragged ? " unaligned + tail" : "");
  }
  // (threads: the workgroup's size; a row per wave or half wave means threads / G rows per workgroup)
  auto body_for = [&](int threads) {
    std::string b = strf("extern \"C\" __global__ void __launch_bounds__(%d) poly_k(%s) {\n", threads, sig.c_str());
    if (G == 64) {
      b += strf("  const int lane = threadIdx.x & 63;\n  const long long row = (long long)blockIdx.x * %d + (threadIdx.x >> 6);\n", threads / 64);
      b += strf("  if (row < %lldll) {\n", (long long)rows);
    } else if (G == 32) {
      b += strf("  const int lane = threadIdx.x & 31;\n  const long long row = (long long)blockIdx.x * %d + (threadIdx.x >> 5);\n", threads / 32);
      b += strf("  if (row < %lldll) {\n", (long long)rows);
    } else {
      b += "  const int lane = threadIdx.x;\n  const long long row = blockIdx.x;\n  {\n";
    }
    for (size_t ci = 0; ci < cache.size(); ci++) b += strf("    %s c%zu[%d];\n", cache[ci].type.c_str(), ci, cache[ci].nit);
    b += row_decls;
    b += calls + "  }\n}\n";
    return b;
  };
  const std::string body = body_for(256);

  out->items = items;
  out->launch_item = last_item;
  out->internal_slots.assign(internal.begin(), internal.end());
  out->arg_slots = arg_slots;
  RenderedKernel &rk = out->rk;
  rk = RenderedKernel();
  rk.source = std::string(hip_prelude()) + code + body;
  rk.entry = "poly_k";
  rk.launch.grid[0] = (unsigned)(G == 256 ? rows : G == 32 ? std::ceil(rows / 8) : std::ceil(rows / 4));
  rk.launch.block[0] = 256;
  rk.klass = KernelClass::ROW_REDUCE;
  rk.strategy = strf("row chain of %zu kernels (%s) G=%d R=%lld rows=%.0f", phases.size(), strat.c_str(), G, (long long)R, rows);
  if (n_cached_uses) rk.strategy += strf(", %d row loads kept in registers", n_cached_uses);
  if (row_V) rk.strategy += ", intermediate rows kept in registers";
  if (n_exported) rk.strategy += strf(", %d row values stored for later kernels", n_exported);
  if (g_narrow_store_slot >= 0 && !narrow_stored) FA_REJECT();
  if (narrow_stored) {
    rk.strategy += ", result stored as the bf16 values that its fp32 values are casts of";
  }
  out->row_chain_from = a_item;
  {
    const KernelGraph &gl = sc.graphs[(size_t)phases.back().m.item];
    out->row_chain_stores = phases.back().is_map ? sc.slot(phases.back().m.item, gl.param_slot(gl.stores[0].param)) : -1;
  }
  rk.n_params = (int)arg_slots.size();
  rk.bytes = bytes - (narrow_stored ? (double)s->buf_slots[g_narrow_store_slot].nbytes / 2 : 0.0);      // (a buffer stored as bf16 values is half written)
  rk.rereads_inputs = n_walked_phases > 1;
  rk.bytes_written = bytes_written - (narrow_stored ? (double)s->buf_slots[g_narrow_store_slot].nbytes / 2 : 0.0);
  // Candidates for on-device tuning: the same rows on smaller workgroups (fewer rows to a
  // workgroup, more workgroups).  Which lanes add which elements of a row, and in what
  // order, stays as it is -- the width of a row's group of lanes and of its loads would
  // change that, so they are not candidates.
  if (matmul_tuning_enabled() && G != 256) {
    rk.variants.push_back({"default", rk.source, rk.strategy, rk.launch});
    for (int threads : {128, 64}) {
      LaunchSpec ls = rk.launch;
      ls.grid[0] = (unsigned)std::ceil(rows / (double)(threads / G));
      ls.block[0] = (unsigned)threads;
      rk.variants.push_back({strf("rows_wg%d", threads), std::string(hip_prelude()) + code + body_for(threads),
                             rk.strategy + strf(", workgroups of %d threads", threads), ls});
    }
  }
  return true;
}

static bool match_row_chain(const Sched &sc, int a_item, const std::vector<char> &taken, FusedGroup *out) {
  fa_item = a_item;
  // first with side reductions, then with maps in the middle of the chain (their rows kept in
  // registers), then the plain form
  if (!getenv("POLY_HIP_NO_SIDE_REDUCE") && match_row_chain_impl(sc, a_item, taken, out, true, true)) return true;
  return match_row_chain_impl(sc, a_item, taken, out, true) || match_row_chain_impl(sc, a_item, taken, out, false);
}

// A kernel that only moves data: out[store index] = in[load index], both affine in the
// kernel's ranges, the store covering its buffer densely (row-major in some order of the
// ranges).  Then element p of the output is element src(p) of the input, with
// src(p) = c0 + sum_i ((p / stride_i) % extent_i) * coef_i.
struct CopyMap {
  int item = -1, src_slot = -1;
  int64_t c0 = 0;
  struct Digit { int64_t stride, extent, coef; };
  std::vector<Digit> digits;   // by decreasing stride
};

static bool match_copy(const Sched &sc, int item, CopyMap *cm) {
  const KernelGraph &g = sc.graphs[(size_t)item];
  if (!g.reduces.empty() || g.stores.size() != 1 || g.stores[0].gate >= 0 || !g.vars.empty()) return false;
  const StoreInfo &st = g.stores[0];
  const KNode &v = g.n(st.value);
  if (v.op != POLY_OP_LOAD || v.guard >= 0 || v.dt != g.n(st.param).dt) return false;
  const KNode &ix = g.n(v.src[0]);
  if (ix.src.size() != 2) return false;
  const int ll = g.n(ix.src[1]).lin, ls = g.n(g.n(st.index).src[1]).lin;
  if (ll < 0 || ls < 0) return false;
  RangeMap id;
  for (int r : st.ranges) id[r] = r;
  Aff as, al;
  if (!lin_to_aff(g, g.lins[(size_t)ls], id, &as) || !lin_to_aff(g, g.lins[(size_t)ll], id, &al)) return false;
  if (as.c0 != 0 || as.c.size() != st.ranges.size()) return false;
  std::vector<CopyMap::Digit> d;
  for (auto &kv : as.c) {
    if (kv.second <= 0) return false;
    auto it = al.c.find(kv.first);
    d.push_back({kv.second, g.ranges[(size_t)kv.first].extent, it == al.c.end() ? 0 : it->second});
  }
  std::sort(d.begin(), d.end(), [](const CopyMap::Digit &a, const CopyMap::Digit &b) { return a.stride > b.stride; });
  int64_t expect = 1;
  for (size_t i = d.size(); i-- > 0;) {
    if (d[i].extent <= 0 || d[i].stride != expect) return false;
    expect *= d[i].extent;
  }
  const int out_slot = sc.slot(item, g.param_slot(st.param));
  if (expect != sc.s->buf_slots[out_slot].numel) return false;
  cm->item = item;
  cm->src_slot = sc.slot(item, g.param_slot(ix.src[0]));
  cm->c0 = al.c0;
  cm->digits = d;
  return cm->src_slot != out_slot;
}

// Tries to grow an attention group from the matmul at schedule item `s_item`.
// Which (block of 128 queries, z) each workgroup of the attention kernel takes.  Under a
// causal mask block b has b + 1 times the work of block 0, every workgroup is resident from
// the start (three per CU) and the hardware puts workgroups j, j + 32, j + 64 of an XCD on
// the same CU (ids go round the 8 XCDs first), so the order decides how evenly the CUs are
// loaded: heaviest first, and within each later round of 32 the heaviest goes to the CU
// that has the least so far.  For 8 blocks x 12 z per XCD the CUs then carry 13 or 14 units
// each instead of 10 to 17.  (Without such a mask all workgroups weigh the same and any
// order does.)  Emitted as a table indexed by the workgroup's number within its XCD.
static std::string attention_order(int64_t MB, int64_t Z) {
  if (measurement_env("POLY_HIP_FA_PLAIN_ORDER") || Z % 8 != 0 || MB < 2) return "";
  const int64_t ZX = Z / 8, n = MB * ZX;
  if (n > 8192) return "";
  constexpr int CUS = 32;
  std::vector<int> items((size_t)n);                 // mb * ZX + z', heaviest first
  for (int64_t i = 0; i < n; i++) items[(size_t)i] = (int)((MB - 1 - i / ZX) * ZX + i % ZX);
  std::vector<int> order((size_t)n);
  std::vector<int64_t> load(CUS, 0);
  for (int64_t r0 = 0; r0 < n; r0 += CUS) {
    const int k = (int)std::min<int64_t>(CUS, n - r0);
    std::vector<int> cu((size_t)k);
    for (int c = 0; c < k; c++) cu[(size_t)c] = c;
    std::stable_sort(cu.begin(), cu.end(), [&](int a, int b) { return load[(size_t)a] < load[(size_t)b]; });
    for (int i = 0; i < k; i++) {
      const int item = items[(size_t)(r0 + i)];
      order[(size_t)(r0 + cu[(size_t)i])] = item;
      load[(size_t)cu[(size_t)i]] += item / ZX + 1;
    }
  }
  std::string t = strf("#define POLY_FA_ORDER 1\n__constant__ unsigned short poly_fa_order[%lld] = {", (long long)n);
  for (int64_t i = 0; i < n; i++) t += strf("%s%d", i ? "," : "", order[(size_t)i]);
  return t + "};\n";
}

static bool match_attention(const Sched &sc, int s_item, const std::vector<char> &taken, FusedGroup *out) {
  const PolySchedule *s = sc.s;
  const KernelGraph &gS = sc.graphs[(size_t)s_item];
  MatmulMatch mS;
  if (!match_matmul(gS, &mS, nullptr)) return false;   // not a matmul: not a candidate, no diagnostics
  if (mS.K != 64 || mS.M % 128 != 0 || mS.N % 64 != 0 || mS.Z > (1 << 20)) FA_REJECT();
  if (mS.ka.kb < mS.K || mS.kb.kb < mS.K || mS.ka.s_lo != 1 || mS.kb.s_lo != 1) FA_REJECT();   // features contiguous
  if (mS.nd_full.size() != 1 || mS.nd_full[0].cut != 1) FA_REJECT();                         // keys: one plain range
  const int n_master = mS.nd_full[0].ord;
  const StoreInfo &stS = gS.stores[0];
  const DT tin = mS.A.dt;
  if (tin != DT_BF16 && tin != DT_F16) FA_REJECT();
  if (gS.n(stS.value).dt != tin) FA_REJECT();
  std::vector<int64_t> mext(gS.ranges.size());
  for (size_t i = 0; i < gS.ranges.size(); i++) mext[i] = gS.ranges[i].extent;
  RangeMap idS;
  for (int r : stS.ranges) idS[r] = r;
  const int lsi = gS.n(gS.n(stS.index).src[1]).lin;
  Aff aS;
  if (lsi < 0 || !lin_to_aff(gS, gS.lins[(size_t)lsi], idS, &aS)) FA_REJECT();
  if (aS.c.size() != stS.ranges.size()) FA_REJECT();   // the store covers a dense [z, m, n] box

  std::vector<Member> members;      // S, E*, MAX, SUM, P, PV in this order
  std::set<int> internal;           // slots that stay inside the fused kernel
  { Member m; m.item = s_item; m.rm = idS; members.push_back(m); }
  int cur = sc.slot(s_item, gS.param_slot(stS.param));
  const int64_t big_numel = s->buf_slots[cur].numel;

  auto only_group_reads = [&](int sl, std::set<int> expect) {
    if (!s->buf_slots[sl].is_intermediate) return false;
    std::set<int> r(sc.readers[(size_t)sl].begin(), sc.readers[(size_t)sl].end());
    return r == expect && sc.writers[(size_t)sl].size() == 1;
  };
  // pointwise consumer of `cur`: maps its ranges, presets its loads of cur, checks its store
  auto pointwise = [&](int item, Member *m, const char *value_name) {
    const KernelGraph &g = sc.graphs[(size_t)item];
    if (!g.reduces.empty() || g.stores.size() != 1 || g.stores[0].gate >= 0 || !g.vars.empty()) return false;
    std::vector<LoadRef> lds;
    const int p = sc.param_of(item, cur);
    if (p < 0 || !loads_of(g, p, &lds) || lds.empty()) return false;
    m->item = item;
    for (const LoadRef &l : lds) {
      if (!derive_map(g, g.lins[(size_t)l.lin], aS, mext, &m->rm)) return false;
      m->preset[l.node] = value_name;
    }
    for (int r : g.stores[0].ranges) if (!m->rm.count(r)) return false;
    const int li = g.n(g.n(g.stores[0].index).src[1]).lin;
    Aff a;
    if (li < 0 || !lin_to_aff(g, g.lins[(size_t)li], m->rm, &a) || !(a == aS)) return false;
    const int outp = g.param_slot(g.stores[0].param);
    if (s->buf_slots[sc.slot(item, outp)].numel != big_numel) return false;
    return true;
  };

  // ── the pointwise chain ────────────────────────────────────────────────
  std::vector<int> tail;
  for (int depth = 0;; depth++) {
    std::vector<int> rd = sc.readers[(size_t)cur];
    if (!s->buf_slots[cur].is_intermediate || sc.writers[(size_t)cur].size() != 1) FA_REJECT();
    if (rd.size() == 3) { tail = rd; break; }
    if (rd.size() != 1 || depth >= 4) FA_REJECT();
    Member m;
    if (taken[(size_t)rd[0]] || !pointwise(rd[0], &m, "x")) FA_REJECT();
    const KernelGraph &g = sc.graphs[(size_t)rd[0]];
    if (g.n(g.stores[0].value).dt != tin) FA_REJECT();
    internal.insert(cur);
    members.push_back(m);
    cur = sc.slot(rd[0], g.param_slot(g.stores[0].param));
  }
  const size_t n_chain = members.size() - 1;
  internal.insert(cur);

  // ── MAX, SUM, P ────────────────────────────────────────────────────────
  int i_max = -1, i_sum = -1, i_p = -1;
  for (int it : tail) {
    if (taken[(size_t)it]) FA_REJECT();
    const KernelGraph &g = sc.graphs[(size_t)it];
    if (g.reduces.empty()) { if (i_p >= 0) FA_REJECT(); i_p = it; continue; }
    if (g.reduces.size() != 1) FA_REJECT();
    const PolyOps op = reduce_op(g.n(g.reduces[0]));
    if (op == POLY_OP_MAX) { if (i_max >= 0) FA_REJECT(); i_max = it; }
    else if (op == POLY_OP_ADD) { if (i_sum >= 0) FA_REJECT(); i_sum = it; }
    else FA_REJECT();
  }
  if (i_max < 0 || i_sum < 0 || i_p < 0) FA_REJECT();

  // a row reduction over the key axis whose body reads `cur` at the producer's index
  auto row_reduce = [&](int item, Member *m, int *body, Aff *store_aff) {
    const KernelGraph &g = sc.graphs[(size_t)item];
    if (g.stores.size() != 1 || g.stores[0].gate >= 0 || !g.vars.empty()) return false;
    const int red = g.reduces[0];
    const KNode &R = g.n(red);
    if (R.src.size() != 2 || R.dt != DT_F32 || g.stores[0].value != red) return false;
    std::vector<LoadRef> lds;
    const int p = sc.param_of(item, cur);
    if (p < 0 || !loads_of(g, p, &lds) || lds.size() != 1) return false;
    m->item = item;
    if (!derive_map(g, g.lins[(size_t)lds[0].lin], aS, mext, &m->rm)) return false;
    m->preset[lds[0].node] = "x";
    const int kr = g.range_ord.at(R.src[1]);
    if (!m->rm.count(kr) || m->rm[kr] != n_master) return false;
    for (int r : g.stores[0].ranges) if (!m->rm.count(r)) return false;
    const int li = g.n(g.n(g.stores[0].index).src[1]).lin;
    if (li < 0 || !lin_to_aff(g, g.lins[(size_t)li], m->rm, store_aff)) return false;
    if (store_aff->c.count(n_master)) return false;
    *body = R.src[0];
    return true;
  };
  auto strip_cast = [](const KernelGraph &g, int node) {
    const KNode &k = g.n(node);
    return (k.op == POLY_OP_CAST && k.dt == DT_F32) ? k.src[0] : node;
  };

  Member mMax, mSum, mP;
  int body_max = -1, body_sum = -1;
  Aff aMax, aSum;
  if (!row_reduce(i_max, &mMax, &body_max, &aMax)) FA_REJECT();
  {
    // the maximum is taken over the stored values themselves, so it is one of them
    const KernelGraph &g = sc.graphs[(size_t)i_max];
    if (!mMax.preset.count(strip_cast(g, body_max))) FA_REJECT();
  }
  const int sl_max = sc.slot(i_max, sc.graphs[(size_t)i_max].param_slot(sc.graphs[(size_t)i_max].stores[0].param));
  if (!row_reduce(i_sum, &mSum, &body_sum, &aSum)) FA_REJECT();
  const int sl_sum = sc.slot(i_sum, sc.graphs[(size_t)i_sum].param_slot(sc.graphs[(size_t)i_sum].stores[0].param));
  // term = exp2((cast(x) - mx) * c), c > 0: this is what makes term(a, m2) = term(a, m1) * term(m1, m2)
  // and term monotone in x.  Returns the SUB node's operands and c.
  auto match_term = [&](const KernelGraph &g, int node, int *x_node, int *mx_node, double *c_out) {
    const KNode &e = g.n(node);
    if (e.op != POLY_OP_EXP2 || e.dt != DT_F32) return false;
    const KNode &mul = g.n(e.src[0]);
    if (mul.op != POLY_OP_MUL) return false;
    int sub = -1;
    for (int side = 0; side < 2; side++) {
      const KNode &c = g.n(mul.src[(size_t)side]);
      if (c.op == POLY_OP_CONST && c.u->arg.kind == POLY_ARG_FLOAT && c.u->arg.f > 0) { sub = mul.src[(size_t)(1 - side)]; *c_out = c.u->arg.f; }
    }
    if (sub < 0 || g.n(sub).op != POLY_OP_SUB) return false;
    *x_node = strip_cast(g, g.n(sub).src[0]);
    *mx_node = g.n(sub).src[1];
    return true;
  };
  double c_sum = 0;
  {
    const KernelGraph &g = sc.graphs[(size_t)i_sum];
    int xn, mn;
    if (!match_term(g, body_sum, &xn, &mn, &c_sum) || !mSum.preset.count(xn)) FA_REJECT();
    std::vector<LoadRef> lm;
    const int pm = sc.param_of(i_sum, sl_max);
    if (pm < 0 || !loads_of(g, pm, &lm) || lm.size() != 1 || lm[0].node != mn) FA_REJECT();
    Aff a;
    if (!lin_to_aff(g, g.lins[(size_t)lm[0].lin], mSum.rm, &a) || !(a == aMax)) FA_REJECT();
    mSum.preset[lm[0].node] = "mx";
  }
  if (!pointwise(i_p, &mP, "x")) FA_REJECT();
  {
    const KernelGraph &g = sc.graphs[(size_t)i_p];
    if (g.n(g.stores[0].value).dt != tin) FA_REJECT();
    for (int which = 0; which < 2; which++) {
      std::vector<LoadRef> l;
      const int p = sc.param_of(i_p, which == 0 ? sl_max : sl_sum);
      if (p < 0 || !loads_of(g, p, &l) || l.empty()) FA_REJECT();
      for (const LoadRef &r : l) {
        Aff a;
        if (!lin_to_aff(g, g.lins[(size_t)r.lin], mP.rm, &a) || !(a == (which == 0 ? aMax : aSum))) FA_REJECT();
        mP.preset[r.node] = which == 0 ? "mx" : "sum";
      }
    }
  }
  // When p = cast(term(x, mx) / sum) with the very term of the sum kernel, a key block whose
  // terms are all exactly zero has probabilities that are all exactly zero (for a finite,
  // non-zero sum), and pass 2 may skip it.
  bool p_is_term_over_sum = false;
  {
    const KernelGraph &g = sc.graphs[(size_t)i_p];
    int v = g.stores[0].value;
    if (g.n(v).op == POLY_OP_CAST) v = g.n(v).src[0];
    const KNode &q = g.n(v);
    int num = -1, den = -1;
    if (q.op == POLY_OP_FDIV) { num = q.src[0]; den = q.src[1]; }
    else if (q.op == POLY_OP_MUL) {
      for (int side = 0; side < 2; side++) {
        const KNode &r = g.n(q.src[(size_t)side]);
        if (r.op == POLY_OP_RECIPROCAL) { den = r.src[0]; num = q.src[(size_t)(1 - side)]; }
      }
    }
    int xn, mn;
    double c_p = 0;
    if (num >= 0 && q.dt == DT_F32 && match_term(g, num, &xn, &mn, &c_p) && c_p == c_sum && mP.preset.count(xn) &&
        mP.preset.count(mn) && mP.preset[mn] == "mx" && mP.preset.count(den) && mP.preset[den] == "sum" && mP.preset[xn] == "x")
      p_is_term_over_sum = true;
  }
  const int sl_p = sc.slot(i_p, sc.graphs[(size_t)i_p].param_slot(sc.graphs[(size_t)i_p].stores[0].param));
  if (!only_group_reads(cur, {i_max, i_sum, i_p}) || !only_group_reads(sl_max, {i_sum, i_p}) || !only_group_reads(sl_sum, {i_p})) FA_REJECT();
  if (sc.readers[(size_t)sl_p].size() != 1 || !s->buf_slots[sl_p].is_intermediate || sc.writers[(size_t)sl_p].size() != 1) FA_REJECT();
  internal.insert(sl_max); internal.insert(sl_sum); internal.insert(sl_p);

  // ── PV ─────────────────────────────────────────────────────────────────
  const int i_pv = sc.readers[(size_t)sl_p][0];
  if (taken[(size_t)i_pv]) FA_REJECT();
  const KernelGraph &gP = sc.graphs[(size_t)i_pv];
  MatmulMatch mV;
  if (!match_matmul(gP, &mV, nullptr)) FA_REJECT();
  if (mV.A.dt != tin || sc.slot(i_pv, mV.A.param) != sl_p || sc.slot(i_pv, mV.B.param) == sl_p) FA_REJECT();
  if (mV.M != mS.M || mV.Z != mS.Z || mV.K != mS.N || mV.N != 64) FA_REJECT();
  if (mV.ka.kb < mV.K || mV.kb.kb < mV.K) FA_REJECT();
  if (mV.nd.size() != 1 || mV.nd[0].cb != 1) FA_REJECT();      // V features contiguous
  if (mV.nd_full.size() != 1 || mV.nd_full[0].cut != 1) FA_REJECT();   // features: one plain range
  const int d_ord = mV.nd_full[0].ord;
  // P is read where it was written: the A operand index identifies PV's ranges (z, m and
  // its reduce range) with master ranges; PV's own numbering of z is never used
  Member mPV;
  mPV.item = i_pv;
  if (!derive_map(gP, gP.lins[(size_t)mV.A.lin], aS, mext, &mPV.rm)) FA_REJECT();
  if (!mPV.rm.count(mV.kr) || mPV.rm[mV.kr] != n_master) FA_REJECT();
  Aff aV;   // index of V in master coordinates, without the feature term
  {
    RangeMap with_d = mPV.rm;
    with_d[d_ord] = -1;   // placeholder coordinate for the feature range
    if (!lin_to_aff(gP, gP.lins[(size_t)mV.B.lin], with_d, &aV)) FA_REJECT();
    if (!aV.c.count(-1) || aV.c[-1] != 1) FA_REJECT();
    aV.c.erase(-1);
    for (const MmDim &d : mS.md_full) if (aV.c.count(d.ord)) FA_REJECT();   // V does not depend on the query
  }
  const StoreInfo &stP = gP.stores[0];
  const int out_slot = sc.slot(i_pv, gP.param_slot(stP.param));

  // ── schedule constraints: the group runs where PV ran ───────────────────
  std::vector<Member> all = members;
  all.push_back(mMax); all.push_back(mSum); all.push_back(mP);
  all.push_back(mPV);
  std::set<int> group_items;
  for (const Member &m : all) group_items.insert(m.item);
  if (group_items.size() != all.size()) FA_REJECT();
  const int last_step = sc.step_of[(size_t)i_pv];
  int first_step = sc.step_of[(size_t)s_item];
  for (int it : group_items) if (sc.step_of[(size_t)it] < first_step || sc.step_of[(size_t)it] > last_step) FA_REJECT();
  // Operands that are plain copies of a slice of another buffer (the q / k / v split of a
  // fused projection) are read from that buffer directly: the copy kernel joins the group
  // and its output is never materialised.  Needs the 64 features of a row to stay
  // contiguous and 64-aligned through the copy.
  const int op_slot[3] = {sc.slot(s_item, mS.A.param), sc.slot(s_item, mS.B.param), sc.slot(i_pv, mV.B.param)};
  const int op_reader[3] = {s_item, s_item, i_pv};
  CopyMap folded[3];
  std::vector<int> copy_items;
  auto multiple_of_64 = [&](const std::vector<MmDim> &dims, bool use_a) {
    for (const MmDim &d : dims) if ((use_a ? d.ca : d.cb) % 64) return false;
    return true;
  };
  bool op_aligned[3] = {mS.a_c0 % 64 == 0 && multiple_of_64(mS.zd, true) && multiple_of_64(mS.md, true),
                        mS.b_c0 % 64 == 0 && multiple_of_64(mS.zd, false) && multiple_of_64(mS.nd, false), aV.c0 % 64 == 0};
  for (auto &kv : aV.c) if (kv.second % 64) op_aligned[2] = false;
  for (int o = 0; o < 3; o++) {
    const int sl = op_slot[o];
    if (getenv("POLY_HIP_NO_COPY_FOLD") || !op_aligned[o] || !s->buf_slots[sl].is_intermediate || internal.count(sl)) continue;
    if (sc.writers[(size_t)sl].size() != 1 || sc.readers[(size_t)sl].size() != 1 || sc.readers[(size_t)sl][0] != op_reader[o]) continue;
    if ((o == 0 && sl == op_slot[1]) || (o == 1 && sl == op_slot[0])) continue;   // Q and K from one buffer: keep it simple
    const int w = sc.writers[(size_t)sl][0];
    CopyMap cm;
    if (taken[(size_t)w] || group_items.count(w) || sc.step_of[(size_t)w] > sc.step_of[(size_t)op_reader[o]] || !match_copy(sc, w, &cm)) continue;
    if (cm.digits.empty() || cm.digits.back().extent % 64 || cm.digits.back().coef != 1 || cm.c0 % 8) continue;
    bool ok = true;
    for (size_t i = 0; i + 1 < cm.digits.size(); i++) if (cm.digits[i].coef % 8) ok = false;
    if (!ok || internal.count(cm.src_slot)) continue;
    folded[o] = cm;
    copy_items.push_back(w);
    group_items.insert(w);
    internal.insert(sl);
    first_step = std::min(first_step, sc.step_of[(size_t)w]);
  }
    std::set<int> inputs;
  std::map<int, int> first_read;   // input slot -> earliest original step of a member reading it
  for (int it : group_items) {
    const PolyExecItem &e = s->items[it];
    for (int i = 0; i < e.n_buf_slots; i++) {
      const int sl = e.buf_slot_indices[i];
      if (internal.count(sl) || sl == out_slot) continue;
      if (sc.graphs[(size_t)it].params[(size_t)i].written) FA_REJECT();
      inputs.insert(sl);
      const int st = sc.step_of[(size_t)it];
      if (!first_read.count(sl) || st < first_read[sl]) first_read[sl] = st;
    }
  }
  // a member that read an input at its own step now reads it at the group's step: the
  // input must not change in between
  for (int sl : inputs)
    for (int w : sc.writers[(size_t)sl])
      if (sc.step_of[(size_t)w] >= first_read[sl] && sc.step_of[(size_t)w] <= last_step) FA_REJECT();
  for (int w : sc.writers[(size_t)out_slot]) if (w != i_pv && sc.step_of[(size_t)w] >= first_step && sc.step_of[(size_t)w] <= last_step) FA_REJECT();
  for (int r : sc.readers[(size_t)out_slot]) if (sc.step_of[(size_t)r] >= first_step && sc.step_of[(size_t)r] <= last_step && r != i_pv) FA_REJECT();
  if (internal.count(out_slot) || inputs.count(out_slot)) FA_REJECT();

  // every load of an internal buffer must have been replaced by a value
  for (const Member &m : all) {
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    for (int id = 0; id < (int)g.nodes.size(); id++) {
      if (g.n(id).op != POLY_OP_LOAD) continue;
      const int p = g.param_slot(g.n(g.n(id).src[0]).src[0]);
      if (!internal.count(sc.slot(m.item, p))) continue;
      // loads the template performs itself: P, and operands folded into their source
      const bool by_template = (m.item == i_pv && (id == mV.A.load || id == mV.B.load)) ||
                               (m.item == s_item && (id == mS.A.load || id == mS.B.load));
      if (!m.preset.count(id) && !by_template) FA_REJECT();
    }
  }

  // ── code generation ────────────────────────────────────────────────────
  std::vector<int> arg_slots;
  arg_slots.push_back(out_slot);
  for (int sl : inputs) arg_slots.push_back(sl);
  auto arg_of = [&](int sl) { return (int)(std::find(arg_slots.begin(), arg_slots.end(), sl) - arg_slots.begin()); };
  auto call_args = [&](int item) {
    const KernelGraph &g = sc.graphs[(size_t)item];
    std::string c;
    for (size_t i = 0; i < g.params.size(); i++) {
      const int sl = sc.slot(item, (int)i);
      if (i) c += ", ";
      if (internal.count(sl)) c += strf("(%s%s*)0", g.params[i].written ? "" : "const ", dt_cname(g.params[i].dt));
      else c += strf("fa%d", arg_of(sl));
    }
    return c;
  };
  std::string sig;
  for (size_t j = 0; j < arg_slots.size(); j++) {
    DT dt = DT_VOID;
    for (int it : group_items) {
      const int p = sc.param_of(it, arg_slots[j]);
      if (p >= 0) dt = sc.graphs[(size_t)it].params[(size_t)p].dt;
    }
    if (j) sig += ", ";
    sig += j == 0 ? strf("%s* fa%zu", dt_cname(dt), j) : strf("const %s* __restrict__ fa%zu", dt_cname(dt), j);
  }

  const std::string master_decomp = matmul_decompose(mS, nullptr);
  const char *tn = dt_cname(tin);
  std::string cfg;
  bool failed = false;
  // one device function per kernel of the group: value of `node` with the member's presets
  // The softmax terms use the bare exp2 instruction: a term below 2^-126 of the row's
  // largest (which is exactly 1, so the sum is at least 1) cannot change the fp32 sum, and
  // the probability it would give is below the smallest normal 16-bit float.
  const bool online = p_is_term_over_sum && !getenv("POLY_HIP_EXACT_ATTENTION");
  auto value_fn = [&](const Member &m, const char *name, const char *ret, const char *lead_args, int node,
                      const std::map<int, std::string> &extra_preset) {
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    Emitter em(g);
    em.raw_exp2 = (m.item == i_sum || m.item == i_p);
    em.pow2_mul16_exact = online;
    Scope S0;
    S0.indent = 1;
    for (auto &kv : m.rm) { em.bind_range(kv.first, strf("r%d", kv.second)); S0.avail |= (uint64_t)1 << kv.first; }
    for (auto &kv : m.preset) em.preset(kv.first, kv.second);
    for (auto &kv : extra_preset) em.preset(kv.first, kv.second);
    std::string v = em.emit(node, &S0);
    if (em.failed() || em.uses_threefry) failed = true;
    cfg += strf("__device__ __forceinline__ %s %s(%s, int m, int n, int z, %s) {\n", ret, name, lead_args, params_decl(g).c_str());
    cfg += master_decomp + S0.code;
    cfg += strf("  return %s;\n}\n", v.c_str());
  };
  cfg += strf("#define POLY_TIN %s\n", tn);
  cfg += strf("#define POLY_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_%s(a, b, c, 0, 0, 0)\n", tin == DT_BF16 ? "bf16" : "f16");
  cfg += strf("#define POLY_FA_M %lld\n#define POLY_FA_N %lld\n#define POLY_FA_Z %lld\n", (long long)mS.M, (long long)mS.N, (long long)mS.Z);
  cfg += attention_order(mS.M / 128, mS.Z);
  auto operand_arg = [&](int o) { return arg_of(folded[o].item >= 0 ? folded[o].src_slot : op_slot[o]); };
  cfg += strf("#define POLY_Q_PTR fa%d\n#define POLY_K_PTR fa%d\n#define POLY_V_PTR fa%d\n", operand_arg(0), operand_arg(1), operand_arg(2));
  // position in the operand's own buffer -> position in the buffer it was copied from
  const char *src_name[3] = {"poly_fa_qsrc", "poly_fa_ksrc", "poly_fa_vsrc"};
  for (int o = 0; o < 3; o++) {
    std::string f = strf("__device__ __forceinline__ int %s(int p) {\n", src_name[o]);
    if (folded[o].item < 0) f += "  return p;\n}\n";
    else {
      f += strf("  int off = %lld;\n", (long long)folded[o].c0);
      for (const CopyMap::Digit &d : folded[o].digits)
        f += strf("  off += ((p / %lld) %% %lld) * %lld;\n", (long long)d.stride, (long long)d.extent, (long long)d.coef);
      f += "  return off;\n}\n";
    }
    cfg += f;
  }
  cfg += matmul_offset_fn("poly_fa_qz", mS.zd, true, mS.a_c0) + matmul_offset_fn("poly_fa_qm", mS.md, true, 0);
  cfg += matmul_offset_fn("poly_fa_kz", mS.zd, false, mS.b_c0) + matmul_offset_fn("poly_fa_kn", mS.nd, false, 0);
  // Row offsets as the kernel sees them: source position of row x (query or key) of batch z.
  // When that is affine in x for every z -- the usual case -- the z part is evaluated once
  // and the row part is a multiplication; otherwise the general digit form is kept.
  auto eval_src = [&](int o, int64_t p) {
    if (folded[o].item < 0) return p;
    int64_t off = folded[o].c0;
    for (const CopyMap::Digit &d : folded[o].digits) off += ((p / d.stride) % d.extent) * d.coef;
    return off;
  };
  auto raw_off = [&](int o, int64_t z, int64_t x) {
    if (o == 0) return mS.a_c0 + matmul_eval_offset(mS.zd, true, z) + matmul_eval_offset(mS.md, true, x);
    if (o == 1) return mS.b_c0 + matmul_eval_offset(mS.zd, false, z) + matmul_eval_offset(mS.nd, false, x);
    int64_t v = aV.c0;
    for (auto &kv : aV.c) v += kv.second * matmul_range_value(mS, kv.first, 0, x, z);
    return v;
  };
  std::string v_expr = strf("%lld", (long long)aV.c0);
  for (auto &kv : aV.c) v_expr += strf(" + %lld * r%d", (long long)kv.second, kv.first);
  int64_t k_pitch = 0;      // elements from one key to the next in the keys' buffer, when that is one number
  const char *off_name[3] = {"poly_q_off", "poly_k_off", "poly_v_off"};
  const std::string general[3] = {
      "__device__ __forceinline__ int poly_fa_q0(int z, int m) { return poly_fa_qz(z) + poly_fa_qm(m); }\n",
      "__device__ __forceinline__ int poly_fa_k0(int z, int n) { return poly_fa_kz(z) + poly_fa_kn(n); }\n",
      "__device__ __forceinline__ int poly_fa_v0(int z, int n) {\n  const int m = 0;\n" + master_decomp + "  return " + v_expr + ";\n}\n"};
  const char *raw_name[3] = {"poly_fa_q0", "poly_fa_k0", "poly_fa_v0"};
  for (int o = 0; o < 3; o++) {
    cfg += general[o];
    const int64_t X = o == 0 ? mS.M : mS.N;
    bool affine = mS.Z * X <= (int64_t)1 << 24;
    const int64_t step = eval_src(o, raw_off(o, 0, 1)) - eval_src(o, raw_off(o, 0, 0));
    for (int64_t z = 0; z < mS.Z && affine; z++) {
      const int64_t base = eval_src(o, raw_off(o, z, 0));
      for (int64_t x = 0; x < X; x++)
        if (eval_src(o, raw_off(o, z, x)) != base + x * step) { affine = false; break; }
    }
    if (o == 1 && affine) k_pitch = step;
    if (affine)
      cfg += strf("__device__ __forceinline__ int %s(int z, int x) { return %s(%s(z, 0)) + x * %lld; }\n", off_name[o], src_name[o],
                  raw_name[o], (long long)step);
    else
      cfg += strf("__device__ __forceinline__ int %s(int z, int x) { return %s(%s(z, x)); }\n", off_name[o], src_name[o], raw_name[o]);
  }
  cfg += strf("#define POLY_SIGNATURE %s\n", sig.c_str());
  cfg += strf("#define POLY_FA_SKIP_DEAD_BLOCKS %d\n", p_is_term_over_sum ? 1 : 0);
  // Do the keys lie in their buffer the way a row-major matrix product of `k_pitch` columns
  // would have left them -- key block kb of z = (b, h) as the 64 x 64 block at row
  // b * N + 64 kb, column c0 + 64 h?  Then that product can say how large the keys of every
  // block are (key_bounds; find_fused_groups asks it to).
  FusedGroup::KeyBounds kbnd;
  if (k_pitch >= 64 && mS.N % 64 == 0 && mS.N / 64 <= 64 && mS.K == 64) {
    const int64_t T = mS.N, NKB = T / 64, c0 = eval_src(1, raw_off(1, 0, 0)) % k_pitch;
    // z counts (b, h) with either of the two running fastest
    const bool heads_fastest = mS.Z > 1 && eval_src(1, raw_off(1, 1, 0)) % k_pitch != c0;
    int64_t H = mS.Z, B = 1;
    if (heads_fastest) {
      for (int64_t z = 1; z < mS.Z; z++)
        if (eval_src(1, raw_off(1, z, 0)) % k_pitch == c0) { H = z; break; }
      B = mS.Z / H;
    } else {
      B = mS.Z;
      for (int64_t z = 1; z < mS.Z; z++)
        if (eval_src(1, raw_off(1, z, 0)) % k_pitch != c0) { B = z; break; }
      H = mS.Z / B;
    }
    bool ok = c0 % 64 == 0 && B * H == mS.Z && c0 + H * 64 <= k_pitch;
    for (int64_t z = 0; z < mS.Z && ok; z++)
      for (int64_t kb = 0; kb < NKB && ok; kb++) {
        const int64_t f = eval_src(1, raw_off(1, z, kb * 64));
        const int64_t b = heads_fastest ? z / H : z % B, h = heads_fastest ? z % H : z / B;
        ok = f / k_pitch == b * T + kb * 64 && f % k_pitch == c0 + h * 64;
      }
    if (ok) {
      kbnd.possible = true;
      kbnd.slot = folded[1].item >= 0 ? folded[1].src_slot : op_slot[1];
      kbnd.pitch = k_pitch;
      kbnd.rows = B * T;
      kbnd.lo = c0;
      kbnd.hi = c0 + H * 64;
      const std::string zexpr = heads_fastest ? strf("((m) / %lld) * %lld + ((n) - %lld) / 64", (long long)T, (long long)H, (long long)c0)
                                              : strf("(((n) - %lld) / 64) * %lld + (m) / %lld", (long long)c0, (long long)B, (long long)T);
      kbnd.index = strf("(%s) * %lld + ((m) %% %lld) / 64", zexpr.c_str(), (long long)NKB, (long long)T);
      kbnd.bytes = (size_t)(mS.Z * NKB) * sizeof(unsigned);
    }
  }

  // score: epilogue of S, then the pointwise chain
  {
    const Member &m = all[0];
    value_fn(m, "poly_fa_s", tn, "float acc", stS.value, {{mS.red, "acc"}});
  }
  std::string score = strf("poly_fa_s(acc, m, n, z, %s)", call_args(s_item).c_str());
  for (size_t e = 1; e <= n_chain; e++) {
    const Member &m = all[e];
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    const std::string fn = strf("poly_fa_e%zu", e);
    value_fn(m, fn.c_str(), tn, strf("%s x", tn).c_str(), g.stores[0].value, {});
    score = strf("%s(%s, m, n, z, %s)", fn.c_str(), score.c_str(), call_args(m.item).c_str());
  }
  cfg += strf("#define POLY_FA_SCORE(acc, m, n, z) %s\n", score.c_str());
  bool mask_table = false;   // a kernel ahead of this one looks at the mask once for all z
  int mask_arg = -1;         // which argument of the fused kernel the mask is
  // An additive mask: the stored score is cast(f(acc) + mask[...]) with f made of casts
  // and products with positive constants, and the mask a bf16 buffer read at consecutive
  // positions for consecutive keys.  The kernel then loads the mask entries of a tile
  // itself (POLY_FA_MASK_PTR), gets the chain with the entry as an argument
  // (POLY_FA_SCORE_MASK) and the value of f alone (POLY_FA_SCORE_NOMASK), and treats tiles
  // whose entries are all one value specially: all zero, the score is f(acc) itself
  // (f(acc) is a 16-bit value, adding zero and rounding again change nothing); all one
  // other value, the score is a non-decreasing function of acc alone, so the score of the
  // tile's largest product bounds them all.
  if (online && tin == DT_BF16 && !getenv("POLY_HIP_NO_MASK_PATHS") && mS.nd_full.size() == 1) {
    const Member &lm = all[n_chain];
    const KernelGraph &g = sc.graphs[(size_t)lm.item];
    auto strip = [&](int v) { while (g.n(v).op == POLY_OP_CAST && dt_is_float(g.n(v).dt) && dt_is_float(g.n(g.n(v).src[0]).dt)) v = g.n(v).src[0]; return v; };
    const int top = strip(n_chain ? g.stores[0].value : stS.value);
    int mask_ld = -1, other = -1;
    bool mask_z_free = false;   // the mask entry does not depend on z
    if (g.n(top).op == POLY_OP_ADD && g.n(top).dt == tin)
      for (int side = 0; side < 2; side++) {
        const int cand = g.n(top).src[(size_t)side];
        if (g.n(cand).op != POLY_OP_LOAD || g.n(cand).dt != tin || lm.preset.count(cand) || g.n(cand).guard >= 0) continue;
        const KNode &ix = g.n(g.n(cand).src[0]);
        Aff a;
        if (ix.src.size() != 2 || g.n(ix.src[1]).lin < 0 || !lin_to_aff(g, g.lins[(size_t)g.n(ix.src[1]).lin], lm.rm, &a)) continue;
        auto it = a.c.find(mS.nd_full[0].ord);
        if (it == a.c.end() || it->second != 1) continue;
        mask_ld = cand;
        other = g.n(top).src[(size_t)(1 - side)];
        mask_arg = arg_of(sc.slot(lm.item, g.param_slot(ix.src[0])));
        mask_z_free = true;
        for (const auto &d : mS.zd) {
          auto zc = a.c.find(d.ord);
          if (zc != a.c.end() && zc->second != 0) mask_z_free = false;
        }
      }
    // f: from acc (or the chain input x) through casts and products with positive constants
    std::function<bool(int)> plain = [&](int id) -> bool {
      const KNode &k = g.n(id);
      if (n_chain == 0 && id == mS.red) return true;
      auto pr = lm.preset.find(id);
      if (pr != lm.preset.end()) return pr->second == "x";
      if (!dt_is_float(k.dt)) return false;
      if (k.op == POLY_OP_CAST) return dt_is_float(g.n(k.src[0]).dt) && plain(k.src[0]);
      if (k.op == POLY_OP_MUL)
        for (int side = 0; side < 2; side++) {
          const KNode &c = g.n(k.src[(size_t)side]);
          if (c.op == POLY_OP_CONST && c.u->arg.kind == POLY_ARG_FLOAT && c.u->arg.f > 0) return plain(k.src[(size_t)(1 - side)]);
        }
      return false;
    };
    bool ok = mask_ld >= 0 && g.n(other).dt == tin && plain(other);
    // the members in front of the last one must be monotone in acc as well: only the S epilogue
    // (a cast) is accepted there
    if (ok && n_chain > 1) ok = false;
    if (ok && n_chain == 1) {
      const KernelGraph &g0 = sc.graphs[(size_t)all[0].item];
      int v = stS.value;
      while (g0.n(v).op == POLY_OP_CAST && dt_is_float(g0.n(v).dt)) v = g0.n(v).src[0];
      ok = v == mS.red;
    }
    if (ok) {
      const size_t before = cfg.size();
      const bool failed_before = failed;
      // address of the mask entry
      {
        Emitter em(g);
        Scope S0;
        S0.indent = 1;
        for (auto &kv : lm.rm) { em.bind_range(kv.first, strf("r%d", kv.second)); S0.avail |= (uint64_t)1 << kv.first; }
        const KNode &ix = g.n(g.n(mask_ld).src[0]);
        const std::string idx = em.emit(ix.src[1], &S0);
        if (em.failed()) failed = true;
        cfg += strf("__device__ __forceinline__ const %s* poly_fa_mask_ptr(int m, int n, int z, %s) {\n", tn, params_decl(g).c_str());
        cfg += master_decomp + S0.code + strf("  return data%d + %s;\n}\n", g.param_slot(ix.src[0]), idx.c_str());
        cfg += strf("#define POLY_FA_MASK_PTR(m, n, z) poly_fa_mask_ptr(m, n, z, %s)\n", call_args(lm.item).c_str());
      }
      const std::string head = n_chain ? strf("poly_fa_s(acc, m, n, z, %s)", call_args(s_item).c_str()) : std::string("acc");
      const char *lead = n_chain ? "%s x, %s mk" : "float acc, %s mk";
      std::map<int, std::string> pre_mask{{mask_ld, "mk"}};
      if (!n_chain) pre_mask[mS.red] = "acc";
      // f(acc) = cast(acc) * 2^k with nothing else in it: the kernel multiplies Q by 2^k
      // once when it stages it instead (products and sums of a dot product scale exactly
      // with a power of two, and so does every rounding on the way, as long as nothing
      // becomes subnormal), and the chain is emitted with that constant as 1.  For bf16 only:
      // it has the exponent range of fp32, so the scaled Q loses nothing; an fp16 Q below
      // 2^-11 would lose mantissa bits, and the reference's cast of an unscaled sum to fp16
      // can overflow where the scaled one does not.
      int scale_const = -1;
      double qscale = 1.0;
      if (!getenv("POLY_HIP_NO_QSCALE") && tin == DT_BF16) {
        int muls = 0, v = other;
        while (true) {
          const KNode &k = g.n(v);
          if (k.op == POLY_OP_CAST) { v = k.src[0]; continue; }
          if (k.op != POLY_OP_MUL) break;
          int side = -1;
          for (int sd = 0; sd < 2; sd++) {
            const KNode &cn = g.n(k.src[(size_t)sd]);
            if (cn.op == POLY_OP_CONST && cn.u->arg.kind == POLY_ARG_FLOAT && cn.u->arg.f > 0) side = sd;
          }
          if (side < 0) break;
          muls++;
          scale_const = k.src[(size_t)side];
          qscale = g.n(scale_const).u->arg.f;
          v = k.src[(size_t)(1 - side)];
        }
        int e2 = 0;
        const bool pow2 = muls == 1 && std::frexp(qscale, &e2) == 0.5 && e2 > -100 && e2 < 100;
        int uses = 0;
        if (pow2)
          for (const KNode &k : g.nodes) for (int sN : k.src) if (sN == scale_const) uses++;
        if (!pow2 || uses != 1) scale_const = -1;
      }
      std::map<int, std::string> pre_acc;
      if (!n_chain) pre_acc[mS.red] = "acc";
      if (scale_const >= 0) {
        pre_mask[scale_const] = "1.0f";
        pre_acc[scale_const] = "1.0f";
        cfg += strf("#define POLY_FA_QSCALE %s\n", Emitter::float_literal(qscale, DT_F32).c_str());
      }
      value_fn(lm, "poly_fa_score_mask", tn, n_chain ? strf(lead, tn, tn).c_str() : strf(lead, tn).c_str(), n_chain ? g.stores[0].value : stS.value, pre_mask);
      cfg += strf("#define POLY_FA_SCORE_MASK(acc, mk, m, n, z) poly_fa_score_mask(%s, mk, m, n, z, %s)\n", head.c_str(), call_args(lm.item).c_str());
      value_fn(lm, "poly_fa_score_nomask", "float", n_chain ? strf("%s x", tn).c_str() : "float acc", other, pre_acc);
      cfg += strf("#define POLY_FA_SCORE_NOMASK(acc, m, n, z) poly_fa_score_nomask(%s, m, n, z, %s)\n", head.c_str(), call_args(lm.item).c_str());
      if (failed && !failed_before) { failed = false; cfg.resize(before); }
      else if (!failed && mask_z_free && !getenv("POLY_HIP_NO_MASK_TABLE")) mask_table = true;
    }
  }
  // Single-pass form when the group is a plain softmax: p = cast(term / sum) with
  // term = exp2((x - max) * c) and the maximum taken over the scores themselves.
  cfg += strf("#define POLY_FA_ONLINE %d\n#define POLY_FA_C %s\n", online ? 1 : 0, Emitter::float_literal(c_sum, DT_F32).c_str());
  value_fn(mMax, "poly_fa_maxv", "float", strf("%s x", tn).c_str(), body_max, {});
  cfg += strf("#define POLY_FA_MAXV(x, m, n, z) poly_fa_maxv(x, m, n, z, %s)\n", call_args(i_max).c_str());
  value_fn(mSum, "poly_fa_term", "float", strf("%s x, float mx", tn).c_str(), body_sum, {});
  cfg += strf("#define POLY_FA_TERM(x, mx, m, n, z) poly_fa_term(x, mx, m, n, z, %s)\n", call_args(i_sum).c_str());
  value_fn(mP, "poly_fa_p", tn, strf("%s x, float mx, float sum", tn).c_str(), sc.graphs[(size_t)i_p].stores[0].value, {});
  cfg += strf("#define POLY_FA_P(x, mx, sum, m, n, z) poly_fa_p(x, mx, sum, m, n, z, %s)\n", call_args(i_p).c_str());
  {
    // output: epilogue of PV; its z and m ranges in master coordinates, its feature range = d
    Emitter em(gP);
    Scope S0;
    S0.indent = 1;
    for (int r : stP.ranges) {
      S0.avail |= (uint64_t)1 << r;
      if (r == d_ord) em.bind_range(r, "d");
      else if (mPV.rm.count(r)) em.bind_range(r, strf("r%d", mPV.rm[r]));
      else failed = true;
    }
    std::string decomp = "  const int n = 0;\n" + master_decomp;
    em.preset(mV.red, "acc");
    std::string val = em.emit(stP.value, &S0);
    std::string idx = em.emit(gP.n(stP.index).src[1], &S0);
    if (em.failed() || em.uses_threefry) failed = true;
    cfg += strf("__device__ __forceinline__ void poly_fa_out(float acc, int m, int d, int z, %s) {\n", params_decl(gP).c_str());
    cfg += decomp + S0.code;
    cfg += strf("  data%d[%s] = %s;\n}\n", gP.param_slot(stP.param), idx.c_str(), val.c_str());
    cfg += strf("#define POLY_FA_OUT(acc, m, d, z) poly_fa_out(acc, m, d, z, %s)\n", call_args(i_pv).c_str());
  }
  if (failed) FA_REJECT();

  out->items.clear();
  for (int w : copy_items) out->items.push_back(w);
  for (const Member &m : all) out->items.push_back(m.item);
  out->launch_item = i_pv;
  out->internal_slots.assign(internal.begin(), internal.end());
  out->arg_slots = arg_slots;
  RenderedKernel &rk = out->rk;
  rk = RenderedKernel();
  // timing experiments: extra macro definitions, "NAME=VALUE;NAME=VALUE"
  if (const char *e = measurement_env("POLY_HIP_FA_DEFS")) {
    std::string d(e);
    size_t pos = 0;
    while (pos < d.size()) {
      size_t end = d.find(';', pos);
      if (end == std::string::npos) end = d.size();
      std::string item = d.substr(pos, end - pos);
      const size_t eq = item.find('=');
      if (!item.empty()) cfg += "#define " + (eq == std::string::npos ? item + " 1" : item.substr(0, eq) + " " + item.substr(eq + 1)) + "\n";
      pos = end + 1;
    }
  }
  if (mask_table) {
    // One word per 32 x 32 tile and one per block of 128 queries x 64 keys, written by a
    // first kernel into scratch memory that the main kernel takes as its last argument.
    const std::string from = strf("#define POLY_SIGNATURE %s\n", sig.c_str());
    const size_t at = cfg.find(from);
    if (at == std::string::npos) FA_REJECT();
    cfg.replace(at, from.size(), strf("#define POLY_SIGNATURE %s, unsigned int* poly_scratch\n#define POLY_FA_MASK_TABLE poly_scratch\n", sig.c_str()));
    RenderedKernel::Pre pre;
    pre.source = std::string(hip_prelude()) + cfg + "#define POLY_FA_CLASSIFY 1\n" + kAttentionTemplate;
    pre.entry = "poly_k";
    pre.launch.grid[0] = (unsigned)((mS.M / 128) * (mS.N / 64));
    pre.launch.block[0] = 512;
    rk.pres.push_back(pre);
    rk.scratch_bytes = (size_t)((mS.M / 32) * (mS.N / 32) + (mS.M / 128) * (mS.N / 64)) * sizeof(unsigned);
    // the words depend on the mask buffer alone
    rk.pres_key = pre.source;
    rk.pre_reads.assign(1, mask_arg);
    if (kbnd.possible && online) {
      out->key_bounds = kbnd;
      out->key_bounds.offset = (rk.scratch_bytes + 255) / 256 * 256;
      if (g_key_bounds_slot == kbnd.slot) {
        // the product that writes the keys leaves the block maxima behind the mask words
        out->key_bounds.used = true;
        cfg += strf("#define POLY_FA_KMAX_TABLE ((const unsigned int*)poly_scratch + %zu)\n", out->key_bounds.offset / sizeof(unsigned));
        rk.scratch_bytes = out->key_bounds.offset + kbnd.bytes;
        rk.pres_key += "// (scratch memory with key bounds)\n";     // shared only among launches that also get them
      }
    }
  }
  rk.source = std::string(hip_prelude()) + cfg + kAttentionTemplate;
  const std::string fa_cfg = cfg;
  rk.entry = "poly_k";
  rk.launch.grid[0] = (unsigned)((mS.M / 128) * mS.Z);
  rk.launch.block[0] = 256;
  rk.klass = KernelClass::ATTENTION;
  rk.strategy = strf("fused attention (%zu kernels): mfma 32x32x16 %s Z=%lld M=%lld N=%lld D=64, %s", all.size() + copy_items.size(),
                     tin == DT_BF16 ? "bf16" : "f16", (long long)mS.Z, (long long)mS.M, (long long)mS.N,
                     cfg.find("#define POLY_FA_ONLINE 1") != std::string::npos ? "one pass, online softmax" : "two passes over keys, exact roundings");
  if (mask_table) rk.strategy += ", mask tiles classified by a first kernel";
  if (out->key_bounds.used) rk.strategy += ", products of masked key blocks bounded by the block maxima the keys' product leaves";
  if (matmul_tuning_enabled()) {
    // the register budget (waves per SIMD) changes the schedule of the instructions, not
    // one value: candidates of the search that POLY_BEAM switches on
    rk.variants.push_back({"default", rk.source, rk.strategy, rk.launch});
    for (int occ : {2, 4})
      rk.variants.push_back({strf("attn_occ%d", occ), std::string(hip_prelude()) + strf("#define POLY_FA_OCC %d\n", occ) + fa_cfg + kAttentionTemplate,
                             rk.strategy + strf(", %d waves per SIMD", occ), rk.launch});
  }
  rk.n_params = (int)arg_slots.size();
  rk.n_vars = 0;
  rk.flops = 2.0 * (double)mS.Z * (double)mS.M * (double)mS.N * (double)(mS.K + mV.N);
  double bytes = 0;
  for (int sl : arg_slots) bytes += (double)s->buf_slots[sl].nbytes;
  rk.bytes = bytes;
  return true;
}

// ── pointwise kernels over the same positions ─────────────────────────────────
//
// An optimizer step reaches the backend as four kernels per parameter (reference:
// src/instance.c:1152-1224): the new parameter into a temporary, the copy back, the two
// moments -- each walks the same N positions with one flat range and reads and writes
// element p of its buffers only.  Run back to back they move 13 streams of N floats; one
// launch in which a thread does all four for its positions moves 7 (p, m, v, g in; p, m, v
// out) and never materialises the temporary.  In general: consecutive kernels of the
// schedule, each without a reduction and with a single ungated store at the flat position,
// all of the same extent, whose loads are at the flat position or at a fixed index, and no
// buffer written twice.  A member's load of what an earlier member stored takes that
// value; a load of what a later member will store reads memory, and every store happens
// after every load of the thread.
static bool match_pointwise_group(const Sched &sc, int a_item, const std::vector<char> &taken, FusedGroup *out) {
  const PolySchedule *s = sc.s;
  if (getenv("POLY_HIP_NO_POINTWISE_GROUPS")) return false;
  struct Pw { int item, ord, out_slot; };
  auto flat_member = [&](int item, int64_t *extent, Pw *pw) {
    const KernelGraph &g = sc.graphs[(size_t)item];
    if (!g.reduces.empty() || g.stores.size() != 1 || g.stores[0].gate >= 0 || !g.vars.empty()) return false;
    if (g.stores[0].ranges.size() != 1 || g.ranges.size() != 1) return false;
    const int ord = g.stores[0].ranges[0];
    auto is_flat = [&](const Lin &l) {
      if (l.c0 != 0 || l.terms.size() != 1 || l.terms[0].coef != 1) return false;
      const Atom &a = g.atoms[(size_t)l.terms[0].atom];
      return a.kind == Atom::RANGE && g.range_ord.at(a.node) == ord;
    };
    const int li = g.n(g.n(g.stores[0].index).src[1]).lin;
    if (li < 0 || !is_flat(g.lins[(size_t)li])) return false;
    if (g.n(g.stores[0].value).dt != g.n(g.stores[0].param).dt) return false;
    for (size_t p = 0; p < g.params.size(); p++) {
      if (!dt_is_float(g.params[p].dt)) return false;      // (float buffers only: what the vector helpers are used with elsewhere)
      std::vector<LoadRef> lds;
      if (!loads_of(g, (int)p, &lds)) return false;
      for (const LoadRef &l : lds) {
        const Lin &lin = g.lins[(size_t)l.lin];
        if (!is_flat(lin) && !lin.terms.empty()) return false;
      }
    }
    *extent = g.ranges[(size_t)ord].extent;
    *pw = {item, ord, sc.slot(item, g.param_slot(g.stores[0].param))};
    return *extent > 0 && *extent < 2147483647LL;
  };
  int64_t E = 0;
  Pw first;
  if (!flat_member(a_item, &E, &first)) return false;
  std::vector<Pw> members{first};
  std::set<int> touched;
  for (int i = 0; i < s->items[a_item].n_buf_slots; i++) touched.insert(s->items[a_item].buf_slot_indices[i]);
  for (int st = sc.step_of[(size_t)a_item] + 1; st < s->n_items && members.size() < 8; st++) {
    const int k = s->exec_order[st];
    int64_t e2 = 0;
    Pw pw;
    if (taken[(size_t)k] || !flat_member(k, &e2, &pw) || e2 != E) break;
    bool shares = false;
    for (int i = 0; i < s->items[k].n_buf_slots; i++) shares = shares || touched.count(s->items[k].buf_slot_indices[i]);
    if (!shares) break;
    bool twice = false;
    for (const Pw &m : members) twice = twice || m.out_slot == pw.out_slot;
    if (twice) break;
    for (int i = 0; i < s->items[k].n_buf_slots; i++) touched.insert(s->items[k].buf_slot_indices[i]);
    members.push_back(pw);
  }
  if (members.size() < 2) return false;
  // what the group writes it may only read at the flat position (a fixed index would be
  // another thread's element)
  for (const Pw &w : members)
    for (const Pw &m : members) {
      const KernelGraph &g = sc.graphs[(size_t)m.item];
      const int p = sc.param_of(m.item, w.out_slot);
      if (p < 0) continue;
      std::vector<LoadRef> lds;
      loads_of(g, p, &lds);
      for (const LoadRef &l : lds) if (g.lins[(size_t)l.lin].terms.empty()) return false;
    }
  // a slot is internal when the group writes it and nobody outside ever touches it
  std::set<int> in_group;
  for (const Pw &m : members) in_group.insert(m.item);
  std::set<int> internal;
  for (const Pw &m : members) {
    if (!s->buf_slots[m.out_slot].is_intermediate) continue;
    bool outside = false;
    for (int r : sc.readers[(size_t)m.out_slot]) outside = outside || !in_group.count(r);
    for (int w : sc.writers[(size_t)m.out_slot]) outside = outside || !in_group.count(w);
    if (!outside) internal.insert(m.out_slot);
  }
  // every buffer position must hold numel == E elements for the flat index to mean the same in all members
  for (int sl : touched) {
    bool flat_use = false;
    for (const Pw &m : members) {
      const KernelGraph &g = sc.graphs[(size_t)m.item];
      const int p = sc.param_of(m.item, sl);
      if (p < 0) continue;
      std::vector<LoadRef> lds;
      loads_of(g, p, &lds);
      for (const LoadRef &l : lds) flat_use = flat_use || !g.lins[(size_t)l.lin].terms.empty();
      if (m.out_slot == sl) flat_use = true;
    }
    if (flat_use && s->buf_slots[sl].numel < E) return false;
  }
  std::vector<int> arg_slots;
  for (const Pw &m : members)
    for (int i = 0; i < s->items[m.item].n_buf_slots; i++) {
      const int sl = s->items[m.item].buf_slot_indices[i];
      if (!internal.count(sl) && std::find(arg_slots.begin(), arg_slots.end(), sl) == arg_slots.end()) arg_slots.push_back(sl);
    }
  auto arg_of = [&](int sl) { return (int)(std::find(arg_slots.begin(), arg_slots.end(), sl) - arg_slots.begin()); };
  // vector width: 16 bytes of the widest element touched at the flat position
  int maxsz = 1;
  std::map<int, DT> slot_dt;
  std::set<int> written;
  for (const Pw &m : members) {
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    for (size_t p = 0; p < g.params.size(); p++) {
      maxsz = std::max(maxsz, dt_size(g.params[p].dt));
      slot_dt[sc.slot(m.item, (int)p)] = g.params[p].dt;
    }
    written.insert(m.out_slot);
  }
  int V = std::max(1, 16 / maxsz);
  // Very long runs over many buffers at once (the optimizer update of 355 M parameters: p, m,
  // v read and written, g read) move faster with one 4-byte access per thread and buffer
  // than with 16-byte ones: 1.85 -> 1.65 ms for 9.9 GB, 5.4 -> 6.0 TB/s (8 bytes: 1.79 ms,
  // 32 bytes: 1.87 ms); the per-tensor updates of a training step (4 M positions each) do not
  // change.
  if (E >= ((int64_t)1 << 25) && arg_slots.size() >= 4) V = std::max(1, 4 / maxsz);
  if (const char *e = measurement_env("POLY_HIP_PW_BYTES")) V = std::max(1, atoi(e) / maxsz);   // tuning experiments: bytes per thread and buffer
  while (V > 1 && E % V != 0) V /= 2;
  // the members as functions of the flat position (passed as `m`)
  std::string code, body;
  std::map<int, std::string> value_of_slot;   // what the group has stored so far, by slot
  std::set<int> read_from_memory;
  double bytes = 0, bytes_written = 0;
  for (size_t mi = 0; mi < members.size(); mi++) {
    const Pw &pw = members[mi];
    const KernelGraph &g = sc.graphs[(size_t)pw.item];
    Member m;
    m.item = pw.item;
    m.range_expr[pw.ord] = "m";
    std::string lead, lead_call;
    for (size_t p = 0; p < g.params.size(); p++) {
      const int sl = sc.slot(pw.item, (int)p);
      std::vector<LoadRef> lds;
      loads_of(g, (int)p, &lds);
      if (lds.empty()) continue;
      if (!value_of_slot.count(sl)) { read_from_memory.insert(sl); continue; }
      const std::string nm = strf("fw%zu", p);
      for (const LoadRef &l : lds) {
        if (g.lins[(size_t)l.lin].terms.empty()) return false;     // a fixed index into what the group itself writes
        m.preset[l.node] = nm;
      }
      lead += strf("%s%s %s", lead.empty() ? "" : ", ", dt_cname(g.params[p].dt), nm.c_str());
      lead_call += strf("%s%s", lead_call.empty() ? "" : ", ", value_of_slot[sl].c_str());
    }
    if (!internal_loads_replaced(sc, m, internal, -1)) return false;
    if (lead.empty()) { lead = "int poly_unused"; lead_call = "0"; }
    const std::string fn = strf("poly_pw_%zu", mi);
    const DT odt = g.n(g.stores[0].value).dt;
    if (!emit_member_fn(sc, m, "", fn.c_str(), dt_cname(odt), lead, g.stores[0].value, {}, false, false, &code)) return false;
    std::string args;
    for (size_t p = 0; p < g.params.size(); p++) {
      const int sl = sc.slot(pw.item, (int)p);
      if (p) args += ", ";
      if (internal.count(sl)) args += strf("(%s%s*)0", g.params[p].written ? "" : "const ", dt_cname(g.params[p].dt));
      else args += strf("fa%d", arg_of(sl));
    }
    body += strf("    o%zu[u] = %s(%s, pos + u, 0, 0, %s);\n", mi, fn.c_str(), lead_call.c_str(), args.c_str());
    value_of_slot[pw.out_slot] = strf("o%zu[u]", mi);
  }
  std::string sig;
  for (size_t j = 0; j < arg_slots.size(); j++) {
    const int sl = arg_slots[j];
    if (j) sig += ", ";
    // (a buffer the group both reads and writes is not declared restrict)
    if (written.count(sl)) sig += strf("%s* fa%zu", dt_cname(slot_dt[sl]), j);
    else sig += strf("const %s* __restrict__ fa%zu", dt_cname(slot_dt[sl]), j);
    // (a buffer updated in place moves twice: in and out)
    bytes += (double)s->buf_slots[sl].nbytes * ((read_from_memory.count(sl) ? 1 : 0) + (written.count(sl) ? 1 : 0));
    if (written.count(sl)) bytes_written += (double)s->buf_slots[sl].nbytes;
  }
  // the kernel for V positions per thread (the members themselves are per position)
  const auto kernel_for = [&](int V) {
    std::string src = std::string(hip_prelude()) + code;
    src += strf("extern \"C\" __global__ void __launch_bounds__(256) poly_k(%s) {\n", sig.c_str());
    src += strf("  const long long pos_ll = ((long long)blockIdx.x * 256 + threadIdx.x) * %d;\n  if (pos_ll >= %lldll) return;\n  const int pos = (int)pos_ll;\n", V, (long long)E);
    for (size_t mi = 0; mi < members.size(); mi++)
      src += strf("  %s o%zu[%d];\n", dt_cname(sc.graphs[(size_t)members[mi].item].n(sc.graphs[(size_t)members[mi].item].stores[0].value).dt), mi, V);
    src += strf("#pragma unroll\n  for (int u = 0; u < %d; u++) {\n", V) + body + "  }\n";
    for (size_t mi = 0; mi < members.size(); mi++) {
      const Pw &pw = members[mi];
      if (internal.count(pw.out_slot)) continue;
      const char *tn = dt_cname(slot_dt[pw.out_slot]);
      src += strf("  { poly_vec<%s, %d> st; for (int u = 0; u < %d; u++) st.v[u] = o%zu[u]; poly_vstore<%s, %d>(fa%d + pos, st); }\n", tn, V, V, mi, tn, V,
                  arg_of(pw.out_slot));
    }
    src += "}\n";
    return src;
  };
  const auto strategy_for = [&](int V) {
    return strf("%zu pointwise kernels over the same %lld positions as one, vec%d, %zu buffers never written out", members.size(), (long long)E, V,
                internal.size());
  };
  const std::string src = kernel_for(V);
  out->items.clear();
  for (const Pw &m : members) out->items.push_back(m.item);
  out->launch_item = members.back().item;
  out->internal_slots.assign(internal.begin(), internal.end());
  out->arg_slots = arg_slots;
  RenderedKernel &rk = out->rk;
  rk = RenderedKernel();
  rk.source = src;
  rk.entry = "poly_k";
  rk.launch.grid[0] = (unsigned)((E / V + 255) / 256);
  rk.launch.block[0] = 256;
  rk.klass = KernelClass::ELEMENTWISE;
  rk.strategy = strategy_for(V);
  rk.n_params = (int)arg_slots.size();
  rk.n_vars = 0;
  rk.bytes = bytes;
  rk.bytes_written = bytes_written;
  rk.flops = 0;
  if (matmul_tuning_enabled()) {
    // other widths of a thread's accesses: candidates of the search that POLY_BEAM switches on
    rk.variants.push_back({"default", rk.source, rk.strategy, rk.launch});
    for (int bytes_per : {16, 8, 4}) {
      const int v = std::max(1, bytes_per / maxsz);
      bool seen = v == V || E % v != 0;
      for (const RenderedKernel::Variant &o : rk.variants) if (o.label == strf("pw_vec%d", v)) seen = true;
      if (seen) continue;
      LaunchSpec ls = rk.launch;
      ls.grid[0] = (unsigned)((E / v + 255) / 256);
      rk.variants.push_back({strf("pw_vec%d", v), kernel_for(v), strategy_for(v), ls});
    }
    if (rk.variants.size() < 2) rk.variants.clear();
  }
  return true;
}

// ── small independent pointwise kernels, side by side ──────────────────────────
//
// A training step casts every fp32 bias and LayerNorm parameter to bf16 before the forward
// pass uses it: a kernel of one workgroup each, six per block of the model, spread over the
// schedule, and a launch costs more than its work.  Kernels of at most 16 384 positions
// without a reduction, with one ungated store at the flat position, that read only buffers
// nobody has written before them in the schedule (parameters, inputs) and whose output
// nobody else writes can run at the place of the first of them, in one launch: member i
// owns the workgroups [first_i, first_i+1) of the grid.
static bool match_side_by_side(const Sched &sc, int a_item, const std::vector<char> &taken, FusedGroup *out) {
  const PolySchedule *s = sc.s;
  if (getenv("POLY_HIP_NO_SIDE_BY_SIDE")) return false;
  struct Sb { int item, ord, out_slot, V; int64_t E; unsigned blocks; };
  auto candidate = [&](int item, Sb *sb) {
    const KernelGraph &g = sc.graphs[(size_t)item];
    if (!g.reduces.empty() || g.stores.size() != 1 || g.stores[0].gate >= 0 || !g.vars.empty()) return false;
    if (g.stores[0].ranges.size() != 1 || g.ranges.size() != 1) return false;
    const int ord = g.stores[0].ranges[0];
    const int64_t E = g.ranges[(size_t)ord].extent;
    if (E <= 0 || E > 16384) return false;
    auto is_flat = [&](const Lin &l) {
      if (l.c0 != 0 || l.terms.size() != 1 || l.terms[0].coef != 1) return false;
      const Atom &a = g.atoms[(size_t)l.terms[0].atom];
      return a.kind == Atom::RANGE && g.range_ord.at(a.node) == ord;
    };
    const int li = g.n(g.n(g.stores[0].index).src[1]).lin;
    if (li < 0 || !is_flat(g.lins[(size_t)li])) return false;
    if (g.n(g.stores[0].value).dt != g.n(g.stores[0].param).dt) return false;
    const int out_slot = sc.slot(item, g.param_slot(g.stores[0].param));
    if (!s->buf_slots[out_slot].is_intermediate || sc.writers[(size_t)out_slot].size() != 1 || s->buf_slots[out_slot].numel < E) return false;
    // (nobody reads the output in front of the kernel: such a reader would see it filled early)
    for (int r : sc.readers[(size_t)out_slot]) if (sc.step_of[(size_t)r] <= sc.step_of[(size_t)item]) return false;
    int maxsz = 1;
    for (size_t p = 0; p < g.params.size(); p++) {
      if (!dt_is_float(g.params[p].dt)) return false;
      maxsz = std::max(maxsz, dt_size(g.params[p].dt));
      const int sl = sc.slot(item, (int)p);
      if (sl == out_slot) { if (g.params[p].read) return false; continue; }
      // nobody writes what it reads before it runs (then it may as well run earlier)
      for (int w : sc.writers[(size_t)sl]) if (sc.step_of[(size_t)w] <= sc.step_of[(size_t)item]) return false;
      std::vector<LoadRef> lds;
      if (!loads_of(g, (int)p, &lds)) return false;
      for (const LoadRef &l : lds) {
        const Lin &lin = g.lins[(size_t)l.lin];
        if (!is_flat(lin) && !lin.terms.empty()) return false;
        if (is_flat(lin) && s->buf_slots[sl].numel < E) return false;
      }
    }
    // the output is not read before the member's own place in the schedule anyway; nobody
    // may read it in front of the launch either (nobody can: it has one writer, this kernel)
    int V = std::max(1, 16 / maxsz);
    while (V > 1 && E % V != 0) V /= 2;
    *sb = {item, ord, out_slot, V, E, (unsigned)((E / V + 255) / 256)};
    return true;
  };
  Sb first;
  if (!candidate(a_item, &first)) return false;
  std::vector<Sb> members{first};
  for (int st = sc.step_of[(size_t)a_item] + 1; st < s->n_items && members.size() < 24; st++) {
    const int k = s->exec_order[st];
    Sb sb;
    if (taken[(size_t)k] || !candidate(k, &sb)) continue;
    members.push_back(sb);
  }
  if (members.size() < 2) return false;
  std::vector<int> arg_slots;
  std::map<int, DT> slot_dt;
  std::set<int> written;
  for (const Sb &m : members) {
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    for (size_t p = 0; p < g.params.size(); p++) {
      const int sl = sc.slot(m.item, (int)p);
      if (written.count(sl)) return false;        // (a member reading another member's output: not independent)
      slot_dt[sl] = g.params[p].dt;
      if (std::find(arg_slots.begin(), arg_slots.end(), sl) == arg_slots.end()) arg_slots.push_back(sl);
    }
    written.insert(m.out_slot);
  }
  for (const Sb &m : members) {
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    for (size_t p = 0; p < g.params.size(); p++) {
      const int sl = sc.slot(m.item, (int)p);
      if (sl != m.out_slot && written.count(sl)) return false;
    }
  }
  auto arg_of = [&](int sl) { return (int)(std::find(arg_slots.begin(), arg_slots.end(), sl) - arg_slots.begin()); };
  std::string code, body;
  double bytes = 0;
  unsigned first_block = 0;
  for (size_t mi = 0; mi < members.size(); mi++) {
    const Sb &sb = members[mi];
    const KernelGraph &g = sc.graphs[(size_t)sb.item];
    Member m;
    m.item = sb.item;
    m.range_expr[sb.ord] = "m";
    const std::string fn = strf("poly_sb_%zu", mi);
    const DT odt = g.n(g.stores[0].value).dt;
    if (!emit_member_fn(sc, m, "", fn.c_str(), dt_cname(odt), "int poly_unused", g.stores[0].value, {}, false, false, &code)) return false;
    std::string args;
    for (size_t p = 0; p < g.params.size(); p++) args += strf("%sfa%d", p ? ", " : "", arg_of(sc.slot(sb.item, (int)p)));
    const char *tn = dt_cname(odt);
    body += strf("  %sif (blockIdx.x < %uu) {\n", mi ? "else " : "", first_block + sb.blocks);
    body += strf("    const int pos = (int)((blockIdx.x - %uu) * 256u + threadIdx.x) * %d;\n    if (pos < %lld) {\n", first_block, sb.V, (long long)sb.E);
    body += strf("      poly_vec<%s, %d> st;\n#pragma unroll\n      for (int u = 0; u < %d; u++) st.v[u] = %s(0, pos + u, 0, 0, %s);\n", tn, sb.V, sb.V, fn.c_str(), args.c_str());
    body += strf("      poly_vstore<%s, %d>(fa%d + pos, st);\n    }\n  }\n", tn, sb.V, arg_of(sb.out_slot));
    first_block += sb.blocks;
  }
  std::string sig;
  for (size_t j = 0; j < arg_slots.size(); j++) {
    const int sl = arg_slots[j];
    if (j) sig += ", ";
    if (written.count(sl)) sig += strf("%s* fa%zu", dt_cname(slot_dt[sl]), j);
    else sig += strf("const %s* __restrict__ fa%zu", dt_cname(slot_dt[sl]), j);
    bytes += (double)s->buf_slots[sl].nbytes;
  }
  std::string src = std::string(hip_prelude()) + code;
  src += strf("extern \"C\" __global__ void __launch_bounds__(256) poly_k(%s) {\n", sig.c_str()) + body + "}\n";
  out->items.clear();
  for (const Sb &m : members) out->items.push_back(m.item);
  out->launch_item = members.front().item;
  out->internal_slots.clear();
  out->arg_slots = arg_slots;
  RenderedKernel &rk = out->rk;
  rk = RenderedKernel();
  rk.source = src;
  rk.entry = "poly_k";
  rk.launch.grid[0] = first_block;
  rk.launch.block[0] = 256;
  rk.klass = KernelClass::ELEMENTWISE;
  rk.strategy = strf("%zu small independent pointwise kernels side by side in one launch", members.size());
  rk.n_params = (int)arg_slots.size();
  rk.n_vars = 0;
  rk.bytes = bytes;
  return true;
}

// ── ordered column sums, side by side ─────────────────────────────────────────
//
// The order-preserving column sums of a training step (bias and LayerNorm-parameter
// gradients that accumulate in bf16) are two kernels each: the terms, over the whole chip,
// and an adder of one thread per output whose time is a chain of dependent additions
// (48 us for 4096 terms) however few outputs there are.  Several of them that depend on
// nothing between them run as one pair of launches at the place of the first: the terms
// kernels on consecutive ranges of workgroups, and so the adders, each with its own part of
// the scratch memory.  The members are rendered as they would be alone and called as device
// functions with their workgroup number passed in.
static bool match_ordered_sums_side_by_side(const Sched &sc, int a_item, const std::vector<char> &taken, FusedGroup *out) {
  const PolySchedule *s = sc.s;
  if (getenv("POLY_HIP_NO_MERGED_ADDERS")) return false;
  struct Ad { int item, out_slot; RenderedKernel rk; };
  auto candidate = [&](int item, Ad *ad) {
    const KernelGraph &g = sc.graphs[(size_t)item];
    if (g.reduces.size() != 1 || g.stores.size() != 1 || !g.vars.empty()) return false;
    const int out_slot = sc.slot(item, g.param_slot(g.stores[0].param));
    if (s->buf_slots[out_slot].numel > 16384 || sc.writers[(size_t)out_slot].size() != 1) return false;
    // (nobody reads the output in front of the kernel: such a reader would see it filled early)
    for (int r : sc.readers[(size_t)out_slot]) if (sc.step_of[(size_t)r] <= sc.step_of[(size_t)item]) return false;
    std::string err;
    RenderedKernel rk;
    if (!render_kernel(g, "poly_m", RenderOptions(), &rk, &err)) return false;
    if (rk.klass != KernelClass::THREAD_REDUCE || rk.pres.size() != 1 || rk.strategy.rfind("ordered reduce, stage 1", 0) != 0 || !rk.guards.empty() ||
        !rk.tables.empty() || rk.variants.size() > 1 || rk.n_vars != 0 || !rk.fallback_source.empty() || rk.n_params != (int)g.params.size())
      return false;
    if (rk.launch.block[0] != 64 || rk.pres[0].launch.block[0] != 256 || rk.launch.grid[1] != 1 || rk.pres[0].launch.grid[1] != 1) return false;
    ad->item = item;
    ad->out_slot = out_slot;
    ad->rk = std::move(rk);
    return true;
  };
  std::vector<Ad> members(1);
  if (!candidate(a_item, &members[0])) return false;
  const int first_step = sc.step_of[(size_t)a_item];
  std::set<int> outs{members[0].out_slot};
  uint64_t threads = (uint64_t)members[0].rk.launch.grid[0] * 64;
  for (int st = first_step + 1; st < s->n_items && st < first_step + 96 && members.size() < 8; st++) {
    const int k = s->exec_order[st];
    if (taken[(size_t)k] || sc.graphs[(size_t)k].reduces.size() != 1) continue;
    // what it reads is there before the first member runs, and is no member's output
    const KernelGraph &g = sc.graphs[(size_t)k];
    bool ready = true;
    for (size_t p = 0; p < g.params.size() && ready; p++) {
      const int sl = sc.slot(k, (int)p);
      if (outs.count(sl)) ready = false;
      if (!g.params[p].read) continue;
      for (int w : sc.writers[(size_t)sl]) if (w != k && sc.launch_step[(size_t)w] >= first_step) ready = false;
    }
    if (!ready) continue;
    Ad ad;
    if (!candidate(k, &ad)) continue;
    if (threads + (uint64_t)ad.rk.launch.grid[0] * 64 > 65536) break;
    threads += (uint64_t)ad.rk.launch.grid[0] * 64;
    outs.insert(ad.out_slot);
    members.push_back(std::move(ad));
  }
  if (members.size() < 2) return false;
  // a kernel as a device function of its workgroup number
  const std::string prelude = hip_prelude();
  auto as_device_fn = [&](const std::string &src, const std::string &entry, const std::string &name, std::string *fn) {
    if (src.compare(0, prelude.size(), prelude) != 0) return false;
    std::string t = src.substr(prelude.size());
    const std::string head = "extern \"C\" __global__ void __launch_bounds__(";
    if (t.compare(0, head.size(), head) != 0) return false;        // (helpers of its own in front: names could clash)
    const size_t open = t.find(entry + "(");
    if (open == std::string::npos || open > 128) return false;
    t = "__device__ __forceinline__ void " + name + "(const unsigned int poly_bid, " + t.substr(open + entry.size() + 1);
    for (size_t at = t.find("blockIdx.x"); at != std::string::npos; at = t.find("blockIdx.x", at)) t.replace(at, 10, "poly_bid");
    if (t.find("blockIdx") != std::string::npos || t.find("__shared__") != std::string::npos) return false;
    *fn = t;
    return true;
  };
  std::vector<int> arg_slots;
  std::map<int, DT> slot_dt;
  std::set<int> written;
  for (const Ad &m : members) {
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    for (size_t p = 0; p < g.params.size(); p++) {
      const int sl = sc.slot(m.item, (int)p);
      if (slot_dt.count(sl) && slot_dt[sl] != g.params[p].dt) return false;
      slot_dt[sl] = g.params[p].dt;
      if (g.params[p].written) written.insert(sl);
      if (std::find(arg_slots.begin(), arg_slots.end(), sl) == arg_slots.end()) arg_slots.push_back(sl);
    }
  }
  auto arg_of = [&](int sl) { return (int)(std::find(arg_slots.begin(), arg_slots.end(), sl) - arg_slots.begin()); };
  std::string code, pre_body, main_body;
  size_t scratch = 0;
  unsigned pre_blocks = 0, main_blocks = 0;
  double bytes = 0;
  for (size_t mi = 0; mi < members.size(); mi++) {
    const Ad &m = members[mi];
    const KernelGraph &g = sc.graphs[(size_t)m.item];
    std::string f1, f2;
    if (!as_device_fn(m.rk.pres[0].source, m.rk.pres[0].entry, strf("poly_terms_%zu", mi), &f1) ||
        !as_device_fn(m.rk.source, m.rk.entry, strf("poly_adder_%zu", mi), &f2))
      return false;
    code += f1 + f2;
    std::string args;
    for (size_t p = 0; p < g.params.size(); p++) args += strf("fa%d, ", arg_of(sc.slot(m.item, (int)p)));
    args += strf("(float*)((char*)poly_scratch + %zuull)", scratch);
    pre_body += strf("  %sif (blockIdx.x < %uu) poly_terms_%zu(blockIdx.x - %uu, %s);\n", mi ? "else " : "", pre_blocks + m.rk.pres[0].launch.grid[0], mi,
                     pre_blocks, args.c_str());
    main_body += strf("  %sif (blockIdx.x < %uu) poly_adder_%zu(blockIdx.x - %uu, %s);\n", mi ? "else " : "", main_blocks + m.rk.launch.grid[0], mi,
                      main_blocks, args.c_str());
    pre_blocks += m.rk.pres[0].launch.grid[0];
    main_blocks += m.rk.launch.grid[0];
    scratch += (m.rk.scratch_bytes + 255) / 256 * 256;
    bytes += m.rk.bytes;
  }
  if (scratch > ((size_t)1 << 30)) return false;
  std::string sig;
  for (size_t j = 0; j < arg_slots.size(); j++) {
    const int sl = arg_slots[j];
    if (written.count(sl)) sig += strf("%s* fa%zu, ", dt_cname(slot_dt[sl]), j);
    else sig += strf("const %s* __restrict__ fa%zu, ", dt_cname(slot_dt[sl]), j);
  }
  sig += "float* poly_scratch";
  const std::string common = prelude + code;
  out->items.clear();
  for (const Ad &m : members) out->items.push_back(m.item);
  out->launch_item = members.front().item;
  out->internal_slots.clear();
  out->arg_slots = arg_slots;
  RenderedKernel &rk = out->rk;
  rk = RenderedKernel();
  RenderedKernel::Pre pre;
  pre.source = common + strf("extern \"C\" __global__ void __launch_bounds__(256) poly_k(%s) {\n", sig.c_str()) + pre_body + "}\n";
  pre.entry = "poly_k";
  pre.launch.grid[0] = pre_blocks;
  pre.launch.block[0] = 256;
  rk.pres.push_back(pre);
  rk.source = common + strf("extern \"C\" __global__ void __launch_bounds__(64) poly_k(%s) {\n", sig.c_str()) + main_body + "}\n";
  rk.entry = "poly_k";
  rk.launch.grid[0] = main_blocks;
  rk.launch.block[0] = 64;
  rk.scratch_bytes = scratch;
  rk.klass = KernelClass::THREAD_REDUCE;
  rk.strategy = strf("%zu ordered column sums side by side (terms in one launch, adders in one): ", members.size()) + members[0].rk.strategy;
  rk.n_params = (int)arg_slots.size();
  rk.n_vars = 0;
  rk.bytes = bytes;
  return true;
}

// Which groups launch at a place that breaks a dependence of the schedule: for two items
// that touch the same buffer, at least one of them writing, the launch of the earlier one
// (its group's, if a group has taken it) must not come behind the launch of the later one.
// A check of the matchers from scratch, on the host: they each reason about their own
// members, this looks at every pair.
// Does buffer `slot` only ever receive bf16 values cast to fp32?  (an intermediate with one
// writer, whose one ungated store has such a cast as its value; what the writer leaves out
// is either never read or filled with zeros)
static bool slot_holds_bf16_values(const PolySchedule *s, const std::vector<KernelGraph> &graphs, int slot) {
  if (slot < 0 || slot >= s->n_buf_slots || !s->buf_slots[slot].is_intermediate) return false;
  int writer = -1;
  for (int k = 0; k < s->n_items; k++) {
    const PolyExecItem &it = s->items[k];
    const KernelGraph &g = graphs[(size_t)k];
    for (size_t q = 0; q < g.params.size() && (int)q < it.n_buf_slots; q++)
      if (it.buf_slot_indices[q] == slot && g.params[q].written) {
        if (writer >= 0 && writer != k) return false;
        writer = k;
      }
  }
  if (writer < 0) return false;
  const KernelGraph &g = graphs[(size_t)writer];
  if (g.stores.size() != 1 || g.stores[0].gate >= 0) return false;
  const StoreInfo &st = g.stores[0];
  const int p = g.param_slot(st.param);
  if (p < 0 || p >= s->items[writer].n_buf_slots || s->items[writer].buf_slot_indices[p] != slot) return false;
  const KNode &v = g.n(st.value);
  return g.n(st.param).dt == DT_F32 && v.op == POLY_OP_CAST && v.dt == DT_F32 && v.src.size() == 1 && g.n(v.src[0]).dt == DT_BF16;
}

std::vector<int> matmul_param_kinds_of(const PolySchedule *s, const std::vector<KernelGraph> &graphs, int item, const std::vector<int> &narrow_slots) {
  std::vector<int> kinds;
  if (getenv("POLY_HIP_NO_EXACT16_BUFFERS")) return kinds;
  const PolyExecItem &it = s->items[item];
  const KernelGraph &g = graphs[(size_t)item];
  kinds.assign((size_t)it.n_buf_slots, 0);
  for (int p = 0; p < it.n_buf_slots && (size_t)p < g.params.size(); p++) {
    if (g.params[(size_t)p].dt != DT_F32 || g.params[(size_t)p].written) continue;
    const int sl = it.buf_slot_indices[p];
    if (!slot_holds_bf16_values(s, graphs, sl)) continue;
    kinds[(size_t)p] = std::find(narrow_slots.begin(), narrow_slots.end(), sl) != narrow_slots.end() ? 2 : 1;
  }
  return kinds;
}

std::vector<int> fused_groups_out_of_order(const PolySchedule *s, const std::vector<KernelGraph> &graphs, const std::vector<FusedGroup> &groups) {
  std::vector<int> step_of((size_t)s->n_items, 0), group_of((size_t)s->n_items, -1), pos((size_t)s->n_items, 0);
  for (int st = 0; st < s->n_items; st++) step_of[(size_t)s->exec_order[st]] = st;
  for (size_t gi = 0; gi < groups.size(); gi++) for (int it : groups[gi].items) group_of[(size_t)it] = (int)gi;
  for (int k = 0; k < s->n_items; k++) pos[(size_t)k] = group_of[(size_t)k] >= 0 ? step_of[(size_t)groups[(size_t)group_of[(size_t)k]].launch_item] : step_of[(size_t)k];
  struct Use { int step, item; bool w; };
  std::vector<std::vector<Use>> uses((size_t)s->n_buf_slots);
  for (int k = 0; k < s->n_items; k++) {
    const PolyExecItem &it = s->items[k];
    const KernelGraph &g = graphs[(size_t)k];
    for (int i = 0; i < it.n_buf_slots && i < (int)g.params.size(); i++) {
      const int sl = it.buf_slot_indices[i];
      if (sl < 0 || sl >= s->n_buf_slots) continue;
      uses[(size_t)sl].push_back({step_of[(size_t)k], k, g.params[(size_t)i].written});
    }
  }
  std::set<int> bad;
  for (auto &u : uses) {
    std::sort(u.begin(), u.end(), [](const Use &a, const Use &b) { return a.step < b.step; });
    // (against every write only: two reads need no order)
    for (size_t j = 0; j < u.size(); j++) {
      if (!u[j].w) continue;
      for (size_t i = 0; i < u.size(); i++) {
        if (i == j || u[i].item == u[j].item) continue;
        const Use &a = i < j ? u[i] : u[j], &b = i < j ? u[j] : u[i];
        if (pos[(size_t)a.item] <= pos[(size_t)b.item]) continue;
        if (group_of[(size_t)a.item] >= 0) bad.insert(group_of[(size_t)a.item]);
        if (group_of[(size_t)b.item] >= 0) bad.insert(group_of[(size_t)b.item]);
      }
    }
  }
  return std::vector<int>(bad.begin(), bad.end());
}

void find_fused_groups(const PolySchedule *s, const std::vector<KernelGraph> &graphs, std::vector<FusedGroup> *out) {
  out->clear();
  if (getenv("POLY_HIP_NO_FUSION")) return;
  Sched sc{s, graphs, {}, {}, {}, {}};
  sc.step_of.assign((size_t)s->n_items, 0);
  for (int st = 0; st < s->n_items; st++) sc.step_of[(size_t)s->exec_order[st]] = st;
  sc.launch_step = sc.step_of;
  auto accept = [&](FusedGroup &fg, std::vector<char> &taken) {
    for (int it : fg.items) { taken[(size_t)it] = 1; sc.launch_step[(size_t)it] = sc.step_of[(size_t)fg.launch_item]; }
    out->push_back(std::move(fg));
  };
  sc.readers.assign((size_t)s->n_buf_slots, {});
  sc.writers.assign((size_t)s->n_buf_slots, {});
  for (int k = 0; k < s->n_items; k++) {
    const PolyExecItem &it = s->items[k];
    const KernelGraph &g = graphs[(size_t)k];
    if ((int)g.params.size() != it.n_buf_slots) return;
    for (int i = 0; i < it.n_buf_slots; i++) {
      const int sl = it.buf_slot_indices[i];
      if (sl < 0 || sl >= s->n_buf_slots) return;
      if (g.params[(size_t)i].read) sc.readers[(size_t)sl].push_back(k);
      if (g.params[(size_t)i].written) sc.writers[(size_t)sl].push_back(k);
    }
  }
  for (auto &v : sc.readers) { std::sort(v.begin(), v.end()); v.erase(std::unique(v.begin(), v.end()), v.end()); }
  std::vector<char> taken((size_t)s->n_items, 0);
  for (int st = 0; st < s->n_items; st++) {
    const int k = s->exec_order[st];
    if (taken[(size_t)k] || graphs[(size_t)k].reduces.size() != 1) continue;
    FusedGroup fg;
    if (!match_attention(sc, k, taken, &fg) && !match_matmul_tail(sc, k, taken, &fg) && !match_row_chain(sc, k, taken, &fg)) continue;
    fg.matched_from = k;
    accept(fg, taken);
  }
  // what is left of the pointwise kernels, in runs over the same positions
  for (int st = 0; st < s->n_items; st++) {
    const int k = s->exec_order[st];
    if (taken[(size_t)k] || !graphs[(size_t)k].reduces.empty()) continue;
    FusedGroup fg;
    if (!match_pointwise_group(sc, k, taken, &fg)) continue;
    accept(fg, taken);
  }
  // the order-preserving column sums that are left, several to a launch
  for (int st = 0; st < s->n_items; st++) {
    const int k = s->exec_order[st];
    if (taken[(size_t)k] || graphs[(size_t)k].reduces.size() != 1) continue;
    FusedGroup fg;
    if (!match_ordered_sums_side_by_side(sc, k, taken, &fg)) continue;
    accept(fg, taken);
  }
  // small kernels that depend on nothing computed in the plan, wherever they stand
  for (int st = 0; st < s->n_items; st++) {
    const int k = s->exec_order[st];
    if (taken[(size_t)k] || !graphs[(size_t)k].reduces.empty()) continue;
    FusedGroup fg;
    if (!match_side_by_side(sc, k, taken, &fg)) continue;
    accept(fg, taken);
  }
  // A row chain whose result is an fp32 buffer of bf16 values (the derivative of the scores
  // of attention: a cast of a bf16 product), read by one product that can take it as a
  // 16-bit operand where it lies: the chain stores the bf16 values, the product reads them,
  // and nothing writes or reads the values as fp32 (half the bytes written, no planes).
  for (size_t gi = 0, n0 = out->size(); gi < n0 && !getenv("POLY_HIP_NO_NARROW_STORE"); gi++) {
    const int slot = (*out)[gi].row_chain_stores;
    if (slot < 0 || !slot_holds_bf16_values(s, graphs, slot)) continue;
    if (std::find((*out)[gi].internal_slots.begin(), (*out)[gi].internal_slots.end(), slot) != (*out)[gi].internal_slots.end()) continue;
    const std::vector<int> &rd = sc.readers[(size_t)slot];
    if (rd.size() != 1 || sc.writers[(size_t)slot].size() != 1 || taken[(size_t)rd[0]]) continue;
    const int reader = rd[0];
    if (sc.step_of[(size_t)reader] <= sc.step_of[(size_t)(*out)[gi].launch_item]) continue;
    FusedGroup rg;
    matmul_hint_param_kinds(matmul_param_kinds_of(s, graphs, reader, {slot}));
    std::string err;
    const bool reads = render_kernel(graphs[(size_t)reader], "poly_k", RenderOptions(), &rg.rk, &err) && rg.rk.klass == KernelClass::MATMUL_MFMA &&
                       rg.rk.guards.empty() && rg.rk.n_vars == 0 && rg.rk.n_params == s->items[reader].n_buf_slots;
    matmul_hint_param_kinds({});
    if (!reads) continue;
    // the chain once more, with the other store
    std::vector<char> free_again = taken;
    for (int it : (*out)[gi].items) free_again[(size_t)it] = 0;
    FusedGroup chain;
    g_narrow_store_slot = slot;
    const bool stores = match_row_chain(sc, (*out)[gi].row_chain_from, free_again, &chain) && chain.items == (*out)[gi].items &&
                        chain.launch_item == (*out)[gi].launch_item;
    g_narrow_store_slot = -1;
    if (!stores) continue;
    (*out)[gi] = std::move(chain);
    (*out)[gi].needs_group_at = reader;
    rg.needs_group_at = (*out)[gi].launch_item;
    rg.items = {reader};
    rg.launch_item = reader;
    rg.arg_slots.assign(s->items[reader].buf_slot_indices, s->items[reader].buf_slot_indices + s->items[reader].n_buf_slots);
    accept(rg, taken);
  }
  // An attention kernel that passes over masked key blocks must first compute their
  // products, unless it knows how large the keys can be.  Where the keys are columns of a
  // product's output (the q | k | v projection), that product's epilogue has every key in
  // its registers: it leaves the largest magnitude of each block of 64 keys x 64 features
  // in the attention kernel's scratch memory, and the attention kernel bounds the products
  // of a block by that times the sum of |q|.  Both groups are matched once more, knowing of
  // each other.
  for (size_t gi = 0, n0 = out->size(); gi < n0 && !getenv("POLY_HIP_NO_KEY_BOUNDS"); gi++) {
    const FusedGroup::KeyBounds kb = (*out)[gi].key_bounds;
    if (!kb.possible || kb.used || (*out)[gi].matched_from < 0 || sc.writers[(size_t)kb.slot].size() != 1) continue;
    size_t pj = n0;
    for (size_t j = 0; j < n0; j++)
      if (j != gi && (*out)[j].matched_from >= 0 && (*out)[j].rk.klass == KernelClass::MATMUL_MFMA && !(*out)[j].arg_slots.empty() &&
          (*out)[j].arg_slots[0] == kb.slot && (*out)[j].rk.scratch_of_item < 0 && (*out)[j].needs_group_at < 0 &&
          (*out)[j].launch_item == sc.writers[(size_t)kb.slot][0])
        pj = j;
    if ((*out)[gi].needs_group_at >= 0) continue;
    const int w_item = sc.writers[(size_t)kb.slot][0];
    if (pj == n0 && taken[(size_t)w_item]) continue;
    int first_step = sc.step_of[(size_t)(*out)[gi].items[0]];
    for (int it : (*out)[gi].items) first_step = std::min(first_step, sc.step_of[(size_t)it]);
    if (sc.step_of[(size_t)w_item] >= first_step) continue;
    std::vector<char> free_again = taken;
    FusedGroup product;
    bool writes = false;
    if (pj < n0) {
      // the product and the pointwise kernels in its epilogue
      for (int it : (*out)[pj].items) free_again[(size_t)it] = 0;
      g_block_maxima_hint = kb;
      writes = match_matmul_tail(sc, (*out)[pj].matched_from, free_again, &product) && product.items == (*out)[pj].items &&
               product.launch_item == (*out)[pj].launch_item;
      g_block_maxima_hint = FusedGroup::KeyBounds();
      product.matched_from = (*out)[pj].matched_from;
    } else {
      // a product by itself: lowered here as the plan would lower it, with the wish
      const PolyExecItem &wi = s->items[w_item];
      uint64_t inputs = 0;
      for (int p = 0; p < wi.n_buf_slots && p < 64; p++) {
        const int sl = wi.buf_slot_indices[p];
        if (!s->buf_slots[sl].is_intermediate && sc.writers[(size_t)sl].empty()) inputs |= (uint64_t)1 << p;
      }
      MatmulEpilogue wish;
      wish.block_maxima.wanted = true;
      wish.block_maxima.lo = kb.lo;
      wish.block_maxima.hi = kb.hi;
      wish.block_maxima.index = kb.index;
      wish.block_maxima.bytes = kb.bytes;
      matmul_hint_input_params(inputs);
      matmul_hint_param_kinds(matmul_param_kinds_of(s, graphs, w_item, {}));
      matmul_hint_block_maxima(&wish, kb.rows, kb.pitch);
      std::string err;
      writes = render_kernel(graphs[(size_t)w_item], "poly_k", RenderOptions(), &product.rk, &err) && product.rk.klass == KernelClass::MATMUL_MFMA &&
               product.rk.guards.empty() && product.rk.n_vars == 0 && product.rk.n_params == wi.n_buf_slots;
      matmul_hint_block_maxima(nullptr, 0, 0);
      matmul_hint_param_kinds({});
      matmul_hint_input_params(0);
      product.items = {w_item};
      product.launch_item = w_item;
      product.arg_slots.assign(wi.buf_slot_indices, wi.buf_slot_indices + wi.n_buf_slots);
    }
    writes = writes && product.rk.writes_block_maxima && product.rk.scratch_bytes == kb.bytes && product.rk.pres_key.empty();
    if (!writes) continue;
    free_again = taken;
    for (int it : (*out)[gi].items) free_again[(size_t)it] = 0;
    FusedGroup attention;
    g_key_bounds_slot = kb.slot;
    const bool reads = match_attention(sc, (*out)[gi].matched_from, free_again, &attention) && attention.items == (*out)[gi].items &&
                       attention.launch_item == (*out)[gi].launch_item && attention.key_bounds.used && attention.key_bounds.bytes == kb.bytes;
    g_key_bounds_slot = -1;
    if (!reads) continue;
    attention.matched_from = (*out)[gi].matched_from;
    product.rk.scratch_of_item = attention.launch_item;
    product.rk.scratch_offset = attention.key_bounds.offset;
    product.needs_group_at = attention.launch_item;
    attention.needs_group_at = product.launch_item;
    if (getenv("POLY_HIP_DEBUG"))
      fprintf(stderr, "polygrad: compile_schedule: the product at kernel %d leaves the block maxima of the keys for the attention kernel at kernel %d\n",
              product.launch_item, attention.launch_item);
    (*out)[gi] = std::move(attention);
    if (pj < n0) (*out)[pj] = std::move(product);
    else accept(product, taken);
  }
  // every pair of items that share a buffer keeps its order; a group that breaks one is
  // dropped and its kernels launch one by one at their own places
  for (;;) {
    const std::vector<int> bad = fused_groups_out_of_order(s, graphs, *out);
    if (bad.empty()) break;
    std::vector<int> partners;      // launch items of groups that go with a dropped one
    for (size_t i = bad.size(); i-- > 0;) {
      log_err("compile_schedule", "fused group at kernel %d (%zu kernels: %s) would launch out of order with a kernel it shares a buffer with: dropped",
              (*out)[(size_t)bad[i]].launch_item, (*out)[(size_t)bad[i]].items.size(), (*out)[(size_t)bad[i]].rk.strategy.substr(0, 60).c_str());
      if ((*out)[(size_t)bad[i]].needs_group_at >= 0) partners.push_back((*out)[(size_t)bad[i]].needs_group_at);
      out->erase(out->begin() + bad[i]);
    }
    for (int at : partners)
      for (size_t i = out->size(); i-- > 0;)
        if ((*out)[i].launch_item == at && (*out)[i].needs_group_at >= 0) out->erase(out->begin() + (long)i);
  }
}

}  // namespace polyhip
