// Kernel graph analysis: turns one scheduled kernel root (a SINK over
// END*(STORE(INDEX(PARAM, idx[, gate]), value), RANGE...)) into an indexed DAG
// with per-node range dependencies and a canonical form for every integer
// index expression.  Nothing here touches the GPU.
//
// The shape of a scheduled root follows the reference scheduler's output
// (src/rangeify.c:1527-1699 builds PARAM/INDEX/LOAD/STORE, :2932-3061 wraps
// stores in END over their ranges).
#pragma once
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace polyhip {

// ── canonical integer expressions ─────────────────────────────────────────
// Lin = c0 + sum(coef_i * atom_i).  Atoms are range variables, DEFINE_VARs,
// opaque integer nodes, or floor-div / mod of a non-negative Lin by a positive
// constant.  Bounds are tracked so that (x*c + y)/c -> x and (..)%c -> (..)
// can be applied exactly when the reference's own simplifier would.
struct Term { int64_t coef; int atom; };
struct Lin {
  std::vector<Term> terms;  // sorted by atom id, no zero coefs
  int64_t c0 = 0;
  bool is_const() const { return terms.empty(); }
};
struct Atom {
  enum Kind { RANGE, VAR, OPAQUE, DIV, MOD } kind;
  int node = -1;   // kernel node id for RANGE / VAR / OPAQUE
  Lin inner;       // for DIV / MOD
  int64_t c = 0;   // divisor for DIV / MOD
  int64_t lo = 0, hi = 0;
};

struct KNode {
  const PolyUOp *u = nullptr;
  PolyOps op;
  DT dt = DT_VOID;
  bool is_ptr = false;
  std::vector<int> src;
  uint64_t deps = 0;   // bitset over KernelGraph::ranges ordinals
  int lin = -1;        // index into KernelGraph::lins when integer-analysable
  int n_uses = 0;
  // LOADs whose only consumer is one branch of WHERE(cond, ., .) are predicated
  // on that condition, as the reference folds them into gated loads
  // (cond ? *p : 0); their index may be out of bounds when cond is false.
  // A REDUCE in that position carries the condition too: its serial loop is skipped
  // where the branch is not taken.
  int guard = -1;
  bool guard_neg = false;
};

struct RangeInfo {
  int node;            // KNode id of the RANGE
  int64_t extent;      // constant trip count, or -1 when bound is symbolic
  int bound_node;      // KNode id of the bound expression
  bool is_reduce;      // closed by a REDUCE (true) or by an END (false)
  int64_t axis_id;
};

struct StoreInfo {
  int store;           // STORE node
  int index;           // INDEX node (src[0] of STORE)
  int param;           // PARAM node
  int value;           // stored value node
  int gate = -1;       // optional gate (INDEX src[2])
  std::vector<int> ranges;  // range ordinals, outermost first
};

struct ParamInfo {
  int node;
  int index;           // PARAM arg.i == position in args[]
  DT dt;
  int64_t numel;       // ptr_size (-1 unknown)
  bool written = false;
  bool read = false;
};

struct VarInfo { int node; std::string name; int64_t lo, hi; };

struct KernelGraph {
  std::vector<KNode> nodes;               // topological order, sink last
  std::unordered_map<const PolyUOp *, int> ids;
  std::vector<RangeInfo> ranges;
  std::unordered_map<int, int> range_ord; // RANGE node id -> ordinal
  std::vector<StoreInfo> stores;
  std::vector<ParamInfo> params;          // sorted by PARAM index
  std::vector<VarInfo> vars;              // in first-seen order
  std::vector<int> reduces;               // REDUCE node ids, topological
  std::vector<Atom> atoms;
  std::vector<Lin> lins;
  std::string error;

  // One slab of a kernel, set before build(): RANGE `slab_range` runs over
  // [slab_lo, slab_lo + slab_extent) only (the graph's range counts from 0 and every use
  // sees range + slab_lo), and every STORE takes `slab_value` in place of its value.
  const PolyUOp *slab_range = nullptr, *slab_value = nullptr;
  int64_t slab_lo = 0, slab_extent = 0;
  std::vector<const PolyUOp *> slab_params;   // every PARAM of the whole kernel: a slab keeps its argument list

  bool build(const PolyUOp *root);

  // canonical-expression helpers
  int atom_for_node(int node, Atom::Kind kind, int64_t lo, int64_t hi);
  int intern_atom(const Atom &a);
  Lin lin_const(int64_t c) const { Lin l; l.c0 = c; return l; }
  Lin lin_atom(int atom) const { Lin l; l.terms.push_back({1, atom}); return l; }
  Lin lin_add(const Lin &a, const Lin &b, int64_t sb = 1) const;
  Lin lin_scale(const Lin &a, int64_t s) const;
  Lin lin_recombine(const Lin &a) const;
  Lin lin_div(const Lin &a, int64_t c);
  Lin lin_mod(const Lin &a, int64_t c);
  void lin_bounds(const Lin &a, int64_t *lo, int64_t *hi) const;
  // Set when a coefficient or constant of a canonical form left the 64-bit range (only a
  // damaged graph gets there): build() then fails instead of lowering nonsense.
  mutable bool lin_overflow = false;
  // coefficient of RANGE ordinal `ord` in `l`; *affine=false when `l` holds a
  // non-affine atom that depends on that range.
  int64_t lin_range_coef(const Lin &l, int ord, bool *affine) const;
  bool lin_is_affine(const Lin &l) const;  // only RANGE/VAR atoms
  uint64_t lin_deps(const Lin &l) const;
  uint64_t atom_deps(int atom) const;

  const KNode &n(int id) const { return nodes[(size_t)id]; }
  int param_slot(int param_node) const;   // position in params[]
  // Self-check of the canonical forms: evaluates every index-typed node both from
  // its raw ops and from its Lin at `samples` range assignments (all of them when
  // the iteration space is small).  Returns the number of mismatches.
  int check_lins(int samples, std::string *first_bad) const;
};

const char *op_name(PolyOps op);

}  // namespace polyhip
