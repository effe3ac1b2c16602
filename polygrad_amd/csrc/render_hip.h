// render_hip: lowers one analysed kernel graph to gfx950 HIP C source plus a
// launch description.  Replaces (does not port) the reference's CUDA lowering
// (src/render_cuda.c:176-570, src/codegen.c:4149-4581): all non-reduce ranges
// are flattened over the grid, accesses are vectorised to 128 bit when the
// fastest index is unit-stride, row reductions run one wave or one workgroup
// per row with DPP/ds_swizzle wave reductions, and matmul-shaped reductions are
// handed to the MFMA template.
#pragma once
#include <algorithm>
#include <cstdlib>
#include <functional>
#include <string>
#include <unordered_map>
#include <vector>

#include "kgraph.h"

namespace polyhip {

// How the kernel is launched.  Sizes may depend on DEFINE_VAR values when a
// range bound is symbolic; then `dyn_*` describe how to recompute them.
struct LaunchSpec {
  unsigned grid[3] = {1, 1, 1};
  unsigned block[3] = {256, 1, 1};
  unsigned lds_bytes = 0;
};

enum class KernelClass { ELEMENTWISE, ROW_REDUCE, THREAD_REDUCE, MATMUL_MFMA, GATHER, COPY, ATTENTION };
inline const char *kernel_class_name(KernelClass k) {
  static const char *const names[] = {"elementwise", "row-reduce", "thread-reduce", "matmul-mfma", "gather", "copy", "attention-mfma"};
  const int i = (int)k;
  return i >= 0 && i < (int)(sizeof(names) / sizeof(names[0])) ? names[i] : "unknown";
}

struct RenderedKernel {
  std::string source;      // complete HIP C translation unit
  std::string entry;       // kernel symbol
  LaunchSpec launch;
  KernelClass klass = KernelClass::ELEMENTWISE;
  std::string strategy;    // human-readable summary for dumps and profiles
  int n_params = 0;        // buffer parameters (args[0..n_params-1])
  int n_vars = 0;          // DEFINE_VAR ints appended after the buffers
  std::vector<const void *> var_uops;   // the DEFINE_VAR UOps, in the order of those ints
  // Algorithmic work of one launch, for roofline accounting.
  double bytes = 0;        // distinct buffer elements touched * element size
  double bytes_written = 0;   // the part of `bytes` that the kernel stores (0 where a renderer does not say)
  bool rereads_inputs = false;   // a later phase of the kernel reads from memory what an earlier one read (rows too long to keep)
  double flops = 0;        // 2*M*N*K for matmul-shaped kernels, else 0
  // Guarded fast paths: a small check kernel must succeed for the fast kernel
  // to be valid; otherwise `fallback` runs (always the generic lowering).
  struct Guard {
    std::string source, entry;
    LaunchSpec launch;
    std::vector<int> arg_params;   // which buffer params the check reads
  };
  std::vector<Guard> guards;
  // Lookup tables the kernel reads: `source` holds a kernel `entry(T* out)` that fills
  // `bytes` bytes once, when the runner is created; the table pointers follow the
  // buffer and variable arguments of every launch (before the guard flag).
  struct Table {
    std::string source, entry;
    size_t bytes = 0;
    LaunchSpec launch;
  };
  std::vector<Table> tables;
  std::string fallback_source, fallback_entry;
  LaunchSpec fallback_launch;
  // The same kernel in other configurations (tile shapes): candidates for timing on the
  // device.  Empty unless tuning is enabled; otherwise variants[0] is `source` itself.
  // Every variant takes the same arguments and writes the same values.
  struct Variant {
    std::string label, source, strategy;
    LaunchSpec launch;
  };
  std::vector<Variant> variants;
  // A matrix product whose own first workgroups read operand B into the memory-side cache
  // (the plan then launches nothing ahead of it for that).
  bool reads_b_ahead = false;
  // A product that leaves the largest magnitude of every 64 x 64 block of some of its output
  // columns in its scratch memory (MatmulEpilogue::block_maxima) -- and, set by the plan-level
  // fusion, whose scratch memory that is: the launch that reads the bounds keeps them in its
  // own scratch memory, `scratch_offset` bytes in, and the plan hands this kernel that
  // address as its scratch pointer (`scratch_of_item`: the reader's launch item; -1: none).
  bool writes_block_maxima = false;
  int scratch_of_item = -1;
  size_t scratch_offset = 0;
  // Kernels in two stages (reductions through partial results, matmuls whose operands are
  // prepared first): `pres` run first, in order, with the same arguments plus one more
  // pointer to `scratch_bytes` bytes of device memory that the runner owns; the main
  // kernel takes that pointer too (after the variables and tables).
  struct Pre {
    std::string source, entry;
    LaunchSpec launch;
  };
  std::vector<Pre> pres;
  size_t scratch_bytes = 0;
  // Set when what the first stages leave in the scratch memory depends on nothing but the
  // contents of the buffers bound to the arguments `pre_reads` (indices into the kernel's
  // buffer parameters) and the main kernel only reads it: `pres_key` then identifies the
  // computation (the text of the first stages before they get their symbol names), and a
  // plan runs it once for all launches that share key and buffers, as long as nothing
  // writes those buffers in between.
  std::string pres_key;
  std::vector<int> pre_reads;
  // What the first stages of a product of computed operands leave at the start of the
  // scratch memory: operand A as `parts` bf16 planes per row ([z][row][part][k]), with a
  // description of the operand that does not name ranges -- its arithmetic over its loads,
  // and every load's address as base + by_row[row] + by_k[k] + by_z[z].  A later kernel
  // of the same launch whose operand A is the same values with rows and depth exchanged
  // reads these planes instead of writing its own (the slabs of the derivative of a
  // q | k | v split: dS K and dS^T Q).
  struct OperandPlanes {
    bool valid = false;
    std::string dag;
    struct Load { int param, dt; int64_t base; std::vector<int64_t> by_row, by_k, by_z; };
    std::vector<Load> loads;
    int64_t rows = 0, k = 0, z = 0;
    int parts = 0;
  } a_planes;
  bool reads_planes_before = false;   // this kernel's operand A is the planes of RenderOptions::planes_before
  // loads from fp32 buffers that hold bf16 values instead (matmul_hint_param_kinds, kind 2)
  // that the kernel reads as such; -1: a launch of several kernels, each checked by itself
  int narrow_loads = 0;
};

struct Scope;
class Emitter;
struct RenderOptions {
  bool allow_templates = true;   // MFMA matmul / gather fast paths
  bool allow_vectorize = true;
  bool allow_coop_reduce = true;
  int block = 256;
  // When set, the kernel takes one more argument `const int* poly_flag` after the
  // vars and returns at once if *poly_flag != 0 (the slow twin of a guarded fast path).
  bool exit_if_flag = false;
  // The fast twin: same extra argument, returns at once if *poly_flag == 0.
  bool exit_unless_flag = false;
  // REDUCE nodes whose value the caller computes without a loop (gather fast
  // path); the kernel is then lowered as if it had no such reduction.
  std::unordered_map<int, std::function<std::string(Emitter &, Scope *)>> reduce_override;
  // First stage of a two-stage reduction: the ranges of REDUCE node `promote_reduce` count
  // as output ranges (fastest), the reductions nested in its operand are the ones that run,
  // and what would be one term of that REDUCE goes to poly_scratch[row].
  int promote_reduce = -1;
  // The kernel takes `float* poly_scratch` as its last pointer argument.
  bool scratch_param = false;
  // Another first stage: one thread per (output, part); REDUCE node `slice_reduce` walks
  // range ordinal `slice_range` from its part number in steps of `slice_parts`, and the
  // partial result goes to poly_scratch[output * slice_parts + part].
  int slice_reduce = -1, slice_range = -1, slice_parts = 0;
  // The order-preserving reduction as two kernels: stage 1 writes every term to
  // poly_scratch[((k / 4) * outputs + output) * 4 + k % 4] (four terms per thread, lanes
  // along the outputs), stage 2 adds them in index order, one thread per output.
  // 0: one kernel.
  int ordered_stage = 0;
  // Lanes along the reduce range only when some load is contiguous along it, however few
  // rows there are (otherwise: only from 65536 rows up).
  bool coop_needs_unit_stride = false;
  // Operand planes that an earlier kernel of the same launch leaves at the start of the
  // scratch memory (see RenderedKernel::OperandPlanes).
  const RenderedKernel::OperandPlanes *planes_before = nullptr;
};

// Returns false and sets *err on unsupported graphs (never falls back to a
// host path).
bool render_kernel(const KernelGraph &g, const std::string &fn_name, const RenderOptions &opt,
                   RenderedKernel *out, std::string *err);

// ── expression emitter shared by the generic path and the templates ───────
struct Scope {
  uint64_t avail = 0;   // range ordinals bound in this scope (including parents)
  std::string code;
  std::unordered_map<int, std::string> names;       // node id -> C name
  std::unordered_map<int, std::string> atom_names;  // atom id -> C name
  Scope *parent = nullptr;
  int indent = 1;
};

class Emitter {
 public:
  explicit Emitter(const KernelGraph &g) : g_(g) {}
  // Binds a range ordinal to a C expression (a variable name).
  void bind_range(int ord, const std::string &name) { range_name_[ord] = name; }
  // Overrides the value of a node (vector-loaded values, reduce results, ...).
  void preset(int node, const std::string &expr) { preset_[node] = expr; }
  void clear_preset(int node) { preset_.erase(node); }
  bool is_preset(int node) const { return preset_.count(node) != 0; }
  // a preset that holds one value for all positions the emitted code walks (a row's sum in
  // a kernel that walks the row): what divides by it shares its reciprocal
  void preset_shared(int node) { shared_presets_.push_back(node); }
  bool is_shared_preset(int node) const { return std::find(shared_presets_.begin(), shared_presets_.end(), node) != shared_presets_.end(); }
  // Replaces the serial loop of a REDUCE node by caller-generated code; the
  // callback receives the scope the value is placed in and returns its C name.
  void custom_reduce(int node, std::function<std::string(Scope *)> fn) { custom_[node] = std::move(fn); }
  // The serial loop of REDUCE `node` takes range `ord` from `first` in steps of `step`.
  void slice_reduce(int node, int ord, const std::string &first, int step) { slice_node_ = node; slice_ord_ = ord; slice_first_ = first; slice_step_ = step; }
  bool has_custom(int node) const { return custom_.count(node) != 0; }
  void stmt(Scope *s, const std::string &line);
  std::string emit(int node, Scope *s);
  std::string emit_lin(const Lin &l, Scope *s);
  std::string load_expr(int load_node, Scope *s);
  // Serial reduction of REDUCE node `id` placed in scope `s`.
  std::string emit_reduce_serial(int id, Scope *s);
  static std::string float_literal(double v, DT dt);
  static std::string reduce_identity(PolyOps op, DT dt);
  static std::string reduce_combine(PolyOps op, DT dt, const std::string &acc, const std::string &v);
  bool failed() const { return !error_.empty(); }
  const std::string &error() const { return error_; }
  bool uses_threefry = false;
  // f32 EXP2 as the bare hardware instruction: results below 2^-126 come out as 0 instead
  // of denormals (the library form wraps the instruction in a range-scaling sequence).
  bool raw_exp2 = false;
  // A 16-bit float value times a power-of-two constant is kept in fp32 instead of being
  // rounded back to 16 bits: the product is exactly representable unless it drops below
  // the smallest normal number, so the only values that change are products under 2^-126.
  bool pow2_mul16_exact = false;
  // cast16(a / b) becomes cast16(a * (1 / b)) with the reciprocal placed where b is
  // computed (outside the loops b does not depend on): the fp32 quotient may differ in its
  // last bit, which the 16-bit rounding hides except at rounding ties.
  bool recip_div16 = false;
  // a / b in fp32 where b varies in fewer loops than a: poly_div_shared with the reciprocal
  // of b placed where b is computed (the same quotient, four instructions instead of eleven)
  bool shared_divisor = getenv("POLY_HIP_NO_SHARED_DIVISOR") == nullptr;

 private:
  bool shared_division(DT dt, int num, int den, Scope *t, std::string *e);
  std::string emit_atom(int atom, Scope *s);
  bool light_body(int root, int ord) const;
  std::string emit_raw(int node, Scope *s);
  Scope *place(uint64_t deps, Scope *s);
  const KernelGraph &g_;
  std::unordered_map<int, std::string> range_name_;
  std::unordered_map<int, std::string> preset_;
  std::vector<int> shared_presets_;
  std::unordered_map<int, std::function<std::string(Scope *)>> custom_;
  int slice_node_ = -1, slice_ord_ = -1, slice_step_ = 1;
  std::string slice_first_;
  std::string error_;
};

// Pieces of the generic lowering that fused kernels reuse.
// Can `l` be accessed as a V-wide vector along range ordinal F (unit stride in F, every
// other contribution a multiple of V)?  With `any_alignment` only the unit stride is asked
// for: vector loads and stores to global memory need no more than element alignment.
bool lin_vec_ok(const KernelGraph &g, const Lin &l, int F, int V, bool any_alignment = false);
void mark_reachable(const KernelGraph &g, int root, std::vector<char> &mark);
// Emits V-wide vector loads into `outer` for every LOAD under `roots` that is unit-stride
// along F (starting at the C expression f0) and presets those nodes to "<name>.v[u]";
// returns the preset nodes.
// `wrap`, when given, may replace the load expression of an ungated LOAD node (e.g. by a
// value kept from an earlier pass over the same addresses).
std::vector<int> hoist_vector_loads(const KernelGraph &g, Emitter &em, const std::vector<int> &roots, int F, int V,
                                    const std::string &f0, Scope *outer,
                                    const std::function<std::string(int, const std::string &)> *wrap = nullptr,
                                    bool any_alignment = false);
// C expression reducing `v` over the 64 lanes of a wave.
// (lanes: 64, or 32 for a reduction over each half of the wave by itself)
std::string wave_reduce_call(PolyOps op, DT dt, const std::string &v, int lanes = 64);

// Prelude with the wave/workgroup reduction helpers and small utilities that
// every generated kernel may use.
const char *hip_prelude();

}  // namespace polyhip
