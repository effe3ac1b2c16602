// Pattern matches shared by the single-kernel templates (templates.cc) and the
// plan-level fusion of kernel groups (fusion.cc).
#pragma once
#include <string>
#include <vector>

#include "render_hip.h"

namespace polyhip {

// One operand of a matmul product: LOAD(INDEX(PARAM, lin)) optionally under a CAST to f32.
struct MmOperand {
  int load = -1, param = -1, lin = -1;   // param: position in KernelGraph::params
  DT dt = DT_VOID;
};

// off(k) = (k / kb) * s_hi + (k % kb) * s_lo ; kb >= K means a plain stride s_lo
struct KSplit { int64_t kb, s_hi, s_lo; };

// One output coordinate: a digit of an END range.  A range r that the indices use
// only through r / a, r % b and (r / a) % b is a mixed-radix number; each digit
// d = (r / cut) % extent becomes a coordinate of its own (a plain range is the
// single digit with cut 1).  ca / cb: coefficient in the A / B operand index.
struct MmDim { int ord; int64_t extent, ca, cb; int64_t cut = 1; };

// Structure of a kernel of the form STORE(f(REDUCE(ADD, cast(A[..]) * cast(B[..]), k))).
struct MatmulMatch {
  int red = -1, kr = -1;        // REDUCE node, ordinal of the reduce range
  int64_t K = 0, M = 1, N = 1, Z = 1;
  MmOperand A, B;
  KSplit ka{0, 0, 0}, kb{0, 0, 0};
  // digits of the END ranges, outermost first: those only A depends on (M), only B (N),
  // both or neither (Z); *_full keep every digit, the others merge digits that nest
  std::vector<MmDim> md, nd, zd, md_full, nd_full, zd_full;
  int64_t a_c0 = 0, b_c0 = 0;   // constant parts of the operand indices
};

bool match_matmul(const KernelGraph &g, MatmulMatch *mm, int *reject_line);

// C text that splits the flattened coordinates `m`, `n`, `z` (ints in scope) into the
// kernel's END ranges, declared as `const int r<ord>`; binds them in `em` when given.
std::string matmul_decompose(const MatmulMatch &mm, Emitter *em);
// "__device__ int name(int x)": offset contribution of a flattened coordinate.
std::string matmul_offset_fn(const char *name, const std::vector<MmDim> &dims, bool use_a, int64_t c0);
std::string matmul_k_fn(const char *name, const KSplit &ks, int64_t K);
// Host-side evaluation of the same maps (used to cross-check fused groups).
int64_t matmul_eval_offset(const std::vector<MmDim> &dims, bool use_a, int64_t x);
// value of END range `ord` at flattened coordinates (m, n, z)
int64_t matmul_range_value(const MatmulMatch &mm, int ord, int64_t m, int64_t n, int64_t z);

// What the MFMA template does with each accumulator: the kernel's signature, which of
// its pointers are the operands, device functions, and the statement (in terms of acc, m,
// n, z) that finishes one output element.
struct MatmulEpilogue {
  std::string signature, a_ptr, b_ptr, code;
  std::string call;        // statement storing one element: uses acc, m, n, z
  // Optional split of `call` into value and address, for outputs that are contiguous
  // along n: the template then stores 8 values of a row with one 16-byte store.
  std::string value_call;  // expression of type out_type: uses acc, m, n, z
  std::string value_call_win;   // the same value with table lookups served from LDS windows (sets poly_tmax), or empty
  std::string ptr_call;    // expression of type out_type*: uses m, n, z
  std::string out_type;
  // A value the chain passes through that other kernels read as well (the pre-activation of
  // a layer whose backward pass wants it): stored too, where the output is stored and with
  // its layout (contiguous form only).  Value in terms of acc, m, n, z; address; element type.
  std::string mid_value_call, mid_ptr_call, mid_type;
  bool out_16bit = false;  // the stored element is a 16-bit float, whatever the form of the store
  bool contiguous_n = false;
  int n_params = 0;
  double bytes = 0;    // algorithmic bytes of the whole kernel
  // When `signature` already ends in a `poly_scratch` parameter (operands staged there by
  // first-stage kernels): its element type and the bytes in use, so that a split-K product
  // can put its partial results behind them.  Empty: no such parameter yet.
  std::string scratch_type;
  size_t scratch_used = 0;
  // Lookup tables the epilogue reads (parameters `poly_lut<i>` at the end of `signature`,
  // in front of any scratch pointer), and the argument list that goes with `signature`.
  std::vector<RenderedKernel::Table> tables;
  int table_parts = 0;     // parts of the epilogue that the tables stand for (parts of one load share a table)
  std::string params_call;
  // Operand B is a buffer that nothing in the plan writes (weights): at the time of the
  // launch it is in HBM, not in the caches.
  bool b_from_hbm = false;
  // A later launch reads the columns [lo, hi) of the output (row-major, one z) in blocks of
  // 64 rows x 64 columns and wants the largest magnitude in each: the product then leaves
  // it, as the bits of the float, in word `index` (C text in terms of the block's first
  // row m and column n) of its scratch memory.  Only the template that loads straight into
  // LDS does that, on tiles of whole blocks; RenderedKernel::writes_block_maxima says
  // whether it did.
  struct BlockMaxima {
    bool wanted = false;
    int64_t lo = 0, hi = 0;
    std::string index;
    size_t bytes = 0;      // of the table
  } block_maxima;
};
// Set by the plan compiler around the lowering of one scheduled kernel: bit p says that
// buffer parameter p is an input of the plan that none of its kernels writes.
void matmul_hint_input_params(uint64_t mask);
// Also set around a lowering: what the plan knows of the kernel's buffer parameters that
// are fp32 in the schedule.  kinds[p] = 1: every value the buffer receives is a bf16 value
// cast to fp32 (its one writer stores such a cast), so that a product may take it as the
// one bf16 plane it is.  kinds[p] = 2: the writer was made to store those bf16 values
// themselves, at the same element indices (the buffer read as a 16-bit one); only a product
// that takes the buffer as a plain operand can read that, and render_kernel refuses every
// other use.
void matmul_hint_param_kinds(const std::vector<int> &kinds);
// Also set around a lowering: a later launch wants the block maxima of this product's
// output, which it takes for a row-major matrix of `rows` x `pitch` elements from element 0
// of the buffer (nullptr: no such wish).  The product grants it when its store is that.
struct MatmulEpilogue;
void matmul_hint_block_maxima(const MatmulEpilogue *with_block_maxima, int64_t rows, int64_t pitch);
int matmul_param_kind(int param);
// Is element (m, n + 1) of the kernel's output stored right after (m, n), for every n
// that is not the last of an aligned group of 8?  (store index affine with coefficient 1
// on the innermost digit of n, digits not crossed inside a group)
bool matmul_store_contiguous(const KernelGraph &g, const MatmulMatch &mm, const Lin &store_lin);
// Chooses layouts and tile shape and instantiates kernels/matmul_mfma.hip.  With tuning
// enabled (POLY_BEAM > 0 in the environment, the switch of the reference's own search,
// src/render_c.c:839) the other tile shapes come along as RenderedKernel::variants.
bool matmul_tuning_enabled();
bool render_matmul(const MatmulMatch &mm, const MatmulEpilogue &ep, RenderedKernel *out);

bool try_render_matmul(const KernelGraph &g, const std::string &fn, const RenderOptions &opt, RenderedKernel *out);
// Matmul-shaped reductions of computed operands (mixed dtypes, derivatives fused into an
// operand, several reduce ranges, ragged extents) on the fp32 MFMA template.
bool try_render_matmul_generic(const KernelGraph &g, const std::string &fn, const RenderOptions &opt, RenderedKernel *out);
bool try_render_gather(const KernelGraph &g, const std::string &fn, const RenderOptions &opt, RenderedKernel *out);

}  // namespace polyhip
