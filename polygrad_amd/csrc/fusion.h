// Plan-level fusion of kernel groups (see fusion.cc).
#pragma once
#include <string>
#include <vector>

#include "polygrad_abi.h"
#include "templates.h"

namespace polyhip {

// A set of schedule items replaced by one launch.
struct FusedGroup {
  std::vector<int> items;           // schedule items the fused kernel stands for
  int launch_item = -1;             // the fused kernel runs at this item's place in exec_order
  std::vector<int> internal_slots;  // buffers that are never materialised
  std::vector<int> arg_slots;       // slot of each kernel argument, in order
  RenderedKernel rk;
  // a row chain: the item it was grown from and the buffer its last kernel stores (-1: none)
  int row_chain_from = -1, row_chain_stores = -1;
  // Two groups that only work together (a chain that stores bf16 values into an fp32 buffer
  // and the product that reads them as such) name each other's launch item here: dropping
  // one drops the other.
  int needs_group_at = -1;
  int matched_from = -1;            // the item the matcher started from
  // An attention group whose keys lie in the output of a product, in blocks of 64 keys x 64
  // features that are blocks of 64 rows x 64 columns there (row-major, `pitch` columns,
  // `rows` rows): what that product would have to leave for the kernel to bound the
  // products of masked key blocks without computing them (MatmulEpilogue::block_maxima).
  struct KeyBounds {
    bool possible = false, used = false;
    int slot = -1;
    int64_t pitch = 0, rows = 0, lo = 0, hi = 0;
    std::string index;
    size_t bytes = 0, offset = 0;   // of the table, and where it lies in the kernel's scratch memory
  } key_bounds;
};

// Finds the fusable groups of a schedule.  graphs[k] is the analysed kernel of item k.
// Setting POLY_HIP_NO_FUSION in the environment disables the search.
void find_fused_groups(const PolySchedule *s, const std::vector<KernelGraph> &graphs, std::vector<FusedGroup> *out);
// The groups (indices into `groups`) whose place of launch breaks the order of two kernels
// of the schedule that share a buffer, one of them writing it; find_fused_groups drops such
// groups itself, so that its result always passes.
std::vector<int> fused_groups_out_of_order(const PolySchedule *s, const std::vector<KernelGraph> &graphs, const std::vector<FusedGroup> &groups);

// What matmul_hint_param_kinds takes for the lowering of item `item`: 1 for every fp32
// buffer parameter that is an intermediate of the plan with one writer, whose one store
// puts a bf16 value cast to fp32 there (2 where `narrow_slots` names the buffer: its writer
// has been made to store the bf16 values themselves).
std::vector<int> matmul_param_kinds_of(const PolySchedule *s, const std::vector<KernelGraph> &graphs, int item, const std::vector<int> &narrow_slots);

}  // namespace polyhip
