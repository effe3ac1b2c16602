// Internal C++ face of the device runtime (the C ABI wraps these).
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "common.h"
#include "render_hip.h"

namespace polyhip {

struct Program;  // one kernel entry inside a loaded (shared) module

int runtime_init();
void *runtime_stream();
// Further streams (same priority; k in [0, kSideStreams)) for launches that a plan's
// captured graph lets run beside the main sequence, and the switch that sends the following
// program_launch calls to one of them (nullptr: back to the main stream).
constexpr int kSideStreams = 3;
void *runtime_side_stream(int k);
void runtime_launch_on(void *stream);
void *runtime_alloc(size_t nbytes);
void runtime_free(void *p);
// kind: 0 host->device, 1 device->host, 2 device->device; returns once done
int runtime_copy(void *dst, const void *src, size_t n, int kind);
int runtime_memset(void *p, int value, size_t n);
int runtime_sync();
// Can a kernel dereference `p`?  False for pageable host memory (malloc, numpy arrays, the
// host-side constant registry of the frontend) and for addresses HIP does not know.
bool runtime_device_can_read(const void *p);
// A device buffer of `bytes` bytes filled once by running kernel `entry(T* out)` of
// `source` with the given launch; identical sources share one buffer.
std::shared_ptr<void> runtime_table(const std::string &source, const std::string &entry, size_t bytes, const LaunchSpec &ls);

// Directory of the on-disk caches (code objects, tuning decisions); empty when disabled.
std::string runtime_cache_dir();
bool compile_to_code_object(const std::string &source, std::vector<char> *code, std::string *log);
Program *program_create(const std::string &source, const std::string &entry);
void program_destroy(Program *p);
int program_launch(Program *p, void **kernel_args, const LaunchSpec &ls);

// What program_launch does with a launch besides (or instead of) enqueueing it, for plans
// that keep their launch sequence as a hipGraph:
//   record: the stream is under capture; after the launch, the kernel node it became is
//           appended to `nodes` (failed is set when the capture does not name exactly one);
//   update: nothing is enqueued; the arguments of the call go to node nodes[next++] of the
//           instantiated graph `exec` (hipGraphExecKernelNodeSetParams), the way to bind a
//           captured sequence to other buffers without capturing it again.
struct GraphLaunches {
  std::vector<void *> nodes;     // hipGraphNode_t, in launch order
  void *exec = nullptr;          // hipGraphExec_t (update)
  size_t next = 0;
  bool failed = false;
};
void runtime_graph_record(GraphLaunches *g);    // nullptr: back to plain launches
void runtime_graph_update(GraphLaunches *g);
// While `t` is set every kernel launch carries a pair of events that the dispatch itself
// stamps at the kernel's first and last cycle (hipExtModuleLaunchKernel), appended to
// t->events as (start, stop): what a profiler reports as the kernel's duration, without
// the time a launch waits in the queue.  The caller destroys the events.
struct LaunchTimes { std::vector<void *> events; bool failed = false; };
void runtime_time_launches(LaunchTimes *t);

// One lowered kernel: the program(s) plus how to call them.
struct HipRunner {
  RenderedKernel rk;
  Program *main = nullptr;
  std::vector<Program *> guards;
  Program *fallback = nullptr;
  std::vector<Program *> pres;     // first stage(s) of a two-stage kernel
  void *scratch = nullptr;         // what they leave for the main kernel
  bool owns_scratch = true;        // false: the memory belongs to a pool shared with other runners
  bool skip_pres = false;          // the scratch memory already holds what the first stages would write
  void *flag = nullptr;            // device int written by the guards
  std::vector<std::shared_ptr<void>> tables;   // filled lookup tables (shared between identical kernels)
  std::string name;
  std::vector<void *> vetted;      // per buffer parameter: the last pointer found to be device-readable
  std::vector<void *> ptr_store;   // argument storage reused by every launch
  std::vector<int> var_store;
  std::vector<void *> arg_ptrs;
};

HipRunner *runner_create(const PolyUOp *root, const char *fn_name, int flags);
// From a kernel rendered elsewhere (fused groups); `named` false: the entry is still the
// placeholder poly_k and gets its descriptive symbol here.
HipRunner *runner_from_rendered(const RenderedKernel &rk, const char *fn_name, bool named);
// Replaces the runner's own scratch memory by `pool` (at least rk.scratch_bytes large, owned
// by the caller, who runs the runners sharing it one after the other on the stream).
void runner_share_scratch(HipRunner *r, void *pool);
// Allocates the runner's own scratch memory if its kernel runs in two stages and it has
// none yet (neither its own nor a shared pool).  Launches under stream capture need it in
// place beforehand.
int runner_ensure_scratch(HipRunner *r);
// `scratch_from_caller`, when non-NULL, is used as the two-stage scratch memory of this
// launch (at least rk.scratch_bytes large) and the runner allocates none of its own.
int runner_launch(HipRunner *r, void **args, int n_args, void *scratch_from_caller = nullptr);
// Switches the runner to rk.variants[idx] (compiles it if needed); the runner is unchanged
// when that fails.
int runner_use_variant(HipRunner *r, int idx);
void runner_destroy(HipRunner *r);

}  // namespace polyhip
