"""Runs the generated HIP kernels of a schedule ON THE HOST, thread by thread, under
AddressSanitizer, to check their indexing: every global load and store of every
thread of every workgroup must stay inside its buffer, and every LDS access inside its
array.  The kernels are compiled as plain C++ for x86-64 with a small shim (threadIdx
and friends as globals, GPU intrinsics as pass-throughs, MFMAs as no-ops): values are
meaningless -- there is no cross-lane exchange and no barrier -- but addresses in these
kernels never depend on loaded values, so the access pattern is the real one.

Test infrastructure only: nothing in the product path uses it.  No GPU needed."""
import ctypes as C
import os
import re
import subprocess
import tempfile

from polygrad_amd import _ffi

CLANG = "/opt/rocm/llvm/bin/clang++"

SHIM = r"""
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <cstdint>
struct poly_dim3 { unsigned x, y, z; };
static poly_dim3 threadIdx, blockIdx, blockDim, gridDim;
#define POLY_HOST_ADDRESS_CHECK 1
#define __device__
#define __global__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define amdgpu_waves_per_eu(...)
#define __shared__ static
#define __constant__ static const
#define __syncthreads() ((void)0)
#define __lane_id() (threadIdx.x & 63u)
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) (src)
#define __builtin_amdgcn_ds_swizzle(v, pat) (v)
#define __builtin_amdgcn_readlane(v, lane) (v)
#define __builtin_amdgcn_readfirstlane(v) (v)
#define __builtin_amdgcn_ds_bpermute(addr, v) (v)
#define __builtin_amdgcn_ballot_w64(p) ((p) ? ~0ull : 0ull)
#define __builtin_amdgcn_fence(...) ((void)0)
#define __builtin_amdgcn_wave_barrier() ((void)0)
#define __builtin_amdgcn_sched_barrier(m) ((void)0)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_div_fixupf(q, d, x) (q)
template <class T> static T atomicAdd(T *p, T v) { T old = *p; *p += v; return old; }
template <class T> static T atomicMax(T *p, T v) { T old = *p; if (old < v) *p = v; return old; }
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) (c)
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) (c)
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) (c)
"""

DRIVER_TAIL = r"""
extern "C" float __ocml_sin_f32(float x) { return sinf(x); }
extern "C" double __ocml_sin_f64(double x) { return sin(x); }
int main() {
  gridDim = {GX, GY, GZ};
  blockDim = {BX, 1, 1};
  void *bufs[NBUF + 1];
  static const size_t sizes[NBUF + 1] = {SIZES 0};
  for (int i = 0; i < NBUF; i++) {
    bufs[i] = malloc(sizes[i]);          // exact size: ASan guards both ends
    memset(bufs[i], 1, sizes[i]);        // (no zeros: integer kernels divide by their inputs)
  }
  for (unsigned bz = 0; bz < GZ; bz++)
    for (unsigned by = 0; by < GY; by++)
      for (unsigned bx = 0; bx < GX; bx += STRIDE)
        for (unsigned tx = 0; tx < BX; tx++) {
          blockIdx = {bx, by, bz};
          threadIdx = {tx, 0, 0};
          ENTRY(ARGS);
        }
  for (int i = 0; i < NBUF; i++) free(bufs[i]);
  puts("ok");
  return 0;
}
"""


def _arg_types(source, entry):
    """Parameter types of kernel `entry`, from its definition in the source (templates
    take their parameter list from the POLY_SIGNATURE line of their configuration)."""
    head = source[source.index(" " + entry + "(") + len(entry) + 2:]
    depth, end = 1, 0
    while depth:
        ch = head[end]
        depth += ch == "("
        depth -= ch == ")"
        end += 1
    text = head[:end - 1].strip()
    if text == "POLY_SIGNATURE":
        text = [ln for ln in source.splitlines() if ln.startswith("#define POLY_SIGNATURE ")][0][len("#define POLY_SIGNATURE "):]
    params = [p.strip() for p in text.split(",")]
    return [p.rsplit(" ", 1)[0].replace("__restrict__", "").strip() for p in params]


def _arg_names(source, entry):
    head = source[source.index(" " + entry + "(") + len(entry) + 2:]
    text = head[:head.index(")")].strip()
    if text == "POLY_SIGNATURE":
        text = [ln for ln in source.splitlines() if ln.startswith("#define POLY_SIGNATURE ")][0][len("#define POLY_SIGNATURE "):]
    return [p.strip().rsplit(" ", 1)[-1].lstrip("*") for p in text.split(",")]


def _entry_name(source):
    line = [ln for ln in source.splitlines() if ln.startswith('extern "C" __global__')][-1]
    return [m for m in re.findall(r"(\w+)\s*\(", line) if m.startswith("poly_")][-1]


def check_kernel(source, entry, grid, block, buf_sizes, block_stride=1, timeout=600, scratch_bytes=0):
    """Compiles `source` for the host and runs kernel `entry` over its whole launch (or
    every `block_stride`-th workgroup along x) with exact-size buffers.  Raises with the
    sanitizer's report on an out-of-bounds access."""
    types = _arg_types(source, entry)
    assert len(types) >= len(buf_sizes), (entry, types, buf_sizes)
    # what follows the buffers: DEFINE_VAR ints (passed as 0) and lookup tables (65536 entries of at most 16 bytes)
    names = _arg_names(source, entry)
    buf_sizes = list(buf_sizes) + [scratch_bytes if names[i] == "poly_scratch" else 65536 * 16
                                   for i, t in enumerate(types) if i >= len(buf_sizes) and "*" in t]
    args = ", ".join(f"({t})bufs[{i}]" if "*" in t else "0" for i, t in enumerate(types))
    tail = (DRIVER_TAIL.replace("GX", str(grid[0])).replace("GY", str(grid[1])).replace("GZ", str(grid[2]))
            .replace("BX", str(block)).replace("NBUF", str(len(buf_sizes))).replace("STRIDE", str(block_stride))
            .replace("SIZES", "".join(f"{int(s)}, " for s in buf_sizes)).replace("ENTRY", entry).replace("ARGS", args))
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "k.cc")
        exe = os.path.join(d, "k")
        with open(src, "w") as f:
            f.write(SHIM + source + tail)
        cc = subprocess.run([CLANG, "-std=c++17", "-O1", "-g", "-fsanitize=address", "-fno-omit-frame-pointer", "-w", src, "-o", exe],
                            capture_output=True, text=True)
        if cc.returncode != 0:
            raise RuntimeError(f"host build of {entry} failed:\n{cc.stderr[-3000:]}")
        run = subprocess.run([exe], capture_output=True, text=True, timeout=timeout)
        if run.returncode != 0 or "ok" not in run.stdout:
            raise AssertionError(f"{entry}: out-of-bounds access on the host run\n{run.stderr[-4000:]}")


def _jobs(lib, schedule, max_threads, only, groups):
    s = C.cast(schedule, C.POINTER(_ffi.PolySchedule)).contents
    seen = set()
    for step in range(s.n_items):
        if only is not None and step not in only:
            continue
        it = s.items[s.exec_order[step]]
        launch = (C.c_int * 7)()
        text = _ffi.take_string(lib.poly_hip_render(it.root, b"k", 0, launch))
        if "\n// ---- guard" in text:
            continue                    # guarded fast path: its arguments include a flag set by another kernel
        main = text.split("\n// ---- ")[0]
        sizes = tuple(max(int(s.buf_slots[it.buf_slot_indices[p]].nbytes), 4) for p in range(it.n_buf_slots))
        if (main, sizes) in seen:
            continue
        seen.add((main, sizes))
        grid = (launch[0], launch[1], launch[2])
        scratch = 0
        for unit in text.split("\n// ---- ")[1:]:
            m = re.match(r"first stage ---- grid=(\d+),(\d+) block=(\d+) scratch=(\d+)\n", unit)
            if m:       # first stage of a two-stage kernel: same arguments plus the scratch, its own launch
                scratch = int(m.group(4))
                yield f"step {step} (first stage)", unit[m.end():], (int(m.group(1)), int(m.group(2)), 1), int(m.group(3)), sizes, scratch
        yield f"step {step}", main, grid, launch[3], sizes, scratch
    if not groups or only is not None:
        return
    for gi in range(lib.poly_hip_fused_groups(schedule, -1, None, None)):
        src = C.c_void_p()
        lib.poly_hip_fused_groups(schedule, gi, C.byref(src), None)
        text = _ffi.take_string(src.value)
        main = text.split("\n// ---- ")[0]
        slots = (C.c_int * 64)()
        launch = (C.c_int * 4)()
        n = lib.poly_hip_fused_group_launch(schedule, gi, slots, 64, launch)
        assert 0 < n <= 64
        sizes = tuple(max(int(s.buf_slots[slots[i]].nbytes), 4) for i in range(n))
        if (main, sizes) in seen:
            continue
        seen.add((main, sizes))
        scratch = 0
        for unit in text.split("\n// ---- ")[1:]:
            m = re.match(r"scratch ---- bytes=(\d+)\n", unit)
            if m:       # scratch memory without a first stage (a product that leaves values for a later launch)
                scratch = int(m.group(1))
            m = re.match(r"first stage ---- grid=(\d+),(\d+) block=(\d+) scratch=(\d+)\n", unit)
            if m:
                scratch = int(m.group(4))
                yield f"group {gi} (first stage)", unit[m.end():], (int(m.group(1)), int(m.group(2)), 1), int(m.group(3)), sizes, scratch
        yield f"group {gi}", main, (launch[0], launch[1], launch[2]), launch[3], sizes, scratch


def check_schedule(lib, schedule, max_threads=1 << 21, only=None, groups=True, workers=6):
    """Host-checks every distinct kernel of `schedule`: each scheduled kernel as the
    per-kernel lowering renders it (guarded fast paths aside) and each fused group of the
    plan-level lowering.  Launches larger than `max_threads` threads are sampled by
    workgroup.  Returns the number of kernels checked; raises on the first failure."""
    from concurrent.futures import ThreadPoolExecutor

    def one(job):
        what, main, grid, block, sizes, scratch = job
        threads = grid[0] * grid[1] * grid[2] * block
        try:
            check_kernel(main, _entry_name(main), grid, block, sizes, block_stride=max(1, threads // max_threads), scratch_bytes=scratch)
        except Exception as e:
            raise AssertionError(f"{what}: {e}") from e
        return 1

    with ThreadPoolExecutor(max_workers=workers) as pool:
        return sum(pool.map(one, list(_jobs(lib, schedule, max_threads, only, groups))))
