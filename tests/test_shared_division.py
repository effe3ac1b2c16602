"""Division by a value that many dividends share (a row's sum, a row's deviation): the
generated code multiplies by the divisor's reciprocal and corrects once with the exact
remainder (poly_div_shared in the kernel prelude, csrc/emitter.cc).  The reference's CPU
backend divides (src/render_c.c emits `a / b`), so the result has to be the correctly
rounded quotient.

On the host: the same arithmetic in C (fmaf) against `x / d`, bit for bit, over all
exponents the fast path admits and the significands that make rounding awkward.
On the GPU: the prelude's own function, compiled by the backend, against the division the
same kernel computes, including the operands that must take the full division."""
import ctypes as C
import os
import subprocess
import tempfile

import numpy as np
import pytest

HOST_C = r"""
#include <math.h>
#include <stdint.h>
#include <string.h>
static uint64_t s = 88172645463325252ull;
static uint64_t rnd(void) { s ^= s << 13; s ^= s >> 7; s ^= s << 17; return s; }
static float mk(int elo, int ehi, int kind) {
  uint32_t m = (uint32_t)rnd() & 0x7fffff;
  if (kind == 1) m = 0x7fffff;            /* all ones */
  if (kind == 2) m = 0;                   /* a power of two */
  if (kind == 3) m = 1;                   /* just above one */
  if (kind == 4) m = 0x7ffffe;
  int e = elo + (int)(rnd() % (uint64_t)(ehi - elo + 1));
  uint32_t b = ((uint32_t)(e + 127) << 23) | m | ((rnd() & 1) ? 0x80000000u : 0);
  float f; memcpy(&f, &b, 4); return f;
}
/* the fast path of poly_div_shared */
static float fast(float x, float d, float r) {
  float q = x * r;
  float e = fmaf(-q, d, x);
  return fmaf(e, r, q);
}
/* mismatches with x / d for |d| in 2^[-100, 100], |x| in 2^[xlo, 26] */
long count_mismatches(int xlo, long divisors, long per_divisor) {
  long bad = 0;
  for (long i = 0; i < divisors; i++) {
    float d = mk(-100, 100, (int)(i % 6));
    volatile float r = 1.0f / d;
    for (long j = 0; j < per_divisor; j++) {
      float x = mk(xlo, 25, (int)(j % 7));
      float want = x / d, got = fast(x, d, r);
      if (memcmp(&want, &got, 4) != 0) bad++;
    }
  }
  return bad;
}
/* largest error in units of the last place of the quotient (2^-149 for a subnormal one) for dividends below 2^-102 */
double worst_tiny_ulps(long divisors, long per_divisor) {
  double worst = 0;
  for (long i = 0; i < divisors; i++) {
    float d = mk(-100, 100, (int)(i % 6));
    volatile float r = 1.0f / d;
    for (long j = 0; j < per_divisor; j++) {
      float x = mk(-126, -103, (int)(j % 7));
      float want = x / d, got = fast(x, d, r);
      if (isinf(want) || want != want) continue;
      int ex; frexpf(want, &ex);
      double ulp = ldexp(1.0, (ex - 24 < -149) ? -149 : ex - 24);
      double err = fabs((double)want - (double)got) / ulp;
      if (err > worst) worst = err;
    }
  }
  return worst;
}
"""


@pytest.fixture(scope="module")
def host_lib():
    d = tempfile.mkdtemp(prefix="poly_div_")
    src = os.path.join(d, "div.c")
    with open(src, "w") as f:
        f.write(HOST_C)
    so = os.path.join(d, "div.so")
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-shared", "-fPIC", "-o", so, src, "-lm"], check=True)
    lib = C.CDLL(so)
    lib.count_mismatches.restype = C.c_long
    lib.count_mismatches.argtypes = [C.c_int, C.c_long, C.c_long]
    lib.worst_tiny_ulps.restype = C.c_double
    lib.worst_tiny_ulps.argtypes = [C.c_long, C.c_long]
    return lib


def test_reciprocal_with_one_correction_is_the_rounded_quotient(host_lib):
    # every dividend whose remainder is representable: |x| >= 2^-102
    assert host_lib.count_mismatches(-102, 3000, 4000) == 0


def test_below_the_representable_remainder_the_error_stays_within_one_unit(host_lib):
    assert host_lib.worst_tiny_ulps(2000, 2000) <= 1.0


# ── on the GPU: the prelude's function itself ────────────────────────────────────────────

KERNEL = r"""
extern "C" __global__ void poly_div_test(float* fast, float* full, const float* x, const float* d, int n) {
  const int i = (int)(blockIdx.x * 256 + threadIdx.x);
  if (i >= n) return;
  const float dv = d[i];
  const float r = 1.0f / dv;
  const bool ok = __builtin_fabsf(dv) >= 0x1p-100f && __builtin_fabsf(dv) <= 0x1p+100f;
  fast[i] = poly_div_shared(x[i], dv, r, ok);
  full[i] = x[i] / dv;
}
"""


def _prelude():
    """The kernel prelude as the backend emits it (everything in front of the first kernel
    or row function of a rendered group)."""
    from polygrad_amd import PlanFile, _ffi
    plans = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "polygrad_amd", "plans")
    pf = PlanFile(os.path.join(plans, "rowops_f32_8192_softmax.polyplan"))
    lib = _ffi.load()
    p, n = C.c_void_p(), C.c_int()
    assert lib.poly_hip_fused_groups(pf.schedule, 0, C.byref(p), C.byref(n)) >= 0
    src = _ffi.take_string(p.value)
    cut = src.index("poly_row_p0")
    cut = src.rindex("__device__", 0, cut)
    assert "poly_div_shared" in src[:cut]
    return src[:cut]


def test_prelude_has_the_function_the_row_chain_calls():
    src = _prelude()
    assert "__builtin_amdgcn_div_fixupf" in src and "0x1p+26f" in src


@pytest.mark.gpu
def test_shared_division_on_the_device_equals_the_division():
    import torch
    from polygrad_amd import _ffi
    lib = _ffi.load()
    assert lib.poly_hip_init() == 0
    rng = np.random.default_rng(5)
    special = np.array([0.0, -0.0, 1.0, -1.0, 3.0, 1e-45, -1e-45, 1e-39, 2.0 ** -126, 2.0 ** -103, 2.0 ** -102, 2.0 ** -100,
                        2.0 ** -101, 2.0 ** 26, 2.0 ** 26 * 1.5, 2.0 ** 27, 2.0 ** 100, 2.0 ** 101, 3e38, -3e38, np.inf, -np.inf, np.nan,
                        1.0 + 2.0 ** -23, 2.0 - 2.0 ** -23, 0.1, 1e10, 1e-10, 1e30, 1e-30], dtype=np.float32)
    xs, ds = np.meshgrid(special, special, indexing="ij")
    bits = rng.integers(0, 2 ** 32, size=1 << 20, dtype=np.uint64).astype(np.uint32)
    x = np.concatenate([xs.ravel(), bits[: 1 << 19].view(np.float32), rng.standard_normal(1 << 19).astype(np.float32)])
    d = np.concatenate([ds.ravel(), bits[1 << 19:].view(np.float32), (rng.random(1 << 19).astype(np.float32) * 8192 + 1)])
    n = x.size
    tx, td = torch.from_numpy(x).cuda(), torch.from_numpy(d).cuda()
    fast = torch.full((n,), 7.0, device="cuda")
    full = torch.full((n,), 9.0, device="cuda")
    prog = lib.poly_hip_compile((_prelude() + KERNEL).encode(), b"poly_div_test")
    assert prog
    try:
        vals = [C.c_void_p(fast.data_ptr()), C.c_void_p(full.data_ptr()), C.c_void_p(tx.data_ptr()), C.c_void_p(td.data_ptr()), C.c_int(n)]
        args = (C.c_void_p * 5)(*[C.cast(C.pointer(v), C.c_void_p) for v in vals])
        torch.cuda.synchronize()
        assert lib.poly_hip_launch(prog, args, 5, (n + 255) // 256, 1, 1, 256, 1, 1, 0) == 0
        assert lib.poly_hip_sync() == 0
    finally:
        lib.poly_hip_program_destroy(prog)
    got, want = fast.cpu().numpy(), full.cpu().numpy()
    nan = np.isnan(want)
    assert (np.isnan(got) == nan).all()
    same = got.view(np.uint32) == want.view(np.uint32)
    # dividends below 2^-102 (and not zero) may differ by one unit in the last place
    tiny = (np.abs(x) < np.float32(2.0 ** -102)) & (x != 0)
    strict = ~nan & ~tiny
    assert same[strict].all(), [(float(a), float(b), float(g), float(w)) for a, b, g, w in
                                zip(x[strict & ~same][:5], d[strict & ~same][:5], got[strict & ~same][:5], want[strict & ~same][:5])]
    loose = ~nan & tiny & ~same
    if loose.any():
        ulp = np.maximum(np.spacing(np.abs(want[loose])), np.float32(2.0 ** -149))
        assert (np.abs(got[loose].astype(np.float64) - want[loose].astype(np.float64)) <= ulp.astype(np.float64)).all()
    # the fast path was taken somewhere and the full division somewhere
    assert (strict & (np.abs(x) <= 2.0 ** 26) & (np.abs(d) >= 2.0 ** -100) & (np.abs(d) <= 2.0 ** 100)).sum() > 1000
    assert (strict & (np.abs(x) > 2.0 ** 26)).sum() > 1000
