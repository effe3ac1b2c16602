"""Pins the CPU oracle (oracle/oracle.c) -- CPU only, no GPU needed.

1. Scalar pieces against closed forms and independent implementations.
2. Every committed golden fixture (outputs of the REAL reference CPU backend,
   tests/golden/make_golden.py) -- including the reference's own known-answer
   vectors (matmul 2x3.3x4, threefry key 1337, uniform-logit cross-entropy).
3. Where the reference library is built, random graphs against it, bit for bit.
"""
import math
import os

import numpy as np
import pytest

import fixtures as F

# The oracle restates the reference's arithmetic exactly: every fixture must come out bit for
# bit, except the one whose function it does not restate (sin: libm, within one ulp).
NOT_BIT_EXACT = {"special_sin"}
BIT_EXACT = set(F.case_names()) - NOT_BIT_EXACT


def test_bf16_conversion_is_round_to_nearest_even():
    o = F.oracle()
    # exactly representable, ties, NaN, inf (test/test_f16.c cast patterns)
    cases = {1.0: 0x3F80, -2.0: 0xC000, 0.0: 0x0000, float("inf"): 0x7F80, 1.00390625: 0x3F80, 1.01171875: 0x3F82,
             3.140625: 0x4049, 65280.0: 0x477F}
    for x, bits in cases.items():
        assert o.oracle_f32_to_bf16(x) == bits, x
    assert o.oracle_f32_to_bf16(float("nan")) & 0x7FC0 == 0x7FC0
    # brute force: every bf16 value round-trips; midpoints go to the even neighbour
    for h in range(0, 0x7F80, 97):
        f = o.oracle_bf16_to_f32(h)
        assert o.oracle_f32_to_bf16(f) == h
        up = o.oracle_bf16_to_f32(h + 1)
        mid = np.float32((np.float64(f) + np.float64(up)) / 2)
        assert o.oracle_f32_to_bf16(float(mid)) == (h if h % 2 == 0 else h + 1)


def test_f16_conversion_matches_ieee_half():
    o = F.oracle()
    g = np.random.default_rng(0)
    xs = np.concatenate([g.normal(0, 1000, 2000), g.normal(0, 1e-5, 2000), [0.0, -0.0, 65504, 65519.9, 65520, 1e-8, 5.96e-8, 2.98e-8, 6.1e-5]]).astype(np.float32)
    for x in xs:
        want = int(np.float32(x).astype(np.float16).view(np.uint16))
        assert o.oracle_f32_to_f16(float(x)) == want, x
    for h in range(0, 0x7C00, 53):
        assert o.oracle_f16_to_f32(h) == float(np.uint16(h).view(np.float16))


def test_exp2_log2_closed_forms_and_accuracy():
    o = F.oracle()
    for k in range(-126, 128):
        assert o.oracle_exp2f(float(k)) == 2.0 ** k
        assert o.oracle_log2f(2.0 ** k) == float(k)
    assert o.oracle_exp2f(128.0) == math.inf and o.oracle_exp2f(-151.0) == 0.0
    assert math.isnan(o.oracle_exp2f(math.nan)) and o.oracle_exp2f(-math.inf) == 0.0 and o.oracle_exp2f(math.inf) == math.inf
    assert o.oracle_log2f(0.0) == -math.inf and math.isnan(o.oracle_log2f(-1.0)) and o.oracle_log2f(math.inf) == math.inf
    assert o.oracle_log2f(-0.0) == -math.inf
    g = np.random.default_rng(1)
    for x in g.uniform(-120, 120, 3000).astype(np.float32):
        assert abs(o.oracle_exp2f(float(x)) - 2.0 ** float(x)) <= 4e-7 * 2.0 ** float(x)
    for x in np.exp(g.uniform(-80, 80, 3000)).astype(np.float32):
        assert abs(o.oracle_log2f(float(x)) - math.log2(float(x))) <= 4e-7 * max(1.0, abs(math.log2(float(x))))
    for x in g.uniform(-1000, 1000, 2000):
        assert abs(o.oracle_exp2(float(x)) - 2.0 ** float(x)) <= 1e-15 * 2.0 ** float(x)
    for x in np.exp(g.uniform(-300, 300, 2000)):
        assert abs(o.oracle_log2(float(x)) - math.log2(float(x))) <= 2e-15 * max(1.0, abs(math.log2(float(x))))


def test_threefry_known_answers():
    # JAX threefry2x32, key 1337, counters 0..19 (reference test/test_nn.c:1126-1131, 1161-1169)
    ref32 = [2732499619, 3322027265, 2482432314, 3871860445, 3571867126, 3019569655, 2459680734, 2731866067,
             986922480, 1616040745, 4238711754, 3594775990, 3046419939, 3519108299, 586160567, 3928687287,
             4074505382, 4210472430, 4094881238, 3306411770]
    ref64 = [2091981003842036387, 7289724007706926337, 5665610599518103866, 1710967476831381213,
             10223482319493553654, 17028600460329286135, 17124603982541209566, 3105577853879908307,
             2086892522412654064, 3335679299718140713, 16051258882154404810, 6689751810128997814,
             14143017499898457571, 15433975895207007435, 585627789352245687, 6751685475094430391,
             13535415641566872742, 11824248585908041198, 12094218887010381270, 17901838715724224250]
    o = F.oracle()
    for i in range(20):
        v = o.oracle_threefry(i, 1337)
        assert v == ref64[i]
        assert v & 0xFFFFFFFF == ref32[i]


# Minutes of interpreted evaluation (2 x 1024 x 1024 scores, each through the whole softmax
# chain); the same kernels are pinned bit for bit at 256 positions (attention_bf16_t256).
SLOW_ON_THE_ORACLE = {"attention_bf16_t1024"}


@pytest.mark.parametrize("name", F.case_names())
def test_oracle_reproduces_reference_fixture(name):
    if name in SLOW_ON_THE_ORACLE and not os.environ.get("POLY_SLOW_TESTS"):
        pytest.skip("set POLY_SLOW_TESTS=1 to run the T=1024 attention fixture through the oracle (about 2 minutes)")
    fx = F.Fixture(name)
    got = F.run_oracle_schedule(fx.plan.schedule, fx.n_slots, fx.inputs)
    for slot in fx.external:
        want = fx.expected[slot]
        have = got[slot]
        if name in BIT_EXACT:
            assert have.tobytes() == want.tobytes(), f"{name}: slot {slot} ({fx.plan.names[slot]}) differs from the reference"
        else:
            np.testing.assert_allclose(F.as_float(have), F.as_float(want), rtol=1e-6, atol=1e-7)


def test_kat_values_are_the_published_ones():
    # the fixtures themselves hold the values the reference's tests assert
    fx = F.Fixture("kat_matmul_2x3x4")
    out = [i for i in fx.external if fx.plan.names[i] == "O"][0]
    assert fx.expected[out].tolist() == [38, 44, 50, 56, 83, 98, 113, 128]
    fx = F.Fixture("kat_xent_uniform")
    out = [i for i in fx.external if fx.plan.names[i] == "loss"][0]
    assert abs(float(fx.expected[out][0]) - math.log(3.0)) < 1e-6


def _random_graph(c, R, g, x, y):
    """A random expression over two (6, 8) fp32 tensors: elementwise ops the frontend
    offers, dtype round trips, movement ops and a final optional reduction."""
    vals = [x, y]
    for _ in range(int(g.integers(4, 10))):
        a = vals[int(g.integers(0, len(vals)))]
        b = vals[int(g.integers(0, len(vals)))]
        k = int(g.integers(0, 13))
        if k == 0: v = a + b
        elif k == 1: v = a * b
        elif k == 2: v = a - b
        elif k == 3: v = a / (b * b + c.const(0.5))
        elif k == 4: v = a.maximum(b)
        elif k == 5: v = (a * c.const(0.25)).exp2()
        elif k == 6: v = (a * a + c.const(1e-3)).log2()
        elif k == 7: v = (a * a).sqrt()
        elif k == 8: v = a.lt(b).where(a, b * c.const(-1.5))
        elif k == 9: v = a.cast(R.BF16).cast(R.F32)
        elif k == 10: v = a.cast(R.F16).cast(R.F32)
        elif k == 11: v = (a * c.const(7.0)).cast(R.I32).cast(R.F32)
        else: v = a.permute((1, 0)).flip((0,)).permute((1, 0))
        vals.append(v)
    out = vals[-1]
    mode = int(g.integers(0, 4))
    if mode == 0: return out.sum(-1), (6,)
    if mode == 1: return out.max(-1), (6,)
    if mode == 2: return out.softmax(-1), (6, 8)
    return out, (6, 8)


@pytest.mark.parametrize("seed", range(8))
def test_oracle_matches_live_reference_on_random_graphs(seed):
    """Where the real reference library is built (the build container), random graphs go
    through its CPU backend and through the oracle: results must agree bit for bit."""
    import refpoly as R
    from hipharness import schedule_slots
    if not R.available():
        pytest.skip("reference library not built here")
    g = np.random.default_rng(1000 + seed)
    c = R.Ctx()
    x, y = c.buffer((6, 8), name="x"), c.buffer((6, 8), name="y")
    val, shape = _random_graph(c, R, g, x, y)
    o = c.buffer(shape, name="o")
    sink = c.sink((o, val))
    bx, by, bo = [t for t, _ in c.buffers]
    arrays = {bx: g.normal(0, 2, 48).astype(np.float32), by: g.normal(0, 2, 48).astype(np.float32),
              bo: np.zeros(int(np.prod(shape)), np.float32)}
    want = {t: a.copy() for t, a in arrays.items()}
    c.realize_cpu(sink, want)
    sched = c.schedule(sink)
    slots, n = schedule_slots(c, sched)
    got = F.run_oracle_schedule(sched, n, {i: arrays[t] for i, (t, _) in slots.items()})
    out_slot = [i for i, (t, _) in slots.items() if t is bo][0]
    c.L.poly_schedule_free(sched)
    c.close()
    assert got[out_slot].tobytes() == want[bo].tobytes(), \
        f"seed {seed}: max abs diff {np.nanmax(np.abs(got[out_slot] - want[bo]))}"
