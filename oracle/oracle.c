/*
 * oracle.c -- CPU restatement of how polygrad's CPU backend evaluates a
 * scheduled kernel.  TEST INFRASTRUCTURE ONLY: it is the checker for the HIP
 * backend (tests/, __graft_entry__.smoke(), the cpu_baseline leg of bench.py)
 * and is never linked into, called by, or a fallback for the product library.
 *
 * What it restates, and where the reference defines it (paths relative to the
 * polygrad tree):
 *   - a kernel is a loop nest over its END ranges (outermost first) storing one
 *     value per iteration; REDUCE is an accumulator initialised to the identity
 *     and updated as acc = acc OP x in increasing range order, innermost range
 *     last                                   src/codegen.c:1424-1583, :44-51
 *   - ALU forms: one rounding per node in the node's dtype; 16-bit floats
 *     promote to float and round back after every op; MAX is (a<b)?b:a;
 *     RECIPROCAL is 1/x; MULACC is two roundings; float constants are f32
 *     literals even for 16-bit dtypes        src/render_c.c:928-1031, :849-880,
 *                                            src/codegen.c:1659-1669, :1849-1855
 *   - loads: *(p+idx); gated INDEX and WHERE-selected loads read only when the
 *     condition holds, else 0                src/render_c.c:1380-1401
 *   - CAST is the C cast, BITCAST a memcpy   src/render_c.c:1418-1476
 *   - EXP2 / LOG2 on f32 and f64 are the polynomial decompositions, not libm
 *                                            src/codegen.c:2051-2334
 *   - THREEFRY is threefry2x32 with 20 rounds src/codegen.c:1905-1970
 *   - compile flags: -O2 -fno-math-errno, no fast-math, no FMA contraction on
 *     baseline x86-64                         src/runtime_cpu.c:128-129
 *   - plan execution: intermediates zero-filled, kernels in exec_order,
 *     PARAM i <-> args[i], DEFINE_VARs after the buffers as pointers to int
 *                                            src/exec_plan.c:934-1060
 *
 * Pinned by tests/test_oracle.py against: the reference's own known-answer
 * vectors (matmul 2x3.3x4, broadcast batch, threefry key 1337, uniform-logit
 * cross-entropy = log 3, bf16/fp16 cast bit patterns), closed forms, and the
 * real reference library (oracle/_ref) on random graphs where that is built.
 * Not restated: SIN on f32/f64 uses libm instead of the reference's
 * Payne-Hanek / Cody-Waite polynomial (src/codegen.c:2338-2660).  The fixture
 * special_sin (outputs of the real reference over small, medium, huge and
 * special arguments) pins it to within one ulp of the reference, not bit for
 * bit: SIN is the one function for which this oracle is not bit-exact.  POW
 * and 16-bit transcendentals use libm as the reference does.
 */
#include "oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ── scalar types ─────────────────────────────────────────────────────── */

typedef enum { K_VOID, K_BOOL, K_SINT, K_UINT, K_F16, K_BF16, K_F32, K_F64 } Kind;

typedef struct { Kind kind; int bits; } Ty;

static Ty classify(const PolyDType *d) {
  Ty t = {K_VOID, 0};
  int bits = d->count > 1 ? d->bitsize / d->count : d->bitsize;
  switch (d->priority) {
    case -1: if (bits) { t.kind = K_SINT; t.bits = 32; } break; /* index == int */
    case 0: t.kind = K_BOOL; t.bits = 8; break;
    case 1: case 3: case 5: case 7: t.kind = K_SINT; t.bits = bits; break;
    case 2: case 4: case 6: case 8: t.kind = K_UINT; t.bits = bits; break;
    case 11: t.kind = K_F16; t.bits = 16; break;
    case 12: t.kind = K_BF16; t.bits = 16; break;
    case 13: t.kind = K_F32; t.bits = 32; break;
    case 14: t.kind = K_F64; t.bits = 64; break;
    default: break;
  }
  return t;
}

typedef union { float f; double d; int64_t i; uint64_t u; } Val;

uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

float oracle_bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

uint16_t oracle_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t mant = x & 0x007fffffu;
  int32_t exp = (int32_t)((x >> 23) & 0xff);
  if (exp == 0xff) return (uint16_t)(sign | 0x7c00u | (mant ? (0x0200u | (mant >> 13)) : 0));
  int32_t e = exp - 127 + 15;
  if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
  if (e <= 0) {
    if (e < -10) return (uint16_t)sign;
    mant |= 0x00800000u;
    uint32_t shift = (uint32_t)(14 - e);
    uint32_t half = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t mid = 1u << (shift - 1);
    if (rem > mid || (rem == mid && (half & 1u))) half++;
    return (uint16_t)(sign | half);
  }
  uint32_t half = ((uint32_t)e << 10) | (mant >> 13);
  uint32_t rem = mant & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++;
  return (uint16_t)(sign | half);
}

float oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f;
  uint32_t mant = h & 0x3ffu;
  uint32_t u;
  if (exp == 0) {
    if (mant == 0) u = sign;
    else {
      int e = -1;
      do { e++; mant <<= 1; } while (!(mant & 0x400u));
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
    }
  } else if (exp == 0x1f) u = sign | 0x7f800000u | (mant << 13);
  else u = sign | ((exp + 127 - 15) << 23) | (mant << 13);
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* Rounds a float result to the node's float dtype (identity for f32). */
static inline float round_to(Kind k, float v) {
  if (k == K_BF16) return oracle_bf16_to_f32(oracle_f32_to_bf16(v));
  if (k == K_F16) return oracle_f16_to_f32(oracle_f32_to_f16(v));
  return v;
}

static inline int64_t wrap_int(Ty t, int64_t v) {
  if (t.kind == K_BOOL) return v != 0;
  if (t.kind == K_SINT) {
    switch (t.bits) { case 8: return (int8_t)v; case 16: return (int16_t)v; case 32: return (int32_t)v; default: return v; }
  }
  switch (t.bits) { case 8: return (uint8_t)v; case 16: return (uint16_t)v; case 32: return (uint32_t)v; default: return v; }
}

/* ── transcendental decompositions (f32 and f64) ──────────────────────── */

static inline float bits_f32(int32_t i) { float f; memcpy(&f, &i, 4); return f; }
static inline int32_t f32_bits(float f) { int32_t i; memcpy(&i, &f, 4); return i; }
static inline double bits_f64(int64_t i) { double f; memcpy(&f, &i, 8); return f; }
static inline int64_t f64_bits(double f) { int64_t i; memcpy(&i, &f, 8); return i; }

float oracle_exp2f(float d) {
  /* inf/NaN mapped to 0 for the arithmetic; fixed up at the end */
  float x = (d != INFINITY) ? ((d != d) ? 0.0f : ((d != -INFINITY) ? d : 0.0f)) : 0.0f;
  int32_t q = (int32_t)(x + ((x < 0.0f) ? -0.5f : 0.5f));
  float s = x - (float)q;
  static const float c[7] = {0.1535920892e-3f, 0.1339262701e-2f, 0.9618384764e-2f, 0.5550347269e-1f,
                             0.2402264476e+0f, 0.6931471825e+0f, 1.0f};
  float u = c[0];
  for (int i = 1; i < 7; i++) { u = u * s; u = u + c[i]; }
  int32_t h = q / 2, o = q - h;
  float r = u * bits_f32((int32_t)((uint32_t)(h + 127) << 23));
  r = r * bits_f32((int32_t)((uint32_t)(o + 127) << 23));
  if (!(d < 128.0f)) r = INFINITY;
  if (d < -150.0f) r = 0.0f;
  if (d != d) r = NAN;
  return r;
}

double oracle_exp2(double d) {
  double x = (d != INFINITY) ? ((d != d) ? 0.0 : ((d != -INFINITY) ? d : 0.0)) : 0.0;
  int64_t q = (int64_t)(x + ((x < 0.0) ? -0.5 : 0.5));
  double s = x - (double)q;
  static const double c[12] = {0.4434359082926529454e-9, 0.7073164598085707425e-8, 0.1017819260921760451e-6,
                               0.1321543872511327615e-5, 0.1525273353517584730e-4, 0.1540353045101147808e-3,
                               0.1333355814670499073e-2, 0.9618129107597600536e-2, 0.5550410866482046596e-1,
                               0.2402265069591012214e+0, 0.6931471805599452862e+0, 0.1000000000000000000e+1};
  double u = c[0];
  for (int i = 1; i < 12; i++) { u = u * s; u = u + c[i]; }
  int64_t h = q / 2, o = q - h;
  double r = u * bits_f64((int64_t)((uint64_t)(h + 1023) << 52));
  r = r * bits_f64((int64_t)((uint64_t)(o + 1023) << 52));
  if (!(d < 1024.0)) r = INFINITY;
  if (d < -2000.0) r = 0.0;
  if (d != d) r = NAN;
  return r;
}

float oracle_log2f(float d) {
  int den = d < 1e-4f;
  float a = den ? d * 18446744073709551616.0f : d;
  float as = a * (float)(1.0 / 0.75);
  int32_t ei = ((f32_bits(as) >> 23) & 0xff) - 127;
  float e = (float)ei;
  float m = bits_f32(f32_bits(a) + (int32_t)((uint32_t)((int32_t)(-e)) << 23));
  float ea = den ? e - 64.0f : e;
  float x = (m - 1.0f) / (m + 1.0f);
  float x2 = x * x;
  float t = 0.4374550283f;
  t = t * x2; t = t + 0.5764790177f;
  t = t * x2; t = t + 0.9618012905120f;
  float r = t * (x * x2);
  r = r + ea;
  r = r + x * 2.8853900432586669922f;
  r = r + x * 3.2734474483568488616e-08f;
  if (!(d != INFINITY)) r = INFINITY;
  if (!(d != 0.0f)) r = -INFINITY;
  if (d < -0.0f) r = NAN;
  if (d != d) r = NAN;
  if (!((1.0f / d) != -INFINITY)) r = -INFINITY;
  return r;
}

double oracle_log2(double d) {
  int den = d < 1e-4;
  double a = den ? d * 18446744073709551616.0 : d;
  double as = a * (1.0 / 0.75);
  int64_t ei = ((f64_bits(as) >> 52) & 0x7ff) - 1023;
  double e = (double)ei;
  double m = bits_f64(f64_bits(a) + (int64_t)((uint64_t)((int64_t)(-e)) << 52));
  double ea = den ? e - 64.0 : e;
  double x = (m - 1.0) / (m + 1.0);
  double x2 = x * x;
  static const double c[7] = {0.2211941750456081490e+0, 0.2200768693152277689e+0, 0.2623708057488514656e+0,
                              0.3205977477944495502e+0, 0.4121985945485324709e+0, 0.5770780162997058982e+0,
                              0.96179669392608091449};
  double t = c[0];
  for (int i = 1; i < 7; i++) { t = t * x2; t = t + c[i]; }
  double r = t * (x * x2);
  r = r + ea;
  r = r + x * 2.885390081777926774;
  if (!(d != INFINITY)) r = INFINITY;
  if (!(d != 0.0)) r = -INFINITY;
  if (d < -0.0) r = NAN;
  if (d != d) r = NAN;
  if (!((1.0 / d) != -INFINITY)) r = -INFINITY;
  return r;
}

uint64_t oracle_threefry(uint64_t x, uint64_t key) {
  uint32_t x0 = (uint32_t)x, x1 = (uint32_t)(x >> 32), k0 = (uint32_t)key, k1 = (uint32_t)(key >> 32);
  uint32_t ks[3] = {k1, (k0 ^ k1) ^ 0x1BD11BDAu, k0};
  static const int rot[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
  x0 += ks[2];
  x1 += ks[0];
  for (int i = 0; i < 5; i++) {
    for (int j = 0; j < 4; j++) {
      int r = rot[i & 1][j];
      uint32_t s = x0 + x1;
      x1 = s ^ ((x1 << r) | (x1 >> (32 - r)));
      x0 = s;
    }
    x0 += ks[i % 3];
    x1 += ks[(i + 1) % 3] + (uint32_t)(i + 1);
  }
  return ((uint64_t)x1 << 32) | x0;
}

/* ── kernel evaluator ─────────────────────────────────────────────────── */

typedef struct {
  const PolyUOp *u;
  Ty ty;
  int *src;
  int n_src;
  uint64_t deps;     /* bitset over ranges */
  Val val;
  uint64_t stamp;    /* tick at which val was computed */
  int guard;         /* WHERE condition predicating this LOAD, or -1 */
  int guard_neg;
  int n_uses;
} Node;

typedef struct {
  Node *nodes;
  int n;
  int range_node[64];
  uint64_t range_tick[64];
  int64_t range_val[64];
  int n_ranges;
  uint64_t tick;
  void **args;
  int n_params;
  int n_args;
  char err[256];
} Kern;

typedef struct { const PolyUOp *u; int id; } MapEnt;

/* Open-addressing pointer map: index of the slot holding u, or of the empty
 * slot where it belongs. */
static int map_slot(const MapEnt *m, int cap, const PolyUOp *u) {
  size_t h = ((size_t)u >> 4) * (size_t)2654435761u;
  for (int p = 0; p < cap; p++) {
    int i = (int)((h + (size_t)p) % (size_t)cap);
    if (!m[i].u || m[i].u == u) return i;
  }
  return -1;
}

/* Post-order numbering of the DAG under root (sources before users). */
static int count_nodes(const PolyUOp *root, MapEnt **map_out, int *cap_out, const PolyUOp ***order_out) {
  int cap = 1024, n = 0, ocap = 256, used = 0;
  MapEnt *map = calloc((size_t)cap, sizeof(MapEnt));
  const PolyUOp **order = malloc((size_t)ocap * sizeof(*order));
  typedef struct { const PolyUOp *u; int next; } Fr;
  int scap = 256, sp = 0;
  Fr *st = malloc((size_t)scap * sizeof(Fr));
  st[sp++] = (Fr){root, 0};
  map[map_slot(map, cap, root)] = (MapEnt){root, -1};
  used = 1;
  while (sp > 0) {
    Fr *f = &st[sp - 1];
    if (f->next < (int)f->u->n_src) {
      const PolyUOp *s = f->u->src[f->next++];
      int sl = map_slot(map, cap, s);
      if (!map[sl].u) {
        if ((used + 1) * 2 > cap) {
          int ncap = cap * 2;
          MapEnt *nm = calloc((size_t)ncap, sizeof(MapEnt));
          for (int i = 0; i < cap; i++)
            if (map[i].u) nm[map_slot(nm, ncap, map[i].u)] = map[i];
          free(map); map = nm; cap = ncap;
          sl = map_slot(map, cap, s);
        }
        map[sl] = (MapEnt){s, -1};
        used++;
        if (sp == scap) { scap *= 2; st = realloc(st, (size_t)scap * sizeof(Fr)); }
        st[sp++] = (Fr){s, 0};
      }
    } else {
      map[map_slot(map, cap, f->u)].id = n;
      if (n == ocap) { ocap *= 2; order = realloc(order, (size_t)ocap * sizeof(*order)); }
      order[n++] = f->u;
      sp--;
    }
  }
  free(st);
  *map_out = map; *cap_out = cap; *order_out = order;
  return n;
}

static int lookup_id(MapEnt *map, int cap, const PolyUOp *u) {
  int sl = map_slot(map, cap, u);
  return (sl >= 0 && map[sl].u == u) ? map[sl].id : -1;
}

static int range_ord(Kern *k, int node) {
  for (int r = 0; r < k->n_ranges; r++) if (k->range_node[r] == node) return r;
  return -1;
}

static Val eval(Kern *k, int id);

static inline int truthy(const Node *n, Val v) {
  switch (n->ty.kind) {
    case K_F32: case K_F16: case K_BF16: return v.f != 0.0f;
    case K_F64: return v.d != 0.0;
    default: return v.i != 0;
  }
}

static Val load_elem(Ty t, const void *base, int64_t idx) {
  Val v; v.u = 0;
  switch (t.kind) {
    case K_BOOL: v.i = ((const uint8_t *)base)[idx] != 0; break;
    case K_SINT:
      switch (t.bits) { case 8: v.i = ((const int8_t *)base)[idx]; break; case 16: v.i = ((const int16_t *)base)[idx]; break;
                        case 32: v.i = ((const int32_t *)base)[idx]; break; default: v.i = ((const int64_t *)base)[idx]; }
      break;
    case K_UINT:
      switch (t.bits) { case 8: v.i = ((const uint8_t *)base)[idx]; break; case 16: v.i = ((const uint16_t *)base)[idx]; break;
                        case 32: v.i = ((const uint32_t *)base)[idx]; break; default: v.u = ((const uint64_t *)base)[idx]; }
      break;
    case K_F16: v.f = oracle_f16_to_f32(((const uint16_t *)base)[idx]); break;
    case K_BF16: v.f = oracle_bf16_to_f32(((const uint16_t *)base)[idx]); break;
    case K_F32: v.f = ((const float *)base)[idx]; break;
    case K_F64: v.d = ((const double *)base)[idx]; break;
    default: break;
  }
  return v;
}

static void store_elem(Ty t, void *base, int64_t idx, Val v) {
  switch (t.kind) {
    case K_BOOL: ((uint8_t *)base)[idx] = v.i != 0; break;
    case K_SINT: case K_UINT:
      switch (t.bits) { case 8: ((uint8_t *)base)[idx] = (uint8_t)v.i; break; case 16: ((uint16_t *)base)[idx] = (uint16_t)v.i; break;
                        case 32: ((uint32_t *)base)[idx] = (uint32_t)v.i; break; default: ((uint64_t *)base)[idx] = v.u; }
      break;
    case K_F16: ((uint16_t *)base)[idx] = oracle_f32_to_f16(v.f); break;
    case K_BF16: ((uint16_t *)base)[idx] = oracle_f32_to_bf16(v.f); break;
    case K_F32: ((float *)base)[idx] = v.f; break;
    case K_F64: ((double *)base)[idx] = v.d; break;
    default: break;
  }
}

/* Converts a value of type `from` to type `to` with C cast semantics. */
static Val convert(Ty from, Ty to, Val v) {
  Val r; r.u = 0;
  int from_f32 = from.kind == K_F32 || from.kind == K_F16 || from.kind == K_BF16;
  int to_f32 = to.kind == K_F32 || to.kind == K_F16 || to.kind == K_BF16;
  if (to.kind == K_BOOL) {
    r.i = from_f32 ? (v.f != 0.0f) : from.kind == K_F64 ? (v.d != 0.0) : (v.i != 0);
  } else if (to_f32) {
    float f;
    if (from_f32) f = v.f;
    else if (from.kind == K_F64) f = (float)v.d;
    else if (from.kind == K_UINT && from.bits == 64) f = (float)v.u;
    else f = (float)v.i;
    /* double -> 16-bit goes through one rounding in the reference's C cast on
     * x86 (via float) as well; int -> 16-bit likewise */
    r.f = round_to(to.kind, f);
  } else if (to.kind == K_F64) {
    if (from_f32) r.d = (double)v.f;
    else if (from.kind == K_F64) r.d = v.d;
    else if (from.kind == K_UINT && from.bits == 64) r.d = (double)v.u;
    else r.d = (double)v.i;
  } else { /* integers */
    int64_t i;
    if (from_f32) i = (to.kind == K_UINT && to.bits == 64) ? (int64_t)(uint64_t)v.f : (int64_t)v.f;
    else if (from.kind == K_F64) i = (to.kind == K_UINT && to.bits == 64) ? (int64_t)(uint64_t)v.d : (int64_t)v.d;
    else i = v.i;
    r.i = wrap_int(to, i);
  }
  return r;
}

static PolyOps reduce_op_of(const PolyUOp *u) {
  return u->arg.kind == POLY_ARG_OPS ? u->arg.ops : (PolyOps)u->arg.i;
}

static Val reduce_identity(PolyOps op, Ty t) {
  Val v; v.u = 0;
  double id = op == POLY_OP_MUL ? 1.0 : op == POLY_OP_MAX ? -INFINITY : 0.0;
  switch (t.kind) {
    case K_F32: case K_F16: case K_BF16: v.f = (float)id; break;
    case K_F64: v.d = id; break;
    default:
      if (op == POLY_OP_MAX) {
        if (t.kind == K_SINT) v.i = t.bits == 64 ? INT64_MIN : -((int64_t)1 << (t.bits - 1));
        else v.i = 0;
      } else v.i = (int64_t)id;
  }
  return v;
}

static Val alu(Kern *k, Node *n, PolyOps op, Val a, Val b, Val c, Ty sty) {
  Val r; r.u = 0;
  Ty t = n->ty;
  /* comparisons: computed in the SOURCE type, result bool */
  if (op == POLY_OP_CMPLT || op == POLY_OP_CMPNE || op == POLY_OP_CMPEQ) {
    int res;
    if (sty.kind == K_F32 || sty.kind == K_F16 || sty.kind == K_BF16)
      res = op == POLY_OP_CMPLT ? a.f < b.f : op == POLY_OP_CMPNE ? a.f != b.f : a.f == b.f;
    else if (sty.kind == K_F64)
      res = op == POLY_OP_CMPLT ? a.d < b.d : op == POLY_OP_CMPNE ? a.d != b.d : a.d == b.d;
    else if (sty.kind == K_UINT && sty.bits == 64)
      res = op == POLY_OP_CMPLT ? a.u < b.u : op == POLY_OP_CMPNE ? a.u != b.u : a.u == b.u;
    else
      res = op == POLY_OP_CMPLT ? a.i < b.i : op == POLY_OP_CMPNE ? a.i != b.i : a.i == b.i;
    r.i = res;
    return r;
  }
  if (t.kind == K_F32 || t.kind == K_F16 || t.kind == K_BF16) {
    float x = a.f, y = b.f, z = c.f, o;
    switch (op) {
      case POLY_OP_ADD: o = x + y; break;
      case POLY_OP_SUB: o = x - y; break;
      case POLY_OP_MUL: o = x * y; break;
      case POLY_OP_FDIV: o = x / y; break;
      case POLY_OP_NEG: o = -x; break;
      case POLY_OP_SQRT: o = sqrtf(x); break;
      case POLY_OP_TRUNC: o = truncf(x); break;
      case POLY_OP_RECIPROCAL: o = 1.0f / x; break;
      case POLY_OP_EXP2: o = t.kind == K_F32 ? oracle_exp2f(x) : exp2f(x); break;
      case POLY_OP_LOG2: o = t.kind == K_F32 ? oracle_log2f(x) : log2f(x); break;
      case POLY_OP_SIN: o = sinf(x); break;
      case POLY_OP_POW: o = powf(x, y); break;
      case POLY_OP_MAX: o = (x < y) ? y : x; break;
      case POLY_OP_MULACC: { float m = round_to(t.kind, x * y); o = m + z; break; }
      default: snprintf(k->err, sizeof(k->err), "float op %d unsupported", (int)op); o = 0; break;
    }
    r.f = round_to(t.kind, o);
    return r;
  }
  if (t.kind == K_F64) {
    double x = a.d, y = b.d, z = c.d, o;
    switch (op) {
      case POLY_OP_ADD: o = x + y; break;
      case POLY_OP_SUB: o = x - y; break;
      case POLY_OP_MUL: o = x * y; break;
      case POLY_OP_FDIV: o = x / y; break;
      case POLY_OP_NEG: o = -x; break;
      case POLY_OP_SQRT: o = sqrt(x); break;
      case POLY_OP_TRUNC: o = trunc(x); break;
      case POLY_OP_RECIPROCAL: o = 1.0 / x; break;
      case POLY_OP_EXP2: o = oracle_exp2(x); break;
      case POLY_OP_LOG2: o = oracle_log2(x); break;
      case POLY_OP_SIN: o = sin(x); break;
      case POLY_OP_POW: o = pow(x, y); break;
      case POLY_OP_MAX: o = (x < y) ? y : x; break;
      case POLY_OP_MULACC: o = (x * y) + z; break;
      default: snprintf(k->err, sizeof(k->err), "double op %d unsupported", (int)op); o = 0; break;
    }
    r.d = o;
    return r;
  }
  /* bool and integers */
  int is_u64 = t.kind == K_UINT && t.bits == 64;
  int64_t x = a.i, y = b.i, o = 0;
  switch (op) {
    case POLY_OP_ADD: o = (int64_t)((uint64_t)x + (uint64_t)y); break;
    case POLY_OP_SUB: o = (int64_t)((uint64_t)x - (uint64_t)y); break;
    case POLY_OP_MUL: o = (int64_t)((uint64_t)x * (uint64_t)y); break;
    case POLY_OP_MULACC: o = (int64_t)((uint64_t)x * (uint64_t)y + (uint64_t)c.i); break;
    case POLY_OP_NEG: o = t.kind == K_BOOL ? !x : (int64_t)(0 - (uint64_t)x); break;
    case POLY_OP_IDIV:
      if (y == 0) { o = 0; break; }
      o = is_u64 ? (int64_t)(a.u / b.u) : x / y; break;
    case POLY_OP_MOD:
      if (y == 0) { o = 0; break; }
      o = is_u64 ? (int64_t)(a.u % b.u) : x % y; break;
    case POLY_OP_SHL: o = (int64_t)((uint64_t)x << (y & 63)); break;
    case POLY_OP_SHR: o = (t.kind == K_UINT) ? (int64_t)(a.u >> (y & 63)) : (x >> (y & 63)); break;
    case POLY_OP_AND: o = x & y; break;
    case POLY_OP_OR: o = x | y; break;
    case POLY_OP_XOR: o = x ^ y; break;
    case POLY_OP_MAX: o = is_u64 ? ((a.u < b.u) ? y : x) : ((x < y) ? y : x); break;
    case POLY_OP_THREEFRY: o = (int64_t)oracle_threefry(a.u, b.u); break;
    default: snprintf(k->err, sizeof(k->err), "integer op %d unsupported", (int)op); break;
  }
  r.i = wrap_int(t, o);
  return r;
}

static int node_fresh(Kern *k, Node *n) {
  if (n->stamp == 0) return 0;
  uint64_t d = n->deps;
  while (d) {
    int r = __builtin_ctzll(d);
    d &= d - 1;
    if (k->range_tick[r] > n->stamp) return 0;
  }
  return 1;
}

static Val eval_load(Kern *k, Node *n) {
  Val zero; zero.u = 0;
  Node *ix = &k->nodes[n->src[0]];
  if (ix->u->op != POLY_OP_INDEX || ix->n_src < 2) { snprintf(k->err, sizeof(k->err), "LOAD without INDEX"); return zero; }
  if (ix->n_src >= 3) {
    Val g = eval(k, ix->src[2]);
    if (!truthy(&k->nodes[ix->src[2]], g)) return zero;
  }
  if (n->guard >= 0) {
    Val g = eval(k, n->guard);
    int t = truthy(&k->nodes[n->guard], g);
    if (n->guard_neg ? t : !t) return zero;
  }
  Node *p = &k->nodes[ix->src[0]];
  int64_t idx = eval(k, ix->src[1]).i;
  int pi = (int)p->u->arg.i;
  if (pi < 0 || pi >= k->n_params) { snprintf(k->err, sizeof(k->err), "PARAM %d out of range", pi); return zero; }
  int64_t numel = p->u->dtype.ptr_size;
  if (idx < 0 || (numel > 0 && idx >= numel)) {
    snprintf(k->err, sizeof(k->err), "load index %lld outside buffer %d (numel %lld)", (long long)idx, pi, (long long)numel);
    return zero;
  }
  return load_elem(n->ty, k->args[pi], idx);
}

static Val eval_reduce(Kern *k, Node *n, int id) {
  (void)id;
  PolyOps op = reduce_op_of(n->u);
  int nr = 0;
  int ords[16];
  int64_t ext[16];
  if (n->n_src - 1 > 16) { snprintf(k->err, sizeof(k->err), "REDUCE over more than 16 ranges"); Val z; z.u = 0; return z; }
  /* only RANGE sources loop; an axis of extent 1 may arrive as a constant instead
   * (src/codegen.c:1431-1439), and with no loop at all the result is the value itself,
   * not identity-op-value (src/codegen.c:1444-1450) */
  for (int i = 1; i < n->n_src; i++) {
    if (k->nodes[n->src[i]].u->op != POLY_OP_RANGE) continue;
    ords[nr] = range_ord(k, n->src[i]);
    ext[nr] = eval(k, k->nodes[n->src[i]].src[0]).i;
    nr++;
  }
  if (nr == 0) return eval(k, n->src[0]);
  Val acc = reduce_identity(op, n->ty);
  int64_t total = 1;
  for (int i = 0; i < nr; i++) total *= ext[i] > 0 ? ext[i] : 0;
  int64_t ctr[16] = {0};
  Val zero; zero.u = 0;
  Ty src_ty = k->nodes[n->src[0]].ty;
  for (int64_t it = 0; it < total; it++) {
    k->tick++;
    for (int i = 0; i < nr; i++) { k->range_val[ords[i]] = ctr[i]; k->range_tick[ords[i]] = k->tick; }
    Val v = eval(k, n->src[0]);
    acc = alu(k, n, op, acc, v, zero, src_ty);
    for (int i = nr - 1; i >= 0; i--) { if (++ctr[i] < ext[i]) break; ctr[i] = 0; }
    if (k->err[0]) break;
  }
  return acc;
}

static Val eval(Kern *k, int id) {
  Node *n = &k->nodes[id];
  if (node_fresh(k, n)) return n->val;
  Val r; r.u = 0;
  PolyOps op = n->u->op;
  switch (op) {
    case POLY_OP_CONST:
      switch (n->ty.kind) {
        case K_F32: case K_F16: case K_BF16: r.f = (float)n->u->arg.f; break;
        case K_F64: r.d = n->u->arg.f; break;
        case K_BOOL: r.i = n->u->arg.kind == POLY_ARG_BOOL ? n->u->arg.b : (n->u->arg.i != 0); break;
        default: r.i = wrap_int(n->ty, n->u->arg.i); break;
      }
      break;
    case POLY_OP_RANGE: r.i = k->range_val[range_ord(k, id)]; break;
    case POLY_OP_DEFINE_VAR: {
      /* vars follow the buffers in args[], in order of first appearance */
      int vi = 0;
      for (int j = 0; j < id; j++) if (k->nodes[j].u->op == POLY_OP_DEFINE_VAR) vi++;
      if (k->n_params + vi >= k->n_args) { snprintf(k->err, sizeof(k->err), "missing DEFINE_VAR argument"); break; }
      r.i = *(const int *)k->args[k->n_params + vi];
      break;
    }
    case POLY_OP_LOAD: r = eval_load(k, n); break;
    case POLY_OP_REDUCE: r = eval_reduce(k, n, id); break;
    case POLY_OP_CAST: r = convert(k->nodes[n->src[0]].ty, n->ty, eval(k, n->src[0])); break;
    case POLY_OP_BITCAST: {
      Node *s = &k->nodes[n->src[0]];
      Val v = eval(k, n->src[0]);
      unsigned char buf[8] = {0};
      /* materialise the source in its storage format, reread in the target's */
      store_elem(s->ty, buf, 0, v);
      r = load_elem(n->ty, buf, 0);
      break;
    }
    case POLY_OP_WHERE: {
      Val cnd = eval(k, n->src[0]);
      int t = truthy(&k->nodes[n->src[0]], cnd);
      Node *b = &k->nodes[n->src[t ? 1 : 2]];
      Val v = eval(k, n->src[t ? 1 : 2]);
      /* branches may carry a float literal in a 16-bit node: round on assignment */
      r = convert(b->ty, n->ty, v);
      break;
    }
    default: {
      Val a, b, c; a.u = b.u = c.u = 0;
      Ty sty = n->ty;
      /* late rewrite a * (1/b) -> a / b, reciprocal as the SECOND factor only
       * (src/codegen.c:1867-1883, pattern at :2026-2029) */
      if (op == POLY_OP_MUL && n->n_src == 2 && n->ty.kind >= K_F16) {
        Node *rb = &k->nodes[n->src[1]];
        int den = -1;
        if (rb->u->op == POLY_OP_RECIPROCAL && rb->n_src == 1) den = rb->src[0];
        else if (rb->u->op == POLY_OP_FDIV && rb->n_src == 2 && k->nodes[rb->src[0]].u->op == POLY_OP_CONST &&
                 k->nodes[rb->src[0]].u->arg.kind == POLY_ARG_FLOAT && k->nodes[rb->src[0]].u->arg.f == 1.0)
          den = rb->src[1];
        if (den >= 0) {
          a = eval(k, n->src[0]);
          b = eval(k, den);
          r = alu(k, n, POLY_OP_FDIV, a, b, c, n->ty);
          break;
        }
      }
      if (n->n_src > 0) { a = eval(k, n->src[0]); sty = k->nodes[n->src[0]].ty; }
      if (n->n_src > 1) b = eval(k, n->src[1]);
      if (n->n_src > 2) c = eval(k, n->src[2]);
      r = alu(k, n, op, a, b, c, sty);
      break;
    }
  }
  n->val = r;
  n->stamp = k->tick;
  return r;
}

/* Runs the loop nest of one STORE (ranges outermost first). */
static void run_store(Kern *k, int store_id, const int *ranges, int nr) {
  Node *st = &k->nodes[store_id];
  Node *ix = &k->nodes[st->src[0]];
  Node *p = &k->nodes[ix->src[0]];
  int pi = (int)p->u->arg.i;
  int64_t ext[64], ctr[64] = {0};
  int64_t total = 1;
  for (int i = 0; i < nr; i++) {
    ext[i] = eval(k, k->nodes[k->range_node[ranges[i]]].src[0]).i;
    total *= ext[i] > 0 ? ext[i] : 0;
  }
  Ty vty = k->nodes[st->src[1]].ty;
  for (int64_t it = 0; it < total && !k->err[0]; it++) {
    k->tick++;
    for (int i = 0; i < nr; i++) { k->range_val[ranges[i]] = ctr[i]; k->range_tick[ranges[i]] = k->tick; }
    if (nr == 0) k->tick++;
    int go = 1;
    if (ix->n_src >= 3) go = truthy(&k->nodes[ix->src[2]], eval(k, ix->src[2]));
    if (go) {
      Val v = eval(k, st->src[1]);
      int64_t idx = eval(k, ix->src[1]).i;
      int64_t numel = p->u->dtype.ptr_size;
      if (idx < 0 || (numel > 0 && idx >= numel)) {
        snprintf(k->err, sizeof(k->err), "store index %lld outside buffer %d", (long long)idx, pi);
        return;
      }
      store_elem(p->ty, k->args[pi], idx, convert(vty, p->ty, v));
    }
    for (int i = nr - 1; i >= 0; i--) { if (++ctr[i] < ext[i]) break; ctr[i] = 0; }
  }
}

static void walk_sink(Kern *k, int id, int *ranges, int nr) {
  Node *n = &k->nodes[id];
  if (k->err[0]) return;
  if (n->u->op == POLY_OP_END) {
    int r2[64];
    memcpy(r2, ranges, (size_t)nr * sizeof(int));
    int m = nr;
    for (int s = 1; s < n->n_src; s++) r2[m++] = range_ord(k, n->src[s]);
    walk_sink(k, n->src[0], r2, m);
  } else if (n->u->op == POLY_OP_STORE) {
    run_store(k, id, ranges, nr);
  } else if (n->u->op == POLY_OP_SINK || n->u->op == POLY_OP_GROUP || n->u->op == POLY_OP_NOOP) {
    for (int s = 0; s < n->n_src; s++) walk_sink(k, n->src[s], ranges, nr);
  } else {
    snprintf(k->err, sizeof(k->err), "unexpected op %d under SINK", (int)n->u->op);
  }
}

int oracle_run_kernel(const PolyUOp *root, void **args, int n_args) {
  if (!root || root->op != POLY_OP_SINK) { fprintf(stderr, "oracle: kernel root is not a SINK\n"); return -1; }
  MapEnt *map; int cap; const PolyUOp **order;
  int n = count_nodes(root, &map, &cap, &order);
  Kern k;
  memset(&k, 0, sizeof(k));
  k.nodes = calloc((size_t)n, sizeof(Node));
  k.n = n; k.args = args; k.n_args = n_args; k.tick = 1;
  int max_param = -1;
  for (int i = 0; i < n; i++) {
    Node *nd = &k.nodes[i];
    nd->u = order[i];
    nd->ty = classify(&order[i]->dtype);
    nd->n_src = order[i]->n_src;
    nd->src = malloc((size_t)(nd->n_src > 0 ? nd->n_src : 1) * sizeof(int));
    nd->guard = -1;
    for (int s = 0; s < nd->n_src; s++) {
      nd->src[s] = lookup_id(map, cap, order[i]->src[s]);
      k.nodes[nd->src[s]].n_uses++;
    }
    if (order[i]->op == POLY_OP_RANGE) {
      if (k.n_ranges >= 64) { snprintf(k.err, sizeof(k.err), "more than 64 ranges"); break; }
      k.range_node[k.n_ranges++] = i;
    }
    if (order[i]->op == POLY_OP_PARAM && (int)order[i]->arg.i > max_param) max_param = (int)order[i]->arg.i;
  }
  k.n_params = max_param + 1;
  for (int i = 0; i < n && !k.err[0]; i++) {
    Node *nd = &k.nodes[i];
    uint64_t d = 0;
    if (nd->u->op == POLY_OP_RANGE) d = (uint64_t)1 << range_ord(&k, i);
    for (int s = 0; s < nd->n_src; s++) d |= k.nodes[nd->src[s]].deps;
    if (nd->u->op == POLY_OP_REDUCE || nd->u->op == POLY_OP_END)
      for (int s = 1; s < nd->n_src; s++) { int r = range_ord(&k, nd->src[s]); if (r >= 0) d &= ~((uint64_t)1 << r); }
    nd->deps = d;
  }
  /* loads selected by one branch of a WHERE are predicated on its condition */
  for (int i = 0; i < n; i++) {
    Node *w = &k.nodes[i];
    if (w->u->op != POLY_OP_WHERE || w->n_src != 3) continue;
    for (int b = 1; b <= 2; b++) {
      int c = w->src[b];
      if (k.nodes[c].u->op == POLY_OP_CAST && k.nodes[c].n_uses == 1) c = k.nodes[c].src[0];
      Node *ld = &k.nodes[c];
      if (ld->u->op == POLY_OP_LOAD && ld->n_uses == 1 && ld->guard < 0) { ld->guard = w->src[0]; ld->guard_neg = (b == 2); }
    }
  }
  if (!k.err[0]) {
    if (k.n_params > n_args) snprintf(k.err, sizeof(k.err), "kernel needs %d buffers, got %d args", k.n_params, n_args);
    else { int none[1]; walk_sink(&k, n - 1, none, 0); }
  }
  int rc = 0;
  if (k.err[0]) { fprintf(stderr, "oracle: %s\n", k.err); rc = -1; }
  for (int i = 0; i < n; i++) free(k.nodes[i].src);
  free(k.nodes); free(map); free(order);
  return rc;
}

int oracle_run_schedule(const PolySchedule *s, void **slot_data, int n_slots) {
  if (!s) return -1;
  void **data = calloc((size_t)s->n_buf_slots, sizeof(void *));
  int rc = 0;
  for (int i = 0; i < s->n_buf_slots; i++) {
    if (s->buf_slots[i].is_intermediate) {
      size_t nb = (size_t)(s->buf_slots[i].nbytes > 0 ? s->buf_slots[i].nbytes : 4);
      data[i] = calloc(1, nb);
    } else {
      data[i] = (i < n_slots) ? slot_data[i] : NULL;
    }
  }
  int *vals = calloc((size_t)(s->n_default_vars + 1), sizeof(int));
  for (int step = 0; step < s->n_items && rc == 0; step++) {
    const PolyExecItem *it = &s->items[s->exec_order[step]];
    int na = it->n_buf_slots + it->n_var_uops;
    void **args = calloc((size_t)(na > 0 ? na : 1), sizeof(void *));
    for (int i = 0; i < it->n_buf_slots; i++) {
      args[i] = data[it->buf_slot_indices[i]];
      if (!args[i]) { fprintf(stderr, "oracle: missing data for slot %d\n", it->buf_slot_indices[i]); rc = -1; }
    }
    for (int v = 0; v < it->n_var_uops && rc == 0; v++) {
      int found = 0;
      for (int d = 0; d < s->n_default_vars; d++)
        if (s->default_vars[d].var == it->var_uops[v]) { vals[d] = s->default_vars[d].value; args[it->n_buf_slots + v] = &vals[d]; found = 1; }
      if (!found) { fprintf(stderr, "oracle: no binding for DEFINE_VAR\n"); rc = -1; }
    }
    if (rc == 0) rc = oracle_run_kernel(it->root, args, na);
    free(args);
  }
  for (int i = 0; i < s->n_buf_slots; i++) if (s->buf_slots[i].is_intermediate) free(data[i]);
  free(data); free(vals);
  return rc;
}
