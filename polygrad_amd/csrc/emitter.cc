// Expression emitter: renders kernel-graph nodes as HIP C statements, placing
// each value in the outermost loop scope that binds every range it depends on.
//
// Arithmetic forms follow the reference CPU renderer so that results agree with
// the CPU backend: one typed temporary per node (so 16-bit float ops round after
// every operation, src/render_c.c:1478-1496), MAX as (a<b)?b:a
// (src/codegen.c:1659-1669), RECIPROCAL as 1/x (src/codegen.c:1849-1855), gated
// loads as gate ? *p : 0 (src/render_c.c:1391-1399), float constants as f32
// literals even for 16-bit types (src/render_c.c:849-880).
#include <cmath>
#include <cstring>

#include "render_hip.h"
#include <functional>

namespace polyhip {

const char *hip_prelude() {
  return R"HIP(
extern "C" __device__ float __ocml_sin_f32(float);
extern "C" __device__ double __ocml_sin_f64(double);
typedef float  poly_f32x4 __attribute__((ext_vector_type(4)));
typedef float  poly_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 poly_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 poly_bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 poly_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 poly_f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 poly_f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 poly_f16x2 __attribute__((ext_vector_type(2)));

template <typename T, int N> struct poly_vec { T v[N]; };
// A kernel that streams through more data than the caches hold reads it with the
// nontemporal hint (POLY_NT_LOADS, defined in front of this text for such a kernel), so
// that what it reads once does not push out what it, or the next kernel, reads again.
#ifdef POLY_NT_LOADS
#define POLY_LD(...) __builtin_nontemporal_load(&(__VA_ARGS__))
#else
#define POLY_LD(...) (__VA_ARGS__)
#endif
template <typename T, int N>
__device__ __forceinline__ poly_vec<T, N> poly_vload(const T *p) {
  typedef T vt __attribute__((ext_vector_type(N)));
  typedef vt uvt __attribute__((aligned(sizeof(T))));
#ifdef POLY_NT_LOADS
  vt x = __builtin_nontemporal_load((const uvt *)p);
#else
  vt x = *(const uvt *)p;
#endif
  poly_vec<T, N> r;
#pragma unroll
  for (int i = 0; i < N; i++) r.v[i] = x[i];
  return r;
}
template <typename T, int N>
__device__ __forceinline__ void poly_vstore(T *p, const poly_vec<T, N> &r) {
  typedef T vt __attribute__((ext_vector_type(N)));
  typedef vt uvt __attribute__((aligned(sizeof(T))));
  vt x;
#pragma unroll
  for (int i = 0; i < N; i++) x[i] = r.v[i];
#ifdef POLY_NT_STORES
  __builtin_nontemporal_store(x, (uvt *)p);
#else
  *(uvt *)p = x;
#endif
}

// x / d where many dividends share one divisor (a row's sum, a row's deviation): r = 1 / d
// and `ok` (d finite and between 2^-100 and 2^100 in magnitude) are computed once per
// divisor.  q = x r is within a unit or two of the quotient, the remainder x - q d is exact
// in one fused multiply-add, and q + (x - q d) r is the correctly rounded quotient -- the
// value x / d has -- whenever the remainder is representable, i.e. for |x| >= 2^-102
// (checked on the host against x / d over all exponents and the awkward significands;
// below that the result is within one unit in the last place, of a subnormal result:
// 2^-149).  v_div_fixup gives a zero dividend the sign the quotient has.  Dividends beyond
// 2^26, non-finite ones and every dividend of a divisor outside the range take the full
// division.  Four instructions instead of eleven per quotient.
__device__ __forceinline__ float poly_div_shared(float x, float d, float r, bool ok) {
  if (ok && __builtin_fabsf(x) <= 0x1p+26f) {
    const float q = x * r;
    const float e = __builtin_fmaf(-q, d, x);
    return __builtin_amdgcn_div_fixupf(__builtin_fmaf(e, r, q), d, x);
  }
  return x / d;
}

// ── wave64 reductions: DPP inside a row of 16 lanes, ds_swizzle across rows of
// a 32-lane half, readlane across the two halves.  Every lane returns the total.
template <int CTRL>
__device__ __forceinline__ float poly_dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float poly_swz16_f32(float v) {
  // bitmask mode: and=0x1f, or=0, xor=0x10 -> exchange with lane^16
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401f));
}
#define POLY_WAVE_REDUCE_F32(NAME, COMBINE)                                   \
  __device__ __forceinline__ float NAME(float v) {                            \
    float o;                                                                  \
    o = poly_dpp_f32<0xB1>(v); v = COMBINE(v, o);  /* quad_perm [1,0,3,2] */  \
    o = poly_dpp_f32<0x4E>(v); v = COMBINE(v, o);  /* quad_perm [2,3,0,1] */  \
    o = poly_dpp_f32<0x141>(v); v = COMBINE(v, o); /* row_half_mirror */      \
    o = poly_dpp_f32<0x140>(v); v = COMBINE(v, o); /* row_mirror */           \
    o = poly_swz16_f32(v); v = COMBINE(v, o);                                 \
    float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));  \
    float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32)); \
    return COMBINE(lo, hi);                                                   \
  }
// The same over the 32 lanes of a half wave (two rows to a wave): every lane returns the
// total of its own half.
#define POLY_HALF_REDUCE_F32(NAME, COMBINE)                                   \
  __device__ __forceinline__ float NAME(float v) {                            \
    float o;                                                                  \
    o = poly_dpp_f32<0xB1>(v); v = COMBINE(v, o);                             \
    o = poly_dpp_f32<0x4E>(v); v = COMBINE(v, o);                             \
    o = poly_dpp_f32<0x141>(v); v = COMBINE(v, o);                            \
    o = poly_dpp_f32<0x140>(v); v = COMBINE(v, o);                            \
    o = poly_swz16_f32(v); v = COMBINE(v, o);                                 \
    return v;                                                                 \
  }
#define POLY_COMB_ADD(a, b) ((a) + (b))
#define POLY_COMB_MUL(a, b) ((a) * (b))
#define POLY_COMB_MAX(a, b) (((a) < (b)) ? (b) : (a))
POLY_WAVE_REDUCE_F32(poly_wave_add_f32, POLY_COMB_ADD)
POLY_WAVE_REDUCE_F32(poly_wave_mul_f32, POLY_COMB_MUL)
POLY_WAVE_REDUCE_F32(poly_wave_max_f32, POLY_COMB_MAX)
POLY_HALF_REDUCE_F32(poly_half_add_f32, POLY_COMB_ADD)
POLY_HALF_REDUCE_F32(poly_half_mul_f32, POLY_COMB_MUL)
POLY_HALF_REDUCE_F32(poly_half_max_f32, POLY_COMB_MAX)

// Generic (any 4/8-byte type) fallback through ds_bpermute shuffles.
template <typename T, typename F, int LANES = 64>
__device__ __forceinline__ T poly_wave_reduce_any(T v, F f) {
#pragma unroll
  for (int m = 1; m < LANES; m <<= 1) {
    T o;
    if constexpr (sizeof(T) == 8) {
      long long x = __builtin_bit_cast(long long, v);
      int lo = __builtin_amdgcn_ds_bpermute(((int)__lane_id() ^ m) << 2, (int)x);
      int hi = __builtin_amdgcn_ds_bpermute(((int)__lane_id() ^ m) << 2, (int)(x >> 32));
      o = __builtin_bit_cast(T, ((long long)hi << 32) | (unsigned int)lo);
    } else {
      int x = __builtin_bit_cast(int, v);
      o = __builtin_bit_cast(T, __builtin_amdgcn_ds_bpermute(((int)__lane_id() ^ m) << 2, x));
    }
    v = f(v, o);
  }
  return v;
}

// threefry2x32, 20 rounds, on a packed (hi:lo) 64-bit counter and key.
__device__ __forceinline__ unsigned long long poly_threefry(unsigned long long x, unsigned long long k) {
  unsigned int x0 = (unsigned int)x, x1 = (unsigned int)(x >> 32);
  unsigned int k0 = (unsigned int)k, k1 = (unsigned int)(k >> 32);
  unsigned int ks[3] = {k1, (k0 ^ k1) ^ 0x1BD11BDAu, k0};
  x0 += ks[2]; x1 += ks[0];
  const int rot[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
#pragma unroll
  for (int i = 0; i < 5; i++) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      int r = rot[i & 1][j];
      unsigned int s = x0 + x1;
      x1 = s ^ ((x1 << r) | (x1 >> (32 - r)));
      x0 = s;
    }
    x0 += ks[i % 3];
    x1 += ks[(i + 1) % 3] + (unsigned int)(i + 1);
  }
  return ((unsigned long long)x1 << 32) | x0;
}
)HIP";
}

std::string Emitter::float_literal(double v, DT dt) {
  bool f64 = (dt == DT_F64);
  if (std::isinf(v)) return f64 ? (v > 0 ? "__builtin_inf()" : "(-__builtin_inf())")
                                : (v > 0 ? "__builtin_inff()" : "(-__builtin_inff())");
  if (std::isnan(v)) return f64 ? "__builtin_nan(\"\")" : "__builtin_nanf(\"\")";
  // Hex float literals round-trip exactly.
  if (f64) return strf("(%a)", v);
  return strf("(%af)", (double)(float)v);
}

std::string Emitter::reduce_identity(PolyOps op, DT dt) {
  // identities as in src/codegen.c:44-51: ADD 0, MUL 1, MAX -inf / type minimum
  if (op == POLY_OP_ADD) return dt_is_float(dt) ? float_literal(0.0, dt) : "0";
  if (op == POLY_OP_MUL) return dt_is_float(dt) ? float_literal(1.0, dt) : "1";
  if (op == POLY_OP_MAX) {
    if (dt_is_float(dt)) return float_literal(-INFINITY, dt);
    switch (dt) {
      case DT_BOOL: return "false";
      case DT_I8: return "(-128)";
      case DT_I16: return "(-32768)";
      case DT_I32: case DT_INDEX: return "(-2147483647-1)";
      case DT_I64: return "(-9223372036854775807ll-1)";
      default: return "0";
    }
  }
  return "0";
}

std::string Emitter::reduce_combine(PolyOps op, DT dt, const std::string &acc, const std::string &v) {
  (void)dt;
  if (op == POLY_OP_ADD) return "(" + acc + "+" + v + ")";
  if (op == POLY_OP_MUL) return "(" + acc + "*" + v + ")";
  return "((" + acc + "<" + v + ")?" + v + ":" + acc + ")";
}

void Emitter::stmt(Scope *s, const std::string &line) {
  s->code.append((size_t)s->indent * 2, ' ');
  s->code += line;
  s->code += "\n";
}

Scope *Emitter::place(uint64_t deps, Scope *s) {
  Scope *t = s;
  while (t->parent && (deps & ~t->parent->avail) == 0) t = t->parent;
  return t;
}

std::string Emitter::emit_atom(int atom, Scope *s) {
  const Atom &a = g_.atoms[(size_t)atom];
  switch (a.kind) {
    case Atom::RANGE: {
      int ord = g_.range_ord.at(a.node);
      auto it = range_name_.find(ord);
      if (it == range_name_.end()) { error_ = strf("range %d used outside its loop", ord); return "0"; }
      return it->second;
    }
    case Atom::VAR: return emit(a.node, s);
    case Atom::OPAQUE: return emit_raw(a.node, s);
    case Atom::DIV: case Atom::MOD: {
      Scope *t = place(g_.atom_deps(atom), s);
      auto f = t->atom_names.find(atom);
      if (f != t->atom_names.end()) return f->second;
      std::string inner = emit_lin(a.inner, t);
      std::string name = strf("q%d", atom);
      int64_t lo = 0, hi = 0;
      g_.lin_bounds(a.inner, &lo, &hi);
      if (a.kind == Atom::MOD && lo < 0) {
        // The dividend can be negative only where the value is not used (positions a pad
        // or shrink masks out: `where(valid, x[...], 0)` still evaluates the index).  The
        // reference's CPU code takes a power-of-two modulus as a bit mask there
        // (src/codegen.c:1675-1748), which keeps such an index inside the buffer; C's %
        // would make it negative.  Floor modulus does the same for every divisor.
        if ((a.c & (a.c - 1)) == 0) stmt(t, strf("const int %s = (%s)&%lld;", name.c_str(), inner.c_str(), (long long)(a.c - 1)));
        else stmt(t, strf("const int %s = (((%s)%%%lld)+%lld)%%%lld;", name.c_str(), inner.c_str(), (long long)a.c, (long long)a.c, (long long)a.c));
      } else {
        stmt(t, strf("const int %s = (%s)%s%lld;", name.c_str(), inner.c_str(),
                     a.kind == Atom::DIV ? "/" : "%", (long long)a.c));
      }
      t->atom_names[atom] = name;
      return name;
    }
  }
  return "0";
}

std::string Emitter::emit_lin(const Lin &l, Scope *s) {
  if (l.is_const()) return strf("%lld", (long long)l.c0);
  std::string e;
  for (const Term &t : l.terms) {
    std::string a = emit_atom(t.atom, s);
    std::string part;
    if (t.coef == 1) part = a;
    else if (t.coef == -1) part = "-" + a;
    else part = strf("%lld*%s", (long long)t.coef, a.c_str());
    if (e.empty()) e = part;
    else if (part[0] == '-') e += part;
    else e += "+" + part;
  }
  if (l.c0 > 0) e += strf("+%lld", (long long)l.c0);
  else if (l.c0 < 0) e += strf("%lld", (long long)l.c0);
  return "(" + e + ")";
}

// num / den in fp32 where den is shared by many values of num (it varies in fewer loops, or
// is computed from per-row results alone): poly_div_shared with the reciprocal of den placed
// where den is computed.  False when the division is not of that kind.
bool Emitter::shared_division(DT dt, int num, int den, Scope *t, std::string *e) {
  if (!shared_divisor || dt != DT_F32 || g_.n(num).dt != DT_F32 || g_.n(den).dt != DT_F32) return false;
  const bool fewer_loops = (g_.n(den).deps & ~g_.n(num).deps) == 0 && g_.n(den).deps != g_.n(num).deps;
  // (a divisor computed from shared presets and constants alone is as shared as they are)
  std::function<bool(int, int)> from_shared = [&](int n, int depth) -> bool {
    if (is_shared_preset(n)) return true;
    if (is_preset(n) || depth > 16) return false;
    const KNode &q = g_.n(n);
    if (q.op == POLY_OP_CONST) return true;
    if (q.op == POLY_OP_LOAD || q.op == POLY_OP_RANGE || q.op == POLY_OP_REDUCE || q.op == POLY_OP_DEFINE_VAR || q.src.empty()) return false;
    for (int sN : q.src) if (!from_shared(sN, depth + 1)) return false;
    return true;
  };
  const bool row_value = !shared_presets_.empty() && g_.n(den).op != POLY_OP_CONST && from_shared(den, 0) && !from_shared(num, 0);
  if (!fewer_loops && !row_value) return false;
  Scope *td = place(g_.n(den).deps, t);
  if (row_value) while (td->parent) td = td->parent;
  if (td == t) return false;
  const int key = -2 - den, key_ok = -1000000 - den;
  const std::string dv = emit(den, td);
  std::string rc, ok;
  auto f = td->names.find(key);
  if (f != td->names.end()) rc = f->second;
  else {
    rc = strf("rcp%d", den);
    stmt(td, strf("const float %s = 1.0f / %s;", rc.c_str(), dv.c_str()));
    td->names[key] = rc;
  }
  auto fo = td->names.find(key_ok);
  if (fo != td->names.end()) ok = fo->second;
  else {
    ok = strf("rok%d", den);
    stmt(td, strf("const bool %s = __builtin_fabsf(%s) >= 0x1p-100f && __builtin_fabsf(%s) <= 0x1p+100f;", ok.c_str(), dv.c_str(), dv.c_str()));
    td->names[key_ok] = ok;
  }
  *e = strf("poly_div_shared(%s, %s, %s, %s)", emit(num, t).c_str(), dv.c_str(), rc.c_str(), ok.c_str());
  return true;
}

std::string Emitter::load_expr(int id, Scope *s) {
  const KNode &k = g_.n(id);
  const KNode &ix = g_.n(k.src[0]);
  int p = g_.param_slot(ix.src[0]);
  std::string idx = emit(ix.src[1], s);
  std::string e = strf("POLY_LD(data%d[%s])", p, idx.c_str());
  std::string gate;
  if (ix.src.size() >= 3) gate = emit(ix.src[2], s);
  if (k.guard >= 0) {
    std::string g2 = emit(k.guard, s);
    if (k.guard_neg) g2 = "(!" + g2 + ")";
    gate = gate.empty() ? g2 : "(" + gate + "&&" + g2 + ")";
  }
  if (!gate.empty()) e = strf("(%s?%s:(%s)0)", gate.c_str(), e.c_str(), dt_cname(k.dt));
  return e;
}

// Is the part of `root` that changes with range `ord` small enough to unroll: a few loads
// whose indices need no division or modulus per iteration?
bool Emitter::light_body(int root, int ord) const {
  std::vector<char> mark(g_.nodes.size(), 0);
  mark_reachable(g_, root, mark);
  const uint64_t bit = (uint64_t)1 << ord;
  int loads = 0, divmods = 0, ops = 0;
  for (size_t id = 0; id < g_.nodes.size(); id++) {
    if (!mark[id] || !(g_.n((int)id).deps & bit)) continue;
    const KNode &n = g_.n((int)id);
    if (n.op == POLY_OP_REDUCE) return false;
    if (n.op == POLY_OP_LOAD) {
      loads++;
      const int li = g_.n(g_.n(n.src[0]).src[1]).lin;
      if (li < 0) return false;
      for (const Term &t : g_.lins[(size_t)li].terms) {
        const Atom &a = g_.atoms[(size_t)t.atom];
        if ((a.kind == Atom::DIV || a.kind == Atom::MOD) && (g_.atom_deps(t.atom) & bit)) divmods++;
      }
    } else if (n.lin < 0 && n.op != POLY_OP_INDEX && n.op != POLY_OP_RANGE) {
      ops++;
    }
  }
  return loads <= 4 && divmods == 0 && ops <= 16;
}

std::string Emitter::emit_reduce_serial(int id, Scope *t) {
  const KNode &k = g_.n(id);
  PolyOps rop = k.u->arg.kind == POLY_ARG_OPS ? k.u->arg.ops : (PolyOps)k.u->arg.i;
  std::string acc = strf("acc%d", id);
  stmt(t, strf("%s %s = %s;", dt_cname(k.dt), acc.c_str(), reduce_identity(rop, k.dt).c_str()));
  Scope inner;
  inner.parent = t;
  inner.avail = t->avail;
  inner.indent = t->indent;
  std::string opens;
  for (size_t i = 1; i < k.src.size(); i++) {
    int ord = g_.range_ord.at(k.src[i]);
    const RangeInfo &r = g_.ranges[(size_t)ord];
    std::string rv = strf("r%d", ord);
    std::string bound = r.extent >= 0 ? strf("%lld", (long long)r.extent) : emit(r.bound_node, t);
    // the innermost loop: several iterations' loads in flight (same order of additions)
    if (i + 1 == k.src.size() && (r.extent < 0 || r.extent >= 64) && light_body(k.src[0], ord)) {
      opens.append((size_t)inner.indent * 2, ' ');
      opens += "#pragma unroll 8\n";
    }
    opens.append((size_t)inner.indent * 2, ' ');
    if (id == slice_node_ && ord == slice_ord_)
      opens += strf("for (int %s = %s; %s < %s; %s += %d) {\n", rv.c_str(), slice_first_.c_str(), rv.c_str(), bound.c_str(), rv.c_str(), slice_step_);
    else
    opens += strf("for (int %s = 0; %s < %s; %s++) {\n", rv.c_str(), rv.c_str(), bound.c_str(), rv.c_str());
    bind_range(ord, rv);
    inner.avail |= (uint64_t)1 << ord;
    inner.indent++;
  }
  std::string v = emit(k.src[0], &inner);
  stmt(&inner, strf("%s = %s;", acc.c_str(), reduce_combine(rop, k.dt, acc, v).c_str()));
  std::string closes;
  for (size_t i = k.src.size() - 1; i >= 1; i--) {
    closes.append((size_t)(t->indent + (int)i - 1) * 2, ' ');
    closes += "}\n";
  }
  if (k.guard >= 0) {
    // only the taken branch of the WHERE above needs the sum
    std::string g = emit(k.guard, t);
    if (k.guard_neg) g = "(!" + g + ")";
    std::string pad((size_t)t->indent * 2, ' ');
    opens = pad + "if (" + g + ") {\n" + opens;
    closes += pad + "}\n";
  }
  t->code += opens + inner.code + closes;
  return acc;
}

std::string Emitter::emit(int id, Scope *s) {
  auto pre = preset_.find(id);
  if (pre != preset_.end()) return pre->second;
  const KNode &k = g_.n(id);
  if (k.op == POLY_OP_CONST) {
    if (dt_is_float(k.dt)) return float_literal(k.u->arg.f, k.dt);
    if (k.dt == DT_BOOL) return k.u->arg.b ? "true" : "false";
    if (k.dt == DT_I64) return strf("%lldll", (long long)k.u->arg.i);
    if (k.dt == DT_U64) return strf("%lluull", (unsigned long long)(uint64_t)k.u->arg.i);
    if (k.dt == DT_U32) return strf("%uu", (unsigned)(uint32_t)k.u->arg.i);
    return strf("%lld", (long long)k.u->arg.i);
  }
  if (k.op == POLY_OP_DEFINE_VAR) {
    for (size_t i = 0; i < g_.vars.size(); i++)
      if (g_.vars[i].node == id) return strf("var%zu", i);
    error_ = "unknown DEFINE_VAR";
    return "0";
  }
  if (k.lin >= 0) {
    const Lin &l = g_.lins[(size_t)k.lin];
    bool self_opaque = l.c0 == 0 && l.terms.size() == 1 && l.terms[0].coef == 1 &&
                       g_.atoms[(size_t)l.terms[0].atom].kind == Atom::OPAQUE &&
                       g_.atoms[(size_t)l.terms[0].atom].node == id;
    if (!self_opaque) {
      if (l.is_const() || (l.terms.size() == 1 && l.c0 == 0 && l.terms[0].coef == 1)) return emit_lin(l, s);
      Scope *t = place(g_.lin_deps(l), s);
      auto f = t->names.find(id);
      if (f != t->names.end()) return f->second;
      std::string e = emit_lin(l, t);
      std::string name = strf("i%d", id);
      stmt(t, strf("const int %s = %s;", name.c_str(), e.c_str()));
      t->names[id] = name;
      return name;
    }
  }
  return emit_raw(id, s);
}

std::string Emitter::emit_raw(int id, Scope *s) {
  auto pre = preset_.find(id);
  if (pre != preset_.end()) return pre->second;
  const KNode &k = g_.n(id);
  Scope *t = place(k.deps, s);
  auto f = t->names.find(id);
  if (f != t->names.end()) return f->second;
  if (k.op == POLY_OP_RANGE) {
    int ord = g_.range_ord.at(id);
    auto it = range_name_.find(ord);
    if (it == range_name_.end()) { error_ = strf("range %d used outside its loop", ord); return "0"; }
    return it->second;
  }
  if (k.op == POLY_OP_REDUCE) {
    auto cu = custom_.find(id);
    std::string acc = cu != custom_.end() ? cu->second(t) : emit_reduce_serial(id, t);
    t->names[id] = acc;
    return acc;
  }
  auto S = [&](size_t i) { return emit(k.src[i], t); };
  const char *ct = dt_cname(k.dt);
  std::string e;
  switch (k.op) {
    case POLY_OP_LOAD: e = load_expr(id, t); break;
    case POLY_OP_CAST: {
      DT sdt = g_.n(k.src[0]).dt;
      const KNode &q = g_.n(k.src[0]);
      if (recip_div16 && (k.dt == DT_BF16 || k.dt == DT_F16) && sdt == DT_F32 && !is_preset(k.src[0])) {
        int num = -1, den = -1;
        if (q.op == POLY_OP_FDIV) { num = q.src[0]; den = q.src[1]; }
        else if (q.op == POLY_OP_MUL && g_.n(q.src[1]).op == POLY_OP_RECIPROCAL && !is_preset(q.src[1])) { num = q.src[0]; den = g_.n(q.src[1]).src[0]; }
        if (num >= 0 && (g_.n(den).deps & ~g_.n(num).deps) == 0 && g_.n(den).deps != g_.n(num).deps) {
          // the divisor varies in fewer loops than the dividend: one reciprocal per value of it
          Scope *td = place(g_.n(den).deps, t);
          const int key = -2 - den;
          auto f = td->names.find(key);
          std::string rc;
          if (f != td->names.end()) rc = f->second;
          else {
            rc = strf("rcp%d", den);
            const std::string dv = emit(den, td);
            stmt(td, strf("const float %s = 1.0f / %s;", rc.c_str(), dv.c_str()));
            td->names[key] = rc;
          }
          e = strf("(%s)(%s * %s)", ct, emit(num, t).c_str(), rc.c_str());
          break;
        }
      }
      if (k.dt == DT_BOOL && sdt != DT_BOOL) e = strf("(%s!=0)", S(0).c_str());
      else e = strf("(%s)(%s)", ct, S(0).c_str());
      break;
    }
    case POLY_OP_BITCAST: {
      DT sdt = g_.n(k.src[0]).dt;
      if (dt_size(sdt) != dt_size(k.dt)) { error_ = "BITCAST between different sizes"; return "0"; }
      e = strf("__builtin_bit_cast(%s, (%s)(%s))", ct, dt_cname(sdt), S(0).c_str());
      break;
    }
    case POLY_OP_NEG: e = k.dt == DT_BOOL ? strf("(!%s)", S(0).c_str()) : strf("(-%s)", S(0).c_str()); break;
    case POLY_OP_SQRT: e = k.dt == DT_F64 ? strf("__builtin_sqrt(%s)", S(0).c_str()) : strf("__builtin_sqrtf(%s)", S(0).c_str()); break;
    case POLY_OP_TRUNC: e = k.dt == DT_F64 ? strf("__builtin_trunc(%s)", S(0).c_str()) : strf("__builtin_truncf(%s)", S(0).c_str()); break;
    case POLY_OP_EXP2:
      if (k.dt == DT_F64) e = strf("__builtin_exp2(%s)", S(0).c_str());
      else if (k.dt == DT_F32 && raw_exp2) e = strf("__builtin_amdgcn_exp2f(%s)", S(0).c_str());
      else e = strf("__builtin_exp2f(%s)", S(0).c_str());
      break;
    case POLY_OP_LOG2: e = k.dt == DT_F64 ? strf("__builtin_log2(%s)", S(0).c_str()) : strf("__builtin_log2f(%s)", S(0).c_str()); break;
    // the device library's sin (argument reduction for any magnitude); the builtin would
    // become the hardware approximation, which loses accuracy beyond a few periods
    case POLY_OP_SIN: e = k.dt == DT_F64 ? strf("__ocml_sin_f64(%s)", S(0).c_str()) : strf("__ocml_sin_f32(%s)", S(0).c_str()); break;
    case POLY_OP_RECIPROCAL: e = strf("(1/%s)", S(0).c_str()); break;
    case POLY_OP_ADD: e = strf("(%s+%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_SUB: e = strf("(%s-%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_MUL: {
      // a * (1/b) is a single division, as the reference's late rewrite makes it
      // (src/codegen.c:1867-1883; the reciprocal must be the second factor)
      const KNode &rb = g_.n(k.src[1]);
      if (dt_is_float(k.dt) && rb.op == POLY_OP_RECIPROCAL && rb.src.size() == 1) {
        if (is_preset(k.src[1]) || !shared_division(k.dt, k.src[0], rb.src[0], t, &e)) e = strf("(%s/%s)", S(0).c_str(), emit(rb.src[0], t).c_str());
        break;
      }
      e = strf("(%s*%s)", S(0).c_str(), S(1).c_str());
      break;
    }
    case POLY_OP_FDIV:
      if (!shared_division(k.dt, k.src[0], k.src[1], t, &e)) e = strf("(%s/%s)", S(0).c_str(), S(1).c_str());
      break;
    case POLY_OP_IDIV: e = strf("(%s/%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_MOD: e = strf("(%s%%%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_SHL: e = strf("(%s<<%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_SHR: e = strf("(%s>>%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_AND: e = strf("(%s&%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_OR: e = strf("(%s|%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_XOR: e = strf("(%s^%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_CMPLT: e = strf("(%s<%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_CMPNE: e = strf("(%s!=%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_CMPEQ: e = strf("(%s==%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_MAX: { std::string a = S(0), b = S(1); e = strf("((%s<%s)?%s:%s)", a.c_str(), b.c_str(), b.c_str(), a.c_str()); break; }
    case POLY_OP_POW: e = k.dt == DT_F64 ? strf("__builtin_pow(%s,%s)", S(0).c_str(), S(1).c_str())
                                         : strf("__builtin_powf(%s,%s)", S(0).c_str(), S(1).c_str()); break;
    case POLY_OP_WHERE: e = strf("(%s?%s:%s)", S(0).c_str(), S(1).c_str(), S(2).c_str()); break;
    case POLY_OP_MULACC: e = strf("((%s*%s)+%s)", S(0).c_str(), S(1).c_str(), S(2).c_str()); break;
    case POLY_OP_THREEFRY:
      uses_threefry = true;
      e = strf("(%s)poly_threefry((unsigned long long)%s,(unsigned long long)%s)", ct, S(0).c_str(), S(1).c_str());
      break;
    default:
      error_ = strf("op %s is not supported inside a kernel", op_name(k.op));
      return "0";
  }
  if (failed()) return "0";
  if (pow2_mul16_exact && k.op == POLY_OP_MUL && (k.dt == DT_BF16 || k.dt == DT_F16)) {
    for (int side = 0; side < 2; side++) {
      const KNode &c = g_.n(k.src[(size_t)side]);
      if (c.op != POLY_OP_CONST || c.u->arg.kind != POLY_ARG_FLOAT || g_.n(k.src[(size_t)(1 - side)]).dt != k.dt) continue;
      int ex = 0;
      const double v = c.u->arg.f;
      if (std::isfinite(v) && v != 0 && std::fabs(std::frexp(v, &ex)) == 0.5 && ex > -100 && ex < 100) ct = "float";
    }
  }
  std::string name = strf("v%d", id);
  stmt(t, strf("const %s %s = %s;", ct, name.c_str(), e.c_str()));
  t->names[id] = name;
  return name;
}

}  // namespace polyhip
