// planfile: a portable container for a PolySchedule (kernel roots, slot table,
// execution order, default variable bindings), so that a schedule produced once
// by polygrad's scheduler can be compiled for the GPU without the frontend.
//
// Layout (little endian):
//   "POLYPLN1"  u32 n_slots  u32 n_items  u32 n_vars  u32 n_default_vars
//   vars:       { u16 len, bytes name, i64 min, i64 max }
//   defaults:   { u32 var_id, i32 value }
//   slots:      { u8 dtype, u8 is_intermediate, i32 external_idx, i64 numel, i64 nbytes,
//                 u16 len, bytes name }
//   items:      { u32 n_params, i32 slot[n_params], u32 n_vars, u32 var_id[n_vars],
//                 u32 n_nodes, node[n_nodes] }   (nodes topological, root last)
//   node:       { u16 op, u8 dtype, u8 flags(bit0 ptr, bits1-2 addrspace), u16 count,
//                 u16 vcount, i64 ptr_size, i32 tag, u16 n_src, u32 src[n_src], u8 arg_kind, arg }
//   exec_order: u32[n_items]
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <memory>
#include <unordered_map>

#include "common.h"
#include "polygrad_hip.h"

namespace polyhip {

static const PolyDType &dtype_of_code(int code) {
  static const PolyDType table[POLYHIP_DT_COUNT] = {
      {-1, 0, "void", 0, 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {0, 1, "bool", '?', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {1, 8, "signed char", 'b', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {2, 8, "unsigned char", 'B', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {3, 16, "short", 'h', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {4, 16, "unsigned short", 'H', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {5, 32, "int", 'i', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {6, 32, "unsigned int", 'I', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {7, 64, "long", 'q', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {8, 64, "unsigned long", 'Q', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {11, 16, "__fp16", 'e', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {12, 16, "__bf16", 0, 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {13, 32, "float", 'f', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {14, 64, "double", 'd', 1, false, POLY_ADDR_GLOBAL, 0, 0},
      {-1, 800, "index", 0, 1, false, POLY_ADDR_GLOBAL, 0, 0},
  };
  return table[code >= 0 && code < POLYHIP_DT_COUNT ? code : 0];
}

struct Writer {
  std::vector<unsigned char> b;
  template <typename T> void put(T v) { const unsigned char *p = (const unsigned char *)&v; b.insert(b.end(), p, p + sizeof(T)); }
  void str(const char *s) {
    size_t n = s ? strlen(s) : 0;
    if (n > 65535) n = 65535;
    put<uint16_t>((uint16_t)n);
    b.insert(b.end(), (const unsigned char *)s, (const unsigned char *)s + n);
  }
};

struct Reader {
  const unsigned char *p, *end;
  bool bad = false;
  template <typename T> T get() {
    T v{};
    if ((size_t)(end - p) < sizeof(T)) { bad = true; return v; }
    memcpy(&v, p, sizeof(T));
    p += sizeof(T);
    return v;
  }
  std::string str() {
    uint16_t n = get<uint16_t>();
    if ((size_t)(end - p) < n) { bad = true; return ""; }
    std::string s((const char *)p, n);
    p += n;
    return s;
  }
};

static bool write_item(Writer &w, const PolyExecItem &it, std::unordered_map<const PolyUOp *, uint32_t> &var_ids,
                       std::vector<const PolyUOp *> &vars) {
  // post-order over the DAG
  std::vector<const PolyUOp *> order;
  std::unordered_map<const PolyUOp *, uint32_t> idx;
  struct Frame { const PolyUOp *u; int next; };
  std::vector<Frame> st;
  std::unordered_map<const PolyUOp *, char> seen;
  st.push_back({it.root, 0});
  seen[it.root] = 1;
  while (!st.empty()) {
    Frame &f = st.back();
    if (f.next < (int)f.u->n_src) {
      const PolyUOp *s = f.u->src[f.next++];
      if (!seen.count(s)) { seen[s] = 1; st.push_back({s, 0}); }
    } else {
      idx[f.u] = (uint32_t)order.size();
      order.push_back(f.u);
      st.pop_back();
    }
  }
  auto var_id = [&](const PolyUOp *u) {
    auto f = var_ids.find(u);
    if (f != var_ids.end()) return f->second;
    uint32_t id = (uint32_t)vars.size();
    var_ids[u] = id;
    vars.push_back(u);
    return id;
  };
  w.put<uint32_t>((uint32_t)it.n_buf_slots);
  for (int i = 0; i < it.n_buf_slots; i++) w.put<int32_t>(it.buf_slot_indices[i]);
  w.put<uint32_t>((uint32_t)it.n_var_uops);
  for (int i = 0; i < it.n_var_uops; i++) w.put<uint32_t>(var_id(it.var_uops[i]));
  w.put<uint32_t>((uint32_t)order.size());
  for (const PolyUOp *u : order) {
    DT dt = classify_dtype(u->dtype);
    if (dt == DT_BAD) { log_err("planfile", "unsupported dtype in kernel graph"); return false; }
    w.put<uint16_t>((uint16_t)u->op);
    w.put<uint8_t>((uint8_t)dt);
    w.put<uint8_t>((uint8_t)((u->dtype.is_ptr ? 1 : 0) | ((int)u->dtype.addrspace << 1)));
    w.put<uint16_t>(u->dtype.count);
    w.put<uint16_t>(u->dtype.vcount);
    w.put<int64_t>(u->dtype.ptr_size);
    w.put<int32_t>(u->tag);
    w.put<uint16_t>(u->n_src);
    for (int i = 0; i < (int)u->n_src; i++) w.put<uint32_t>(idx[u->src[i]]);
    w.put<uint8_t>((uint8_t)u->arg.kind);
    switch (u->arg.kind) {
      case POLY_ARG_NONE: case POLY_ARG_INVALID: break;
      case POLY_ARG_INT: w.put<int64_t>(u->arg.i); break;
      case POLY_ARG_FLOAT: w.put<double>(u->arg.f); break;
      case POLY_ARG_BOOL: w.put<uint8_t>(u->arg.b ? 1 : 0); break;
      case POLY_ARG_OPS: w.put<uint32_t>((uint32_t)u->arg.ops); break;
      case POLY_ARG_STRING: w.str(u->arg.str); break;
      case POLY_ARG_INT_TUPLE:
        w.put<uint32_t>((uint32_t)u->arg.int_tuple.n);
        for (int i = 0; i < u->arg.int_tuple.n; i++) w.put<int64_t>(u->arg.int_tuple.vals[i]);
        break;
      case POLY_ARG_PAIR_TUPLE:
        w.put<uint32_t>((uint32_t)u->arg.pair_tuple.n);
        for (int i = 0; i < u->arg.pair_tuple.n; i++) { w.put<int64_t>(u->arg.pair_tuple.pairs[i][0]); w.put<int64_t>(u->arg.pair_tuple.pairs[i][1]); }
        break;
      case POLY_ARG_REDUCE_AXIS:
        w.put<uint32_t>((uint32_t)u->arg.reduce_axis.op);
        w.put<uint32_t>((uint32_t)u->arg.reduce_axis.n);
        for (int i = 0; i < u->arg.reduce_axis.n; i++) w.put<int64_t>(u->arg.reduce_axis.axes[i]);
        break;
      case POLY_ARG_RANGE:
        w.put<int64_t>(u->arg.range.axis_id);
        w.put<uint32_t>((uint32_t)u->arg.range.axis_type);
        w.put<uint32_t>((uint32_t)u->arg.range.n_extra);
        for (int i = 0; i < u->arg.range.n_extra; i++) w.put<int64_t>(u->arg.range.extra[i]);
        break;
      case POLY_ARG_DEFINE_VAR: w.put<uint32_t>(var_id(u)); break;
    }
  }
  return true;
}

}  // namespace polyhip

using namespace polyhip;

struct PolyHipPlanFile {
  PolySchedule sched{};
  std::deque<PolyUOp> uops;                    // stable addresses
  std::deque<std::vector<PolyUOp *>> srcs;
  std::deque<std::vector<int64_t>> ints;
  std::deque<std::string> strings;
  std::vector<PolyUOp *> vars;
  std::vector<PolyScheduleBufSlot> slots;
  std::vector<std::string> slot_names;
  std::vector<PolyExecItem> items;
  std::deque<std::vector<int>> item_slots;
  std::deque<std::vector<PolyUOp *>> item_vars;
  std::vector<int> exec_order;
  std::vector<PolyVarBinding> defaults;
};

extern "C" {

int poly_hip_planfile_save(const PolySchedule *s, const char *const *names, const char *path) {
  if (!s || !path) return -1;
  Writer items;
  std::unordered_map<const PolyUOp *, uint32_t> var_ids;
  std::vector<const PolyUOp *> vars;
  for (int i = 0; i < s->n_default_vars; i++) {
    var_ids[s->default_vars[i].var] = (uint32_t)vars.size();
    vars.push_back(s->default_vars[i].var);
  }
  for (int k = 0; k < s->n_items; k++) {
    if (s->items[k].kind != POLY_EXEC_COMPUTE) { log_err("planfile", "item %d is not a compute item", k); return -1; }
    if (!write_item(items, s->items[k], var_ids, vars)) return -1;
  }
  Writer w;
  w.b.insert(w.b.end(), (const unsigned char *)"POLYPLN1", (const unsigned char *)"POLYPLN1" + 8);
  w.put<uint32_t>((uint32_t)s->n_buf_slots);
  w.put<uint32_t>((uint32_t)s->n_items);
  w.put<uint32_t>((uint32_t)vars.size());
  w.put<uint32_t>((uint32_t)s->n_default_vars);
  for (const PolyUOp *v : vars) {
    if (v->op != POLY_OP_DEFINE_VAR || v->arg.kind != POLY_ARG_DEFINE_VAR) { log_err("planfile", "var is not a DEFINE_VAR"); return -1; }
    w.str(v->arg.define_var.name);
    w.put<int64_t>(v->arg.define_var.min_val);
    w.put<int64_t>(v->arg.define_var.max_val);
  }
  for (int i = 0; i < s->n_default_vars; i++) { w.put<uint32_t>(var_ids[s->default_vars[i].var]); w.put<int32_t>(s->default_vars[i].value); }
  for (int i = 0; i < s->n_buf_slots; i++) {
    const PolyScheduleBufSlot &b = s->buf_slots[i];
    DT dt = classify_dtype(b.dtype);
    if (dt == DT_BAD) { log_err("planfile", "slot %d has an unsupported dtype", i); return -1; }
    w.put<uint8_t>((uint8_t)dt);
    w.put<uint8_t>(b.is_intermediate ? 1 : 0);
    w.put<int32_t>(b.external_buf_idx);
    w.put<int64_t>(b.numel);
    w.put<int64_t>(b.nbytes);
    w.str((names && !b.is_intermediate && names[i]) ? names[i] : "");
  }
  w.b.insert(w.b.end(), items.b.begin(), items.b.end());
  for (int k = 0; k < s->n_items; k++) w.put<uint32_t>((uint32_t)s->exec_order[k]);
  FILE *f = fopen(path, "wb");
  if (!f) { log_err("planfile", "cannot write %s", path); return -1; }
  size_t n = fwrite(w.b.data(), 1, w.b.size(), f);
  fclose(f);
  return n == w.b.size() ? 0 : -1;
}

PolyHipPlanFile *poly_hip_planfile_load(const char *path) {
  FILE *f = path ? fopen(path, "rb") : nullptr;
  if (!f) { log_err("planfile", "cannot open %s", path ? path : "(null)"); return nullptr; }
  std::vector<unsigned char> buf;
  unsigned char tmp[65536];
  size_t n;
  while ((n = fread(tmp, 1, sizeof(tmp), f)) > 0) buf.insert(buf.end(), tmp, tmp + n);
  fclose(f);
  if (buf.size() < 24 || memcmp(buf.data(), "POLYPLN1", 8) != 0) { log_err("planfile", "%s: bad magic", path); return nullptr; }
  Reader r{buf.data() + 8, buf.data() + buf.size()};
  std::unique_ptr<PolyHipPlanFile> pf(new PolyHipPlanFile());
  uint32_t n_slots = r.get<uint32_t>(), n_items = r.get<uint32_t>(), n_vars = r.get<uint32_t>(), n_def = r.get<uint32_t>();
  if (n_slots > (1u << 24) || n_items > (1u << 24) || n_vars > (1u << 16) || n_def > n_vars) { log_err("planfile", "%s: bad header", path); return nullptr; }
  const PolyDType i32 = dtype_of_code(POLYHIP_DT_INT32);
  for (uint32_t i = 0; i < n_vars && !r.bad; i++) {
    pf->strings.push_back(r.str());
    PolyUOp u{};
    u.op = POLY_OP_DEFINE_VAR; u.dtype = i32; u.src = nullptr; u.n_src = 0;
    u.arg.kind = POLY_ARG_DEFINE_VAR;
    u.arg.define_var.name = pf->strings.back().c_str();
    u.arg.define_var.min_val = r.get<int64_t>();
    u.arg.define_var.max_val = r.get<int64_t>();
    pf->uops.push_back(u);
    pf->vars.push_back(&pf->uops.back());
  }
  for (uint32_t i = 0; i < n_def && !r.bad; i++) {
    uint32_t id = r.get<uint32_t>();
    int32_t val = r.get<int32_t>();
    if (id >= n_vars) { r.bad = true; break; }
    pf->defaults.push_back({pf->vars[id], val});
  }
  for (uint32_t i = 0; i < n_slots && !r.bad; i++) {
    PolyScheduleBufSlot b{};
    const uint8_t slot_dt = r.get<uint8_t>();
    if (slot_dt >= POLYHIP_DT_COUNT) { r.bad = true; break; }
    b.dtype = dtype_of_code(slot_dt);
    b.is_intermediate = r.get<uint8_t>() != 0;
    b.external_buf_idx = r.get<int32_t>();
    b.numel = r.get<int64_t>();
    b.nbytes = r.get<int64_t>();
    b.buf_uop = nullptr;
    pf->slot_names.push_back(r.str());
    pf->slots.push_back(b);
  }
  for (uint32_t k = 0; k < n_items && !r.bad; k++) {
    PolyExecItem it{};
    it.kind = POLY_EXEC_COMPUTE;
    uint32_t np = r.get<uint32_t>();
    if (np > 4096) { r.bad = true; break; }
    pf->item_slots.emplace_back();
    for (uint32_t i = 0; i < np; i++) {
      int32_t s = r.get<int32_t>();
      if (s < 0 || (uint32_t)s >= n_slots) r.bad = true;
      pf->item_slots.back().push_back(s);
    }
    uint32_t nv = r.get<uint32_t>();
    if (nv > n_vars) { r.bad = true; break; }
    pf->item_vars.emplace_back();
    for (uint32_t i = 0; i < nv; i++) {
      uint32_t id = r.get<uint32_t>();
      if (id >= n_vars) { r.bad = true; break; }
      pf->item_vars.back().push_back(pf->vars[id]);
    }
    uint32_t nn = r.get<uint32_t>();
    if (nn == 0 || nn > (1u << 24)) { r.bad = true; break; }
    std::vector<PolyUOp *> nodes;
    nodes.reserve(nn);
    for (uint32_t j = 0; j < nn && !r.bad; j++) {
      PolyUOp u{};
      // every enumeration read from the file is range-checked before it becomes one
      const uint16_t op_code = r.get<uint16_t>();
      if (op_code < 1 || op_code >= (uint16_t)POLY_OP_COUNT) { r.bad = true; break; }
      u.op = (PolyOps)op_code;
      const uint8_t dt_code = r.get<uint8_t>();
      if (dt_code >= POLYHIP_DT_COUNT) { r.bad = true; break; }
      u.dtype = dtype_of_code(dt_code);
      uint8_t flags = r.get<uint8_t>();
      if (((flags >> 1) & 3) > (uint8_t)POLY_ADDR_REG) { r.bad = true; break; }
      u.dtype.count = r.get<uint16_t>();
      if (u.dtype.count > 1) u.dtype.bitsize = (uint16_t)(u.dtype.bitsize * u.dtype.count);
      u.dtype.vcount = r.get<uint16_t>();
      u.dtype.ptr_size = r.get<int64_t>();
      u.dtype.is_ptr = flags & 1;
      u.dtype.addrspace = (PolyAddrSpace)((flags >> 1) & 3);
      u.tag = r.get<int32_t>();
      u.n_src = r.get<uint16_t>();
      pf->srcs.emplace_back();
      for (int s = 0; s < (int)u.n_src; s++) {
        uint32_t si = r.get<uint32_t>();
        if (si >= j) { r.bad = true; break; }
        pf->srcs.back().push_back(nodes[si]);
      }
      u.src = pf->srcs.back().empty() ? nullptr : pf->srcs.back().data();
      const uint8_t kind_code = r.get<uint8_t>();
      if (kind_code > (uint8_t)POLY_ARG_INVALID) { r.bad = true; break; }
      u.arg.kind = (PolyArgKind)kind_code;
      auto get_op = [&]() {
        const uint32_t v = r.get<uint32_t>();
        if (v < 1 || v >= (uint32_t)POLY_OP_COUNT) { r.bad = true; return POLY_OP_NOOP; }
        return (PolyOps)v;
      };
      bool is_var = false;
      switch (u.arg.kind) {
        case POLY_ARG_NONE: case POLY_ARG_INVALID: break;
        case POLY_ARG_INT: u.arg.i = r.get<int64_t>(); break;
        case POLY_ARG_FLOAT: u.arg.f = r.get<double>(); break;
        case POLY_ARG_BOOL: u.arg.b = r.get<uint8_t>() != 0; break;
        case POLY_ARG_OPS: u.arg.ops = get_op(); break;
        case POLY_ARG_STRING: pf->strings.push_back(r.str()); u.arg.str = pf->strings.back().c_str(); break;
        case POLY_ARG_INT_TUPLE: {
          uint32_t c = r.get<uint32_t>();
          if (c > (1u << 20)) { r.bad = true; break; }
          pf->ints.emplace_back();
          for (uint32_t i = 0; i < c; i++) pf->ints.back().push_back(r.get<int64_t>());
          u.arg.int_tuple.vals = pf->ints.back().data();
          u.arg.int_tuple.n = (int)c;
          break;
        }
        case POLY_ARG_PAIR_TUPLE: {
          uint32_t c = r.get<uint32_t>();
          if (c > (1u << 20)) { r.bad = true; break; }
          pf->ints.emplace_back();
          for (uint32_t i = 0; i < 2 * c; i++) pf->ints.back().push_back(r.get<int64_t>());
          u.arg.pair_tuple.pairs = (int64_t(*)[2])pf->ints.back().data();
          u.arg.pair_tuple.n = (int)c;
          break;
        }
        case POLY_ARG_REDUCE_AXIS: {
          u.arg.reduce_axis.op = get_op();
          uint32_t c = r.get<uint32_t>();
          if (c > (1u << 20)) { r.bad = true; break; }
          pf->ints.emplace_back();
          for (uint32_t i = 0; i < c; i++) pf->ints.back().push_back(r.get<int64_t>());
          u.arg.reduce_axis.axes = pf->ints.back().data();
          u.arg.reduce_axis.n = (int)c;
          break;
        }
        case POLY_ARG_RANGE: {
          u.arg.range.axis_id = r.get<int64_t>();
          const uint32_t axis_type = r.get<uint32_t>();
          if (axis_type > (uint32_t)POLY_AXIS_PLACEHOLDER) { r.bad = true; break; }
          u.arg.range.axis_type = (PolyAxisType)axis_type;
          uint32_t c = r.get<uint32_t>();
          if (c > (1u << 20)) { r.bad = true; break; }
          pf->ints.emplace_back();
          for (uint32_t i = 0; i < c; i++) pf->ints.back().push_back(r.get<int64_t>());
          u.arg.range.extra = c ? pf->ints.back().data() : nullptr;
          u.arg.range.n_extra = (int)c;
          break;
        }
        case POLY_ARG_DEFINE_VAR: {
          uint32_t id = r.get<uint32_t>();
          if (id >= n_vars) { r.bad = true; break; }
          nodes.push_back(pf->vars[id]);   // shared DEFINE_VAR node
          is_var = true;
          break;
        }
        default: r.bad = true; break;
      }
      if (is_var) continue;
      pf->uops.push_back(u);
      nodes.push_back(&pf->uops.back());
    }
    if (r.bad) break;
    it.root = nodes.back();
    it.buf_slot_indices = pf->item_slots.back().data();
    it.n_buf_slots = (int)np;
    it.var_uops = pf->item_vars.back().empty() ? nullptr : pf->item_vars.back().data();
    it.n_var_uops = (int)nv;
    pf->items.push_back(it);
  }
  for (uint32_t k = 0; k < n_items && !r.bad; k++) {
    uint32_t e = r.get<uint32_t>();
    if (e >= n_items) r.bad = true;
    pf->exec_order.push_back((int)e);
  }
  if (r.bad) { log_err("planfile", "%s: truncated or corrupt", path); return nullptr; }
  PolySchedule &s = pf->sched;
  s.entrypoint_name = "planfile";
  s.mode = POLY_MODE_CALL;
  s.buf_slots = pf->slots.data();
  s.n_buf_slots = (int)pf->slots.size();
  s.items = pf->items.data();
  s.n_items = (int)pf->items.size();
  s.exec_order = pf->exec_order.data();
  s.default_vars = pf->defaults.empty() ? nullptr : pf->defaults.data();
  s.n_default_vars = (int)pf->defaults.size();
  s.loss_buf_slot = -1;
  s.grad_buf_slots = nullptr;
  return pf.release();
}

const PolySchedule *poly_hip_planfile_schedule(const PolyHipPlanFile *pf) { return pf ? &pf->sched : nullptr; }

const char *poly_hip_planfile_slot_name(const PolyHipPlanFile *pf, int slot) {
  if (!pf || slot < 0 || slot >= (int)pf->slot_names.size()) return "";
  return pf->slot_names[(size_t)slot].c_str();
}

void poly_hip_planfile_free(PolyHipPlanFile *pf) { delete pf; }

}  // extern "C"
