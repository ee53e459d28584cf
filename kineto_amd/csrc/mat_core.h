/*
 * mat_core.h — turns one raw record plus its join results into a MatRow (host/device).
 *
 * Accessor semantics being reproduced (paths relative to the pytorch/kineto tree):
 *   libkineto/include/GenericTraceActivity.h:45-100   GenericTraceActivity accessors
 *   libkineto/src/RocprofActivity.h:37-162             RocprofActivity / GpuActivity / RuntimeActivity
 *   libkineto/src/CuptiTimestamp.h:29-51               timestamp / duration of CUPTI-shaped rows
 *   libkineto/src/output_json.cpp:871-891              "External id" rule
 */
#ifndef KTJ_MAT_CORE_H_
#define KTJ_MAT_CORE_H_

#include "fmt_core.h"

namespace ktj {

struct ClockDev {
  uint64_t t0_approx;
  int64_t t0;
  uint64_t scale_bits;
  int64_t async_offset;
  uint32_t runtime_mode;
  uint32_t device_mode;
};

/* RocprofActivityApi.cpp:166-175: begin and end are converted separately */
KTJ_HD inline void convert_range(const ClockDev& c, uint32_t mode, uint64_t* begin, uint64_t* end) {
  if (mode == KTJ_CLOCK_CONVERT) {
    *begin = (uint64_t)convert_timestamp(*begin, c.t0_approx, c.t0, c.scale_bits);
    *end = (uint64_t)convert_timestamp(*end, c.t0_approx, c.t0, c.scale_bits);
  } else if (mode == KTJ_CLOCK_OFFSET) {
    *begin += (uint64_t)c.async_offset;
    *end += (uint64_t)c.async_offset;
  }
}

/* The kind of a device row: the low 16 bits of `domain`; kinds this engine does not know are
 * kernel dispatches, as in GpuActivity's constructor (RocprofActivity.h:88-97). */
KTJ_HD inline uint32_t device_row_domain(uint32_t raw) {
  const uint32_t d = KTJ_ROW_DOMAIN(raw);
  return d <= KTJ_DOM_MEMSET ? d : KTJ_DOM_KERNEL_DISPATCH;
}
/* resourceId() of a device row as submitted: a memset row's stream id is 32 bits wide (ktj_memset_rec) */
KTJ_HD inline int64_t device_row_stream(uint32_t dom, uint64_t stream) {
  return dom == KTJ_DOM_MEMSET ? (int64_t)(stream & 0xFFFFFFFFull) : (int64_t)stream;
}

/* timestamp()/duration() of a device row after clock conversion */
KTJ_HD inline void device_times(uint32_t domain, uint64_t begin, uint64_t end, int64_t* ts, int64_t* dur) {
  if (domain == KTJ_DOM_MEMSET) {
    *ts = (int64_t)begin;
    *dur = (int64_t)end - (int64_t)begin;
  } else { /* RocprofActivity.h:122-127 */
    *ts = (int64_t)(begin + 1);
    *dur = (int64_t)(end - (begin + 1));
  }
}

/* GenericActivityProfiler::outOfRange: GenericActivityProfiler.cpp:329-340 */
KTJ_HD inline bool out_of_range(int64_t ts, int64_t dur, int64_t win_start, int64_t win_end) {
  return ts < win_start || (ts + dur) > win_end;
}

/* key under which the profiler looks a correlation id up: linkedActivity(int32_t, …)
 * (GenericActivityProfiler.cpp:397-408) narrows it to int32 and widens it again */
KTJ_HD inline uint64_t narrow_corr_key(uint64_t id) { return (uint64_t)(int64_t)(int32_t)(uint32_t)id; }

KTJ_HD inline bool type_hides_own_external_id(uint32_t type) { /* output_json.cpp:878-887 */
  switch (type) {
    case KTJ_TYPE_GPU_MEMCPY: case KTJ_TYPE_GPU_MEMSET: case KTJ_TYPE_CONCURRENT_KERNEL:
    case KTJ_TYPE_CUDA_RUNTIME: case KTJ_TYPE_CUDA_DRIVER: case KTJ_TYPE_XPU_RUNTIME:
    case KTJ_TYPE_XPU_DRIVER: case KTJ_TYPE_PRIVATEUSE1_RUNTIME: case KTJ_TYPE_PRIVATEUSE1_DRIVER:
      return true;
    default: return false;
  }
}

/* deviceId() of a generic record: the 32-bit field, or the args slot before the record's values */
KTJ_HD inline int64_t generic_device(const ktj_generic_rec& g, const uint64_t* args, uint64_t n_args) {
  if ((g.flags & KTJ_GF_WIDE_DEVICE) && g.args_off >= 1 && g.args_off - 1 < n_args) return (int64_t)args[g.args_off - 1];
  return g.device;
}

KTJ_HD inline MatRow mat_generic(const ktj_generic_rec& g, int64_t device) {
  MatRow m;
  m.ts = g.start_ns;
  m.dur = g.end_ns - g.start_ns;
  m.dev = device;
  m.res = g.resource;
  m.flow_id = g.flow_id;
  uint32_t meta = (g.type & KTJ_M_TYPE_MASK) | (KTJ_CLASS_GENERIC << KTJ_M_CLASS_SHIFT) | KTJ_M_VALID;
  /* instant and counter events (output_json.cpp:842-856, 660-716): no flow, no External id */
  const bool instant = g.type == KTJ_TYPE_CPU_INSTANT_EVENT || g.type == KTJ_TYPE_HARDWARE_COUNTERS ||
                       g.type == KTJ_TYPE_MTIA_COUNTERS || g.type == KTJ_TYPE_XPU_SCOPE_PROFILER;
  if (!instant && g.flow_id > 0 && (g.flow_type == KTJ_LINK_FWDBWD || g.flow_type == KTJ_LINK_ASYNC_CPU_GPU)) {
    meta |= KTJ_M_FLOW;
    if (g.flags & KTJ_GF_FLOW_START) meta |= KTJ_M_FLOW_START;
    if (g.flow_type == KTJ_LINK_FWDBWD) meta |= KTJ_M_FLOW_FWDBWD;
  }
  if (g.name_id == KTJ_NONE) { meta |= KTJ_M_NAME_BUILTIN; m.name_id = KTJ_NAME_EMPTY; }
  else m.name_id = g.name_id;
  m.meta = meta;
  if (instant) m.ext = 0;
  else if (g.flags & KTJ_GF_LINKED) m.ext = g.linked_id;
  else m.ext = type_hides_own_external_id(g.type) ? 0 : g.id;
  m.aux = g.schema_id;
  m.p[0] = g.args_off; m.p[1] = 0; m.p[2] = 0; m.p[3] = 0; m.p[4] = 0;
  return m;
}

/* grid[0..2] and workgroup[0..2] of a kernel-launch row as three 64-bit words */
KTJ_HD inline void pack_grid(const ktj_runtime_rec& r, uint64_t g[3]) {
  g[0] = (uint64_t)r.u.kernel.grid[0] | ((uint64_t)r.u.kernel.grid[1] << 32);
  g[1] = (uint64_t)r.u.kernel.grid[2] | ((uint64_t)r.u.kernel.workgroup[0] << 32);
  g[2] = (uint64_t)r.u.kernel.workgroup[1] | ((uint64_t)r.u.kernel.workgroup[2] << 32);
}

/* name_id: dictionary id of the API name, KTJ_NONE when the cid is outside the API table */
KTJ_HD inline MatRow mat_runtime(const ktj_runtime_rec& r, int64_t ts, int64_t dur, bool valid, int32_t ext,
                                 uint32_t name_id, bool flow_start, bool is_malloc_cid) {
  MatRow m;
  m.ts = ts; m.dur = dur;
  m.dev = (int64_t)r.pid; m.res = (int64_t)r.tid;        /* RocprofActivity.h:141-146 */
  m.flow_id = (int64_t)r.id;                              /* RocprofActivity.h:60-62 */
  const uint32_t kind = r.kind <= KTJ_RT_MALLOC ? r.kind : KTJ_RT_DEFAULT;
  uint32_t meta = KTJ_TYPE_CUDA_RUNTIME | (KTJ_CLASS_RUNTIME << KTJ_M_CLASS_SHIFT) | (kind << KTJ_M_KIND_SHIFT);
  if (valid) meta |= KTJ_M_VALID;
  if ((int64_t)r.id > 0) { meta |= KTJ_M_FLOW; if (flow_start) meta |= KTJ_M_FLOW_START; }
  if (name_id == KTJ_NONE) { meta |= KTJ_M_NAME_BUILTIN; m.name_id = KTJ_NAME_UNKNOWN_OP; }
  else m.name_id = name_id;
  m.ext = ext;
  m.aux = r.cid;
  m.p[0] = m.p[1] = m.p[2] = m.p[3] = m.p[4] = 0;
  if (kind == KTJ_RT_KERNEL) {
    pack_grid(r, m.p);
    m.p[3] = r.u.kernel.group_segment_size;
    m.p[4] = r.u.kernel.kernel_name_id;
    if (r.u.kernel.kernel_name_id != KTJ_NONE) meta |= KTJ_M_HAS_KERNEL_ARG;
  } else if (kind == KTJ_RT_COPY) {
    m.p[0] = r.u.copy.src; m.p[1] = r.u.copy.dst; m.p[2] = r.u.copy.size; m.p[3] = r.u.copy.copy_kind;
  } else if (kind == KTJ_RT_MALLOC) {
    m.p[0] = r.u.malloc_.ptr; m.p[1] = r.u.malloc_.size;
    if (is_malloc_cid) meta |= KTJ_M_MALLOC_BYTES;
  }
  m.meta = meta;
  return m;
}

/* res: resourceId() after stream back-fill.  grid: packed grid and block of the launching kernel
 * row that the reference hands over (null = none); size: bytes handed over by a copy/malloc row. */
/* coll: 1 + index of the collective metadata of the linked CPU op, 0 = none (kernels only) */
KTJ_HD inline MatRow mat_device_v(const ktj_device_rec& d, int64_t ts, int64_t dur, int64_t res, bool valid, int32_t ext,
                                  bool has_grid, uint64_t g0, uint64_t g1, uint64_t g2, bool has_size, uint64_t size,
                                  uint32_t coll) {
  MatRow m;
  m.ts = ts; m.dur = dur; m.dev = (int64_t)d.device; m.res = res;
  m.flow_id = (int64_t)d.id;
  const uint32_t dom = device_row_domain(d.domain);
  const uint32_t type = dom == KTJ_DOM_MEMSET ? KTJ_TYPE_GPU_MEMSET
                      : dom == KTJ_DOM_MEMORY_COPY ? KTJ_TYPE_GPU_MEMCPY : KTJ_TYPE_CONCURRENT_KERNEL;
  uint32_t meta = type | (KTJ_CLASS_DEVICE << KTJ_M_CLASS_SHIFT) | (dom << KTJ_M_KIND_SHIFT);
  if (valid) meta |= KTJ_M_VALID;
  if ((int64_t)d.id > 0) meta |= KTJ_M_FLOW;             /* flowStart() is false for device rows */
  m.ext = ext;
  m.aux = d.op;
  m.p[0] = m.p[1] = m.p[2] = m.p[4] = 0;
  m.p[3] = d.queue;
  if (dom == KTJ_DOM_MEMSET) { /* the row's ktj_memset_rec view */
    meta |= KTJ_M_NAME_BUILTIN; m.name_id = KTJ_NAME_MEMSET;
    m.aux = (d.domain >> 16) & 0xFFFFu;              /* channel type | memory kind << 8 */
    m.p[0] = d.bytes;
    m.p[1] = (uint64_t)d.op | ((uint64_t)d.name_id << 32); /* graph node id */
    m.p[2] = (d.stream >> 32) | (d.queue & 0xFFFFFFFF00000000ull); /* graph id | channel id << 32 */
    m.p[3] = d.queue & 0xFFFFFFFFull;                 /* context id */
  } else {
    if (dom == KTJ_DOM_MEMORY_COPY) {
      meta |= KTJ_M_NAME_BUILTIN;
      m.name_id = (d.op >= KTJ_COPY_H2H && d.op <= KTJ_COPY_D2D) ? d.op : KTJ_NAME_MEMCPY_UNKNOWN;
    } else if (d.name_id == KTJ_NONE) { meta |= KTJ_M_NAME_BUILTIN; m.name_id = KTJ_NAME_UNKNOWN_OP; }
    else m.name_id = d.name_id;
    if (has_size) { meta |= KTJ_M_HAS_SIZE; m.p[0] = size; }
    else if (has_grid) {
      meta |= KTJ_M_HAS_GRID;
      m.p[0] = g0; m.p[1] = g1; m.p[2] = g2;
    }
    if (dom == KTJ_DOM_KERNEL_DISPATCH) m.p[4] = coll;
  }
  m.meta = meta;
  return m;
}
KTJ_HD inline MatRow mat_device(const ktj_device_rec& d, int64_t ts, int64_t dur, int64_t res, bool valid,
                                int32_t ext, const uint64_t* grid, bool has_size, uint64_t size, uint32_t coll = 0) {
  return mat_device_v(d, ts, dur, res, valid, ext, grid != nullptr, grid ? grid[0] : 0, grid ? grid[1] : 0, grid ? grid[2] : 0,
                      has_size, size, coll);
}

}  // namespace ktj
#endif
