// Host-side simulation of the engine's data path, for CPU tests only.
//
// The engine's per-record logic (mat_core.h, fmt_core.h) and its host-formatted events
// (host_events.cpp) compile as plain C++.  This file drives them sequentially in the same order
// and with the same join semantics as the HIP kernels (last writer wins by arrival index,
// output-partitioned tiles with clipping and deferred string copies), with std containers standing
// in for the GPU hash tables, radix sort and scan.  It lets the byte-level logic be compared with
// the oracle without a GPU.  It is not linked into libktj.so.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "../../kineto_amd/csrc/host_events.h"
#include "../../kineto_amd/csrc/mat_core.h"

using namespace ktj;

namespace {

struct Views {
  std::string name_blob, arg_blob, raw_blob;
  std::vector<uint64_t> name_off, arg_off;
  std::vector<uint32_t> flags;
};

// same transformation the dictionary kernels perform
void build_views(const ktj_stream* s, Views& v) {
  v.name_off.push_back(0);
  v.arg_off.push_back(0);
  for (uint64_t i = 0; i < s->n_strings; ++i) {
    const char* p = s->str_blob + s->str_off[i];
    const uint64_t n = s->str_off[i + 1] - s->str_off[i];
    uint32_t fl = 0;
    bool blank = true, unknown = false;
    std::string arg, name;
    for (uint64_t k = 0; k < n; ++k) {
      unsigned char c = (unsigned char)p[k];
      if (c == '\n') continue;
      if (c == '\\') c = '/';
      arg += (char)c;
      if (!(c == ' ' || c == '\t' || c == '\v' || c == '\f' || c == '\r')) blank = false;
      if (c < 0x20 || c > 0x7e) unknown = true;
      if (c == '"') name += '\\';
      name += (char)c;
    }
    if (n == 6 && memcmp(p, "kernel", 6) == 0) name = "Kernel";
    else if (unknown) { name = "unknown"; fl |= KTJ_SF_NAME_UNKNOWN; }
    if (blank) fl |= KTJ_SF_ARG_BLANK;
    if (n == 11 && memcmp(p, "Stream Sync", 11) == 0) fl |= KTJ_SF_STREAM_SYNC;
    v.name_blob += name; v.name_off.push_back(v.name_blob.size());
    v.arg_blob += arg; v.arg_off.push_back(v.arg_blob.size());
    v.flags.push_back(fl);
  }
}

}  // namespace

extern "C" {

// Returns a malloc'ed buffer with the complete document.
int ktjsim_render(const ktj_stream* s, uint32_t tile_bytes, char** out, uint64_t* out_n) {
  Views v;
  build_views(s, v);
  EmitCtx ctx;
  ctx.dict.name_blob = v.name_blob.data(); ctx.dict.name_off = v.name_off.data();
  ctx.dict.arg_blob = v.arg_blob.data(); ctx.dict.arg_off = v.arg_off.data();
  v.raw_blob.assign(s->str_blob ? s->str_blob : "", s->n_strings ? s->str_off[s->n_strings] : 0);
  v.raw_blob.append(16, '\0'); /* string copies load whole aligned words */
  ctx.dict.raw_blob = v.raw_blob.data(); ctx.dict.raw_off = s->str_off;
  ctx.dict.flags = v.flags.data(); ctx.dict.n = (uint32_t)s->n_strings;
  ctx.fields = s->fields; ctx.schemas = s->schemas; ctx.n_schemas = (uint32_t)s->n_schemas;
  ctx.args = s->args; ctx.n_args = s->n_args; ctx.base_time_ns = s->base_time_ns;
  ctx.create_flags = s->create_flags;
  // collective metadata: the arguments of every entry in one blob
  std::vector<ktj::CollectiveInfo> collectives;
  std::string coll_blob;
  std::vector<uint64_t> coll_off(1, 0);
  for (uint64_t k = 0; k < s->n_collectives; ++k) {
    collectives.push_back(ktj::make_collective(s->collectives[k]));
    coll_blob += collectives.back().args;
    coll_off.push_back(coll_blob.size());
  }
  coll_blob.append(16, '\0');
  ctx.coll_blob = coll_blob.data(); ctx.coll_off = coll_off.data(); ctx.n_coll = (uint32_t)s->n_collectives;

  ClockDev clk;
  clk.t0_approx = s->clock.t0_approx; clk.t0 = s->clock.t0; memcpy(&clk.scale_bits, &s->clock.scale, 8);
  clk.async_offset = s->clock.async_offset; clk.runtime_mode = s->clock.runtime_mode; clk.device_mode = s->clock.device_mode;

  const uint64_t ng = s->n_generic, nr = s->n_runtime, nd = s->n_device;
  std::vector<MatRow> mat(ng + nr + nd);

  // tables (value = winning source index)
  std::unordered_map<uint64_t, uint64_t> extcorr;          // correlation -> external id (last wins)
  for (uint64_t i = 0; i < s->n_extcorr; ++i) extcorr[s->extcorr[i].correlation] = s->extcorr[i].external_id;
  std::unordered_map<uint64_t, uint64_t> cpu_ids;          // CPU op id -> generic idx (last wins)
  for (uint64_t i = 0; i < ng; ++i) cpu_ids[(uint64_t)(int64_t)s->generic[i].id] = i;
  auto coll_of = [&](uint64_t id) -> uint32_t {            // collective metadata of the linked CPU op
    auto it = extcorr.find(narrow_corr_key(id));
    if (it == extcorr.end()) return 0;
    auto ci = cpu_ids.find(it->second);
    return ci == cpu_ids.end() ? 0 : collective_for_linked(s->generic[ci->second], ctx);
  };
  auto ext_of = [&](uint64_t id) -> int32_t {
    auto it = extcorr.find(narrow_corr_key(id));
    if (it == extcorr.end()) return 0;
    if (!cpu_ids.count(it->second)) return 0;
    return (int32_t)(int64_t)it->second;
  };
  std::vector<uint8_t> flow_start(s->n_cids ? s->n_cids : 1, 0);
  for (uint64_t i = 0; i < s->n_flow_start; ++i) if (s->flow_start_cids[i] < s->n_cids) flow_start[s->flow_start_cids[i]] = 1;

  for (uint64_t i = 0; i < ng; ++i) {
    mat[i] = mat_generic(s->generic[i], generic_device(s->generic[i], s->args, s->n_args));
    if (!generic_record_prints(s->generic[i], ctx)) mat[i].meta &= ~KTJ_M_VALID;
    attach_own_collective(mat[i], s->generic[i], ctx);
  }

  std::unordered_map<uint64_t, uint64_t> stream_src;       // full id -> runtime idx (last wins)
  std::unordered_map<uint64_t, uint64_t> kernel_src, size_src;  // int-truncated id -> runtime idx (in range, last wins)
  for (uint64_t i = 0; i < nr; ++i) {
    const ktj_runtime_rec& r = s->runtime[i];
    uint64_t b = r.begin, e = r.end;
    convert_range(clk, clk.runtime_mode, &b, &e);
    const int64_t ts = (int64_t)b, dur = (int64_t)(e - b);
    const bool valid = !out_of_range(ts, dur, s->window_start_ns, s->window_end_ns);
    const uint32_t name = r.cid < s->n_cids ? s->cid_name_ids[r.cid] : KTJ_NONE;
    mat[ng + i] = mat_runtime(r, ts, dur, valid, ext_of(r.id), name, r.cid < s->n_cids && flow_start[r.cid], r.cid == s->malloc_cid);
    const uint64_t sid = r.kind == KTJ_RT_KERNEL ? r.u.kernel.stream : r.kind == KTJ_RT_COPY ? r.u.copy.stream : 0;
    if (sid) stream_src[r.id] = i;
    if (valid) {
      const uint64_t key = narrow_corr_key(r.id);
      if (r.kind == KTJ_RT_KERNEL) kernel_src[key] = i;
      else if (r.kind == KTJ_RT_COPY || r.kind == KTJ_RT_MALLOC) size_src[key] = i;
    }
  }
  // stream back-fill
  std::vector<uint64_t> dstream(nd);
  for (uint64_t i = 0; i < nd; ++i) dstream[i] = s->device[i].stream;
  if (!stream_src.empty()) {
    for (uint64_t i = 0; i < nd; ++i) {
      const ktj_device_rec& d = s->device[i];
      if (device_row_domain(d.domain) == KTJ_DOM_MEMSET || dstream[i]) continue;
      auto it = stream_src.find(d.id);
      if (it != stream_src.end()) {
        const ktj_runtime_rec& r = s->runtime[it->second];
        dstream[i] = r.kind == KTJ_RT_KERNEL ? r.u.kernel.stream : r.u.copy.stream;
      }
    }
    std::unordered_map<uint64_t, uint64_t> by_queue;
    std::unordered_set<uint64_t> ambiguous;
    for (uint64_t i = 0; i < nd; ++i) {
      const ktj_device_rec& d = s->device[i];
      if (device_row_domain(d.domain) == KTJ_DOM_MEMSET || !dstream[i] || !d.queue) continue;
      auto it = by_queue.find(d.queue);
      if (it == by_queue.end()) by_queue[d.queue] = dstream[i];
      else if (it->second != dstream[i]) ambiguous.insert(d.queue);
    }
    for (uint64_t i = 0; i < nd; ++i) {
      const ktj_device_rec& d = s->device[i];
      if (device_row_domain(d.domain) == KTJ_DOM_MEMSET || dstream[i]) continue;
      auto it = by_queue.find(d.queue);
      if (it != by_queue.end() && !ambiguous.count(d.queue)) dstream[i] = it->second;
    }
    // dense index = 1 + number of distinct keys of the same device first seen earlier
    struct Ent { int32_t dev; uint64_t key; uint64_t first; };
    std::vector<Ent> ents;
    auto key_of = [&](uint64_t i, uint64_t* key) {
      const ktj_device_rec& d = s->device[i];
      if (device_row_domain(d.domain) == KTJ_DOM_MEMSET) return false;
      if (dstream[i]) *key = dstream[i]; else if (d.queue) *key = d.queue | (1ULL << 63); else return false;
      return true;
    };
    for (uint64_t i = 0; i < nd; ++i) {
      uint64_t key;
      if (!key_of(i, &key)) continue;
      bool found = false;
      for (auto& e : ents) if (e.dev == s->device[i].device && e.key == key) { found = true; break; }
      if (!found) ents.push_back({s->device[i].device, key, i});
    }
    for (uint64_t i = 0; i < nd; ++i) {
      uint64_t key;
      if (!key_of(i, &key)) continue;
      uint64_t my_first = 0, rank = 1;
      for (auto& e : ents) if (e.dev == s->device[i].device && e.key == key) my_first = e.first;
      for (auto& e : ents) if (e.dev == s->device[i].device && e.first < my_first) ++rank;
      dstream[i] = rank;
    }
  }
  for (uint64_t i = 0; i < nd; ++i) {
    const ktj_device_rec& d = s->device[i];
    uint64_t b = d.begin, e = d.end;
    convert_range(clk, clk.device_mode, &b, &e);
    int64_t ts, dur;
    device_times(device_row_domain(d.domain), b, e, &ts, &dur);
    const bool valid = !out_of_range(ts, dur, s->window_start_ns, s->window_end_ns);
    const int64_t res = device_row_domain(d.domain) == KTJ_DOM_MEMSET ? device_row_stream(KTJ_DOM_MEMSET, d.stream) : (int64_t)(dstream[i] ? dstream[i] : d.queue);
    const uint64_t key = narrow_corr_key(d.id);
    const ktj_runtime_rec* ksrc = nullptr;
    bool has_size = false;
    uint64_t size = 0;
    if (device_row_domain(d.domain) != KTJ_DOM_MEMSET) {
      auto si = size_src.find(key);
      if (si != size_src.end()) {
        const ktj_runtime_rec& r = s->runtime[si->second];
        has_size = true;
        size = r.kind == KTJ_RT_COPY ? r.u.copy.size : r.u.malloc_.size;
      } else {
        auto ki = kernel_src.find(key);
        if (ki != kernel_src.end()) ksrc = &s->runtime[ki->second];
      }
    }
    uint64_t grid[3];
    if (ksrc) pack_grid(*ksrc, grid);
    mat[ng + nr + i] = mat_device(d, ts, dur, res, valid, ext_of(d.id), ksrc ? grid : nullptr, has_size, size, coll_of(d.id));
  }

  // GPU user annotations (GenericActivityProfiler.cpp:277-327, 423-433): one span per (device,
  // resource, annotation) over the in-window device rows, appended in the profiler's log order
  if (s->n_usercorr) {
    std::unordered_map<uint64_t, uint64_t> user;
    for (uint64_t i = 0; i < s->n_usercorr; ++i) user[s->usercorr[i].correlation] = s->usercorr[i].external_id;
    struct Span { int64_t dev, res, id, start, end; uint64_t op; };
    std::vector<Span> spans;
    std::map<std::pair<int64_t, int64_t>, std::unordered_map<int64_t, size_t>> streams;
    for (uint64_t i = 0; i < nd; ++i) {
      const MatRow& m = mat[ng + nr + i];
      if (!(m.meta & KTJ_M_VALID)) continue;
      auto ui = user.find(s->device[i].id);
      if (ui == user.end()) continue;
      auto ci = cpu_ids.find(ui->second);
      if (ci == cpu_ids.end()) continue;
      const int64_t id = s->generic[ci->second].id;
      auto& per_stream = streams[{m.dev, m.res}];
      auto it = per_stream.find(id);
      if (it == per_stream.end()) {
        it = per_stream.insert({id, spans.size()}).first;
        spans.push_back({m.dev, m.res, id, m.ts, m.ts + m.dur, ci->second});
      }
      Span& sp = spans[it->second];
      if (m.ts < sp.start || sp.start == 0) sp.start = m.ts;
      if (m.ts + m.dur > sp.end) sp.end = m.ts + m.dur;
    }
    for (const auto& stream : streams) {
      for (const auto& entry : stream.second) {
        const Span& sp = spans[entry.second];
        ktj_generic_rec r;
        memset(&r, 0, sizeof r);
        r.start_ns = sp.start; r.end_ns = sp.end; r.resource = sp.res; r.device = (int32_t)sp.dev;
        r.id = (int32_t)sp.id; r.name_id = s->generic[sp.op].name_id; r.schema_id = KTJ_NONE;
        r.type = KTJ_TYPE_GPU_USER_ANNOTATION;
        mat.push_back(mat_generic(r, sp.dev));
      }
    }
  }

  // canonical order over valid rows
  std::vector<uint64_t> perm;
  for (uint64_t a = 0; a < mat.size(); ++a) if (mat[a].meta & KTJ_M_VALID) perm.push_back(a);
  std::stable_sort(perm.begin(), perm.end(), [&](uint64_t x, uint64_t y) {
    const MatRow &a = mat[x], &b = mat[y];
    if (a.dev != b.dev) return a.dev < b.dev;
    if (a.res != b.res) return a.res < b.res;
    return a.ts < b.ts;
  });
  {
    // Stream Sync rows: the first activity of each (device, row) key in emission order announces the row
    std::set<uint64_t> announced;
    for (uint64_t a : perm) {
      if (a >= ng) continue;
      MatRow probe = mat[a];
      mark_stream_sync(probe, ctx, false);
      if (!(probe.meta & KTJ_M_SYNC)) continue;
      const bool first = announced.insert(stream_sync_key(mat[a].dev, mat[a].res)).second;
      mark_stream_sync(mat[a], ctx, first);
    }
  }
  std::vector<uint64_t> offs(perm.size() + 1, 0);
  for (size_t i = 0; i < perm.size(); ++i) {
    CountWriter cw;
    format_activity(cw, mat[perm[i]], ctx);
    offs[i + 1] = offs[i] + cw.n;
  }
  const uint64_t act_bytes = offs.back();

  std::string prefix, suffix;
  append_trace_start(prefix, s->meta_kv, s->n_meta, s->device_properties, s->base_time_ns);
  for (uint64_t i = 0; i < s->n_device_infos; ++i) append_device_info(prefix, s->device_infos[i], s->base_time_ns);
  for (uint64_t i = 0; i < s->n_resource_infos; ++i) append_resource_info(prefix, s->resource_infos[i], s->base_time_ns);
  for (uint64_t i = 0; i < s->n_overhead_infos; ++i) append_overhead_info(prefix, s->overhead_infos[i], s->base_time_ns);
  for (uint64_t i = 0; i < s->n_spans; ++i) append_trace_span(suffix, s->spans[i], s->base_time_ns);
  std::vector<ktj::CollectiveUse> uses; // every activity that prints collective metadata, in emission order
  for (uint64_t a : perm) {
    const uint32_t k = collective_of(mat[a]);
    const uint32_t cls = (mat[a].meta & KTJ_M_CLASS_MASK) >> KTJ_M_CLASS_SHIFT;
    if (k) uses.push_back(ktj::CollectiveUse{k - 1, cls == KTJ_CLASS_GENERIC && (mat[a].meta & KTJ_M_TYPE_MASK) == KTJ_TYPE_MTIA_CCP_EVENTS});
  }
  append_trace_end(suffix, s->end_time_ns, s->base_time_ns, s->trace_name, ktj::distributed_info_text(collectives, uses));

  const uint64_t total = prefix.size() + act_bytes + suffix.size();
  char* buf = (char*)aligned_alloc(64, (total + 64 + 63) / 64 * 64);
  if (!buf) return -1;
  memset(buf, '#', total);
  memcpy(buf, prefix.data(), prefix.size());
  memcpy(buf + prefix.size() + act_bytes, suffix.data(), suffix.size());

  // output-partitioned tiles, exactly as the emit kernel lays them out: tile k owns the
  // document bytes [k*T, (k+1)*T) clipped to the activity section; tile-local coordinate
  // L = absolute offset - k*T
  if (tile_bytes == 0) {
    // direct variant: one "lane" per activity, aligned 16-byte blocks; the buffer is over-allocated
    // so that aligned accesses at the end stay inside it
    std::vector<uint32_t> kinds(perm.size());
    for (size_t i = 0; i < perm.size(); ++i) {
      const MatRow& m = mat[perm[i]];
      kinds[i] = tail_kind(m, has_args(m, ctx));
    }
    const uint64_t P = prefix.size();
    for (size_t i = 0; i < perm.size(); ++i) {
      BlockWriter w;
      w.begin(buf, P + offs[i], i ? kinds[i - 1] : 0u, i == 0);
      format_activity(w, mat[perm[i]], ctx);
      if (w.position(buf) != P + offs[i + 1]) { free(buf); return -2; }
      w.end(i + 1 == perm.size());
    }
    *out = buf;
    *out_n = total;
    return 0;
  }
  const uint64_t T = tile_bytes;
  if (T % 8) { free(buf); return -3; }
  std::vector<uint64_t> tile_store(T / 8 + 1);
  char* tile = reinterpret_cast<char*>(tile_store.data());
  std::vector<CopyJob> jobs(64);
  const uint64_t P = prefix.size();
  if (act_bytes) {
    for (uint64_t k = P / T; k * T < P + act_bytes; ++k) {
      const uint64_t t0 = k * T;
      const uint64_t abs_lo = t0 > P ? t0 : P;
      const uint64_t abs_hi = std::min<uint64_t>(t0 + T, P + act_bytes);
      const uint64_t lo = abs_lo - P, hi = abs_hi - P;  // activity-relative
      size_t r0 = std::upper_bound(offs.begin(), offs.end(), lo) - offs.begin() - 1;
      size_t r1 = std::lower_bound(offs.begin(), offs.end(), hi) - offs.begin();  // exclusive
      uint32_t nj = 0;
      memset(tile, 0, T);
      for (size_t r = r0; r < r1; ++r) {
        if (offs[r + 1] == offs[r]) continue;
        TileWriter w;
        w.buf = tile; w.size = (uint32_t)T;
        w.jobs = jobs.data(); w.n_jobs = &nj; w.max_jobs = (uint32_t)jobs.size();
        w.begin((int32_t)((int64_t)(offs[r] + P) - (int64_t)t0));
        format_activity(w, mat[perm[r]], ctx);
        w.end();
        if ((int64_t)w.position() != (int64_t)(offs[r + 1] + P) - (int64_t)t0) { free(buf); return -2; }
      }
      const uint32_t done = nj < jobs.size() ? nj : (uint32_t)jobs.size();
      for (uint32_t j = 0; j < done; ++j) memcpy(tile + jobs[j].dst, jobs[j].src, jobs[j].len);
      memcpy(buf + abs_lo, tile + (abs_lo - t0), abs_hi - abs_lo);
    }
  }
  *out = buf;
  *out_n = total;
  return 0;
}

void ktjsim_free(char* p) { free(p); }

}  // extern "C"
