/* host_events.cpp — see host_events.h.  Plain host C++; one std::string append per piece. */
#include "host_events.h"

#include <unordered_map>

#include <cstdint>
#include <cstdlib>

namespace ktj {
namespace {

std::string fmt_ts(int64_t ns) { /* fmtTs, output_json.cpp:124-126: "{}.{:03}" */
  const int64_t q = ns / 1000, r = ns % 1000;
  std::string s = std::to_string(q);
  s += '.';
  /* fmt's {:03} is a minimum width of 3 with zero fill after the sign */
  const int64_t a = r < 0 ? -r : r;
  std::string d = std::to_string(a);
  if (r < 0) { s += '-'; if (d.size() < 2) s.append(2 - d.size(), '0'); }
  else if (d.size() < 3) s.append(3 - d.size(), '0');
  s += d;
  return s;
}

int64_t rel_time(int64_t t, int64_t base) { /* transToRelativeTime, output_json.cpp:144-153 */
  const int64_t r = t - base;
  return r < 0 ? 0 : r;
}

int64_t abs_tid(int64_t tid) { /* sanitizeTid, output_json.cpp:114-121 */
  if (tid == INT64_MIN) return 0;
  return tid < 0 ? -tid : tid;
}

/* sanitizeStrForJSON (:72-78) then escapeQuotesForJSON (:86-91) */
std::string clean_label(const char* s) {
  std::string r;
  for (const char* p = s ? s : ""; *p; ++p) {
    char c = *p;
    if (c == '\n') continue;
    if (c == '\\') c = '/';
    if (c == '"') r += '\\';
    r += c;
  }
  return r;
}

std::string sanitize_only(const char* s) {
  std::string r;
  for (const char* p = s ? s : ""; *p; ++p) {
    if (*p == '\n') continue;
    r += (*p == '\\') ? '/' : *p;
  }
  return r;
}

/* writeMetadataEvent, output_json.cpp:214-235 */
void metadata_event(std::string& out, const char* name, int64_t ts, const std::string& pid,
                    const std::string& tid, const char* arg_key, const std::string& arg_value) {
  out += "\n  {\n    \"ph\": \"M\",\n    \"name\": \"";
  out += name;
  out += "\",\n    \"ts\": ";
  out += fmt_ts(ts);
  out += ",\n    \"pid\": ";
  out += pid;
  out += ",\n    \"tid\": ";
  out += tid;
  out += ",\n    \"args\": {\n      \"";
  out += arg_key;
  out += "\": ";
  out += arg_value;
  out += "\n    }\n  },";
}

}  // namespace

void append_trace_start(std::string& out, const char* const* meta_kv, size_t n_kv,
                        const char* device_properties, int64_t base_time_ns, bool display_ns) {
  out += " {\n    \"schemaVersion\": 1,\n    \"deviceProperties\": [";
  out += device_properties ? device_properties : "";
  out += "],\n    ";
  for (size_t i = 0; i < n_kv; ++i) {
    out += "\n      \"";
    out += meta_kv[2 * i];
    out += "\": ";
    out += sanitize_only(meta_kv[2 * i + 1]);
    out += ',';
  }
  out += display_ns ? "\n    \"displayTimeUnit\": \"ns\",\n    \"baseTimeNanoseconds\": "   /* DISPLAY_TRACE_IN_NS, output_json.cpp:451-454 */
                    : "\n    \"displayTimeUnit\": \"ms\",\n    \"baseTimeNanoseconds\": ";
  out += std::to_string(base_time_ns);
  out += ",\n    \"traceEvents\": [\n    ";
}

void append_device_info(std::string& out, const ktj_device_info& info, int64_t base) {
  const int64_t t = rel_time(info.time_ns, base);
  const std::string pid = std::to_string(info.id);
  metadata_event(out, "process_name", t, pid, "0", "name", "\"" + clean_label(info.name) + "\"");
  metadata_event(out, "process_labels", t, pid, "0", "labels", "\"" + clean_label(info.label) + "\"");
  metadata_event(out, "process_sort_index", t, pid, "0", "sort_index", std::to_string(info.sort_index));
}

void append_resource_info(std::string& out, const ktj_resource_info& info, int64_t base) {
  std::string name = info.name ? info.name : "";
  if (info.host_thread) name = "thread " + std::to_string(info.id) + " (" + name + ")";
  const int64_t t = rel_time(info.time_ns, base);
  const std::string pid = std::to_string(info.device_id);
  const std::string tid = std::to_string(abs_tid(info.id));
  metadata_event(out, "thread_name", t, pid, tid, "name", "\"" + clean_label(name.c_str()) + "\"");
  metadata_event(out, "thread_sort_index", t, pid, tid, "sort_index", std::to_string(info.sort_index));
}

void append_overhead_info(std::string& out, const ktj_overhead_info& info, int64_t base) {
  const int64_t t = rel_time(info.time_ns, base);
  metadata_event(out, "process_name", t, "-1", "0", "name", "\"" + clean_label(info.name) + "\"");
  metadata_event(out, "process_sort_index", t, "-1", "0", "sort_index", std::to_string(0x100000All));
}

void append_trace_span(std::string& out, const ktj_trace_span& sp, int64_t base) {
  const int64_t start = rel_time(sp.start_ns, base);
  const int64_t dur = sp.end_ns == 0 ? 0 : sp.end_ns - sp.start_ns;
  const std::string name = sp.name ? sp.name : "";
  /* writeCompleteEvent, output_json.cpp:237-259 */
  out += "\n  {\n    \"ph\": \"X\",\n    \"cat\": \"Trace\",\n    \"name\": \"";
  out += sp.prefix ? sp.prefix : "";
  out += name;
  out += " (" + std::to_string(sp.iteration) + ")";
  out += "\",\n    \"pid\": \"Spans\",\n    \"tid\": \"" + name + "\",\n    \"ts\": ";
  out += fmt_ts(start);
  out += ",\n    \"dur\": ";
  out += fmt_ts(dur);
  out += "\n    ,\n    \"args\": {\n      \"Op count\": " + std::to_string(sp.op_count) + "\n    }\n  },";
  metadata_event(out, "process_sort_index", start, "\"Spans\"", "0", "sort_index", std::to_string(0x20000000ll));
  /* addIterationMarker → writeInstantEvent, output_json.cpp:261-292, 642-658 */
  out += "\n  {\n    \"ph\": \"i\",\n    \n    \"s\": \"g\",\n    \"name\": \"Iteration Start: " + name;
  out += "\",\n    \"pid\": \"Traces\",\n    \"tid\": \"Trace " + name + "\",\n    \"ts\": ";
  out += fmt_ts(start);
  out += "\n    \n  },";
}

void append_trace_end(std::string& out, int64_t end_time_ns, int64_t base, const std::string& file_name,
                      const std::string& distributed_info) {
  out += "\n  {\n    \"ph\": \"i\",\n    \n    \"s\": \"g\",\n    \"name\": \"Record Window End\",\n    \"pid\": \"\",\n    \"tid\": \"\",\n    \"ts\": ";
  out += fmt_ts(rel_time(end_time_ns, base));
  out += "\n    \n  }";
  out += "\n  ],";
  out += distributed_info;
  out += "\"traceName\": \"" + sanitize_only(file_name.c_str()) + "\" }";
}

namespace {
std::string value_of(const char* p) { return p ? std::string(p) : std::string(); }
/* stripQuotes (output_json.cpp:57-63): one surrounding pair of double quotes goes */
std::string unquoted(const char* p) {
  std::string v = value_of(p);
  if (v.size() >= 2 && v.front() == '"' && v.back() == '"') v = v.substr(1, v.size() - 2);
  return v;
}
struct ArgList { /* ArgsBuilder (output_json.cpp:157-212): entries joined by a bare comma */
  std::string text;
  void raw(const char* key, const std::string& v) {
    if (!text.empty()) text += ',';
    text += '"'; text += key; text += "\": "; text += v;
  }
  void quoted(const char* key, const std::string& v) { raw(key, '"' + v + '"'); }
};
}  // namespace

CollectiveInfo make_collective(const ktj_collective_meta& m) {
  CollectiveInfo c;
  ArgList a;
  const std::string name = unquoted(m.collective_name), dtype = unquoted(m.dtype);
  const std::string in_n = value_of(m.in_msg_nelems), out_n = value_of(m.out_msg_nelems), group = value_of(m.group_size);
  if (!name.empty() && !in_n.empty() && !out_n.empty() && !group.empty() && !dtype.empty()) { /* all five or none: :731-738 */
    a.quoted("Collective name", name);
    a.raw("In msg nelems", in_n);
    a.raw("Out msg nelems", out_n);
    a.raw("Group size", group);
    a.quoted("dtype", dtype);
  }
  const std::string in_start = unquoted(m.in_tensors_start), out_start = unquoted(m.out_tensors_start);
  if (!in_start.empty()) a.quoted("Input Tensors start", in_start);
  if (!out_start.empty()) a.quoted("Output Tensors start", out_start);
  const std::string in_split = unquoted(m.in_split), out_split = unquoted(m.out_split);
  if (!in_split.empty() && !out_split.empty()) { /* all_to_all only, both or none: :752-759 */
    a.quoted("In split size", in_split);
    a.quoted("Out split size", out_split);
  }
  c.pg_name = unquoted(m.pg_name);
  c.pg_desc = unquoted(m.pg_desc);
  c.ranks = unquoted(m.group_ranks);
  c.group_size = group;
  c.rank = value_of(m.rank);
  if (!c.pg_name.empty()) a.quoted("Process Group Name", c.pg_name);
  if (!c.pg_desc.empty()) a.quoted("Process Group Description", c.pg_desc);
  if (!c.ranks.empty()) a.quoted("Process Group Ranks", c.ranks);
  const std::string dst = value_of(m.dst_rank), src = value_of(m.src_rank), seq = value_of(m.seq), comms = value_of(m.comms_id);
  if (!dst.empty()) a.raw("Dst Rank", dst);
  if (!src.empty()) a.raw("Src Rank", src);
  if (!seq.empty()) a.raw("Seq", seq);
  if (!comms.empty()) a.raw("Comms Id", comms);
  c.args = std::move(a.text);
  return c;
}

std::string distributed_info_text(const std::vector<CollectiveInfo>& collectives, const std::vector<CollectiveUse>& uses) {
  struct Group { std::string desc, backend_config, size, ranks; };
  std::unordered_map<std::string, Group> groups; /* pgMap_ (output_json.h:233): the first entry of a name stays */
  std::string backend, rank, world_size, nccl_version;
  for (const CollectiveUse& u : uses) {
    if (u.index >= collectives.size()) continue;
    const CollectiveInfo& c = collectives[u.index];
    if (backend.empty() && c.pg_desc == "default_pg") { /* :807-817 */
      backend = u.hccl ? "hccl" : "nccl";
      rank = c.rank;
      world_size = c.group_size;
      nccl_version = u.hccl ? "" : "unknown";
    }
    groups.insert({c.pg_name, Group{c.pg_desc, u.hccl ? "mtia:hccl" : "cuda:nccl", c.group_size, c.ranks}});
  }
  if (backend.empty()) return std::string();
  std::string out = "\n  \"distributedInfo\": {\"backend\": \"" + backend + "\", \"rank\": " + rank + ", \"world_size\": " +
                    world_size + ", \"pg_count\": " + std::to_string(groups.size()) + ", \"pg_config\": [";
  bool first = true;
  for (const auto& g : groups) {
    if (!first) out += ',';
    first = false;
    out += "{\"pg_name\": \"" + g.first + "\", \"pg_desc\": \"" + g.second.desc + "\", \"backend_config\": \"" +
           g.second.backend_config + "\", \"pg_size\": " + g.second.size + ", \"ranks\": \"" + g.second.ranks + "\"}";
  }
  out += "], \"nccl_version\": \"" + nccl_version + "\"},";
  return out;
}

}  // namespace ktj
