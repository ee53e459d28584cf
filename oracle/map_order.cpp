/*
 * map_order.cpp — TEST INFRASTRUCTURE ONLY, part of the CPU checker.
 *
 * ChromeTraceLogger keeps its process groups in a std::unordered_map<std::string, pgConfig>
 * (libkineto/src/output_json.h:233) and lists them in that map's iteration order
 * (output_json.cpp:1046-1062).  That order is a property of the C++ standard library the logger
 * is built with, not of the logger, so the checker asks the same library rather than restating it.
 * The same holds for the GPU user-annotation spans, kept per stream in a
 * std::map<std::pair<int64_t, int64_t>, std::unordered_map<int64_t, ...>>
 * (libkineto/src/GenericActivityProfiler.h:341-346) and logged in iteration order (.cpp:313-319).
 */
#include <cstdint>
#include <map>
#include <string>
#include <unordered_map>
#include <utility>

extern "C" void ktj_oracle_string_map_order(const char* const* keys, uint64_t n, uint64_t* order) {
  std::unordered_map<std::string, uint64_t> m;
  for (uint64_t i = 0; i < n; ++i) m.insert({std::string(keys[i]), i}); /* distinct keys, insertion order */
  uint64_t k = 0;
  for (const auto& kv : m) order[k++] = kv.second;
}

/* keys in insertion order (distinct triples); order receives the logEvents() sequence */
extern "C" void ktj_oracle_span_map_order(const int64_t* device, const int64_t* resource, const int64_t* id, uint64_t n,
                                          uint64_t* order) {
  std::map<std::pair<int64_t, int64_t>, std::unordered_map<int64_t, uint64_t>> streams;
  for (uint64_t i = 0; i < n; ++i) streams[{device[i], resource[i]}].insert({id[i], i});
  uint64_t k = 0;
  for (const auto& st : streams)
    for (const auto& sp : st.second) order[k++] = sp.second;
}
