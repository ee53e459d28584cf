/*
 * map_order.cpp — TEST INFRASTRUCTURE ONLY, part of the CPU checker.
 *
 * ChromeTraceLogger keeps its process groups in a std::unordered_map<std::string, pgConfig>
 * (libkineto/src/output_json.h:233) and lists them in that map's iteration order
 * (output_json.cpp:1046-1062).  That order is a property of the C++ standard library the logger
 * is built with, not of the logger, so the checker asks the same library rather than restating it.
 */
#include <cstdint>
#include <string>
#include <unordered_map>

extern "C" void ktj_oracle_string_map_order(const char* const* keys, uint64_t n, uint64_t* order) {
  std::unordered_map<std::string, uint64_t> m;
  for (uint64_t i = 0; i < n; ++i) m.insert({std::string(keys[i]), i}); /* distinct keys, insertion order */
  uint64_t k = 0;
  for (const auto& kv : m) order[k++] = kv.second;
}
