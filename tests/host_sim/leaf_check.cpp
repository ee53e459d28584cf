// Host build of the engine's formatting core: leaf functions for known-answer tests on the CPU.
#include <cstring>
#include "../../kineto_amd/csrc/fmt_core.h"
extern "C" {
int ktjsim_fmt_double(double v, char* out) { uint64_t b; memcpy(&b, &v, 8); int n = ktj::format_double(b, out); out[n] = 0; return n; }
long long ktjsim_convert_ts(unsigned long long t, unsigned long long t0a, long long t0, double scale) {
  uint64_t b; memcpy(&b, &scale, 8); return ktj::convert_timestamp(t, t0a, t0, b); }
}
