// ASan/UBSan run of the host-side code paths: generator, CPU checker, host build of the formatter
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <initializer_list>
#include "../../include/ktj.h"
#include "../../include/ktj_stream.h"
extern "C" {
#include "../../oracle/ktj_oracle.h"
int ktjsim_render(const ktj_stream* s, uint32_t tile_bytes, char** out, uint64_t* out_n);
}
int main() {
  int bad = 0;
  const uint64_t sizes[] = {1, 3, 257, 4097, 20000};
  for (uint32_t cfg = 1; cfg <= 5; ++cfg)
    for (uint64_t n : sizes) {
      ktj_synth_params p; memset(&p, 0, sizeof p);
      p.config = cfg; p.n_device = n; p.base_time_ns = 1790857026000000000LL; p.host_name = "san"; p.trace_name = "san.json";
      ktj_stream* s = ktj_synth_generate(&p);
      if (!s) { printf("synth failed %u %llu\n", cfg, (unsigned long long)n); return 2; }
      ktj_oracle* o = ktj_oracle_run(s);
      const char* want; uint64_t want_n;
      ktj_oracle_output(o, &want, &want_n);
      for (uint32_t tile : {0u, 8192u}) {
        char* got = nullptr; uint64_t got_n = 0;
        const int rc = ktjsim_render(s, tile, &got, &got_n);
        const bool same = rc == 0 && got_n == want_n && memcmp(got, want, want_n) == 0;
        if (!same) { printf("MISMATCH cfg %u n %llu tile %u rc %d (%llu vs %llu bytes)\n", cfg, (unsigned long long)n, tile, rc, (unsigned long long)got_n, (unsigned long long)want_n); ++bad; }
        free(got);
      }
      ktj_oracle_free(o);
      ktj_synth_free(s);
      printf("cfg %u n %llu ok (%llu bytes)\n", cfg, (unsigned long long)n, (unsigned long long)want_n);
    }
  return bad != 0;
}
