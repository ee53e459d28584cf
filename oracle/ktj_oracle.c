/*
 * ktj_oracle.c — CPU restatement of the reference's records → Chrome-trace JSON path.
 *
 * TEST INFRASTRUCTURE ONLY (see ktj_oracle.h).  Plain C, single thread, written to follow the
 * reference function by function; every function cites the reference lines it restates (paths
 * relative to the pytorch/kineto tree).
 *
 * How each part is pinned (tests/test_oracle_*.py):
 *   - logger templates, args assembly, name pipeline, flow events, header/footer:
 *       byte-compared with the real ChromeTraceLogger built from the reference sources
 *       (oracle/_ref) on all five synthetic configurations and on hand-made edge cases, and
 *       against literal strings observed from the real logger (tests/golden/kat_events.json).
 *   - typed-metadata rendering (ints, doubles, arrays, strings): the real
 *       JsonTypedMetadataVisitor inside oracle/_ref renders the same typed values; plus the
 *       literal pins of test/TypedMetadataTest.cpp:164-244.
 *   - double formatting: compared with fmt's "{}" through oracle/_ref on a few million random and
 *       boundary doubles; implemented here by shortest-precision search with printf/strtod, i.e.
 *       independently of the integer algorithm the GPU uses.
 *   - clock conversion: x86 `long double` arithmetic, the very expression of
 *       ApproximateClock.cpp:83-90; checked against exact rational arithmetic in the tests.
 *   - join (external correlation, stream back-fill, grid/block/bytes hand-over, window filter,
 *       timestamp-order counter, GPU user-annotation spans): the reference's own
 *       GenericActivityProfiler::processTraceInternal with the ROCm handlers and the real logger,
 *       run by oracle/_ref/profiler_ref_driver on rows placed in memory; every event it writes and
 *       its counters are compared on seeded cases (tests/test_rocm_wrappers.py).  Also a
 *       brute-force nested-loop re-implementation in the tests on small streams, and the
 *       expectations of test/RocmActivityProfilerTest.cpp:370-397, 486-503, 552-554.
 *   - canonical order: stable merge sort here; std::stable_sort on tuples inside oracle/_ref.
 *   - instant events and the Stream Sync row remap: byte-compared with the real logger on a
 *       hand-made case (tests/kat_cases.py: case_instant_and_stream_sync).
 *   - counter events: byte-compared with the real logger on a hand-made case
 *       (tests/kat_cases.py: case_counter_events) and inside the seeded random streams.
 *   - collective metadata and the "distributedInfo" footer entry: the inputs and expected
 *       values of test/OutputJsonTest.cpp:81-225, and byte-compared with the real logger on
 *       hand-made cases (tests/kat_cases.py: case_collective_*).  The order of the process groups
 *       is the iteration order of a std::unordered_map and is taken from the C++ library
 *       (map_order.cpp), as the logger takes it.
 *   - GPU user-annotation spans: the expectations of test/RocmActivityProfilerTest.cpp:770-833 and
 *       the sequential Python statement of tests/test_join_bruteforce.py; the spans' relative order
 *       is the iteration order of the profiler's own maps, taken from the C++ library (map_order.cpp).
 *   - rocprofiler-sdk buffer records -> device rows (sdk_rows.c): against the reference's own
 *       RocprofLogger::buffer_callback, run by oracle/_ref/sdk_ref_driver on records built in
 *       memory (tests/test_sdk_ingest.py).
 *   - the ROCm wrapper layer (what runtime and device rows report as activities: names, the args'
 *       keys, order and values, the hand-over of grid, block and size from runtime rows to device
 *       rows, device timestamps, flow starts): against the reference's own RuntimeActivity<T> and
 *       GpuActivity classes, run by the same driver on packed rows (tests/test_rocm_wrappers.py);
 *       the stream back-fill against the reference's own detail::backfillAsyncStreams
 *       (RocmStreamQueue.h:42-136) on seeded rows, same driver, same test file.
 *   - memset rows, which are CUDA-shaped (CuptiActivity.h:682-719): against the reference's own
 *       GpuActivity<CUpti_ActivityMemsetType>, run by oracle/_ref/cupti_ref_driver on records built
 *       in memory, compiled against the CUDA 12 and CUPTI headers of this image
 *       (tests/test_cuda_memset_rows.py): name, type, times, ids and every args key and value, with
 *       the four keys that the reference prints for CUDA >= 12 (KTJ_CREATE_CUDA12_ARGS) and without.
 */
#define _GNU_SOURCE
#include "ktj_oracle.h"

#include <ctype.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

/* ------------------------------------------------------------------------------------------ */
/* small utilities                                                                              */
/* ------------------------------------------------------------------------------------------ */
typedef struct sbuf {
  char* p;
  size_t n, cap;
} sbuf;

static void sb_reserve(sbuf* b, size_t extra) {
  if (b->n + extra <= b->cap) return;
  size_t nc = b->cap ? b->cap : 1024;
  while (nc < b->n + extra) nc *= 2;
  char* np = (char*)realloc(b->p, nc);
  if (!np) abort();
  b->p = np;
  b->cap = nc;
}
static void sb_put(sbuf* b, const char* s, size_t n) {
  if (n == 0) return;
  sb_reserve(b, n);
  memcpy(b->p + b->n, s, n);
  b->n += n;
}
static void sb_puts(sbuf* b, const char* s) { sb_put(b, s, strlen(s)); }
static void sb_putc(sbuf* b, char c) { sb_put(b, &c, 1); }

static double now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

/* open-addressing map uint64 → uint64 (insert-or-assign, find) */
typedef struct umap {
  uint64_t* k;
  uint64_t* v;
  uint8_t* used;
  uint64_t cap, n;
} umap;
static uint64_t hash64(uint64_t x) {
  x ^= x >> 33; x *= 0xff51afd7ed558ccdULL; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ULL; x ^= x >> 33;
  return x;
}
static void umap_init(umap* m, uint64_t expected) {
  uint64_t cap = 16;
  while (cap < expected * 2 + 16) cap <<= 1;
  m->cap = cap; m->n = 0;
  m->k = (uint64_t*)malloc(cap * 8);
  m->v = (uint64_t*)malloc(cap * 8);
  m->used = (uint8_t*)calloc(cap, 1);
  if (!m->k || !m->v || !m->used) abort();
}
static void umap_free(umap* m) { free(m->k); free(m->v); free(m->used); memset(m, 0, sizeof *m); }
static void umap_grow(umap* m);
static uint64_t* umap_slot(umap* m, uint64_t key, int* inserted) {
  if ((m->n + 1) * 2 > m->cap) umap_grow(m);
  uint64_t i = hash64(key) & (m->cap - 1);
  while (m->used[i]) {
    if (m->k[i] == key) { if (inserted) *inserted = 0; return &m->v[i]; }
    i = (i + 1) & (m->cap - 1);
  }
  m->used[i] = 1; m->k[i] = key; m->v[i] = 0; m->n++;
  if (inserted) *inserted = 1;
  return &m->v[i];
}
static void umap_grow(umap* m) {
  umap o = *m;
  umap_init(m, o.cap);
  for (uint64_t i = 0; i < o.cap; ++i)
    if (o.used[i]) *umap_slot(m, o.k[i], NULL) = o.v[i];
  umap_free(&o);
}
static const uint64_t* umap_find(const umap* m, uint64_t key) {
  uint64_t i = hash64(key) & (m->cap - 1);
  while (m->used[i]) {
    if (m->k[i] == key) return &m->v[i];
    i = (i + 1) & (m->cap - 1);
  }
  return NULL;
}
static void umap_erase_mark(umap* m, uint64_t key, uint64_t tomb) {
  /* used only for the queue map of the stream fallback: mark instead of erase */
  uint64_t* v = umap_slot(m, key, NULL);
  *v = tomb;
}

/* (device, stream key) → dense per-device index in first-seen order
 * (std::unordered_map<int, std::unordered_map<uint64_t, uint64_t>> of RocmStreamQueue.h:112-135) */
typedef struct dense_ent { int32_t device; uint64_t key; uint64_t index; } dense_ent;
typedef struct dense_map { dense_ent* e; uint64_t n, cap; umap per_dev; } dense_map;
static void dense_init(dense_map* m) { m->e = NULL; m->n = m->cap = 0; umap_init(&m->per_dev, 64); }
static void dense_free(dense_map* m) { free(m->e); umap_free(&m->per_dev); }
static uint64_t dense_index(dense_map* m, int32_t device, uint64_t key) {
  for (uint64_t i = 0; i < m->n; ++i)
    if (m->e[i].device == device && m->e[i].key == key) return m->e[i].index;
  if (m->n == m->cap) {
    m->cap = m->cap ? m->cap * 2 : 64;
    m->e = (dense_ent*)realloc(m->e, m->cap * sizeof *m->e);
    if (!m->e) abort();
  }
  uint64_t* c = umap_slot(&m->per_dev, (uint64_t)(int64_t)device, NULL);
  *c += 1;
  m->e[m->n].device = device; m->e[m->n].key = key; m->e[m->n].index = *c;
  return m->e[m->n++].index;
}

/* ------------------------------------------------------------------------------------------ */
/* leaf formatting                                                                              */
/* ------------------------------------------------------------------------------------------ */

/* libkineto/include/ActivityType.h:80-111 */
static const char* const kTypeNames[KTJ_TYPE_COUNT + 1] = {
    "cpu_op", "user_annotation", "gpu_user_annotation", "gpu_memcpy", "gpu_memset", "kernel",
    "external_correlation", "cuda_runtime", "cuda_driver", "cpu_instant_event", "python_function",
    "overhead", "mtia_runtime", "mtia_ccp_events", "mtia_insight", "cuda_sync", "cuda_event",
    "mtia_counters", "glow_runtime", "cuda_profiler_range", "hpu_op", "xpu_runtime", "xpu_driver",
    "collective_comm", "privateuse1_runtime", "privateuse1_driver", "xpu_scope_profiler", "xpu_sync",
    "hardware_counters", "ENUM_COUNT"};
const char* ktj_oracle_type_name(int type) {
  if (type < 0 || type > KTJ_TYPE_COUNT) return "";
  return kTypeNames[type];
}

static size_t fmt_i64(int64_t v, char* out) { return (size_t)sprintf(out, "%lld", (long long)v); }
static size_t fmt_u64(uint64_t v, char* out) { return (size_t)sprintf(out, "%llu", (unsigned long long)v); }

/* fmtTs: libkineto/src/output_json.cpp:124-126 — fmt "{}.{:03}" of ns/1000 and ns%1000.
 * For a negative remainder fmt's {:03} pads after the sign ("-05"); C's %03lld does the same. */
size_t ktj_oracle_fmt_ts(int64_t ns, char* out) {
  return (size_t)sprintf(out, "%lld.%03lld", (long long)(ns / 1000), (long long)(ns % 1000));
}

/* fmt "{}" on a double (libkineto/include/TypedMetadataJson.h:172-178 → fmt/format.h
 * write_float with default specs): shortest digits that round-trip, fixed notation iff the
 * decimal exponent is in [-4, 16), else d[.ddd]e±XX. */
size_t ktj_oracle_fmt_double(double v, char* out) {
  if (isnan(v)) return (size_t)sprintf(out, signbit(v) ? "-nan" : "nan");
  if (isinf(v)) return (size_t)sprintf(out, v < 0 ? "-inf" : "inf");
  char* o = out;
  if (signbit(v)) { *o++ = '-'; v = -v; }
  if (v == 0.0) { *o++ = '0'; *o = 0; return (size_t)(o - out); }
  /* Shortest-precision search: the first precision p at which some p-digit decimal reads back
   * as v.  printf gives the p-digit decimal nearest to v; at a power of two the rounding
   * interval is lopsided, so the p-digit neighbours are tried as well (the closest wins). */
  char digits[24];
  int nd = 0, E = 0;
  for (int prec = 1; prec <= 17 && nd == 0; ++prec) {
    char tmp[48];
    snprintf(tmp, sizeof tmp, "%.*e", prec - 1, v);
    unsigned long long m = 0;
    const char* q = tmp;
    for (; *q && *q != 'e'; ++q)
      if (*q >= '0' && *q <= '9') m = m * 10 + (unsigned long long)(*q - '0');
    const int e10 = atoi(q + 1);          /* v ~ m * 10^(e10 - (prec - 1)) */
    unsigned long long best_m = 0;
    int have = 0;
    long double best_err = 0;
    for (int delta = 0; delta < 3; ++delta) {
      unsigned long long c = delta == 0 ? m : (delta == 1 ? m + 1 : m - 1);
      if (c == 0) continue;
      char cand[64];
      snprintf(cand, sizeof cand, "%llue%d", c, e10 - (prec - 1));
      if (strtod(cand, NULL) != v) continue;
      long double err = fabsl(strtold(cand, NULL) - (long double)v);
      if (!have || err < best_err) { have = 1; best_err = err; best_m = c; }
    }
    if (have) {
      nd = snprintf(digits, sizeof digits, "%llu", best_m);
      E = e10 - (prec - 1) + (nd - 1);    /* scientific exponent of the chosen digits */
    }
  }
  while (nd > 1 && digits[nd - 1] == '0') --nd; /* shortest form has no trailing zeros */
  if (E >= -4 && E < 16) {
    if (E >= 0) {
      int i = 0;
      for (; i <= E; ++i) *o++ = i < nd ? digits[i] : '0';
      if (nd > E + 1) {
        *o++ = '.';
        for (; i < nd; ++i) *o++ = digits[i];
      }
    } else {
      *o++ = '0'; *o++ = '.';
      for (int i = 0; i < -E - 1; ++i) *o++ = '0';
      for (int i = 0; i < nd; ++i) *o++ = digits[i];
    }
  } else {
    *o++ = digits[0];
    if (nd > 1) {
      *o++ = '.';
      for (int i = 1; i < nd; ++i) *o++ = digits[i];
    }
    *o++ = 'e';
    int a = E;
    if (a < 0) { *o++ = '-'; a = -a; } else *o++ = '+';
    if (a >= 100) { *o++ = (char)('0' + a / 100); a %= 100; }
    *o++ = (char)('0' + a / 10);
    *o++ = (char)('0' + a % 10);
  }
  *o = 0;
  return (size_t)(o - out);
}

/* sanitizeStrForJSON: libkineto/src/output_json.cpp:72-78 */
size_t ktj_oracle_sanitize_str(const char* in, size_t n, char* out) {
  size_t w = 0;
  for (size_t i = 0; i < n; ++i) {
    char c = in[i];
    if (c == '\\') c = '/';
    if (c == '\n') continue;
    out[w++] = c;
  }
  return w;
}

/* Name pipeline of handleActivity: libkineto/src/output_json.cpp:946-949 with
 * sanitizeStrForJSON (:72-78), sanitizeForNonReadableChars (:103-112; std::isprint in the "C"
 * locale: 0x20..0x7e) and escapeQuotesForJSON (:86-91). */
size_t ktj_oracle_sanitize_name(const char* in, size_t n, char* out) {
  if (n == 6 && memcmp(in, "kernel", 6) == 0) { memcpy(out, "Kernel", 6); return 6; }
  char* tmp = (char*)malloc(n + 1);
  if (!tmp) abort();
  size_t m = ktj_oracle_sanitize_str(in, n, tmp);
  for (size_t i = 0; i < m; ++i) {
    unsigned char c = (unsigned char)tmp[i];
    if (c < 0x20 || c > 0x7e) {
      free(tmp);
      memcpy(out, "unknown", 7);
      return 7;
    }
  }
  size_t w = 0;
  for (size_t i = 0; i < m; ++i) {
    if (tmp[i] == '"') out[w++] = '\\';
    out[w++] = tmp[i];
  }
  free(tmp);
  return w;
}

/* Time converter: libkineto/src/ApproximateClock.cpp:83-90.  scale_factor is a long double that
 * holds a double value (:51-57); the product is taken in extended precision and truncated. */
int64_t ktj_oracle_convert_ts(const ktj_clock_model* m, uint64_t t) {
  int64_t t_approx = (int64_t)t;
  int64_t t0_approx = (int64_t)m->t0_approx;
  long double scale_factor = (long double)m->scale;
  if (!(t_approx > t0_approx)) return 0;
  /* the sum wraps where the reference's signed addition overflows, as its machine code does */
  const int64_t scaled = (int64_t)((double)(t_approx - t0_approx) * scale_factor);
  return (int64_t)((uint64_t)scaled + (uint64_t)m->t0);
}

/* ------------------------------------------------------------------------------------------ */
/* the oracle object                                                                            */
/* ------------------------------------------------------------------------------------------ */
enum { /* built-in strings appended to the stream's dictionary */
  BS_DEVICE, BS_STREAM, BS_HSA_QUEUE, BS_CORRELATION, BS_KIND, BS_BYTES, BS_BANDWIDTH, BS_GRID,
  BS_BLOCK, BS_CID, BS_SHARED_MEMORY, BS_SRC, BS_DST, BS_PTR, BS_KERNEL, BS_CONTEXT,
  BS_DISPATCH_KERNEL, BS_HTOH, BS_HTOD, BS_DTOH, BS_DTOD, BS_UNKNOWN_KIND,
  BS_MEMSET_UNKNOWN, BS_MEMSET_PAGEABLE, BS_MEMSET_PINNED, BS_MEMSET_DEVICE, BS_MEMSET_ARRAY, BS_MEMSET_MANAGED,
  BS_MEMSET_DEVICE_STATIC, BS_MEMSET_MANAGED_STATIC, BS_MEMSET_UNRECOGNIZED,
  BS_GRAPH_ID, BS_GRAPH_NODE_ID, BS_CHANNEL, BS_CHANNEL_TYPE, BS_EMPTY, BS_COUNT
};
static const char* const kBuiltin[BS_COUNT] = {
    "device", "stream", "hsa_queue", "correlation", "kind", "bytes", "memory bandwidth (GB/s)", "grid",
    "block", "cid", "shared memory", "src", "dst", "ptr", "kernel", "context",
    "Dispatch Kernel", "HtoH", "HtoD", "DtoH", "DtoD", "<unknown>",
    /* "Memset ({})" of memoryKindString, cupti_strings.cpp:42-66 */
    "Memset (Unknown)", "Memset (Pageable)", "Memset (Pinned)", "Memset (Device)", "Memset (Array)", "Memset (Managed)",
    "Memset (Device Static)", "Memset (Managed Static)", "Memset (Unrecognized)",
    "graph id", "graph node id", "channel", "channel_type", ""};

struct ktj_oracle {
  const ktj_stream* s;
  /* string table */
  sbuf xblob;            /* extra strings */
  uint64_t* xoff;        /* offsets of extra strings (n_x + 1) */
  uint64_t n_x, cap_x;
  uint32_t builtin0;
  /* materialised activities */
  ktj_mat_activity* acts;
  uint64_t n_acts, cap_acts;
  uint64_t* order;
  /* per-activity metadata storage */
  ktj_field* fpool; uint64_t n_fpool, cap_fpool;
  uint64_t* spool; uint64_t n_spool, cap_spool;
  uint64_t* act_f0; /* first field / slot per activity (offsets; pointers fixed up at the end) */
  uint64_t* act_s0;
  /* output */
  sbuf out;
  uint64_t out_of_range, out_of_order, n_flow, n_linked, n_blank;
  /* (device << 32 | virtual tid) keys whose Stream-Sync row header was written: output_json.h
   * syncStreamMetadataEmitted_ */
  int64_t* sync_seen; uint64_t n_sync_seen, cap_sync_seen;
  /* distInfo_ and pgMap_ (output_json.h:229-233); process groups in insertion order */
  char *dist_backend, *dist_rank, *dist_world_size, *dist_nccl_version;
  struct pg_entry { char *name, *desc, *backend_config, *size, *ranks; } *pgs;
  uint64_t n_pgs, cap_pgs;
  double t_join, t_sort, t_emit;
  int64_t win_start, win_end;
};

static uint32_t add_xstring(ktj_oracle* o, const char* p, size_t n) {
  if (o->n_x + 2 > o->cap_x) {
    o->cap_x = o->cap_x ? o->cap_x * 2 : 256;
    o->xoff = (uint64_t*)realloc(o->xoff, o->cap_x * 8);
    if (!o->xoff) abort();
  }
  if (o->n_x == 0) o->xoff[0] = 0;
  sb_put(&o->xblob, p, n);
  o->n_x++;
  o->xoff[o->n_x] = o->xblob.n;
  return (uint32_t)(o->s->n_strings + o->n_x - 1);
}

void ktj_oracle_string(const ktj_oracle* o, uint32_t id, const char** p, uint64_t* n) {
  const ktj_stream* s = o->s;
  if (id < s->n_strings) {
    *p = s->str_blob + s->str_off[id];
    *n = s->str_off[id + 1] - s->str_off[id];
  } else if (id - s->n_strings < o->n_x) {
    uint64_t k = id - s->n_strings;
    *p = o->xblob.p + o->xoff[k];
    *n = o->xoff[k + 1] - o->xoff[k];
  } else {
    *p = "";
    *n = 0;
  }
}
uint64_t ktj_oracle_n_strings(const ktj_oracle* o) { return o->s->n_strings + o->n_x; }

static ktj_mat_activity* new_act(ktj_oracle* o) {
  if (o->n_acts == o->cap_acts) {
    o->cap_acts = o->cap_acts ? o->cap_acts * 2 : 1024;
    o->acts = (ktj_mat_activity*)realloc(o->acts, o->cap_acts * sizeof *o->acts);
    o->act_f0 = (uint64_t*)realloc(o->act_f0, o->cap_acts * 8);
    o->act_s0 = (uint64_t*)realloc(o->act_s0, o->cap_acts * 8);
    if (!o->acts || !o->act_f0 || !o->act_s0) abort();
  }
  ktj_mat_activity* a = &o->acts[o->n_acts];
  memset(a, 0, sizeof *a);
  o->act_f0[o->n_acts] = o->n_fpool;
  o->act_s0[o->n_acts] = o->n_spool;
  o->n_acts++;
  return a;
}
/* one visitor.visit(field, value) call */
static void visit(ktj_oracle* o, ktj_mat_activity* a, uint32_t key_id, uint16_t type, uint16_t count,
                  const uint64_t* vals) {
  if (o->n_fpool == o->cap_fpool) {
    o->cap_fpool = o->cap_fpool ? o->cap_fpool * 2 : 4096;
    o->fpool = (ktj_field*)realloc(o->fpool, o->cap_fpool * sizeof *o->fpool);
    if (!o->fpool) abort();
  }
  if (o->n_spool + count > o->cap_spool) {
    o->cap_spool = o->cap_spool ? o->cap_spool * 2 : 8192;
    while (o->n_spool + count > o->cap_spool) o->cap_spool *= 2;
    o->spool = (uint64_t*)realloc(o->spool, o->cap_spool * 8);
    if (!o->spool) abort();
  }
  ktj_field* f = &o->fpool[o->n_fpool++];
  f->key_id = key_id; f->type = type; f->count = count;
  memcpy(o->spool + o->n_spool, vals, 8 * (size_t)count);
  o->n_spool += count;
  a->n_fields++;
}
/* slots of one KTJ_F_SHAPES value that starts at args[at] (see include/ktj.h), clipped to the blob
 * and to what a field's 16-bit count can say */
static uint64_t shapes_encoded_slots(const uint64_t* args, uint64_t n_args, uint64_t at) {
  if (at >= n_args) return 0;
  uint64_t p = at + 1;
  for (uint64_t e = 0; e < args[at] && p < n_args; ++e) {
    const uint64_t head = args[p++], m = head & 0xFFFFFFFFull;
    if (head & KTJ_SHAPE_LIST) {
      for (uint64_t t = 0; t < m && p < n_args; ++t) p += 1 + (args[p] & 0xFFFFFFFFull);
    } else p += m;
  }
  if (p > n_args) p = n_args;
  return p - at > 65535 ? 65535 : p - at;
}
static void visit1(ktj_oracle* o, ktj_mat_activity* a, int builtin_key, uint16_t type, uint64_t v) {
  visit(o, a, o->builtin0 + (uint32_t)builtin_key, type, 1, &v);
}
static uint64_t dbits(double d) { uint64_t u; memcpy(&u, &d, 8); return u; }

/* ------------------------------------------------------------------------------------------ */
/* stage 2: clock conversion, joins, window filter — the profiler half                          */
/* ------------------------------------------------------------------------------------------ */

/* GenericActivityProfiler::outOfRange: libkineto/src/GenericActivityProfiler.cpp:329-340 */
static int out_of_range(ktj_oracle* o, int64_t ts, int64_t dur) {
  int r = ts < o->win_start || (ts + dur) > o->win_end;
  if (r) o->out_of_range++;
  return r;
}

/* GenericActivityProfiler::checkTimestampOrder: GenericActivityProfiler.cpp:363-395.
 * map value packs (is_runtime, ts) of the first activity seen with this correlation id. */
typedef struct order_ent { int64_t ts; int is_runtime; } order_ent;
static void check_ts_order(ktj_oracle* o, umap* seen, order_ent** ents, uint64_t* n_ents,
                           uint64_t* cap_ents, int64_t corr, int is_runtime, int64_t ts) {
  int inserted;
  uint64_t* v = umap_slot(seen, (uint64_t)corr, &inserted);
  if (inserted) {
    if (*n_ents == *cap_ents) {
      *cap_ents = *cap_ents ? *cap_ents * 2 : 1024;
      *ents = (order_ent*)realloc(*ents, *cap_ents * sizeof **ents);
      if (!*ents) abort();
    }
    (*ents)[*n_ents].ts = ts;
    (*ents)[*n_ents].is_runtime = is_runtime;
    *v = (*n_ents)++;
    return;
  }
  order_ent act1 = {ts, is_runtime};
  order_ent act2 = (*ents)[*v];
  if (act2.is_runtime) { order_ent t = act1; act1 = act2; act2 = t; }
  if (act2.ts == 0) return;
  if (act1.ts > act2.ts) o->out_of_order++;
}

/* GenericActivityProfiler::linkedActivity: GenericActivityProfiler.cpp:397-408 — the
 * correlation id is narrowed to int32 by the parameter type. Returns index of the generic
 * record or -1. */
static int64_t linked_activity(const umap* cpu_corr, const umap* activity_map, uint64_t id) {
  int32_t narrowed = (int32_t)(uint32_t)id;
  const uint64_t* ext = umap_find(cpu_corr, (uint64_t)(int64_t)narrowed);
  if (!ext) return -1;
  const uint64_t* act = umap_find(activity_map, *ext);
  return act ? (int64_t)*act : -1;
}

/* 1 + the slot value of a record's leading KTJ_F_COLLECTIVE field, 0 if it has none */
static uint32_t collective_index(const ktj_stream* s, const ktj_generic_rec* r) {
  if (r->schema_id == KTJ_NONE || r->schema_id >= s->n_schemas) return 0;
  const ktj_schema_desc* d = &s->schemas[r->schema_id];
  if (d->n_fields == 0 || s->fields[d->first_field].type != KTJ_F_COLLECTIVE || r->args_off >= s->n_args) return 0;
  const uint64_t k = s->args[r->args_off];
  return k < s->n_collectives ? (uint32_t)k + 1u : 0u;
}

static uint32_t ptr_string(ktj_oracle* o, uint64_t p) { /* fmt "{}" of const void* */
  char b[32];
  int n = sprintf(b, "0x%llx", (unsigned long long)p);
  return add_xstring(o, b, (size_t)n);
}

/* a GPU-side span of one user annotation on one stream (GenericActivityProfiler.h:324-347) */
typedef struct user_span {
  int64_t device, resource, cpu_id, start, end;
  uint64_t cpu_row;
} user_span;
void ktj_oracle_span_map_order(const int64_t* device, const int64_t* resource, const int64_t* id, uint64_t n,
                               uint64_t* order); /* map_order.cpp */

static int stage_join(ktj_oracle* o) {
  const ktj_stream* s = o->s;
  const ktj_clock_model* cm = &s->clock;
  o->win_start = s->window_start_ns;
  o->win_end = s->window_end_ns;

  /* activityMap_[act->correlationId()] = act  (GenericActivityProfiler.cpp:262) */
  umap activity_map; umap_init(&activity_map, s->n_generic);
  /* cpuCorrelationMap_[correlationId] = externalId  (RocmActivityProfiler.cpp:135-148) */
  umap cpu_corr; umap_init(&cpu_corr, s->n_extcorr);
  /* correlatedCudaActivities_ (GenericActivityProfiler.cpp:363-395) */
  umap seen; umap_init(&seen, s->n_runtime + s->n_device);
  order_ent* ents = NULL; uint64_t n_ents = 0, cap_ents = 0;
  /* thread_local correlationToGrid/Block/Size keyed by int (RocprofActivity_inl.h:28-30):
   * value = index of the runtime row that wrote it last */
  umap corr_to_kernel; umap_init(&corr_to_kernel, s->n_runtime);
  umap corr_to_size; umap_init(&corr_to_size, s->n_runtime / 4);

  /* ---- generic records: logged as they are (output_json.cpp:837-971 via
   *      GenericTraceActivity::log, GenericTraceActivity.cpp:50-52) ---- */
  for (uint64_t i = 0; i < s->n_generic; ++i) {
    const ktj_generic_rec* r = &s->generic[i];
    ktj_mat_activity* a = new_act(o);
    a->ts = r->start_ns;
    a->dur = r->end_ns - r->start_ns;
    /* a deviceId beyond 32 bits travels in the args slot before the record's values (include/ktj.h) */
    a->device = ((r->flags & KTJ_GF_WIDE_DEVICE) && r->args_off >= 1 && r->args_off - 1 < s->n_args)
                    ? (int64_t)s->args[r->args_off - 1] : r->device;
    a->resource = r->resource;
    a->corr = r->id;
    a->flow_id = r->flow_id;
    a->flow_type = r->flow_type;
    a->flow_start = (r->flags & KTJ_GF_FLOW_START) ? 1 : 0;
    a->type = r->type;
    a->has_linked = (r->flags & KTJ_GF_LINKED) ? 1 : 0;
    a->linked_corr = r->linked_id;
    a->name_id = r->name_id == KTJ_NONE ? o->builtin0 + BS_EMPTY : r->name_id;
    a->arrival = i;
    if (r->schema_id != KTJ_NONE && r->schema_id < s->n_schemas) {
      const ktj_schema_desc* d = &s->schemas[r->schema_id];
      uint64_t slot = r->args_off;
      for (uint32_t f = 0; f < d->n_fields; ++f) {
        const ktj_field* fd = &s->fields[d->first_field + f];
        if (fd->type == KTJ_F_SHAPES) { /* the value's encoding lives elsewhere in the blob: materialised inline */
          const uint64_t at = slot < s->n_args ? s->args[slot] : s->n_args;
          const uint64_t len = shapes_encoded_slots(s->args, s->n_args, at);
          visit(o, a, fd->key_id, fd->type, (uint16_t)len, len ? s->args + at : NULL);
        } else if (fd->type != KTJ_F_COLLECTIVE) visit(o, a, fd->key_id, fd->type, fd->count, s->args + slot);
        slot += fd->count;
      }
    }
    /* an activity that arrives with its record_param_comms op resolved (output_json.cpp:899-908) */
    if (a->has_linked && (r->type == KTJ_TYPE_CONCURRENT_KERNEL || r->type == KTJ_TYPE_MTIA_CCP_EVENTS))
      a->collective = collective_index(s, r);
    *umap_slot(&activity_map, (uint64_t)(int64_t)r->id, NULL) = i;
  }
  for (uint64_t i = 0; i < s->n_extcorr; ++i)
    *umap_slot(&cpu_corr, s->extcorr[i].correlation, NULL) = s->extcorr[i].external_id;
  umap user_corr; umap_init(&user_corr, s->n_usercorr); /* userCorrelationMap_: RocmActivityProfiler.cpp:141-142 */
  for (uint64_t i = 0; i < s->n_usercorr; ++i)
    *umap_slot(&user_corr, s->usercorr[i].correlation, NULL) = s->usercorr[i].external_id;
  user_span* spans = NULL; uint64_t n_spans = 0, cap_spans = 0;

  /* ---- stream back-fill: libkineto/src/RocmStreamQueue.h:42-136 ---- */
  uint64_t* dev_stream = (uint64_t*)malloc(8 * (s->n_device ? s->n_device : 1));
  if (!dev_stream) abort();
  {
    umap by_corr; umap_init(&by_corr, s->n_runtime);
    for (uint64_t i = 0; i < s->n_runtime; ++i) {
      const ktj_runtime_rec* r = &s->runtime[i];
      uint64_t sid = r->kind == KTJ_RT_KERNEL ? r->u.kernel.stream
                   : r->kind == KTJ_RT_COPY ? r->u.copy.stream : 0;
      if (sid != 0) *umap_slot(&by_corr, r->id, NULL) = sid;
    }
    for (uint64_t i = 0; i < s->n_device; ++i) dev_stream[i] = s->device[i].stream;
    if (by_corr.n != 0) {
      for (uint64_t i = 0; i < s->n_device; ++i) {
        const ktj_device_rec* d = &s->device[i];
        if (KTJ_ROW_DOMAIN(d->domain) == KTJ_DOM_MEMSET || dev_stream[i] != 0) continue;
        const uint64_t* f = umap_find(&by_corr, d->id);
        if (f) dev_stream[i] = *f;
      }
      /* fallback: infer the stream from the HSA queue when that is unambiguous */
      const uint64_t AMBIG = ~0ULL;
      umap by_queue; umap_init(&by_queue, 1024);
      for (uint64_t i = 0; i < s->n_device; ++i) {
        const ktj_device_rec* d = &s->device[i];
        if (KTJ_ROW_DOMAIN(d->domain) == KTJ_DOM_MEMSET || dev_stream[i] == 0 || d->queue == 0) continue;
        int inserted;
        uint64_t* v = umap_slot(&by_queue, d->queue, &inserted);
        if (inserted) *v = dev_stream[i];
        else if (*v != AMBIG && *v != dev_stream[i]) umap_erase_mark(&by_queue, d->queue, AMBIG);
      }
      for (uint64_t i = 0; i < s->n_device; ++i) {
        const ktj_device_rec* d = &s->device[i];
        if (KTJ_ROW_DOMAIN(d->domain) == KTJ_DOM_MEMSET || dev_stream[i] != 0) continue;
        const uint64_t* f = umap_find(&by_queue, d->queue);
        if (f && *f != AMBIG) dev_stream[i] = *f;
      }
      umap_free(&by_queue);
      /* dense per-device index in first-seen order; queue id tagged with the high bit when
       * there is still no stream */
      dense_map dense; dense_init(&dense);
      for (uint64_t i = 0; i < s->n_device; ++i) {
        const ktj_device_rec* d = &s->device[i];
        if (KTJ_ROW_DOMAIN(d->domain) == KTJ_DOM_MEMSET) continue;
        uint64_t key;
        if (dev_stream[i] != 0) key = dev_stream[i];
        else if (d->queue != 0) key = d->queue | (1ULL << 63);
        else continue;
        dev_stream[i] = dense_index(&dense, d->device, key);
      }
      dense_free(&dense);
    }
    umap_free(&by_corr);
  }

  /* flow-start cid set */
  uint8_t* flow_start = (uint8_t*)calloc(s->n_cids ? s->n_cids : 1, 1);
  for (uint64_t i = 0; i < s->n_flow_start; ++i)
    if (s->flow_start_cids[i] < s->n_cids) flow_start[s->flow_start_cids[i]] = 1;

  /* ---- runtime rows: RocprofActivityApi.cpp:145-179 + RocmActivityProfiler.cpp:150-169 ---- */
  for (uint64_t i = 0; i < s->n_runtime; ++i) {
    const ktj_runtime_rec* r = &s->runtime[i];
    uint64_t begin = r->begin, end = r->end;
    if (cm->runtime_mode == KTJ_CLOCK_CONVERT) {
      begin = (uint64_t)ktj_oracle_convert_ts(cm, begin);
      end = (uint64_t)ktj_oracle_convert_ts(cm, end);
    } else if (cm->runtime_mode == KTJ_CLOCK_OFFSET) {
      begin += (uint64_t)cm->async_offset;
      end += (uint64_t)cm->async_offset;
    }
    int64_t ts = (int64_t)begin;          /* RocprofActivity::timestamp  (RocprofActivity.h:42-44) */
    int64_t dur = (int64_t)(end - begin); /* RocprofActivity::duration   (RocprofActivity.h:45-47) */
    int64_t linked = linked_activity(&cpu_corr, &activity_map, r->id);
    check_ts_order(o, &seen, &ents, &n_ents, &cap_ents, (int64_t)r->id, 1, ts);
    if (out_of_range(o, ts, dur)) continue;

    ktj_mat_activity* a = new_act(o);
    a->ts = ts; a->dur = dur;
    a->device = r->pid; a->resource = r->tid;   /* RocprofActivity.h:141-146 */
    a->corr = (int64_t)r->id;
    a->flow_id = a->corr;                       /* RocprofActivity.h:60-62 */
    a->flow_type = KTJ_LINK_ASYNC_CPU_GPU;
    a->flow_start = r->cid < s->n_cids ? flow_start[r->cid] : 0; /* RocprofActivity_inl.h:185-200 */
    a->type = KTJ_TYPE_CUDA_RUNTIME;
    a->arrival = s->n_generic + i;
    if (linked >= 0) { a->has_linked = 1; a->linked_corr = s->generic[linked].id; o->n_linked++; }
    if (r->cid < s->n_cids && s->cid_name_ids[r->cid] != KTJ_NONE) a->name_id = s->cid_name_ids[r->cid];
    else { /* RocprofLogger::opString fallback: RocprofLogger.cpp:751-760 */
      char b[64];
      int n = sprintf(b, "<unknown operation:%u>", r->cid);
      a->name_id = add_xstring(o, b, (size_t)n);
    }
    int key = (int)(uint32_t)r->id;             /* unordered_map<int,…> key */
    switch (r->kind) {
      case KTJ_RT_KERNEL: { /* RocprofActivity_inl.h:208-232 */
        if (r->u.kernel.kernel_name_id != KTJ_NONE) visit1(o, a, BS_KERNEL, KTJ_F_STR, r->u.kernel.kernel_name_id);
        *umap_slot(&corr_to_kernel, (uint64_t)(int64_t)key, NULL) = i;
        visit1(o, a, BS_CID, KTJ_F_U64, r->cid);
        visit1(o, a, BS_CORRELATION, KTJ_F_U64, r->id);
        uint64_t g3[3] = {r->u.kernel.grid[0], r->u.kernel.grid[1], r->u.kernel.grid[2]};
        uint64_t b3[3] = {r->u.kernel.workgroup[0], r->u.kernel.workgroup[1], r->u.kernel.workgroup[2]};
        visit(o, a, o->builtin0 + BS_GRID, KTJ_F_I64_ARRAY, 3, g3);
        visit(o, a, o->builtin0 + BS_BLOCK, KTJ_F_I64_ARRAY, 3, b3);
        visit1(o, a, BS_SHARED_MEMORY, KTJ_F_U64, r->u.kernel.group_segment_size);
        break;
      }
      case KTJ_RT_COPY: { /* RocprofActivity_inl.h:243-255 */
        *umap_slot(&corr_to_size, (uint64_t)(int64_t)key, NULL) = r->u.copy.size;
        visit1(o, a, BS_CID, KTJ_F_U64, r->cid);
        visit1(o, a, BS_CORRELATION, KTJ_F_U64, r->id);
        visit1(o, a, BS_SRC, KTJ_F_STR, ptr_string(o, r->u.copy.src));
        visit1(o, a, BS_DST, KTJ_F_STR, ptr_string(o, r->u.copy.dst));
        visit1(o, a, BS_BYTES, KTJ_F_U64, r->u.copy.size);
        char b[16];
        int n = sprintf(b, "%d", (int)r->u.copy.copy_kind);
        visit1(o, a, BS_KIND, KTJ_F_STR, add_xstring(o, b, (size_t)n));
        break;
      }
      case KTJ_RT_MALLOC: { /* RocprofActivity_inl.h:265-277 */
        *umap_slot(&corr_to_size, (uint64_t)(int64_t)key, NULL) = r->u.malloc_.size;
        if (r->cid == s->malloc_cid) visit1(o, a, BS_BYTES, KTJ_F_U64, r->u.malloc_.size);
        visit1(o, a, BS_CID, KTJ_F_U64, r->cid);
        visit1(o, a, BS_CORRELATION, KTJ_F_U64, r->id);
        visit1(o, a, BS_PTR, KTJ_F_STR, ptr_string(o, r->u.malloc_.ptr));
        break;
      }
      default: /* RocprofActivity_inl.h:294-299 */
        visit1(o, a, BS_CID, KTJ_F_U64, r->cid);
        visit1(o, a, BS_CORRELATION, KTJ_F_U64, r->id);
        break;
    }
  }

  /* ---- device rows: RocprofActivityApi.cpp:166-170, RocmActivityProfiler.cpp:171-178,
   *      GenericActivityProfiler.cpp:410-435 ---- */
  for (uint64_t i = 0; i < s->n_device; ++i) {
    const ktj_device_rec* d = &s->device[i];
    uint64_t begin = d->begin, end = d->end;
    if (cm->device_mode == KTJ_CLOCK_CONVERT) {
      begin = (uint64_t)ktj_oracle_convert_ts(cm, begin);
      end = (uint64_t)ktj_oracle_convert_ts(cm, end);
    } else if (cm->device_mode == KTJ_CLOCK_OFFSET) {
      begin += (uint64_t)cm->async_offset;
      end += (uint64_t)cm->async_offset;
    }
    int64_t ts, dur, resource;
    if (KTJ_ROW_DOMAIN(d->domain) == KTJ_DOM_MEMSET) {
      /* CuptiActivity.h GpuActivity<T>::timestamp/duration via CuptiTimestamp.h:29-51 */
      ts = (int64_t)begin;
      dur = (int64_t)end - (int64_t)begin;
      resource = (int64_t)(uint32_t)d->stream; /* streamId is 32 bits wide: ktj_memset_rec */
    } else {
      /* RocprofActivity.h:122-127 */
      ts = (int64_t)(begin + 1);
      dur = (int64_t)(end - (begin + 1));
      resource = (int64_t)(dev_stream[i] != 0 ? dev_stream[i] : d->queue); /* RocprofActivity.h:100-102 */
    }
    int64_t linked = linked_activity(&cpu_corr, &activity_map, d->id);
    if (out_of_range(o, ts, dur)) continue;
    check_ts_order(o, &seen, &ents, &n_ents, &cap_ents, (int64_t)d->id, 0, ts);

    ktj_mat_activity* a = new_act(o);
    a->ts = ts; a->dur = dur; a->device = d->device; a->resource = resource;
    a->corr = (int64_t)d->id;
    a->flow_id = a->corr;
    a->flow_type = KTJ_LINK_ASYNC_CPU_GPU;
    a->flow_start = 0;
    a->arrival = s->n_generic + s->n_runtime + i;
    if (s->n_usercorr) { /* handleGpuActivity: GenericActivityProfiler.cpp:423-433 */
      const uint64_t* ext = umap_find(&user_corr, d->id);
      const uint64_t* op = ext ? umap_find(&activity_map, *ext) : NULL;
      if (op) { /* GpuUserEventMap::insertOrExtendEvent: :292-311 */
        const int64_t cpu_id = s->generic[*op].id;
        user_span* sp = NULL;
        for (uint64_t k = 0; k < n_spans && !sp; ++k)
          if (spans[k].device == a->device && spans[k].resource == a->resource && spans[k].cpu_id == cpu_id) sp = &spans[k];
        if (!sp) { /* createUserGpuSpan: :277-290 */
          if (n_spans == cap_spans) {
            cap_spans = cap_spans ? cap_spans * 2 : 64;
            spans = (user_span*)realloc(spans, cap_spans * sizeof *spans);
            if (!spans) abort();
          }
          sp = &spans[n_spans++];
          sp->device = a->device; sp->resource = a->resource; sp->cpu_id = cpu_id; sp->cpu_row = *op;
          sp->start = ts; sp->end = ts + dur;
        }
        if (ts < sp->start || sp->start == 0) sp->start = ts;
        if (ts + dur > sp->end) sp->end = ts + dur;
      }
    }
    if (linked >= 0) {
      a->has_linked = 1; a->linked_corr = s->generic[linked].id; o->n_linked++;
      const ktj_generic_rec* op = &s->generic[linked]; /* the op hands its collective metadata to kernels */
      if (KTJ_ROW_DOMAIN(d->domain) != KTJ_DOM_MEMSET && KTJ_ROW_DOMAIN(d->domain) != KTJ_DOM_MEMORY_COPY && op->type != KTJ_TYPE_CONCURRENT_KERNEL &&
          op->type != KTJ_TYPE_MTIA_CCP_EVENTS)
        a->collective = collective_index(s, op);
    }
    int key = (int)(uint32_t)d->id;
    if (KTJ_ROW_DOMAIN(d->domain) == KTJ_DOM_MEMSET) { /* CuptiActivity.h:682-719 */
      ktj_memset_rec m;
      memcpy(&m, d, sizeof m);
      a->type = KTJ_TYPE_GPU_MEMSET;
      a->name_id = o->builtin0 + (m.memory_kind <= KTJ_MEMKIND_MANAGED_STATIC ? BS_MEMSET_UNKNOWN + m.memory_kind : BS_MEMSET_UNRECOGNIZED);
      visit1(o, a, BS_DEVICE, KTJ_F_I64, (uint64_t)(int64_t)m.device);
      visit1(o, a, BS_CONTEXT, KTJ_F_U64, m.context);
      visit1(o, a, BS_STREAM, KTJ_F_I64, m.stream);
      visit1(o, a, BS_CORRELATION, KTJ_F_U64, m.id);
      visit1(o, a, BS_BYTES, KTJ_F_U64, m.bytes);
      if (dur != 0) /* addBandwidthTypedMetadata, CuptiActivity.h:460-470 */
        visit1(o, a, BS_BANDWIDTH, KTJ_F_F64, dbits((double)m.bytes / (double)dur));
      if (s->create_flags & KTJ_CREATE_CUDA12_ARGS) { /* CUDA_VERSION >= 12000: CuptiActivity.h:424-458 */
        visit1(o, a, BS_GRAPH_ID, KTJ_F_U64, m.graph_id);
        visit1(o, a, BS_GRAPH_NODE_ID, KTJ_F_U64, (uint64_t)m.graph_node_lo | ((uint64_t)m.graph_node_hi << 32));
        visit1(o, a, BS_CHANNEL, KTJ_F_U64, m.channel_id);
        visit1(o, a, BS_CHANNEL_TYPE, KTJ_F_I64, m.channel_type);
      }
      continue;
    }
    int kind_str;
    if (KTJ_ROW_DOMAIN(d->domain) == KTJ_DOM_MEMORY_COPY) { /* RocprofActivity_inl.h:50-94, 98-127 */
      a->type = KTJ_TYPE_GPU_MEMCPY;
      const char *ks, *src, *dst;
      switch (d->op) {
        case KTJ_COPY_H2H: ks = "HtoH"; src = "Host"; dst = "Host"; kind_str = BS_HTOH; break;
        case KTJ_COPY_H2D: ks = "HtoD"; src = "Host"; dst = "Device"; kind_str = BS_HTOD; break;
        case KTJ_COPY_D2H: ks = "DtoH"; src = "Device"; dst = "Host"; kind_str = BS_DTOH; break;
        case KTJ_COPY_D2D: ks = "DtoD"; src = "Device"; dst = "Device"; kind_str = BS_DTOD; break;
        default: ks = "<unknown>"; src = "?"; dst = "?"; kind_str = BS_UNKNOWN_KIND; break;
      }
      char b[96];
      int n = sprintf(b, "Memcpy %s (%s -> %s)", ks, src, dst);
      a->name_id = add_xstring(o, b, (size_t)n);
    } else {
      a->type = KTJ_TYPE_CONCURRENT_KERNEL;
      kind_str = BS_DISPATCH_KERNEL;
      if (d->name_id != KTJ_NONE) a->name_id = d->name_id;
      else {
        char b[64];
        int n = sprintf(b, "<unknown operation:%u>", d->op);
        a->name_id = add_xstring(o, b, (size_t)n);
      }
    }
    /* GpuActivity::visitTypedMetadata: RocprofActivity_inl.h:147-180 */
    visit1(o, a, BS_DEVICE, KTJ_F_I64, (uint64_t)(int64_t)d->device);
    visit1(o, a, BS_STREAM, KTJ_F_I64, (uint64_t)resource);
    visit1(o, a, BS_HSA_QUEUE, KTJ_F_U64, d->queue);
    visit1(o, a, BS_CORRELATION, KTJ_F_U64, d->id);
    visit1(o, a, BS_KIND, KTJ_F_STR, o->builtin0 + (uint32_t)kind_str);
    const uint64_t* sz = umap_find(&corr_to_size, (uint64_t)(int64_t)key);
    if (sz) {
      visit1(o, a, BS_BYTES, KTJ_F_U64, *sz);
      uint64_t raw_dur = end - begin;
      if (raw_dur != 0) /* RocprofActivity_inl.h:129-139 */
        visit1(o, a, BS_BANDWIDTH, KTJ_F_F64, dbits((double)*sz / (double)raw_dur));
    } else {
      const uint64_t* kr = umap_find(&corr_to_kernel, (uint64_t)(int64_t)key);
      if (kr) {
        const ktj_runtime_rec* r = &s->runtime[*kr];
        uint64_t g3[3] = {r->u.kernel.grid[0], r->u.kernel.grid[1], r->u.kernel.grid[2]};
        uint64_t b3[3] = {r->u.kernel.workgroup[0], r->u.kernel.workgroup[1], r->u.kernel.workgroup[2]};
        visit(o, a, o->builtin0 + BS_GRID, KTJ_F_I64_ARRAY, 3, g3);
        visit(o, a, o->builtin0 + BS_BLOCK, KTJ_F_I64_ARRAY, 3, b3);
      }
    }
  }

  /* GpuUserEventMap::logEvents (GenericActivityProfiler.cpp:313-319, called at :726): after every
   * GPU activity, stream by stream (std::map order) and, inside a stream, in the iteration order
   * of a std::unordered_map keyed by the annotation's id (taken from the C++ library) */
  if (n_spans) {
    int64_t* kd = (int64_t*)malloc(8 * n_spans); int64_t* kr = (int64_t*)malloc(8 * n_spans);
    int64_t* ki = (int64_t*)malloc(8 * n_spans); uint64_t* ord = (uint64_t*)malloc(8 * n_spans);
    if (!kd || !kr || !ki || !ord) abort();
    for (uint64_t k = 0; k < n_spans; ++k) { kd[k] = spans[k].device; kr[k] = spans[k].resource; ki[k] = spans[k].cpu_id; }
    ktj_oracle_span_map_order(kd, kr, ki, n_spans, ord);
    for (uint64_t k = 0; k < n_spans; ++k) {
      const user_span* sp = &spans[ord[k]];
      const ktj_generic_rec* op = &s->generic[sp->cpu_row];
      ktj_mat_activity* a = new_act(o);
      a->ts = sp->start; a->dur = sp->end - sp->start;
      a->device = sp->device; a->resource = sp->resource;
      a->corr = sp->cpu_id;
      a->type = KTJ_TYPE_GPU_USER_ANNOTATION;
      a->name_id = op->name_id == KTJ_NONE ? o->builtin0 + BS_EMPTY : op->name_id;
      a->arrival = s->n_generic + s->n_runtime + s->n_device + k;
    }
    free(kd); free(kr); free(ki); free(ord);
  }
  free(spans);
  umap_free(&user_corr);
  free(flow_start);
  free(dev_stream);
  free(ents);
  umap_free(&activity_map); umap_free(&cpu_corr); umap_free(&seen);
  umap_free(&corr_to_kernel); umap_free(&corr_to_size);
  for (uint64_t i = 0; i < o->n_acts; ++i) {
    o->acts[i].fields = o->fpool + o->act_f0[i];
    o->acts[i].slots = o->spool + o->act_s0[i];
  }
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* stage 3: canonical order — stable sort by (deviceId, resourceId, timestamp)                  */
/* ------------------------------------------------------------------------------------------ */
static int act_less(const ktj_mat_activity* a, const ktj_mat_activity* b) {
  if (a->device != b->device) return a->device < b->device;
  if (a->resource != b->resource) return a->resource < b->resource;
  return a->ts < b->ts;
}
static void merge_sort(const ktj_mat_activity* acts, uint64_t* idx, uint64_t* tmp, uint64_t n) {
  if (n < 2) return;
  uint64_t h = n / 2;
  merge_sort(acts, idx, tmp, h);
  merge_sort(acts, idx + h, tmp, n - h);
  uint64_t i = 0, j = h, k = 0;
  while (i < h && j < n) {
    if (act_less(&acts[idx[j]], &acts[idx[i]])) tmp[k++] = idx[j++];
    else tmp[k++] = idx[i++];
  }
  while (i < h) tmp[k++] = idx[i++];
  while (j < n) tmp[k++] = idx[j++];
  memcpy(idx, tmp, n * 8);
}

/* ------------------------------------------------------------------------------------------ */
/* stage 4: the logger                                                                          */
/* ------------------------------------------------------------------------------------------ */
static int64_t rel_time(const ktj_oracle* o, int64_t t) { /* output_json.cpp:144-153 */
  int64_t r = t - o->s->base_time_ns;
  return r < 0 ? 0 : r;
}
static int64_t sanitize_tid(int64_t tid) { /* output_json.cpp:114-121 */
  if (tid == INT64_MIN) return 0;
  return tid < 0 ? -tid : tid;
}

/* sanitizeStrForJSON + escapeQuotesForJSON on a C string (info names) */
static void put_info_string(sbuf* b, const char* s) {
  size_t n = strlen(s);
  char* t = (char*)malloc(n + 1);
  if (!t) abort();
  size_t m = ktj_oracle_sanitize_str(s, n, t);
  for (size_t i = 0; i < m; ++i) {
    if (t[i] == '"') sb_putc(b, '\\');
    sb_putc(b, t[i]);
  }
  free(t);
}

/* writeMetadataEvent: output_json.cpp:214-235 */
static void write_metadata_event(ktj_oracle* o, const char* name, int64_t ts, const char* pid,
                                 const char* tid, const char* arg_key, const char* arg_value,
                                 size_t arg_value_n) {
  char t[40];
  ktj_oracle_fmt_ts(ts, t);
  sbuf* b = &o->out;
  sb_puts(b, "\n  {\n    \"ph\": \"M\",\n    \"name\": \""); sb_puts(b, name);
  sb_puts(b, "\",\n    \"ts\": "); sb_puts(b, t);
  sb_puts(b, ",\n    \"pid\": "); sb_puts(b, pid);
  sb_puts(b, ",\n    \"tid\": "); sb_puts(b, tid);
  sb_puts(b, ",\n    \"args\": {\n      \""); sb_puts(b, arg_key);
  sb_puts(b, "\": "); sb_put(b, arg_value, arg_value_n);
  sb_puts(b, "\n    }\n  },");
}
static void write_metadata_event_i(ktj_oracle* o, const char* name, int64_t ts, int64_t pid,
                                   int64_t tid, const char* arg_key, const char* arg_value,
                                   size_t n) { /* output_json.cpp:348-357 */
  char p[24], t[24];
  fmt_i64(pid, p);
  fmt_i64(tid, t);
  write_metadata_event(o, name, ts, p, t, arg_key, arg_value, n);
}

/* ArgsBuilder::renderField: output_json.cpp:193-203 */
static void put_args_field(sbuf* b, const sbuf* args) {
  if (args->n == 0) return;
  sb_puts(b, ",\n    \"args\": {\n      ");
  sb_put(b, args->p, args->n);
  sb_puts(b, "\n    }");
}

/* writeCompleteEvent: output_json.cpp:237-259 */
static void write_complete_event(ktj_oracle* o, const char* cat, const char* name, size_t name_n,
                                 const char* pid, const char* tid, int64_t ts, int64_t dur,
                                 const sbuf* args) {
  char t1[40], t2[40];
  ktj_oracle_fmt_ts(ts, t1);
  ktj_oracle_fmt_ts(dur, t2);
  sbuf* b = &o->out;
  sb_puts(b, "\n  {\n    \"ph\": \"X\",\n    \"cat\": \""); sb_puts(b, cat);
  sb_puts(b, "\",\n    \"name\": \""); sb_put(b, name, name_n);
  sb_puts(b, "\",\n    \"pid\": "); sb_puts(b, pid);
  sb_puts(b, ",\n    \"tid\": "); sb_puts(b, tid);
  sb_puts(b, ",\n    \"ts\": "); sb_puts(b, t1);
  sb_puts(b, ",\n    \"dur\": "); sb_puts(b, t2);
  sb_puts(b, "\n    ");
  put_args_field(b, args);
  sb_puts(b, "\n  },");
}

/* writeInstantEvent: output_json.cpp:261-292 */
static void write_instant_event(ktj_oracle* o, const char* cat, const char* scope, const char* name,
                                const char* pid, const char* tid, int64_t ts, const sbuf* args,
                                int final_event) {
  char t[40];
  ktj_oracle_fmt_ts(ts, t);
  sbuf* b = &o->out;
  sb_puts(b, "\n  {\n    \"ph\": \"i\",\n    ");
  if (cat[0]) { sb_puts(b, "\n    \"cat\": \""); sb_puts(b, cat); sb_puts(b, "\","); }
  sb_puts(b, "\n    \"s\": \""); sb_puts(b, scope);
  sb_puts(b, "\",\n    \"name\": \""); sb_puts(b, name);
  sb_puts(b, "\",\n    \"pid\": "); sb_puts(b, pid);
  sb_puts(b, ",\n    \"tid\": "); sb_puts(b, tid);
  sb_puts(b, ",\n    \"ts\": "); sb_puts(b, t);
  sb_puts(b, "\n    ");
  put_args_field(b, args);
  sb_puts(b, "\n  }");
  if (!final_event) sb_putc(b, ',');
}

/* writeFlowEvent: output_json.cpp:318-345 */
static void write_flow_event(ktj_oracle* o, char type, int64_t id, int64_t pid, int64_t tid, int64_t ts,
                             const char* name) {
  char t[40], a[24], p[24], q[24];
  ktj_oracle_fmt_ts(ts, t);
  fmt_i64(id, a); fmt_i64(pid, p); fmt_i64(tid, q);
  sbuf* b = &o->out;
  sb_puts(b, "\n  {\n    \"ph\": \""); sb_putc(b, type);
  sb_puts(b, "\",\n    \"id\": "); sb_puts(b, a);
  sb_puts(b, ",\n    \"pid\": "); sb_puts(b, p);
  sb_puts(b, ",\n    \"tid\": "); sb_puts(b, q);
  sb_puts(b, ",\n    \"ts\": "); sb_puts(b, t);
  sb_puts(b, ",\n    \"cat\": \""); sb_puts(b, name);
  sb_puts(b, "\",\n    \"name\": \""); sb_puts(b, name);
  sb_puts(b, "\"\n    ");
  if (type == 'f') sb_puts(b, ", \"bp\": \"e\"");
  sb_puts(b, "\n  },");
}

/* handleTraceStart + metadataToJSON: output_json.cpp:414-479 */
static void handle_trace_start(ktj_oracle* o) {
  const ktj_stream* s = o->s;
  sbuf* b = &o->out;
  char n[32];
  sb_puts(b, " {\n    \"schemaVersion\": 1,\n    \"deviceProperties\": [");
  sb_puts(b, s->device_properties ? s->device_properties : "");
  sb_puts(b, "],\n    ");
  for (uint64_t i = 0; i < s->n_meta; ++i) {
    const char* k = s->meta_kv[2 * i];
    const char* v = s->meta_kv[2 * i + 1];
    size_t vn = strlen(v);
    char* t = (char*)malloc(vn + 1);
    if (!t) abort();
    size_t m = ktj_oracle_sanitize_str(v, vn, t);
    sb_puts(b, "\n      \""); sb_puts(b, k); sb_puts(b, "\": "); sb_put(b, t, m); sb_putc(b, ',');
    free(t);
  }
  sb_puts(b, "\n    \"displayTimeUnit\": \"ms\",\n    \"baseTimeNanoseconds\": ");
  fmt_i64(s->base_time_ns, n);
  sb_puts(b, n);
  sb_puts(b, ",\n    \"traceEvents\": [\n    ");
}

/* handleDeviceInfo: output_json.cpp:507-542 */
static void handle_device_info(ktj_oracle* o, const ktj_device_info* info) {
  sbuf v = {0};
  char n[24];
  int64_t t = rel_time(o, info->time_ns);
  sb_putc(&v, '"'); put_info_string(&v, info->name); sb_putc(&v, '"');
  write_metadata_event_i(o, "process_name", t, info->id, 0, "name", v.p, v.n);
  v.n = 0;
  sb_putc(&v, '"'); put_info_string(&v, info->label); sb_putc(&v, '"');
  write_metadata_event_i(o, "process_labels", t, info->id, 0, "labels", v.p, v.n);
  size_t k = fmt_i64(info->sort_index, n);
  write_metadata_event_i(o, "process_sort_index", t, info->id, 0, "sort_index", n, k);
  free(v.p);
}

/* handleResourceInfo: output_json.cpp:544-577 */
static void handle_resource_info(ktj_oracle* o, const ktj_resource_info* info) {
  sbuf raw = {0}, v = {0};
  char n[24];
  if (info->host_thread) {
    sb_puts(&raw, "thread "); fmt_i64(info->id, n); sb_puts(&raw, n);
    sb_puts(&raw, " ("); sb_puts(&raw, info->name); sb_puts(&raw, ")");
  } else sb_puts(&raw, info->name);
  sb_putc(&raw, 0);
  sb_putc(&v, '"'); put_info_string(&v, raw.p); sb_putc(&v, '"');
  int64_t t = rel_time(o, info->time_ns);
  int64_t tid = sanitize_tid(info->id);
  write_metadata_event_i(o, "thread_name", t, info->device_id, tid, "name", v.p, v.n);
  size_t k = fmt_i64(info->sort_index, n);
  write_metadata_event_i(o, "thread_sort_index", t, info->device_id, tid, "sort_index", n, k);
  free(raw.p); free(v.p);
}

/* handleOverheadInfo: output_json.cpp:579-607 */
static void handle_overhead_info(ktj_oracle* o, const ktj_overhead_info* info) {
  sbuf v = {0};
  int64_t t = rel_time(o, info->time_ns);
  sb_putc(&v, '"'); put_info_string(&v, info->name); sb_putc(&v, '"');
  write_metadata_event_i(o, "process_name", t, -1, 0, "name", v.p, v.n);
  write_metadata_event_i(o, "process_sort_index", t, -1, 0, "sort_index", "16777226", 8); /* 0x100000A */
  free(v.p);
}

/* handleTraceSpan + addIterationMarker: output_json.cpp:609-658 */
static void handle_trace_span(ktj_oracle* o, const ktj_trace_span* sp) {
  int64_t start = rel_time(o, sp->start_ns);
  int64_t dur = sp->end_ns == 0 ? 0 : sp->end_ns - sp->start_ns;
  sbuf args = {0}, name = {0}, tid = {0};
  char n[24];
  sb_puts(&args, "\"Op count\": "); fmt_i64(sp->op_count, n); sb_puts(&args, n);
  sb_puts(&name, sp->prefix); sb_puts(&name, sp->name); sb_puts(&name, " (");
  fmt_i64(sp->iteration, n); sb_puts(&name, n); sb_puts(&name, ")");
  sb_putc(&tid, '"'); sb_puts(&tid, sp->name); sb_putc(&tid, '"'); sb_putc(&tid, 0);
  write_complete_event(o, "Trace", name.p, name.n, "\"Spans\"", tid.p, start, dur, &args);
  write_metadata_event(o, "process_sort_index", start, "\"Spans\"", "0", "sort_index", "536870912", 9);
  sbuf iname = {0}, itid = {0}, none = {0};
  sb_puts(&iname, "Iteration Start: "); sb_puts(&iname, sp->name); sb_putc(&iname, 0);
  sb_puts(&itid, "\"Trace "); sb_puts(&itid, sp->name); sb_puts(&itid, "\""); sb_putc(&itid, 0);
  write_instant_event(o, "", "g", iname.p, "\"Traces\"", itid.p, start, &none, 0);
  free(args.p); free(name.p); free(tid.p); free(iname.p); free(itid.p);
}

/* JsonTypedMetadataVisitor: libkineto/include/TypedMetadataJson.h:38-205 */
static void render_metadata(const ktj_oracle* o, const ktj_mat_activity* a, sbuf* json) {
  const uint64_t* slot = a->slots;
  int first = 1;
  char n[48];
  for (uint32_t f = 0; f < a->n_fields; ++f) {
    const ktj_field* fd = &a->fields[f];
    const char* p; uint64_t len;
    if (fd->key_id != KTJ_NONE) { /* appendKey: TypedMetadataJson.h:145-152 */
      if (!first) sb_puts(json, ", ");
      first = 0;
      ktj_oracle_string(o, fd->key_id, &p, &len);
      sb_putc(json, '"'); sb_put(json, p, len); sb_puts(json, "\": ");
    }
    switch (fd->type) {
      case KTJ_F_I64: sb_put(json, n, fmt_i64((int64_t)slot[0], n)); break;
      case KTJ_F_U64: sb_put(json, n, fmt_u64(slot[0], n)); break;
      case KTJ_F_F64: { /* appendDoubleValue: TypedMetadataJson.h:172-178 */
        double d; memcpy(&d, &slot[0], 8);
        size_t k = ktj_oracle_fmt_double(d, n);
        if (isfinite(d)) sb_put(json, n, k);
        else { sb_putc(json, '"'); sb_put(json, n, k); sb_putc(json, '"'); }
        break;
      }
      case KTJ_F_BOOL: sb_puts(json, slot[0] ? "true" : "false"); break;
      case KTJ_F_STR:
        ktj_oracle_string(o, (uint32_t)slot[0], &p, &len);
        sb_putc(json, '"'); sb_put(json, p, len); sb_putc(json, '"');
        break;
      case KTJ_F_RAW:
        ktj_oracle_string(o, (uint32_t)slot[0], &p, &len);
        sb_put(json, p, len);
        break;
      case KTJ_F_I64_ARRAY: /* appendArray: TypedMetadataJson.h:52-64 */
        sb_putc(json, '[');
        for (uint32_t k = 0; k < fd->count; ++k) {
          if (k) sb_puts(json, ", ");
          sb_put(json, n, fmt_i64((int64_t)slot[k], n));
        }
        sb_putc(json, ']');
        break;
      case KTJ_F_STR_ARRAY: /* appendArray over appendQuoted: TypedMetadataJson.h:52-64, 184-186 */
        sb_putc(json, '[');
        for (uint32_t k = 0; k < fd->count; ++k) {
          if (k) sb_puts(json, ", ");
          ktj_oracle_string(o, (uint32_t)slot[k], &p, &len);
          sb_putc(json, '"'); sb_put(json, p, len); sb_putc(json, '"');
        }
        sb_putc(json, ']');
        break;
      case KTJ_F_DICT_BEGIN: sb_putc(json, '{'); first = 1; break;  /* beginDict: TypedMetadataJson.h:128-132 */
      case KTJ_F_DICT_END: sb_putc(json, '}'); first = 0; break;    /* endDict: :134-137 */
      case KTJ_F_UNSUPPORTED: sb_puts(json, "\"<unsupported metadata type>\""); break; /* :122-126 */
      case KTJ_F_SHAPES: { /* appendArray over the nested shapes: TypedMetadataJson.h:186-201; inline encoding */
        const uint64_t* q = slot; const uint64_t* end = slot + fd->count;
        const uint64_t entries = q < end ? *q++ : 0;
        sb_putc(json, '[');
        for (uint64_t e = 0; e < entries && q < end; ++e) {
          if (e) sb_puts(json, ", ");
          const uint64_t head = *q++, m = head & 0xFFFFFFFFull;
          const uint64_t tensors = (head & KTJ_SHAPE_LIST) ? m : 1;
          if (head & KTJ_SHAPE_LIST) sb_putc(json, '[');
          for (uint64_t t = 0; t < tensors && ((head & KTJ_SHAPE_LIST) == 0 || q < end); ++t) {
            if (t) sb_puts(json, ", ");
            const uint64_t rank = (head & KTJ_SHAPE_LIST) ? (*q++ & 0xFFFFFFFFull) : m;
            sb_putc(json, '[');
            for (uint64_t k = 0; k < rank; ++k) {
              if (k) sb_puts(json, ", ");
              sb_put(json, n, fmt_i64(q < end ? (int64_t)*q : 0, n));
              if (q < end) ++q;
            }
            sb_putc(json, ']');
          }
          if (head & KTJ_SHAPE_LIST) sb_putc(json, ']');
        }
        sb_putc(json, ']');
        break;
      }
      default: break;
    }
    slot += fd->count;
  }
}

static int is_whitespace(const char* p, size_t n) { /* output_json.cpp:128-131 */
  for (size_t i = 0; i < n; ++i)
    if (!isspace((unsigned char)p[i])) return 0;
  return 1;
}

#define SYNC_STREAM_TID_OFFSET 1000000 /* output_json.h: kSyncStreamTidOffset */
static int is_stream_sync(const ktj_oracle* o, const ktj_mat_activity* a) { /* :915, :1011 */
  if (a->type != KTJ_TYPE_CUDA_SYNC) return 0;
  const char* nm; uint64_t nl;
  ktj_oracle_string(o, a->name_id, &nm, &nl);
  return nl == 11 && memcmp(nm, "Stream Sync", 11) == 0;
}
/* handleGenericInstantEvent: output_json.cpp:660-677.  Name and metadata are printed as they are. */
static void handle_instant_event(ktj_oracle* o, const ktj_mat_activity* a) {
  sbuf args = {0}, meta = {0};
  render_metadata(o, a, &meta);
  if (meta.n && !is_whitespace(meta.p, meta.n)) sb_put(&args, meta.p, meta.n);
  const char* nm; uint64_t nl;
  ktj_oracle_string(o, a->name_id, &nm, &nl);
  char* name = (char*)malloc(nl + 1);
  if (!name) abort();
  memcpy(name, nm, nl);
  name[nl] = 0;
  char pid[24], tid[24];
  fmt_i64(a->device, pid);
  fmt_i64(sanitize_tid(a->resource), tid);
  write_instant_event(o, ktj_oracle_type_name(a->type), "t", name, pid, tid, rel_time(o, a->ts), &args, 0);
  free(name); free(args.p); free(meta.p);
}

/* writeCounterEvent: output_json.cpp:294-316.  The args object is printed even when empty. */
static void write_counter_event(ktj_oracle* o, const char* cat, const char* name, size_t name_n,
                                const char* pid, const char* tid, int64_t ts, const sbuf* args) {
  char t[40];
  ktj_oracle_fmt_ts(ts, t);
  sbuf* b = &o->out;
  sb_puts(b, "\n  {\n    \"ph\": \"C\",\n    \"cat\": \""); sb_puts(b, cat);
  sb_puts(b, "\",\n    \"name\": \""); sb_put(b, name, name_n);
  sb_puts(b, "\",\n    \"pid\": "); sb_puts(b, pid);
  sb_puts(b, ",\n    \"tid\": "); sb_puts(b, tid);
  sb_puts(b, ",\n    \"ts\": "); sb_puts(b, t);
  sb_puts(b, ",\n    \"args\": {\n      "); sb_put(b, args->p, args->n);
  sb_puts(b, "\n    }\n  },");
}

static int is_counter_type(int type) { /* output_json.cpp:847-856 */
  return type == KTJ_TYPE_HARDWARE_COUNTERS || type == KTJ_TYPE_MTIA_COUNTERS || type == KTJ_TYPE_XPU_SCOPE_PROFILER;
}
/* handleCounterEvent: output_json.cpp:679-716.  counterValues() of a record are the keyed
 * double fields of its schema, in schema order; its other fields are never printed.  Names are
 * printed as they are, values by fmt "{}" (non-finite ones bare). */
static void handle_counter_event(ktj_oracle* o, const ktj_mat_activity* a) {
  const int64_t ts = rel_time(o, a->ts);
  const char* cat = ktj_oracle_type_name(a->type);
  char pid[48], tid[24], n[48];
  fmt_i64(sanitize_tid(a->resource), tid);
  const int hw = a->type == KTJ_TYPE_HARDWARE_COUNTERS;
  if (hw) sprintf(pid, "\"GPU %lld Counters\"", (long long)a->device); /* :688 */
  else fmt_i64(a->device, pid);
  sbuf args = {0};
  const uint64_t* slot = a->slots;
  for (uint32_t f = 0; f < a->n_fields; slot += a->fields[f].count, ++f) {
    const ktj_field* fd = &a->fields[f];
    if (fd->type != KTJ_F_F64 || fd->key_id == KTJ_NONE) continue;
    const char* kp; uint64_t kl;
    ktj_oracle_string(o, fd->key_id, &kp, &kl);
    double d; memcpy(&d, &slot[0], 8);
    const size_t vn = ktj_oracle_fmt_double(d, n);
    if (hw) { /* one event per counter on the device's counter track: :687-701 */
      sbuf one = {0};
      sb_puts(&one, "\"\": "); sb_put(&one, n, vn);
      write_counter_event(o, cat, kp, kl, pid, tid, ts, &one);
      free(one.p);
    } else {  /* ArgsBuilder::addRaw :161-164 */
      if (args.n) sb_putc(&args, ',');
      sb_putc(&args, '"'); sb_put(&args, kp, kl); sb_puts(&args, "\": "); sb_put(&args, n, vn);
    }
  }
  if (!hw) {
    const char* nm; uint64_t nl;
    ktj_oracle_string(o, a->name_id, &nm, &nl);
    write_counter_event(o, cat, nm, nl, pid, tid, ts, &args);
  }
  free(args.p);
}

/* ---- collective metadata: output_json.cpp:718-835 ---- */
void ktj_oracle_string_map_order(const char* const* keys, uint64_t n, uint64_t* order); /* map_order.cpp */

static char* dup_value(const char* p) { return strdup(p ? p : ""); }
/* stripQuotes: output_json.cpp:57-63 */
static char* strip_quotes(const char* p) {
  if (!p) p = "";
  size_t n = strlen(p);
  if (n >= 2 && p[0] == '"' && p[n - 1] == '"') { p += 1; n -= 2; }
  char* r = (char*)malloc(n + 1);
  if (!r) abort();
  memcpy(r, p, n);
  r[n] = 0;
  return r;
}
static void args_add_raw(sbuf* args, const char* key, const char* value) { /* ArgsBuilder::addRaw :161-164 */
  if (args->n) sb_putc(args, ',');
  sb_putc(args, '"'); sb_puts(args, key); sb_puts(args, "\": "); sb_puts(args, value);
}
static void args_add_quoted(sbuf* args, const char* key, const char* value) { /* ArgsBuilder::addQuoted :167-170 */
  if (args->n) sb_putc(args, ',');
  sb_putc(args, '"'); sb_puts(args, key); sb_puts(args, "\": \""); sb_puts(args, value); sb_putc(args, '"');
}
/* appendCollectiveArgs: output_json.cpp:718-797 */
static void append_collective_args(sbuf* args, const ktj_collective_meta* m) {
  char* name = strip_quotes(m->collective_name);
  char* in_n = dup_value(m->in_msg_nelems);
  char* out_n = dup_value(m->out_msg_nelems);
  char* group = dup_value(m->group_size);
  char* dtype = strip_quotes(m->dtype);
  if (name[0] && in_n[0] && out_n[0] && group[0] && dtype[0]) {
    args_add_quoted(args, "Collective name", name);
    args_add_raw(args, "In msg nelems", in_n);
    args_add_raw(args, "Out msg nelems", out_n);
    args_add_raw(args, "Group size", group);
    args_add_quoted(args, "dtype", dtype);
  }
  char* in_start = strip_quotes(m->in_tensors_start);
  char* out_start = strip_quotes(m->out_tensors_start);
  if (in_start[0]) args_add_quoted(args, "Input Tensors start", in_start);
  if (out_start[0]) args_add_quoted(args, "Output Tensors start", out_start);
  char* in_split = strip_quotes(m->in_split);
  char* out_split = strip_quotes(m->out_split);
  if (in_split[0] && out_split[0]) {
    args_add_quoted(args, "In split size", in_split);
    args_add_quoted(args, "Out split size", out_split);
  }
  char* pg_name = strip_quotes(m->pg_name);
  if (pg_name[0]) args_add_quoted(args, "Process Group Name", pg_name);
  char* pg_desc = strip_quotes(m->pg_desc);
  if (pg_desc[0]) args_add_quoted(args, "Process Group Description", pg_desc);
  char* ranks = strip_quotes(m->group_ranks);
  if (ranks[0]) args_add_quoted(args, "Process Group Ranks", ranks);
  if (m->dst_rank && m->dst_rank[0]) args_add_raw(args, "Dst Rank", m->dst_rank);
  if (m->src_rank && m->src_rank[0]) args_add_raw(args, "Src Rank", m->src_rank);
  if (m->seq && m->seq[0]) args_add_raw(args, "Seq", m->seq);
  if (m->comms_id && m->comms_id[0]) args_add_raw(args, "Comms Id", m->comms_id);
  free(name); free(in_n); free(out_n); free(group); free(dtype); free(in_start); free(out_start);
  free(in_split); free(out_split); free(pg_name); free(pg_desc); free(ranks);
}
/* appendCollectiveMetadata: output_json.cpp:799-835 */
static void append_collective_metadata(ktj_oracle* o, sbuf* args, const ktj_collective_meta* m, const char* backend,
                                       const char* backend_config) {
  append_collective_args(args, m);
  char* pg_name = strip_quotes(m->pg_name);
  char* pg_desc = strip_quotes(m->pg_desc);
  if (!o->dist_backend && strcmp(pg_desc, "default_pg") == 0) { /* :807-817 */
    o->dist_backend = dup_value(backend);
    o->dist_rank = dup_value(m->rank);
    o->dist_world_size = dup_value(m->group_size);
    o->dist_nccl_version = dup_value(strcmp(backend, "nccl") == 0 ? "unknown" : "");
  }
  int known = 0; /* pgMap_.insert: the first entry of a name stays */
  for (uint64_t k = 0; k < o->n_pgs && !known; ++k) known = strcmp(o->pgs[k].name, pg_name) == 0;
  if (!known) {
    if (o->n_pgs == o->cap_pgs) {
      o->cap_pgs = o->cap_pgs ? o->cap_pgs * 2 : 8;
      o->pgs = (struct pg_entry*)realloc(o->pgs, o->cap_pgs * sizeof *o->pgs);
      if (!o->pgs) abort();
    }
    struct pg_entry* e = &o->pgs[o->n_pgs++];
    e->name = pg_name; pg_name = NULL;
    e->desc = pg_desc; pg_desc = NULL;
    e->backend_config = dup_value(backend_config);
    e->size = dup_value(m->group_size);
    e->ranks = strip_quotes(m->group_ranks);
  }
  free(pg_name); free(pg_desc);
}
/* addOnDemandDistMetadata: output_json.cpp:1030-1064 */
static void add_dist_metadata(ktj_oracle* o) {
  if (!o->dist_backend) return;
  sbuf* b = &o->out;
  char n[24];
  sb_puts(b, "\n  \"distributedInfo\": {\"backend\": \""); sb_puts(b, o->dist_backend);
  sb_puts(b, "\", \"rank\": "); sb_puts(b, o->dist_rank);
  sb_puts(b, ", \"world_size\": "); sb_puts(b, o->dist_world_size);
  sb_puts(b, ", \"pg_count\": "); sb_put(b, n, fmt_u64(o->n_pgs, n));
  sb_puts(b, ", \"pg_config\": [");
  const char** names = (const char**)malloc(sizeof(char*) * (o->n_pgs ? o->n_pgs : 1));
  uint64_t* order = (uint64_t*)malloc(8 * (o->n_pgs ? o->n_pgs : 1));
  if (!names || !order) abort();
  for (uint64_t k = 0; k < o->n_pgs; ++k) names[k] = o->pgs[k].name;
  ktj_oracle_string_map_order(names, o->n_pgs, order);
  for (uint64_t k = 0; k < o->n_pgs; ++k) {
    const struct pg_entry* e = &o->pgs[order[k]];
    if (k) sb_putc(b, ',');
    sb_puts(b, "{\"pg_name\": \""); sb_puts(b, e->name);
    sb_puts(b, "\", \"pg_desc\": \""); sb_puts(b, e->desc);
    sb_puts(b, "\", \"backend_config\": \""); sb_puts(b, e->backend_config);
    sb_puts(b, "\", \"pg_size\": "); sb_puts(b, e->size);
    sb_puts(b, ", \"ranks\": \""); sb_puts(b, e->ranks); sb_puts(b, "\"}");
  }
  sb_puts(b, "], \"nccl_version\": \""); sb_puts(b, o->dist_nccl_version); sb_puts(b, "\"},");
  free(names); free(order);
}

/* handleActivity + handleGenericLink + handleLink: output_json.cpp:837-1021. */
static void handle_activity(ktj_oracle* o, const ktj_mat_activity* a) {
  if (a->type == KTJ_TYPE_CPU_INSTANT_EVENT) { handle_instant_event(o, a); return; } /* :842-845 */
  if (is_counter_type(a->type)) { handle_counter_event(o, a); return; }               /* :847-856 */
  int64_t ts = a->ts;
  int64_t duration = a->dur < 0 ? 0 : a->dur;              /* :860 */
  if (a->type == KTJ_TYPE_GPU_USER_ANNOTATION) { ts -= 1; duration += 2; } /* :862-869 */
  int external_id = 0;                                      /* :871-891 */
  if (a->has_linked) external_id = (int)a->linked_corr;
  else {
    switch (a->type) {
      case KTJ_TYPE_GPU_MEMCPY: case KTJ_TYPE_GPU_MEMSET: case KTJ_TYPE_CONCURRENT_KERNEL:
      case KTJ_TYPE_CUDA_RUNTIME: case KTJ_TYPE_CUDA_DRIVER: case KTJ_TYPE_XPU_RUNTIME:
      case KTJ_TYPE_XPU_DRIVER: case KTJ_TYPE_PRIVATEUSE1_RUNTIME: case KTJ_TYPE_PRIVATEUSE1_DRIVER:
        break;
      default: external_id = (int)a->corr;
    }
  }
  sbuf args = {0};
  char n[48];
  if (external_id != 0) {                                   /* :892-895 */
    sb_puts(&args, "\"External id\": ");
    sb_put(&args, n, fmt_i64(external_id, n));
  }
  sbuf meta = {0};
  render_metadata(o, a, &meta);
  if (meta.n) meta.n = ktj_oracle_sanitize_str(meta.p, meta.n, meta.p); /* :896-897 */
  if (meta.n && !is_whitespace(meta.p, meta.n)) {           /* appendFragment :173-181 */
    if (args.n) sb_putc(&args, ',');
    sb_put(&args, meta.p, meta.n);
  }
  const char* nm; uint64_t nl;
  ktj_oracle_string(o, a->name_id, &nm, &nl);
  if (a->has_linked && a->collective) {                     /* :899-908: the linked op is a record_param_comms */
    const ktj_collective_meta* m = &o->s->collectives[a->collective - 1];
    if (a->type == KTJ_TYPE_CONCURRENT_KERNEL) append_collective_metadata(o, &args, m, "nccl", "cuda:nccl");
    else if (a->type == KTJ_TYPE_MTIA_CCP_EVENTS && nl >= 6 && memcmp(nm, "hccl::", 6) == 0)
      append_collective_metadata(o, &args, m, "hccl", "mtia:hccl");
  }
  char* name = (char*)malloc(nl * 2 + 8);
  if (!name) abort();
  size_t name_n = ktj_oracle_sanitize_name(nm, nl, name);   /* :946-949 */
  if (name_n == 7 && memcmp(name, "unknown", 7) == 0 && !(nl == 7 && memcmp(nm, "unknown", 7) == 0))
    o->n_blank++;
  char pid[24], tid[24];
  fmt_i64(a->device, pid);
  int64_t resource = a->resource;
  const int sync = is_stream_sync(o, a);
  if (sync) { /* :913-943: own row per stream, announced once per (device, row) */
    const int64_t sync_tid = (int64_t)((uint64_t)resource + SYNC_STREAM_TID_OFFSET); /* wraps like the logger's own sum */
    const int64_t key = (int64_t)(((uint64_t)a->device << 32) | (uint64_t)sync_tid);
    int seen = 0;
    for (uint64_t k = 0; k < o->n_sync_seen && !seen; ++k) seen = o->sync_seen[k] == key;
    if (!seen) {
      if (o->n_sync_seen == o->cap_sync_seen) {
        o->cap_sync_seen = o->cap_sync_seen ? o->cap_sync_seen * 2 : 64;
        o->sync_seen = (int64_t*)realloc(o->sync_seen, o->cap_sync_seen * 8);
        if (!o->sync_seen) abort();
      }
      o->sync_seen[o->n_sync_seen++] = key;
      char t[40], st[24], rs[24];
      ktj_oracle_fmt_ts(rel_time(o, ts), t);
      fmt_i64(sync_tid, st);
      fmt_i64(resource, rs);
      sbuf* b = &o->out;
      sb_puts(b, "\n  {\n    \"name\": \"thread_name\", \"ph\": \"M\", \"ts\": "); sb_puts(b, t);
      sb_puts(b, ", \"pid\": "); sb_puts(b, pid); sb_puts(b, ", \"tid\": "); sb_puts(b, st);
      sb_puts(b, ",\n    \"args\": {\n      \"name\": \"stream "); sb_puts(b, rs);
      sb_puts(b, " (sync)\"\n    }\n  },");
      sb_puts(b, "\n  {\n    \"name\": \"thread_sort_index\", \"ph\": \"M\", \"ts\": "); sb_puts(b, t);
      sb_puts(b, ", \"pid\": "); sb_puts(b, pid); sb_puts(b, ", \"tid\": "); sb_puts(b, st);
      sb_puts(b, ",\n    \"args\": {\n      \"sort_index\": "); sb_puts(b, rs);
      sb_puts(b, "\n    }\n  },");
    }
    resource = sync_tid;
  }
  fmt_i64(sanitize_tid(resource), tid);
  write_complete_event(o, ktj_oracle_type_name(a->type), name, name_n, pid, tid, rel_time(o, ts),
                       duration, &args);
  if (a->flow_id > 0) {                                     /* :960-962, 973-995 */
    const char* fname = a->flow_type == (int)KTJ_LINK_FWDBWD ? "fwdbwd"
                      : a->flow_type == (int)KTJ_LINK_ASYNC_CPU_GPU ? "ac2g" : NULL;
    if (fname) {
      write_flow_event(o, a->flow_start ? 's' : 'f', a->flow_id, a->device,
                       sanitize_tid(sync ? (int64_t)((uint64_t)a->resource + SYNC_STREAM_TID_OFFSET) : a->resource),
                       rel_time(o, a->ts), fname);          /* handleLink :997-1021 */
      o->n_flow++;
    }
  }
  free(name); free(args.p); free(meta.p);
}

/* finalizeTrace: output_json.cpp:1066-1108 (file handling is the caller's business) */
static void finalize_trace(ktj_oracle* o) {
  const ktj_stream* s = o->s;
  sbuf none = {0};
  write_instant_event(o, "", "g", "Record Window End", "\"\"", "\"\"", rel_time(o, s->end_time_ns), &none, 1);
  sb_puts(&o->out, "\n  ],");
  add_dist_metadata(o);                                     /* :1094-1096 */
  sb_puts(&o->out, "\"traceName\": \"");
  size_t n = strlen(s->trace_name);
  char* t = (char*)malloc(n + 1);
  if (!t) abort();
  size_t m = ktj_oracle_sanitize_str(s->trace_name, n, t); /* :1071 */
  sb_put(&o->out, t, m);
  free(t);
  sb_puts(&o->out, "\" }");
}

/* ------------------------------------------------------------------------------------------ */
ktj_oracle* ktj_oracle_run(const ktj_stream* s) {
  ktj_oracle* o = (ktj_oracle*)calloc(1, sizeof *o);
  if (!o) return NULL;
  o->s = s;
  o->builtin0 = (uint32_t)s->n_strings;
  for (int i = 0; i < BS_COUNT; ++i) add_xstring(o, kBuiltin[i], strlen(kBuiltin[i]));

  double t0 = now_s();
  stage_join(o);
  double t1 = now_s();
  o->order = (uint64_t*)malloc(8 * (o->n_acts ? o->n_acts : 1));
  uint64_t* tmp = (uint64_t*)malloc(8 * (o->n_acts ? o->n_acts : 1));
  if (!o->order || !tmp) abort();
  for (uint64_t i = 0; i < o->n_acts; ++i) o->order[i] = i;
  merge_sort(o->acts, o->order, tmp, o->n_acts);
  free(tmp);
  double t2 = now_s();

  /* emission order of the reference's buffering logger: libkineto/src/output_membuf.h:91-107 */
  handle_trace_start(o);
  for (uint64_t i = 0; i < s->n_device_infos; ++i) handle_device_info(o, &s->device_infos[i]);
  for (uint64_t i = 0; i < s->n_resource_infos; ++i) handle_resource_info(o, &s->resource_infos[i]);
  for (uint64_t i = 0; i < s->n_overhead_infos; ++i) handle_overhead_info(o, &s->overhead_infos[i]);
  for (uint64_t i = 0; i < o->n_acts; ++i) handle_activity(o, &o->acts[o->order[i]]);
  for (uint64_t i = 0; i < s->n_spans; ++i) handle_trace_span(o, &s->spans[i]);
  finalize_trace(o);
  double t3 = now_s();
  o->t_join = t1 - t0; o->t_sort = t2 - t1; o->t_emit = t3 - t2;
  return o;
}

void ktj_oracle_free(ktj_oracle* o) {
  if (!o) return;
  free(o->xblob.p); free(o->xoff); free(o->acts); free(o->order); free(o->fpool); free(o->spool);
  free(o->act_f0); free(o->act_s0); free(o->out.p); free(o->sync_seen);
  free(o->dist_backend); free(o->dist_rank); free(o->dist_world_size); free(o->dist_nccl_version);
  for (uint64_t k = 0; k < o->n_pgs; ++k) {
    free(o->pgs[k].name); free(o->pgs[k].desc); free(o->pgs[k].backend_config); free(o->pgs[k].size); free(o->pgs[k].ranks);
  }
  free(o->pgs);
  free(o);
}
void ktj_oracle_output(const ktj_oracle* o, const char** bytes, uint64_t* n) { *bytes = o->out.p; *n = o->out.n; }
void ktj_oracle_activities(const ktj_oracle* o, const ktj_mat_activity** acts, uint64_t* n) { *acts = o->acts; *n = o->n_acts; }
void ktj_oracle_order(const ktj_oracle* o, const uint64_t** order, uint64_t* n) { *order = o->order; *n = o->n_acts; }
void ktj_oracle_counters(const ktj_oracle* o, uint64_t* out_of_range, uint64_t* out_of_order,
                         uint64_t* n_flow_events, uint64_t* n_linked, uint64_t* n_blank_names) {
  if (out_of_range) *out_of_range = o->out_of_range;
  if (out_of_order) *out_of_order = o->out_of_order;
  if (n_flow_events) *n_flow_events = o->n_flow;
  if (n_linked) *n_linked = o->n_linked;
  if (n_blank_names) *n_blank_names = o->n_blank;
}
void ktj_oracle_timings(const ktj_oracle* o, double* secs3) {
  secs3[0] = o->t_join; secs3[1] = o->t_sort; secs3[2] = o->t_emit;
}
