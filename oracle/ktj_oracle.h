/*
 * ktj_oracle.h — CPU restatement of the reference's records → Chrome-trace JSON path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (kineto_amd/, libktj.so) may include, link
 * or call this.  It exists so that tests, the smoke check and the benchmark's CPU-baseline leg
 * can compare the HIP engine's bytes with an independent single-threaded implementation that
 * follows the reference's structure: one materialised activity per record, string temporaries,
 * one formatted write per event.
 */
#ifndef KTJ_ORACLE_H_
#define KTJ_ORACLE_H_

#include "../include/ktj_stream.h"

#ifdef __cplusplus
extern "C" {
#endif

/* One activity as the reference's ITraceActivity accessors would report it
 * (libkineto/include/ITraceActivity.h:24-76) after the profiler's join stage. */
typedef struct ktj_mat_activity {
  int64_t ts;           /* timestamp()                                                         */
  int64_t dur;          /* duration() (may be negative)                                        */
  int64_t device;       /* deviceId()                                                          */
  int64_t resource;     /* resourceId()                                                        */
  int64_t corr;         /* correlationId()                                                     */
  int64_t flow_id;      /* flowId()                                                            */
  int64_t linked_corr;  /* linkedActivity()->correlationId() if has_linked                     */
  uint64_t arrival;     /* arrival index (generic, then runtime, then device rows)             */
  const uint64_t* slots;   /* typed metadata values in visit order                             */
  const ktj_field* fields; /* typed metadata fields in visit order                             */
  uint32_t n_fields;
  uint32_t name_id;     /* id in the oracle's string table (ktj_oracle_string)                 */
  int32_t type;         /* KTJ_TYPE_*                                                          */
  int32_t flow_type;    /* flowType()                                                          */
  int32_t flow_start;   /* flowStart()                                                         */
  int32_t has_linked;
  uint32_t collective;  /* 1 + index (ktj_stream::collectives) of the metadata of the linked
                           record_param_comms op, 0 = the linked op is no such op                */
  uint32_t pad;
} ktj_mat_activity;

typedef struct ktj_oracle ktj_oracle;

/* Runs the whole path.  Returns NULL on allocation failure. */
ktj_oracle* ktj_oracle_run(const ktj_stream* s);
void ktj_oracle_free(ktj_oracle* o);

/* The finished JSON document. */
void ktj_oracle_output(const ktj_oracle* o, const char** bytes, uint64_t* n);
/* Activities after join + window filter, in arrival order (before the canonical sort). */
void ktj_oracle_activities(const ktj_oracle* o, const ktj_mat_activity** acts, uint64_t* n);
/* Order in which activities are emitted: indices into the array above. */
void ktj_oracle_order(const ktj_oracle* o, const uint64_t** order, uint64_t* n);
/* String table = the stream's dictionary followed by strings the join stage created. */
void ktj_oracle_string(const ktj_oracle* o, uint32_t id, const char** p, uint64_t* n);
uint64_t ktj_oracle_n_strings(const ktj_oracle* o);
/* Error counters of the post-processing stage. */
void ktj_oracle_counters(const ktj_oracle* o, uint64_t* out_of_range, uint64_t* out_of_order,
                         uint64_t* n_flow_events, uint64_t* n_linked, uint64_t* n_blank_names);
/* Seconds spent in: [0] join+materialise, [1] sort, [2] emit. */
void ktj_oracle_timings(const ktj_oracle* o, double* secs3);

/* Leaf functions, exposed for known-answer tests. */
size_t ktj_oracle_fmt_double(double v, char* out /* >= 40 bytes */);
size_t ktj_oracle_fmt_ts(int64_t ns, char* out /* >= 32 bytes */);
int64_t ktj_oracle_convert_ts(const ktj_clock_model* m, uint64_t t);
/* name pipeline of ChromeTraceLogger::handleActivity; out needs 2*n+8 bytes */
size_t ktj_oracle_sanitize_name(const char* in, size_t n, char* out);
/* sanitizeStrForJSON only; out needs n bytes */
size_t ktj_oracle_sanitize_str(const char* in, size_t n, char* out);
const char* ktj_oracle_type_name(int type);

#ifdef __cplusplus
}
#endif
#endif
