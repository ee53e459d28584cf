/*
 * ktj_stream.h — one complete input of the engine as a plain bundle of pointers: what a caller
 * would pass through the ktj_* calls of ktj.h, gathered in one struct so that the synthetic
 * generator, the engine's test glue and the CPU checker all consume the same bytes.
 */
#ifndef KTJ_STREAM_H_
#define KTJ_STREAM_H_

#include "ktj.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ktj_schema_desc {
  uint32_t first_field; /* index into ktj_stream::fields */
  uint32_t n_fields;
} ktj_schema_desc;

typedef struct ktj_stream {
  /* header */
  int64_t base_time_ns;
  const char* trace_name;         /* file name printed as "traceName"                          */
  const char* device_properties;  /* verbatim inside "deviceProperties": [...]                  */
  const char* const* meta_kv;     /* 2*n_meta pointers, emission order                          */
  uint64_t n_meta;

  /* string dictionary */
  const char* str_blob;
  const uint64_t* str_off;        /* n_strings + 1                                              */
  uint64_t n_strings;

  /* args schemas + blob */
  const ktj_field* fields;
  uint64_t n_fields;
  const ktj_schema_desc* schemas;
  uint64_t n_schemas;
  const uint64_t* args;           /* 8-byte slots                                               */
  uint64_t n_args;

  /* runtime API table */
  const uint32_t* cid_name_ids;
  uint64_t n_cids;
  const uint32_t* flow_start_cids;
  uint64_t n_flow_start;
  uint32_t malloc_cid;            /* the cid of hipMalloc (its rows carry a "bytes" arg)         */
  uint32_t create_flags;          /* the ktj_create flags that change the document
                                     (KTJ_CREATE_CUDA12_ARGS); the engine takes them at ktj_create */

  /* clock + window */
  ktj_clock_model clock;
  int64_t window_start_ns;
  int64_t window_end_ns;
  int64_t end_time_ns;            /* finalizeTrace endTime                                      */

  /* records, arrival order within each class */
  const ktj_generic_rec* generic;
  uint64_t n_generic;
  const ktj_runtime_rec* runtime;
  uint64_t n_runtime;
  const ktj_device_rec* device;
  uint64_t n_device;
  const ktj_extcorr_rec* extcorr;
  uint64_t n_extcorr;

  /* small events, in the order the reference's memory logger replays them
   * (libkineto/src/output_membuf.h:91-107): device infos, resource infos, [activities], spans */
  const ktj_device_info* device_infos;
  uint64_t n_device_infos;
  const ktj_resource_info* resource_infos;
  uint64_t n_resource_infos;
  const ktj_overhead_info* overhead_infos;
  uint64_t n_overhead_infos;
  const ktj_trace_span* spans;
  uint64_t n_spans;

  /* collective metadata, indexed by the slots of KTJ_F_COLLECTIVE fields */
  const ktj_collective_meta* collectives;
  uint64_t n_collectives;

  /* external correlation of the user domain (KTJ_REC_USERCORR), arrival order */
  const ktj_extcorr_rec* usercorr;
  uint64_t n_usercorr;
} ktj_stream;

/* ------------------------------------------------------------------------------------------
 * Synthetic streams (libktj_synth): the five benchmark configurations, generated with integer
 * arithmetic only from a counter-based RNG so that the same bytes come out on every machine.
 * ---------------------------------------------------------------------------------------- */
typedef struct ktj_synth_params {
  uint32_t config;        /* 1..5                                                              */
  uint32_t pad;
  uint64_t n_device;      /* number of device records (0 = the configuration's full size);
                             every other count scales with it                                   */
  int64_t base_time_ns;   /* all wall-clock timestamps are base_time_ns + offset                */
  const char* host_name;  /* "host_name" header metadata; NULL = none                           */
  const char* trace_name; /* NULL = "synthetic.json"                                            */
} ktj_synth_params;

/* Returns NULL on allocation failure or bad parameters.  The stream owns all memory it points
 * to; release with ktj_synth_free. */
ktj_stream* ktj_synth_generate(const ktj_synth_params* params);
void ktj_synth_free(ktj_stream* s);

#ifdef __cplusplus
}
#endif
#endif /* KTJ_STREAM_H_ */
