/*
 * ktj_device.h — data layouts shared by the HIP kernels and the host side of the engine.
 */
#ifndef KTJ_DEVICE_H_
#define KTJ_DEVICE_H_

#include <stdint.h>

#include "../../include/ktj_stream.h"

#if defined(__HIPCC__)
#define KTJ_HD __host__ __device__
#else
#define KTJ_HD
#endif

/* One joined activity, self-contained for formatting (except generic args, which stay in the
 * args blob).  96 bytes = 6 x 16. */
struct MatRow {
  int64_t ts;        /* timestamp(): absolute ns                                                */
  int64_t dur;       /* duration(), unclamped                                                   */
  int64_t dev;       /* deviceId()                                                              */
  int64_t res;       /* resourceId()                                                            */
  int64_t flow_id;   /* flowId()                                                                */
  uint32_t name_id;  /* dictionary id, or a KTJ_NAME_* code when KTJ_M_NAME_BUILTIN              */
  uint32_t meta;     /* KTJ_M_* bit fields                                                      */
  int32_t ext;       /* "External id" value, 0 = none                                           */
  uint32_t aux;      /* generic: schema id; runtime: cid; device: op                            */
  uint64_t p[5];     /* payload, see below                                                      */
};
/* payload by class:
 *   generic          p0 = args_off, p1 = 1 + index of the collective metadata the row prints (0 = none)
 *   runtime KERNEL   p0 = grid0 | grid1<<32, p1 = grid2 | wg0<<32, p2 = wg1 | wg2<<32, p3 = group
 *                    segment size, p4 = kernel_name_id
 *   runtime COPY     p0 = src, p1 = dst, p2 = size, p3 = copy_kind
 *   runtime MALLOC   p0 = ptr, p1 = size
 *   device kernel    p0..p2 = grid/block of the launching row (if KTJ_M_HAS_GRID), p3 = queue,
 *                    p4 = 1 + index of the collective metadata of the linked CPU op (0 = none)
 *   device copy      p0 = bytes of the launching row (if KTJ_M_HAS_SIZE), p3 = queue
 *   device memset    p0 = bytes, p1 = graph node id, p2 = graph id | channel id<<32, p3 = context id;
 *                    aux = channel type | memory kind<<8
 */

#define KTJ_M_TYPE_MASK 0x1Fu
#define KTJ_M_CLASS_SHIFT 5
#define KTJ_M_CLASS_MASK (3u << KTJ_M_CLASS_SHIFT)
#define KTJ_M_KIND_SHIFT 7
#define KTJ_M_KIND_MASK (3u << KTJ_M_KIND_SHIFT)
#define KTJ_M_VALID (1u << 9)
#define KTJ_M_FLOW (1u << 10)
#define KTJ_M_FLOW_START (1u << 11)
#define KTJ_M_FLOW_FWDBWD (1u << 12)
#define KTJ_M_HAS_GRID (1u << 13)
#define KTJ_M_HAS_SIZE (1u << 14)
#define KTJ_M_HAS_KERNEL_ARG (1u << 15)
#define KTJ_M_MALLOC_BYTES (1u << 16)
#define KTJ_M_NAME_BUILTIN (1u << 17)
#define KTJ_M_HAS_STREAM (1u << 18) /* meta column of runtime rows only: the row carries a stream */
#define KTJ_M_SYNC (1u << 19)       /* CUDA_SYNC activity named "Stream Sync": own row at tid + 1000000 */
#define KTJ_M_SYNC_FIRST (1u << 20) /* first such activity of its (device, row) in emission order  */

#define KTJ_CLASS_GENERIC 0u
#define KTJ_CLASS_RUNTIME 1u
#define KTJ_CLASS_DEVICE 2u

/* built-in names */
#define KTJ_NAME_MEMCPY_UNKNOWN 0u /* "Memcpy <unknown> (? -> ?)"; 1..4 = KTJ_COPY_* directions */
#define KTJ_NAME_MEMSET 5u
#define KTJ_NAME_UNKNOWN_OP 6u     /* "<unknown operation:N>", N = aux */
#define KTJ_NAME_EMPTY 7u

/* string dictionary as the kernels see it */
struct DictViews {
  const char* name_blob;     /* names after the logger's name pipeline                         */
  const uint64_t* name_off;  /* n + 1                                                          */
  const char* arg_blob;      /* strings after sanitizeStrForJSON                               */
  const uint64_t* arg_off;   /* n + 1                                                          */
  const char* raw_blob;      /* strings as interned (instant events print them untouched)      */
  const uint64_t* raw_off;   /* n + 1                                                          */
  const uint32_t* flags;     /* KTJ_SF_*                                                       */
  uint32_t n;
};
#define KTJ_SF_ARG_BLANK 1u  /* arg view is empty or whitespace only                           */
#define KTJ_SF_NAME_UNKNOWN 2u /* name view was replaced by "unknown"                          */
#define KTJ_SF_NAME_KERNEL 4u  /* the string is "kernel" (printed as "Kernel")                  */
#define KTJ_SF_STREAM_SYNC 8u  /* the string is "Stream Sync"                                    */
#define KTJ_SYNC_TID_OFFSET 1000000 /* libkineto/src/output_json.h: kSyncStreamTidOffset          */

/* everything format_activity needs besides the row itself */
struct EmitCtx {
  DictViews dict;
  const ktj_field* fields;          /* all schemas' fields                                     */
  const ktj_schema_desc* schemas;
  uint32_t n_schemas;
  const uint64_t* args;             /* 8-byte slots                                            */
  uint64_t n_args;
  int64_t base_time_ns;
  const char* coll_blob;            /* collective arguments of each ktj_add_collective entry   */
  const uint64_t* coll_off;         /* n_coll + 1                                              */
  uint32_t n_coll;
  uint32_t create_flags;            /* ktj_create flags that change the text (KTJ_CREATE_CUDA12_ARGS) */
};

#endif
