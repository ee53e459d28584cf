/*
 * ktj_debug.h — read-back of the engine's intermediate device arrays, for stage-level tests.
 * Not part of the drop-in surface; no counterpart in the reference.
 */
#ifndef KTJ_DEBUG_H_
#define KTJ_DEBUG_H_

#include "ktj.h"

#ifdef __cplusplus
extern "C" {
#endif

enum {
  KTJ_DBG_COL_TS = 0,     /* int64[N]  timestamp() per arrival index            */
  KTJ_DBG_COL_DUR = 1,    /* int64[N]  duration()                               */
  KTJ_DBG_COL_DEV = 2,    /* int64[N]                                           */
  KTJ_DBG_COL_RES = 3,    /* int64[N]  resourceId() after stream back-fill      */
  KTJ_DBG_COL_META = 4,   /* uint32[N] bit 9 = inside the capture window        */
  KTJ_DBG_COL_EXT = 5,    /* int32[N]  "External id" of runtime/device rows     */
  KTJ_DBG_PERM = 6,       /* uint32[N] arrival index per sorted position        */
  KTJ_DBG_LEN = 7,        /* uint32[N] byte length per sorted position          */
  KTJ_DBG_OFFS = 8,       /* uint64[N+1] exclusive scan of the lengths          */
  KTJ_DBG_MAT = 9,        /* 96-byte joined rows per arrival index              */
  KTJ_DBG_SORT_KEYS = 10, /* uint64[N] sorted composite keys (engines created with
                             KTJ_CREATE_PAIR_SORT only: KTJ_ERR_STATE otherwise)  */
  KTJ_DBG_NAME_VIEW = 11, /* bytes: all names after the name pipeline           */
  KTJ_DBG_NAME_OFF = 12,  /* uint64[n_strings+1]                                */
  KTJ_DBG_ARG_VIEW = 13,
  KTJ_DBG_ARG_OFF = 14
};

/* Copies the array to dst (at most cap bytes) and reports its full size.  Valid after
 * ktj_process. */
int ktj_debug_fetch(ktj_engine* e, int what, void* dst, uint64_t cap, uint64_t* n_bytes);

/* Runs a plain device-to-device copy kernel of n_bytes (16 bytes per lane) twice and reports the
 * second run's time: the achievable-bandwidth yardstick and the scale for the HBM counters. */
int ktj_debug_copy_reference(ktj_engine* e, uint64_t n_bytes, float* ms);

/* on != 0: a trace of one sort tile (up to 4096 rows) is sorted by the launches of a large trace
 * (keys, then one scatter per pass) instead of by the one launch that does it all; for the tests
 * that run small cases through both.  Process-wide. */
void ktj_debug_force_sort_passes(int on);

#ifdef __cplusplus
}
#endif
#endif
