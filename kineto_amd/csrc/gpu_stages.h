/*
 * gpu_stages.h — launch interface between the host side of the engine (engine.cpp) and the HIP
 * kernels (kernels.hip).  Every function only enqueues work on the given stream and returns the
 * HIP status of the launch; none of them synchronises or allocates.
 */
#ifndef KTJ_GPU_STAGES_H_
#define KTJ_GPU_STAGES_H_

#include <hip/hip_runtime_api.h>

#include "mat_core.h"

namespace ktj {
namespace gpu {

/* open-addressing hash table in device memory; keys hold KTJ_EMPTY_KEY when free.  Slot `cap` (one
 * past the power-of-two range) is reserved for the key whose value equals KTJ_EMPTY_KEY. */
#define KTJ_EMPTY_KEY 0xFFFFFFFFFFFFFFFFULL
struct Table {
  uint64_t* keys;
  uint32_t* v0;
  uint32_t* v1;
  uint32_t mask; /* cap - 1 */
};

/* columns in arrival order: generic rows, then runtime rows, then device rows */
struct Columns {
  int64_t* ts;    /* raw begin, after convert: timestamp()          */
  int64_t* dur;   /* raw end, after convert: duration()             */
  uint64_t* corr; /* correlation id                                  */
  int64_t* dev;   /* deviceId()                                      */
  int64_t* res;   /* resourceId(); device rows: stream before and after back-fill */
  uint32_t* meta; /* KTJ_M_VALID | class                              */
  int32_t* ext;   /* "External id" value                              */
};

/* small block of scalars the kernels update and the host reads back */
struct Scalars {
  unsigned long long ts_min_biased;   /* min over valid rows of ts ^ 2^63 */
  unsigned long long ts_max_biased;
  unsigned long long out_of_range;
  unsigned long long out_of_order;
  unsigned long long n_flow;
  unsigned long long n_linked;
  unsigned long long n_blank_names;
  unsigned long long n_valid;
  unsigned int error;                 /* KTJ_DEVERR_* bits */
  unsigned int have_stream_src;       /* some runtime row carries a stream */
  unsigned int n_dev_ranks;           /* distinct deviceId values */
  unsigned int n_res_ranks;           /* distinct resourceId values */
  unsigned int n_dense;               /* distinct (device, stream key) pairs */
  unsigned int pad;
};
#define KTJ_DEVERR_TABLE_FULL 1u
#define KTJ_DEVERR_TOO_MANY_DISTINCT 2u
#define KTJ_DEVERR_HASH_COLLISION 4u
#define KTJ_DEVERR_RECORD_TOO_LONG 8u

#define KTJ_SET_CAP 16384u     /* slots of the distinct-value sets (at most half may be used) */
#define KTJ_DENSE_CAP 8192u    /* slots of the (device, stream) table */
#define KTJ_QUEUE_CAP 65536u   /* slots of the queue -> stream table */

struct ApiTable {
  const uint32_t* cid_name_ids;
  uint32_t n_cids;
  const uint32_t* flow_start_bits; /* bitmap over cids */
  uint32_t malloc_cid;
};

/* ---- utilities ---- */
hipError_t fill_u64(uint64_t* p, uint64_t v, uint64_t n, hipStream_t st);
hipError_t fill_u32(uint32_t* p, uint32_t v, uint64_t n, hipStream_t st);
hipError_t init_scalars(Scalars* s, hipStream_t st);
hipError_t copy_reference(const void* src, void* dst, uint64_t bytes, hipStream_t st);

/* exclusive scans; tmp must hold scan_tmp_elems(n) uint64 values */
uint64_t scan_tmp_elems(uint64_t n);
hipError_t scan_u32_to_u64(const uint32_t* in, uint64_t* out /* n+1 */, uint64_t n, uint64_t* tmp, hipStream_t st);
hipError_t scan_u32_inplace(uint32_t* data, uint64_t n, uint64_t* tmp, hipStream_t st);

/* ---- stage 0: dictionary ---- */
hipError_t dict_measure(const char* blob, const uint64_t* off, uint32_t n, uint32_t* name_len, uint32_t* arg_len,
                        uint32_t* flags, hipStream_t st);
hipError_t dict_write(const char* blob, const uint64_t* off, uint32_t n, const uint64_t* name_off,
                      const uint64_t* arg_off, const uint32_t* flags, char* name_blob, char* arg_blob, hipStream_t st);

/* ---- stage 1: decode ---- */
hipError_t decode_generic(const ktj_generic_rec* r, uint64_t n, Columns c, uint64_t first, hipStream_t st);
hipError_t decode_runtime(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first, hipStream_t st);
hipError_t decode_device(const ktj_device_rec* r, uint64_t n, Columns c, uint64_t first, hipStream_t st);

/* ---- stage 2a: clock conversion + window filter (runtime and device rows) ---- */
hipError_t convert_rows(Columns c, uint64_t first_runtime, uint64_t n_runtime, uint64_t n_device, ClockDev clk,
                        int64_t win_start, int64_t win_end, Scalars* sc, hipStream_t st);

/* ---- stage 2b: joins ---- */
hipError_t build_extcorr(const ktj_extcorr_rec* e, uint64_t n, Table t, Scalars* sc, hipStream_t st);
hipError_t build_cpu_ids(const ktj_generic_rec* g, uint64_t n, Table t, Scalars* sc, hipStream_t st);
hipError_t build_runtime(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first_runtime, Table by_id,
                         Table by_narrow, Scalars* sc, hipStream_t st);
hipError_t insert_device_first(const ktj_device_rec* d, uint64_t n, Columns c, uint64_t first_device, Table by_id,
                               Scalars* sc, hipStream_t st);
hipError_t probe_external(Columns c, uint64_t first, uint64_t n, const ktj_extcorr_rec* e, Table ext, Table cpu,
                          Scalars* sc, hipStream_t st);
hipError_t count_out_of_order(Columns c, uint64_t first_runtime, uint64_t n_runtime, uint64_t n_device, Table by_id,
                              Scalars* sc, hipStream_t st);
/* stream back-fill: queue table (keys/vals/ambiguous) and dense table are caller-provided, zeroed */
struct StreamTables {
  uint64_t* q_keys;   /* KTJ_QUEUE_CAP + 1, filled with KTJ_EMPTY_KEY */
  uint64_t* q_stream; /* 0 = unset */
  uint32_t* q_amb;
  uint64_t* d_hash;   /* KTJ_DENSE_CAP + 1, filled with KTJ_EMPTY_KEY */
  uint32_t* d_first;  /* min arrival index, filled with 0xFFFFFFFF */
  int32_t* d_dev;
  uint64_t* d_key;
  uint32_t* d_rank;
};
hipError_t backfill_streams(const ktj_device_rec* d, uint64_t n, const ktj_runtime_rec* r, Columns c,
                            uint64_t first_device, Table by_id, StreamTables t, Scalars* sc, hipStream_t st);

/* ---- stage 3: canonical order ---- */
struct SortSets {
  uint64_t* dev_keys;  /* KTJ_SET_CAP + 1, KTJ_EMPTY_KEY filled */
  uint32_t* dev_rank;
  uint64_t* res_keys;
  uint32_t* res_rank;
};
hipError_t collect_distinct(Columns c, uint64_t n, SortSets s, Scalars* sc, hipStream_t st);
hipError_t rank_distinct(SortSets s, Scalars* sc, hipStream_t st);
/* key = ((rank(dev) << res_bits | rank(res)) << ts_bits) | (ts - ts_min); dropped rows get 1 << key_bits */
hipError_t make_keys(Columns c, uint64_t n, SortSets s, const Scalars* sc, uint32_t ts_bits, uint32_t res_bits,
                     uint32_t key_bits, uint64_t* keys, uint32_t* vals, hipStream_t st);
/* stable LSD radix sort of (key, val) pairs on the low `bits` bits; result ends in keys_out/vals_out
 * pointers returned through *res_keys / *res_vals (one of the two buffer pairs) */
uint64_t radix_tmp_elems(uint64_t n);
hipError_t radix_sort(uint64_t* keys_a, uint32_t* vals_a, uint64_t* keys_b, uint32_t* vals_b, uint64_t n,
                      uint32_t bits, uint32_t* hist /* radix_tmp_elems(n) */, uint64_t* scan_tmp,
                      uint64_t** res_keys, uint32_t** res_vals, hipStream_t st);

/* ---- stage 4a: joined rows + exact byte length (arrival order) ---- */
hipError_t mat_generic_rows(const ktj_generic_rec* g, uint64_t n, EmitCtx ctx, MatRow* mat, uint32_t* len,
                            Scalars* sc, hipStream_t st);
hipError_t mat_runtime_rows(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first, ApiTable api,
                            EmitCtx ctx, MatRow* mat, uint32_t* len, Scalars* sc, hipStream_t st);
hipError_t mat_device_rows(const ktj_device_rec* d, uint64_t n, Columns c, uint64_t first,
                           const ktj_runtime_rec* r, Table by_narrow, EmitCtx ctx, MatRow* mat, uint32_t* len,
                           Scalars* sc, hipStream_t st);
hipError_t gather_len(const uint32_t* perm, const uint32_t* len, uint64_t n, uint32_t* len_sorted, hipStream_t st);

/* ---- stage 4b: emit ---- */
/* tile size (bytes of output per workgroup) for a document whose activity section has act_bytes
 * bytes in n_rows activities, and the number of tiles / entries of tile_start (tiles + 1) */
uint32_t emit_tile_bytes(uint64_t act_bytes, uint64_t n_rows);
uint64_t emit_tile_count(uint64_t prefix_len, uint64_t act_bytes, uint32_t tile);
hipError_t emit(const MatRow* mat, const uint32_t* perm, const uint64_t* offs /* n+1 */, uint64_t n,
                EmitCtx ctx, char* out, uint64_t prefix_len, uint64_t act_bytes, uint32_t tile,
                uint32_t* tile_start /* tiles + 1 */, hipStream_t st);

/* direct variant: one lane per activity, no LDS staging; len_kind is the arrival-order length
 * array whose top two bits carry the tail kind; n_rows = number of activities that are written */
hipError_t emit_direct(const MatRow* mat, const uint32_t* perm, const uint64_t* offs, const uint32_t* len_kind,
                       uint64_t n_rows, EmitCtx ctx, char* out, uint64_t prefix_len, hipStream_t st);

}  // namespace gpu
}  // namespace ktj
#endif
