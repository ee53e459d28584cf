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

/* Join tables in device memory.  A table maps a 64-bit key to a slot index; what is stored per
 * slot lives in separate arrays indexed by it: compact 4-byte arrays for the "winner" indices that
 * are updated with atomics (atomics on neighbouring addresses coalesce; on 48-byte strides they
 * were measured 20 times slower), and payload arrays that the winners fill with plain stores.
 * A table is either direct-addressed (slot = key - base, chosen on the GPU when the keys that
 * will be inserted span less than the capacity: correlation ids are dense counters in practice,
 * so rows that arrive in id order touch consecutive slots and nothing is probed) or an
 * open-addressing hash table over `keys` (any other key set).  A hash slot is free while its key
 * is KTJ_EMPTY_KEY; slot `cap` (one past the power-of-two range) is reserved for the key whose
 * value equals KTJ_EMPTY_KEY.  The mode lives in device memory (TableCtl) so that no host round
 * trip is needed to choose it.  In direct mode a table with keyed_direct == 0 does not touch
 * `keys` at all: an id inside the range that was never inserted simply has empty per-slot
 * values. */
#define KTJ_EMPTY_KEY 0xFFFFFFFFFFFFFFFFULL
struct KeyRange {          /* over the keys that will be inserted; empty while lo > hi */
  unsigned long long lo, hi;
};
struct TableCtl {
  uint64_t base;           /* direct mode: smallest key */
  uint64_t span;           /* direct mode: largest key - base */
  uint32_t direct;
  uint32_t pad;
};
struct Table {
  uint64_t* keys;          /* cap + 1 */
  uint32_t mask;           /* cap - 1, cap a power of two >= 16 */
  uint32_t keyed_direct;   /* 1: a plain set, membership is told by the stored key in both modes */
  const TableCtl* ctl;
};
/* per slot of the table keyed by the full correlation id */
struct FullPay {           /* published by the winning runtime row, read by device rows */
  int64_t first_ts;        /* timestamp of the first runtime row with this id                   */
  uint64_t stream;         /* stream of row stream_src[slot]; 0 = no row carries one            */
};                         /* 16 bytes */
struct FullCols {
  uint32_t* has_runtime;   /* one bit per slot: some runtime row has this id.  Runtime rows arrive
                              before device rows, so where the bit is set the first row of the id is
                              a runtime row and its timestamp is in the payload; the bitmap is small
                              enough to stay in cache, unlike the array of first rows              */
  uint32_t* first;         /* smallest arrival index seen with this id, 0xFFFFFFFF = none (atomicMin);
                              filled for runtime rows only where they share ids, and for device rows
                              whose id no runtime row has                                          */
  uint32_t* stream_src;    /* last runtime row (index + 1) that carries a stream (atomicMax)    */
  FullPay* pay;
};
/* per slot of the table keyed by the int-narrowed correlation id (and by the external-correlation
 * records' full id) */
struct NarrowPay {         /* two writers (external-correlation records, runtime rows), in different passes */
  int32_t ext_val;         /* external id if a CPU op with that id exists, else 0               */
  uint32_t info;           /* bits 0-1: KTJ_DL_HAS_SIZE / KTJ_DL_HAS_GRID, what pay[] holds;
                              bit 2: ext_val names an existing CPU op; bits 3-31: 1 + index of the
                              collective metadata of the linked CPU op, 0 = none                  */
  uint64_t pay[3];         /* bytes of the winning copy / malloc row in pay[0], or packed grid /
                              workgroup of the winning kernel-launch row (see pack_grid)        */
};                         /* 32 bytes: a slot never straddles a line */
#define KTJ_NP_KIND_MASK 3u
#define KTJ_NP_LINKED 4u
#define KTJ_NP_COLL_SHIFT 3
#define KTJ_MAX_COLLECTIVES ((1u << 29) - 2u)
struct NarrowCols {
  uint32_t* ext_src;       /* last external-correlation record (index + 1), 0 = none            */
  uint32_t* kern_src;      /* last in-window kernel-launch row (index + 1)                     */
  uint32_t* copy_src;      /* last in-window copy / malloc row (index + 1)                     */
  NarrowPay* pay;
};
#define KTJ_TBL_FULL 0
#define KTJ_TBL_NARROW 1
#define KTJ_TBL_CPU 2
struct JoinPlan {
  KeyRange range[3];
  TableCtl ctl[3];
};
/* what a device row takes over from the runtime row(s) with its correlation id */
struct DevLink {
  uint64_t p[3];           /* size in p[0], or packed grid / workgroup */
  uint32_t flags;          /* KTJ_DL_* */
  uint32_t coll;           /* 1 + index of the collective metadata of the linked CPU op (kernels) */
};                         /* 32 bytes */
/* the fields of a device row that the stream back-fill passes read */
struct DevBrief {
  uint64_t queue;
  int32_t device;
  uint32_t domain;
};                         /* 16 bytes */
#define KTJ_DL_HAS_SIZE 1u
#define KTJ_DL_HAS_GRID 2u
#define KTJ_DL_ORPHAN 4u   /* no runtime row has the id: the order check runs in a pass of its own */

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
#ifndef KTJ_COUNTER_SHARDS
#define KTJ_COUNTER_SHARDS 64u
#endif
struct Scalars {
  unsigned long long ts_min_biased;   /* min over valid rows of ts ^ 2^63 */
  unsigned long long ts_max_biased;
  unsigned long long out_of_range;
  unsigned long long out_of_order;
  unsigned long long n_flow;
  unsigned long long n_linked;
  unsigned long long n_blank_names;
  unsigned long long n_valid;
  unsigned long long n_unresolved;    /* device rows still without a stream after the correlation pass */
  unsigned long long n_sync_typed;    /* generic rows of type CUDA_SYNC */
  unsigned long long n_device_orphans; /* in-window device rows whose id no runtime row has */
  unsigned int error;                 /* KTJ_DEVERR_* bits */
  unsigned int have_stream_src;       /* some runtime row carries a stream */
  unsigned int n_dev_ranks;           /* distinct deviceId values */
  unsigned int n_res_ranks;           /* distinct resourceId values */
  unsigned int n_dense;               /* distinct (device, stream key) pairs */
  unsigned int runtime_ids_repeat;    /* two runtime rows share a slot of the full table */
  unsigned int n_queues;              /* distinct hardware queues entered into the queue -> stream table */
  unsigned int n_sync_rows;           /* distinct (device, row) pairs of Stream Sync activities */
  unsigned int ext_ids_repeat;        /* two external-correlation records share a correlation id */
  alignas(256) JoinPlan plan;         /* key ranges and modes of the join tables: read by every row of the join
                                         kernels, so kept off the cache lines that take the counters' atomics */
  /* The counters that most workgroups add to (KTJ_CNT_*) are kept in KTJ_COUNTER_SHARDS copies, one
   * 128-byte line each; a workgroup adds to the copy of its index.  Atomics on one address are carried
   * out one after the other, and tens of thousands of workgroups adding to the same few words cost the
   * join more than its table lookups.  k_publish sums the copies into the fields above, which nothing
   * on the device reads; it hands the host everything in front of this array. */
  alignas(128) unsigned long long shard[KTJ_COUNTER_SHARDS][16];
};
enum { KTJ_CNT_OUT_OF_RANGE = 0, KTJ_CNT_OUT_OF_ORDER, KTJ_CNT_FLOW, KTJ_CNT_LINKED, KTJ_CNT_BLANK_NAMES, KTJ_CNT_VALID,
       KTJ_CNT_SYNC_TYPED, KTJ_CNT_COUNT };
#define KTJ_DEVERR_TABLE_FULL 1u         /* a join table sized from the record counts filled up (a defect) */
#define KTJ_DEVERR_DISTINCT_DEVICES 2u   /* more distinct deviceId values than the rank set holds: the sort
                                            takes its slower path without ranks, no error reaches the caller */
#define KTJ_DEVERR_HASH_COLLISION 4u
#define KTJ_DEVERR_RECORD_TOO_LONG 8u
#define KTJ_DEVERR_DISTINCT_RESOURCES 16u /* as DISTINCT_DEVICES, for resourceId values */
#define KTJ_DEVERR_STREAMS 32u            /* more than KTJ_MAX_STREAM_PAIRS (device, stream) pairs */
#define KTJ_DEVERR_QUEUES 64u             /* more than KTJ_MAX_QUEUES hardware queues */
#define KTJ_DEVERR_SYNC_ROWS 128u         /* more than KTJ_MAX_SYNC_ROWS (device, row) pairs of Stream Sync events */

#define KTJ_SET_CAP 16384u     /* slots of the distinct-value sets; KTJ_SET_MAX values get a rank */
#define KTJ_SET_MAX 4096u
#define KTJ_DENSE_CAP (2u * KTJ_MAX_STREAM_PAIRS) /* slots of the (device, stream) table */
#define KTJ_QUEUE_CAP (2u * KTJ_MAX_QUEUES)       /* slots of the queue -> stream table */
#define KTJ_SYNC_CAP (2u * KTJ_MAX_SYNC_ROWS)     /* slots of the Stream Sync (device, row) table */
#define KTJ_TABLE_PROBES 256u  /* linear probing of these small tables gives up after this many slots: a backstop,
                                  the documented limits are enforced by counting the distinct keys */

struct ApiTable {
  const uint32_t* cid_name_ids;
  uint32_t n_cids;
  const uint32_t* flow_start_bits; /* bitmap over cids */
  uint32_t malloc_cid;
};

/* read-backs and text of a pass without the copy engine: sc, *total (may be null) and list[0..n_list)
 * into pinned host memory (device-visible addresses); two pieces of host text to their places in the
 * document (source and destination of a piece must agree modulo 16) */
hipError_t publish(Scalars* sc, const uint64_t* total, const uint32_t* list, uint32_t n_list, Scalars* h_sc,
                   uint64_t* h_total, uint32_t* h_list, hipStream_t st);
hipError_t put_text(const char* src_a, char* dst_a, uint64_t n_a, const char* src_b, char* dst_b, uint64_t n_b, hipStream_t st);
/* pieces of page-locked host memory to their places in device memory, in one launch */
#define KTJ_MAX_PIECES 16u
struct PieceJobs {
  const char* src[KTJ_MAX_PIECES];
  char* dst[KTJ_MAX_PIECES];
  uint64_t n[KTJ_MAX_PIECES];
  uint32_t count;
};
hipError_t put_pieces(const PieceJobs& jobs, hipStream_t st);
/* ---- utilities ---- */
hipError_t fill_u64(uint64_t* p, uint64_t v, uint64_t n, hipStream_t st);
hipError_t fill_u32(uint32_t* p, uint32_t v, uint64_t n, hipStream_t st);
struct FillJobs {          /* up to 12 fills in one launch */
  void* p[12];
  uint64_t value[12];
  uint64_t n[12];
  uint32_t bytes_each[12]; /* 4 or 8 */
  uint32_t count;
  void add(void* ptr, uint64_t v, uint64_t elems, uint32_t width) { p[count] = ptr; value[count] = v; n[count] = elems; bytes_each[count] = width; ++count; }
};
hipError_t fill_many(const FillJobs& jobs, hipStream_t st);
hipError_t init_scalars(Scalars* s, hipStream_t st);
hipError_t copy_reference(const void* src, void* dst, uint64_t bytes, hipStream_t st);

/* Working memory for callers that cannot allocate: a static array in device memory, one copy per
 * GPU, KTJ_NOALLOC_SCRATCH_BYTES long.  Returns the address of the copy on `device` (which must be
 * the current device); the address is looked up once per device and kept. */
hipError_t scratch_address(int device, void** ptr, size_t* bytes);

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
/* id_range / narrow_range: one KeyRange per workgroup (decode_blocks(n) entries), smallest and
 * largest id of the workgroup's records; id_range of decode_generic may be null */
uint64_t decode_blocks(uint64_t n);
hipError_t decode_generic(const ktj_generic_rec* r, uint64_t n, Columns c, uint64_t first, Scalars* sc, EmitCtx ctx,
                          KeyRange* id_range, hipStream_t st);
/* the runtime and device kernels also convert the clock and apply the capture window */
hipError_t decode_runtime(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first, KeyRange* id_range,
                          KeyRange* narrow_range, ClockDev clk, int64_t win_start, int64_t win_end, Scalars* sc, hipStream_t st);
hipError_t decode_device(const ktj_device_rec* r, uint64_t n, Columns c, uint64_t first, DevBrief* brief, KeyRange* id_range,
                         ClockDev clk, int64_t win_start, int64_t win_end, Scalars* sc, hipStream_t st);

/* ---- stage 2b: joins ---- */
/* key ranges of the three tables, then their modes (direct unless force_hash or the span is too wide).
 * parts: the decode kernels' per-workgroup ranges, laid out as [generic ids | runtime ids | runtime ids
 * narrowed | device ids] with decode_blocks() entries each */
hipError_t plan_tables(const KeyRange* parts, uint64_t n_generic, uint64_t n_runtime, uint64_t n_device,
                       const ktj_extcorr_rec* e, uint64_t n_ext, uint32_t cap_full, uint32_t cap_narrow, uint32_t cap_cpu,
                       bool force_hash, Scalars* sc, hipStream_t st);
hipError_t clear_tables(Table tf, FullCols fc, Table tn, NarrowCols nc, Table cpu, hipStream_t st);
hipError_t build_cpu_ids(const ktj_generic_rec* g, uint64_t n, Table cpu, uint32_t* cpu_row, Scalars* sc, hipStream_t st);
/* after build_cpu_ids: enters the external-correlation records and resolves their external ids */
hipError_t build_extcorr(const ktj_extcorr_rec* e, uint64_t n, Table tn, NarrowCols nc, Table cpu, const uint32_t* cpu_row,
                         const ktj_generic_rec* g, EmitCtx ctx, Scalars* sc, hipStream_t st);
hipError_t collective_first(const MatRow* mat, const uint32_t* perm, uint64_t n_rows, uint32_t n_coll, uint32_t* first,
                            hipStream_t st);
/* per device row: "External id", timestamp-order check, stream of the launching row, and the
 * size / grid hand-over (into link[]) */
hipError_t link_device_rows(uint64_t n, Columns c, uint64_t first_device, Table tf, FullCols fc, Table tn, NarrowCols nc,
                            DevLink* link, Scalars* sc, hipStream_t st);
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
hipError_t backfill_streams(const DevBrief* d, uint64_t n, Columns c, uint64_t first_device, StreamTables t,
                            Scalars* sc, hipStream_t st);

/* ---- GPU user annotations (GenericActivityProfiler.cpp:277-327, 423-433): one span per
 * (device, resource, annotation id) over the device rows that the user-domain correlation
 * records lead to.  Tables are caller-provided: u_keys (cap_user + 1, KTJ_EMPTY_KEY), u_src (0),
 * and the span table of cap_span + 1 slots: hash (KTJ_EMPTY_KEY), first (0xFFFFFFFF), lo/hi
 * (biased timestamps: lo ~0, hi 0), zero (0). ---- */
struct SpanTables {
  uint64_t* u_keys; uint32_t* u_src; uint32_t u_mask;   /* correlation id -> last user record (index + 1) */
  uint64_t* hash; uint32_t* first; uint64_t* lo; uint64_t* hi; uint32_t* zero; uint32_t mask;
  int32_t* dev; int64_t* res; uint64_t* ext; uint32_t* name;  /* written by the first row of a span */
};
struct SpanOut {            /* one finished span, read back by the host */
  int64_t res;
  uint64_t ext;             /* the annotation's id (key of the CPU-op table) */
  int64_t start, end;       /* min timestamp, max end over the span's rows */
  int32_t dev;
  uint32_t name;            /* string id of the annotation's name */
  uint32_t first;           /* index of the first device row of the span: insertion order */
  uint32_t zero;            /* some row starts at time 0: the start needs the sequential rule */
};                          /* 48 bytes */
struct SpanMember { uint32_t slot, row; int64_t ts; };  /* rows of spans with `zero` set */
hipError_t build_usercorr(const ktj_extcorr_rec* u, uint64_t n, SpanTables t, Scalars* sc, hipStream_t st);
hipError_t group_spans(const ktj_extcorr_rec* u, const ktj_generic_rec* g, uint64_t n_device, Columns c, uint64_t first_device,
                       Table cpu, const uint32_t* cpu_row, SpanTables t, SpanOut* out, uint32_t* n_out, Scalars* sc,
                       hipStream_t st);
hipError_t span_members(const ktj_extcorr_rec* u, uint64_t n_device, Columns c, uint64_t first_device, Table cpu,
                        SpanTables t, SpanMember* out, uint32_t cap_out, uint32_t* n_out, hipStream_t st);

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
/* for timestamp spans too wide for one composite key: keys = ts - ts_min with vals = arrival
 * index, then keys = composite rank of row order[p] with vals = order[p] (dropped rows get
 * 1 << rank_bits) */
hipError_t make_ts_keys(Columns c, uint64_t n, const Scalars* sc, uint64_t* keys, uint32_t* vals, hipStream_t st);
/* keys[p] = sign-biased column value of row order[p] (validity != 0: 0 for kept rows, 1 for dropped ones) */
hipError_t make_column_keys(const int64_t* column, const uint32_t* meta, const uint32_t* order, uint64_t n, int validity,
                            uint64_t* keys, uint32_t* vals, hipStream_t st);
hipError_t clear_error_bits(Scalars* sc, unsigned int bits, hipStream_t st);
/* The composite-key sort on single 64-bit words (key above the arrival index); perm receives the
 * arrival index per sorted position.  Usable when sort_packed_fits(n, key_bits). */
bool sort_packed_fits(uint64_t n, uint32_t key_bits);
void sort_packed_force_passes(bool on); /* tests: no one-launch sort of a single tile */
hipError_t sort_packed(Columns c, uint64_t n, SortSets s, const Scalars* sc, uint32_t ts_bits, uint32_t res_bits,
                       uint32_t key_bits, uint64_t* buf_a, uint64_t* buf_b, uint32_t* perm, uint32_t* hist, uint64_t* scan_tmp,
                       hipStream_t st);
hipError_t make_rank_keys(Columns c, const uint32_t* order, uint64_t n, SortSets s, uint32_t res_bits, uint32_t rank_bits,
                          uint64_t* keys, uint32_t* vals, hipStream_t st);
/* stable LSD radix sort of (key, val) pairs on the low `bits` bits; result ends in keys_out/vals_out
 * pointers returned through *res_keys / *res_vals (one of the two buffer pairs) */
uint64_t radix_tmp_elems(uint64_t n);
hipError_t radix_sort(uint64_t* keys_a, uint32_t* vals_a, uint64_t* keys_b, uint32_t* vals_b, uint64_t n,
                      uint32_t bits, uint32_t* hist /* radix_tmp_elems(n) */, uint64_t* scan_tmp,
                      uint64_t** res_keys, uint32_t** res_vals, hipStream_t st);

/* ---- stage 4a: joined rows + exact byte length (arrival order) ---- */
/* keys: KTJ_SYNC_CAP + 1, first_pos: KTJ_SYNC_CAP + 1, is_first: n_generic (all caller-provided);
 * dev: the deviceId column */
hipError_t stream_sync_first(const uint32_t* perm, uint64_t n_sorted, const ktj_generic_rec* g, uint64_t n_generic,
                             const int64_t* dev, DictViews d, uint64_t* keys, uint32_t* first_pos, uint32_t* is_first, Scalars* sc,
                             hipStream_t st);
/* sync_first: per generic row, from stream_sync_first, or null when there are no such rows */
/* generic records whose rows start at arrival index `first` */
hipError_t mat_generic_rows(const ktj_generic_rec* g, uint64_t n, uint64_t first, EmitCtx ctx, const uint32_t* sync_first,
                            MatRow* mat, uint32_t* len, Scalars* sc, hipStream_t st);
/* the pass over the runtime rows: publishes what device rows take over (first timestamp, stream, grid,
 * size) into the tables, reads the "External id", makes the joined rows and their lengths; runs
 * after build_extcorr and before link_device_rows */
hipError_t join_runtime_rows(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first, ApiTable api, Table tf, FullCols fc,
                             Table tn, NarrowCols nc, uint32_t* slot_f, uint32_t* slot_n, EmitCtx ctx, MatRow* mat,
                             uint32_t* len, Scalars* sc, hipStream_t st);
/* winners write the payload again and repeated ids are checked; returns at once where no two
 * runtime rows share a slot */
hipError_t republish_runtime_rows(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first, FullCols fc, NarrowCols nc,
                                  const uint32_t* slot_f, const uint32_t* slot_n, Scalars* sc, hipStream_t st);
hipError_t mat_device_rows(const ktj_device_rec* d, uint64_t n, Columns c, uint64_t first, const DevLink* link,
                           EmitCtx ctx, MatRow* mat, uint32_t* len, Scalars* sc, hipStream_t st);
hipError_t gather_len(const uint32_t* perm, const uint32_t* len, uint64_t n, uint32_t* len_sorted, uint8_t* kind_sorted,
                      hipStream_t st);

/* ---- stage 4b: emit ---- */
/* tile size (bytes of output per workgroup) for a document whose activity section has act_bytes
 * bytes in n_rows activities, and the number of tiles / entries of tile_start (tiles + 1) */
uint32_t emit_tile_bytes(uint64_t act_bytes, uint64_t n_rows);
uint64_t emit_tile_count(uint64_t prefix_len, uint64_t act_bytes, uint32_t tile);
hipError_t emit(const MatRow* mat, const uint32_t* perm, const uint64_t* offs /* n+1 */, uint64_t n,
                EmitCtx ctx, char* out, uint64_t prefix_len, uint64_t act_bytes, uint32_t tile,
                uint32_t* tile_start /* tiles + 1 */, hipStream_t st);

/* direct variant: one lane per activity, no LDS staging; kind_sorted holds the tail kind of every
 * activity in emission order (gather_len); n_rows = number of activities that are written */
hipError_t emit_direct(const MatRow* mat, const uint32_t* perm, const uint64_t* offs, const uint8_t* kind_sorted,
                       uint64_t n_rows, uint64_t act_bytes, EmitCtx ctx, char* out, uint64_t prefix_len, hipStream_t st);

}  // namespace gpu
}  // namespace ktj
#endif
