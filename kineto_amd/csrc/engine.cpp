/*
 * engine.cpp — host side of the trace post-processing engine behind the C ABI of include/ktj.h:
 * owns device memory, accepts submissions, orders the kernel stages on one HIP stream, formats
 * the handful of non-activity events and moves the finished document to the host / file.
 *
 * There is no CPU implementation of the activity path in this library: if a HIP call fails the
 * entry point returns KTJ_ERR_HIP.
 */
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <thread>
#include <string>
#include <unistd.h>
#include <unordered_map>
#include <utility>
#include <vector>

#include <rocprofiler-sdk/buffer_tracing.h>

#include "../../include/ktj_debug.h"
#include "../../include/ktj_rocprofiler.h"
#include "gpu_stages.h"
#include "host_events.h"
#include "sdk_api_rows.h"

using namespace ktj;
using namespace ktj::gpu;

namespace {

#define KTJ_INPUT_ARENA_BYTES (1u << 20)   /* device memory for the inputs of small traces */
#define KTJ_INPUT_PIECE_MAX (128u << 10)   /* largest array that takes a piece of it */
#define KTJ_STAGE_SMALL_BYTES (256u << 10) /* pinned ring that small submissions pass through */
#define KTJ_STAGE_SMALL_MAX (64u << 10)    /* largest submission that does */
/* large submissions: pinned chunks, two per copying thread.  Measured for 1.9 GB of records from
 * ordinary memory (one copy through the runtime's staging: 25 GB/s): chunks of 1 / 2 / 4 / 8 / 16 MiB
 * give 30 / 38 / 42 / 46 / 45 GB/s, 3, 4, 8 or 12 threads the same (each copy handed to the copy
 * engine costs some microseconds whatever its size). */
#define KTJ_STAGE_CHUNK (8ull << 20)
#define KTJ_STAGE_BIG_MIN (16ull << 20)    /* smallest submission that is spread over threads */
#define KTJ_STAGE_THREADS_MAX 4
#define KTJ_KIT_DEVICE_BYTES_MAX (64ull << 20) /* working and document memory that waits for the next engine */
#define KTJ_KIT_PINNED_BYTES_MAX (1ull << 20)  /* same, per pinned buffer sized by a document */

/* One working buffer in device memory.  `p` is what the kernels use: either the buffer's own
 * allocation (freed with the engine; the engine's device is current then) or, for the entry point
 * that allocates nothing, a borrowed range that somebody else owns (a piece of the library's static
 * scratch array, or the caller's output buffer).  The own allocation survives a borrow. */
struct DevBuf {
  void* p = nullptr;
  size_t cap = 0;
  void* own = nullptr;
  size_t own_cap = 0;
  DevBuf() = default;
  DevBuf(const DevBuf&) = delete;
  DevBuf& operator=(const DevBuf&) = delete;
  DevBuf& operator=(DevBuf&& o) noexcept {
    if (this != &o) { release(); p = o.p; cap = o.cap; own = o.own; own_cap = o.own_cap; o.p = o.own = nullptr; o.cap = o.own_cap = 0; }
    return *this;
  }
  ~DevBuf() { release(); }
  hipError_t ensure(size_t bytes, bool with_slack = true) {
    if (p != own) { p = own; cap = own_cap; } /* back from a borrowed range */
    if (bytes <= cap) return hipSuccess;
    if (own) { hipError_t e = hipFree(own); p = own = nullptr; cap = own_cap = 0; if (e != hipSuccess) return e; }
    size_t want = bytes + (with_slack ? bytes / 8 : 0) + 256;
    hipError_t e = hipMalloc(&own, want);
    if (e != hipSuccess) { p = own = nullptr; return e; }
    p = own;
    cap = own_cap = want;
    return hipSuccess;
  }
  void borrow(void* ptr, size_t bytes) { p = ptr; cap = bytes; }
  void release() { if (own) (void)hipFree(own); p = own = nullptr; cap = own_cap = 0; }
  template <typename T> T* as() const { return reinterpret_cast<T*>(p); }
};

/* Device memory for the inputs of a small trace: one allocation that the engine's small arrays are
 * carved out of (a trace of a few records otherwise spends more time in hipMalloc than on the GPU).
 * Pieces are never given back; a new engine that inherits the arena starts at its beginning. */
struct InputArena {
  DevBuf mem;
  size_t used = 0;
  void* take(size_t bytes) {
    const size_t off = (used + 255) & ~(size_t)255;
    if (bytes > KTJ_INPUT_PIECE_MAX || !mem.p || off > mem.cap || bytes > mem.cap - off) return nullptr;
    used = off + bytes;
    return static_cast<char*>(mem.p) + off;
  }
};

/* append-only device array fed from host memory */
struct DevVec {
  DevBuf buf;
  size_t bytes = 0;
  /* room for n more bytes behind what is there; what is there moves along.  A small array takes a
   * piece of the engine's input arena instead of an allocation of its own. */
  hipError_t reserve(size_t n, hipStream_t st, InputArena* arena) {
    if (bytes + n + 16 > buf.cap) { /* 16 spare bytes: string copies load whole aligned words */
      DevBuf nb;
      size_t want = (bytes + n) * 2 + 16;
      void* piece = arena ? arena->take(want) : nullptr;
      hipError_t e = hipSuccess;
      if (piece) nb.borrow(piece, want);
      else e = nb.ensure(want);
      if (e != hipSuccess) return e;
      if (bytes) { e = hipMemcpyAsync(nb.p, buf.p, bytes, hipMemcpyDeviceToDevice, st); if (e != hipSuccess) return e; }
      e = hipStreamSynchronize(st);
      if (e != hipSuccess) return e;
      buf = std::move(nb);
    }
    return hipSuccess;
  }
  char* end() const { return static_cast<char*>(buf.p) + bytes; }
  void release() { buf.release(); bytes = 0; }
};

struct RecordSet {
  DevVec owned;
  const void* external = nullptr; /* device pointer supplied by the caller */
  uint64_t n = 0;
  const void* ptr() const { return external ? external : owned.buf.p; }
};

/* read-backs of one pass land in pinned host memory (no staging inside the runtime) */
struct HostCtl {
  Scalars scalars;
  uint64_t act_bytes;
  uint32_t n_out;
  uint32_t pad;
};
#define KTJ_GUESS_BYTES_PER_ROW 480u /* the fixed text of an event with its flow event */
#define KTJ_PINNED_SMALL_BYTES (256u << 10) /* header/footer text and small tables of a pass that may not allocate */

enum { EV_START = 0, EV_DICT, EV_DECODE, EV_CONVERT, EV_JOIN, EV_SORT_A, EV_SORT_B, EV_SORT, EV_SIZE, EV_SCAN,
       EV_EMIT_START, EV_EMIT, EV_COUNT };

}  // namespace

struct ktj_engine {
  std::string out_path, tmp_path, last_error;
  int64_t base_time_ns = 0;
  int device = 0;
  uint32_t flags = 0;
  FILE* sink = nullptr;
  bool bad_sink = false;
  bool started = false;
  bool processed = false;
  hipStream_t stream = nullptr;
  hipEvent_t ev[EV_COUNT] = {};
  hipEvent_t ev_d2h[2] = {};

  /* inputs */
  std::string txt_header, txt_before, txt_after; /* events in front of and behind the activity section, call order */
  bool activities_begun = false;
  DevVec str_blob, str_off; /* str_off holds n_strings + 1 absolute offsets */
  uint64_t n_strings = 0, blob_bytes = 0;
  std::vector<ktj_field> fields;
  std::vector<ktj_schema_desc> schemas;
  DevBuf d_fields, d_schemas;
  bool schemas_dirty = true;
  DevVec args;
  uint64_t n_args = 0;
  std::vector<CollectiveInfo> collectives; /* ktj_add_collective entries */
  bool coll_schemas = false;               /* a schema with a leading KTJ_F_COLLECTIVE field exists */
  bool coll_dirty = true;
  DevBuf d_coll_blob, d_coll_off, d_coll_first, cpu_row;
  /* GPU user annotations: correlation table, span table, finished spans, synthesised records */
  DevBuf u_keys, u_src, sp_hash, sp_first, sp_lo, sp_hi, sp_zero, sp_dev, sp_res, sp_ext, sp_name, sp_out, sp_count, sp_members,
      synth_recs;
  uint64_t n_spans = 0;
  std::vector<uint32_t> coll_first;        /* read back: first use of each entry per backend */
  std::unordered_map<uint64_t, int32_t> sdk_agents;        /* agent handle -> device index */
  std::unordered_map<uint64_t, uint32_t> sdk_kernel_names; /* kernel id -> string id of its name */
  uint32_t sdk_unknown_name = KTJ_NONE;
  std::vector<ktj_device_rec> sdk_rows;                    /* conversion buffer, reused */
  std::vector<ktj_runtime_rec> sdk_api_rows;               /* runtime rows of ktj_submit_sdk_api_record, not yet on the device */
  std::vector<ktj_extcorr_rec> sdk_api_ext, sdk_api_user;  /* their external-correlation pairs */
  std::vector<uint32_t> cid_names, flow_bits;
  uint32_t malloc_cid = KTJ_NONE;
  DevBuf d_cid_names, d_flow_bits;
  bool api_dirty = true;
  ktj_clock_model clock{};
  int64_t win_start = INT64_MIN, win_end = INT64_MAX;
  RecordSet generic, runtime, devrows, extcorr, usercorr;

  /* working buffers */
  DevBuf d_scalars, d_name_len, d_arg_len, d_sflags, d_name_off, d_arg_off, d_name_blob, d_arg_blob;
  DevBuf c_ts, c_dur, c_corr, c_dev, c_res, c_meta, c_ext;
  DevBuf t_full, t_narrow, t_cpu, f_has_runtime, f_first, f_stream_src, f_pay, n_ext_src, n_kern_src, n_copy_src, n_pay, slot_f, slot_n, dev_link, dev_brief, sync_keys, sync_pos, sync_first;
  DevBuf q_keys, q_stream, q_amb, dn_hash, dn_first, dn_dev, dn_key, dn_rank, range_parts;
  DevBuf s_dev_k, s_dev_r, s_res_k, s_res_r;
  DevBuf keys_a, keys_b, vals_a, vals_b, hist, scan_tmp;
  DevBuf mat, len, len_sorted, kind_sorted, offs, out, tile_start;
  void* pinned_small = nullptr; size_t pinned_small_cap = 0;
  HostCtl* h_ctl = nullptr;                  /* pinned: what the device hands back during a pass */
  HostCtl* h_ctl_dev = nullptr;              /* the same memory as the kernels address it */
  char* pinned_small_dev = nullptr;
  /* ktj_process_noalloc: working buffers are carved out of the library's static scratch array */
  bool noalloc = false;
  char* arena = nullptr; size_t arena_cap = 0, arena_used = 0;
  /* ktj_process: one allocation that the working buffers of a pass are carved out of */
  DevBuf pool;
  size_t pool_used = 0, pool_need = 0;
  bool measuring = false;
  char* pinned_out = nullptr; size_t pinned_out_cap = 0;
  char* file_stage[2] = {nullptr, nullptr};   /* pinned staging of the file sink, at most KTJ_FILE_STAGE_BYTES each */
  size_t file_stage_cap[2] = {0, 0};
  hipEvent_t ev_file_stage[2] = {};
  bool host_copy_valid = false;
  /* submissions from ordinary host memory: small ones pass through a pinned ring and are not waited
   * for (the stream orders them before the pass), large ones through pinned chunks that several
   * threads fill while the copy engine empties others */
  InputArena input_arena;
  char* stage_small = nullptr; char* stage_small_dev = nullptr; size_t stage_small_used = 0;
  PieceJobs pieces{}; /* small submissions in the ring that no kernel has moved yet */
  char* stage_big = nullptr; size_t stage_big_chunks = 0;
  hipEvent_t ev_stage_big[2 * KTJ_STAGE_THREADS_MAX] = {};
  bool hip_failed = false; /* a HIP call failed at some point: nothing of this engine is handed on */

  /* results */
  uint64_t N = 0, prefix_len = 0, act_bytes = 0, total_bytes = 0;
  uint32_t* perm = nullptr; uint64_t* sorted_keys = nullptr;
  int sort_mode = 0; /* 0: key and index in one word; 1: (key, index) pairs */
  Scalars scalars{};
  ktj_stats stats{};
};

namespace {

int fail_hip(ktj_engine* e, hipError_t err, const char* what) {
  e->hip_failed = true;
  e->last_error = std::string(what) + ": " + hipGetErrorString(err);
  return KTJ_ERR_HIP;
}
#define HIPCHK(call)                                            \
  do {                                                          \
    hipError_t _e = (call);                                     \
    if (_e != hipSuccess) return fail_hip(e, _e, #call);        \
  } while (0)

/* the ktj_last_error() text for the KTJ_DEVERR_* bits that end a pass */
std::string limit_text(unsigned bits) {
  std::string t;
  auto add = [&](const std::string& x) { t += (t.empty() ? "" : "; ") + x; };
  if (bits & KTJ_DEVERR_STREAMS)
    add("more than KTJ_MAX_STREAM_PAIRS (" + std::to_string(KTJ_MAX_STREAM_PAIRS) + ") distinct (device, stream) pairs among the device records");
  if (bits & KTJ_DEVERR_QUEUES)
    add("more than KTJ_MAX_QUEUES (" + std::to_string(KTJ_MAX_QUEUES) + ") distinct hardware queues among the device records");
  if (bits & KTJ_DEVERR_SYNC_ROWS)
    add("more than KTJ_MAX_SYNC_ROWS (" + std::to_string(KTJ_MAX_SYNC_ROWS) + ") distinct (device, row) pairs of Stream Sync activities");
  if (bits & KTJ_DEVERR_RECORD_TOO_LONG) add("an activity's JSON text is 1 GiB or longer");
  if (bits & KTJ_DEVERR_HASH_COLLISION) add("two (device, stream) pairs share a 64-bit hash");
  if (bits & KTJ_DEVERR_TABLE_FULL) add("a join table sized from the record counts is full (internal error)");
  if (bits & (KTJ_DEVERR_DISTINCT_DEVICES | KTJ_DEVERR_DISTINCT_RESOURCES)) add("distinct-value set overflow after the sort (internal error)");
  return "limit exceeded: " + t + " [bits " + std::to_string(bits) + "]";
}

uint32_t pow2_at_least(uint64_t v) {
  uint64_t c = 1024;
  while (c < v) c <<= 1;
  return (uint32_t)c;
}

std::string default_file_name() { /* output_json.cpp:65-70, 481-483 */
  return "/tmp/libkineto_activities_" + std::to_string((long)getpid()) + ".json";
}

/* Room for `bytes` in a working buffer.  Normally the buffer grows by allocation; in a pass that
 * may not allocate it becomes the next piece of the scratch array (256-byte aligned), or the pass
 * fails with KTJ_ERR_LIMIT. */
int need(ktj_engine* e, DevBuf& b, size_t bytes) {
  if (!e->noalloc) {
    /* The working buffers of a pass share one allocation, the pool: a first pass then makes a handful
     * of allocations instead of sixty.  The pass first asks for everything with `measuring` set, which
     * only adds the sizes up, sizes the pool, and asks again.  What does not fit (buffers whose size a
     * pass learns late) is allocated on its own as before. */
    if (e->measuring) { e->pool_need += (bytes + 255) & ~(size_t)255; return KTJ_OK; }
    const size_t off = (e->pool_used + 255) & ~(size_t)255;
    if (e->pool.p && off <= e->pool.cap && bytes <= e->pool.cap - off) {
      b.borrow(static_cast<char*>(e->pool.p) + off, bytes);
      e->pool_used = off + bytes;
      return KTJ_OK;
    }
    HIPCHK(b.ensure(bytes));
    return KTJ_OK;
  }
  const size_t off = (e->arena_used + 255) & ~(size_t)255;
  if (off > e->arena_cap || bytes > e->arena_cap - off) {
    e->last_error = "ktj_process_noalloc: the trace needs more than the " + std::to_string(e->arena_cap) +
                    " bytes of the static scratch array (asked for " + std::to_string(bytes) + " more at " + std::to_string(off) + ")";
    return KTJ_ERR_LIMIT;
  }
  b.borrow(e->arena + off, bytes);
  e->arena_used = off + bytes;
  return KTJ_OK;
}
#define NEED(buf, bytes)                                  \
  do {                                                    \
    const int _rc = need(e, buf, bytes);                  \
    if (_rc != KTJ_OK) return _rc;                        \
  } while (0)

/* A small host table to the device.  A pass that may not allocate stages it through the pinned
 * buffer of the engine (allocated with the engine) instead of the runtime's own staging. */
int upload_small(ktj_engine* e, DevBuf& dst, const void* src, size_t bytes) {
  /* these tables outlive the pass (they are uploaded only when they change), so outside a pass that
   * may not allocate they keep allocations of their own rather than a piece of the pass's pool */
  if (e->noalloc) NEED(dst, bytes ? bytes : 16);
  else HIPCHK(dst.ensure(bytes ? bytes : 16));
  if (bytes && e->noalloc) {
    if (bytes > e->pinned_small_cap) {
      e->last_error = "ktj_process_noalloc: a table of " + std::to_string(bytes) + " bytes exceeds the pinned staging buffer";
      return KTJ_ERR_LIMIT;
    }
    memcpy(e->pinned_small, src, bytes);
    src = e->pinned_small;
  }
  if (bytes) HIPCHK(hipMemcpyAsync(dst.p, src, bytes, hipMemcpyHostToDevice, e->stream));
  HIPCHK(hipStreamSynchronize(e->stream));
  return KTJ_OK;
}

/* The small submissions gathered in the pinned ring go to their places on the device: one launch for
 * all of them, ordered on the engine's stream like everything else.  Before a pass, before an array
 * they belong to moves, and when the ring or the list is full. */
int put_pending_pieces(ktj_engine* e) {
  if (e->pieces.count == 0) return KTJ_OK;
  HIPCHK(put_pieces(e->pieces, e->stream));
  e->pieces.count = 0;
  return KTJ_OK;
}

/* Is this host memory page-locked for the GPU (ktj_host_alloc, or the caller's own hipHostMalloc)?
 * Such memory is copied from directly. */
bool is_pinned_host(const void* p) {
  hipPointerAttribute_t a;
  memset(&a, 0, sizeof a);
  if (hipPointerGetAttributes(&a, p) != hipSuccess) { (void)hipGetLastError(); return false; }
  return a.type == hipMemoryTypeHost;
}

/* n bytes of host memory behind a device array.  The caller may free or reuse src when this
 * returns; the copy itself is only ordered on the engine's stream, in front of the next pass.
 *   - up to KTJ_STAGE_SMALL_MAX bytes: into the pinned ring, from where one kernel launch takes all
 *     such pieces to their places (put_pending_pieces; a trace of a few records pays a dozen copies
 *     and stream synchronisations otherwise);
 *   - from KTJ_STAGE_BIG_MIN bytes of ordinary memory: threads copy chunks into pinned buffers, two
 *     per thread, and hand each to the copy engine as soon as it is full (one thread's copy through
 *     the runtime's own staging reaches about half of what the link carries);
 *   - everything else, and page-locked sources: one copy, waited for. */
int append_from_host(ktj_engine* e, DevVec& v, const void* src, size_t n) {
  if (n == 0) return KTJ_OK;
  hipStream_t st = e->stream;
  if (v.bytes + n + 16 > v.buf.cap) { /* the array is about to move: the pieces on their way to it go first */
    const int rc = put_pending_pieces(e);
    if (rc != KTJ_OK) return rc;
  }
  HIPCHK(v.reserve(n, st, &e->input_arena));
  char* dst = v.end();
  if (n <= KTJ_STAGE_SMALL_MAX && e->stage_small) {
    /* the piece sits in the ring where its place on the device does, modulo 16 */
    size_t off = ((e->stage_small_used + 63) & ~(size_t)63) + ((uintptr_t)dst & 15u);
    if (off + n > KTJ_STAGE_SMALL_BYTES || e->pieces.count == KTJ_MAX_PIECES) {
      const int rc = put_pending_pieces(e);
      if (rc != KTJ_OK) return rc;
    }
    if (off + n > KTJ_STAGE_SMALL_BYTES) { /* the ring is full: what is in it has to be on the device first */
      HIPCHK(hipStreamSynchronize(st));
      off = (uintptr_t)dst & 15u;
    }
    memcpy(e->stage_small + off, src, n);
    const uint32_t k = e->pieces.count++;
    e->pieces.src[k] = e->stage_small_dev + off;
    e->pieces.dst[k] = dst;
    e->pieces.n[k] = n;
    e->stage_small_used = off + n;
    v.bytes += n;
    return KTJ_OK;
  }
  unsigned n_threads = std::thread::hardware_concurrency() / 2;
  if (n_threads > KTJ_STAGE_THREADS_MAX) n_threads = KTJ_STAGE_THREADS_MAX;
  if (n >= KTJ_STAGE_BIG_MIN && n_threads >= 2 && !is_pinned_host(src)) {
    const size_t slots = 2 * (size_t)n_threads;
    if (e->stage_big_chunks < slots) {
      if (e->stage_big) HIPCHK(hipHostFree(e->stage_big));
      e->stage_big = nullptr; e->stage_big_chunks = 0;
      void* p = nullptr;
      HIPCHK(hipHostMalloc(&p, slots * KTJ_STAGE_CHUNK, hipHostMallocDefault));
      e->stage_big = static_cast<char*>(p);
      e->stage_big_chunks = slots;
    }
    for (size_t k = 0; k < slots; ++k)
      if (!e->ev_stage_big[k]) HIPCHK(hipEventCreateWithFlags(&e->ev_stage_big[k], hipEventDisableTiming));
    const size_t n_chunks = (n + KTJ_STAGE_CHUNK - 1) / KTJ_STAGE_CHUNK;
    hipError_t err[KTJ_STAGE_THREADS_MAX];
    auto worker = [&](unsigned t) {
      err[t] = hipSetDevice(e->device);
      /* thread t takes chunks t, t + T, ...; its two pinned slots alternate */
      for (size_t c = t, turn = 0; c < n_chunks && err[t] == hipSuccess; c += n_threads, ++turn) {
        const size_t slot = 2 * (size_t)t + (turn & 1);
        char* stage = e->stage_big + slot * KTJ_STAGE_CHUNK;
        const size_t off = c * KTJ_STAGE_CHUNK, len = n - off < KTJ_STAGE_CHUNK ? n - off : KTJ_STAGE_CHUNK;
        if (turn >= 2) { err[t] = hipEventSynchronize(e->ev_stage_big[slot]); if (err[t] != hipSuccess) break; }
        memcpy(stage, static_cast<const char*>(src) + off, len);
        err[t] = hipMemcpyAsync(dst + off, stage, len, hipMemcpyHostToDevice, st);
        if (err[t] == hipSuccess) err[t] = hipEventRecord(e->ev_stage_big[slot], st);
      }
    };
    for (auto& x : err) x = hipSuccess;
    std::vector<std::thread> pool;
    unsigned started = 1; /* thread 0 is this one; a thread that cannot be started has its chunks copied here */
    try {
      pool.reserve(n_threads);
      for (; started < n_threads; ++started) pool.emplace_back(worker, started);
    } catch (...) {}
    worker(0);
    for (unsigned t = started; t < n_threads; ++t) worker(t);
    for (auto& th : pool) th.join();
    /* the slots are free for the next call once the stream has passed them */
    const hipError_t done = hipStreamSynchronize(st);
    for (unsigned t = 0; t < n_threads; ++t) HIPCHK(err[t]);
    HIPCHK(done);
    v.bytes += n;
    return KTJ_OK;
  }
  HIPCHK(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, st));
  HIPCHK(hipStreamSynchronize(st)); /* the caller may free src when we return */
  v.bytes += n;
  return KTJ_OK;
}

int bits_for(uint64_t max_value) { /* bits needed to hold values 0..max_value */
  int b = 0;
  while (b < 64 && (max_value >> b) != 0) ++b;
  return b;
}

/* GPU user annotations (GenericActivityProfiler.cpp:277-327, 423-433, 726).  The device groups the
 * in-window device rows by (device, resource, annotation) and reduces each group to its extent;
 * the host puts the finished spans into the order the profiler logs them in — stream by stream
 * (std::map), inside a stream the iteration order of a std::unordered_map keyed by the
 * annotation's id, both filled in the order of the spans' first rows — and hands them back as
 * generic records of type GPU_USER_ANNOTATION whose rows follow the device rows. */
int synthesise_user_spans(ktj_engine* e, Columns c, const EmitCtx& ctx, Table t_cpu, const uint32_t* cpu_row, Scalars* sc,
                          uint64_t first_row) {
  hipStream_t st = e->stream;
  const uint64_t ng = e->generic.n, nr = e->runtime.n, nd = e->devrows.n, nu = e->usercorr.n;
  const ktj_generic_rec* g_recs = static_cast<const ktj_generic_rec*>(e->generic.ptr());
  const ktj_extcorr_rec* u_recs = static_cast<const ktj_extcorr_rec*>(e->usercorr.ptr());
  const uint32_t cap_user = pow2_at_least(2 * nu), cap_span = pow2_at_least(2 * nd);
  NEED(e->u_keys, (cap_user + 1ull) * 8); NEED(e->u_src, (cap_user + 1ull) * 4);
  NEED(e->sp_hash, (cap_span + 1ull) * 8); NEED(e->sp_first, (cap_span + 1ull) * 4);
  NEED(e->sp_lo, (cap_span + 1ull) * 8); NEED(e->sp_hi, (cap_span + 1ull) * 8);
  NEED(e->sp_zero, (cap_span + 1ull) * 4); NEED(e->sp_dev, (cap_span + 1ull) * 4);
  NEED(e->sp_res, (cap_span + 1ull) * 8); NEED(e->sp_ext, (cap_span + 1ull) * 8);
  NEED(e->sp_name, (cap_span + 1ull) * 4); NEED(e->sp_out, (nd + 1ull) * sizeof(SpanOut));
  NEED(e->sp_count, 16);
  SpanTables t{e->u_keys.as<uint64_t>(), e->u_src.as<uint32_t>(), cap_user - 1,
               e->sp_hash.as<uint64_t>(), e->sp_first.as<uint32_t>(), e->sp_lo.as<uint64_t>(), e->sp_hi.as<uint64_t>(),
               e->sp_zero.as<uint32_t>(), cap_span - 1,
               e->sp_dev.as<int32_t>(), e->sp_res.as<int64_t>(), e->sp_ext.as<uint64_t>(), e->sp_name.as<uint32_t>()};
  HIPCHK(fill_u64(t.u_keys, KTJ_EMPTY_KEY, cap_user + 1ull, st)); HIPCHK(fill_u32(t.u_src, 0, cap_user + 1ull, st));
  HIPCHK(fill_u64(t.hash, KTJ_EMPTY_KEY, cap_span + 1ull, st)); HIPCHK(fill_u32(t.first, 0xFFFFFFFFu, cap_span + 1ull, st));
  HIPCHK(fill_u64(t.lo, ~0ull, cap_span + 1ull, st)); HIPCHK(fill_u64(t.hi, 0, cap_span + 1ull, st));
  HIPCHK(fill_u32(t.zero, 0, cap_span + 1ull, st));
  HIPCHK(build_usercorr(u_recs, nu, t, sc, st));
  HIPCHK(group_spans(u_recs, g_recs, nd, c, ng + nr, t_cpu, cpu_row, t, e->sp_out.as<SpanOut>(), e->sp_count.as<uint32_t>(), sc, st));
  HIPCHK(hipMemcpyAsync(&e->h_ctl->n_out, e->sp_count.p, 4, hipMemcpyDeviceToHost, st));
  HIPCHK(hipStreamSynchronize(st));
  const uint32_t n_out = e->h_ctl->n_out;
  if (n_out == 0) return KTJ_OK;
  std::vector<SpanOut> spans(n_out);
  HIPCHK(hipMemcpyAsync(spans.data(), e->sp_out.p, n_out * sizeof(SpanOut), hipMemcpyDeviceToHost, st));
  HIPCHK(hipStreamSynchronize(st));
  std::sort(spans.begin(), spans.end(), [](const SpanOut& a, const SpanOut& b) { return a.first < b.first; });

  /* insertOrExtendEvent's start rule is `if (ts < start || start == 0) start = ts` (:304-306): the
   * plain minimum unless a row of the span starts at time 0, after which the next row's time is
   * taken whatever it is.  Those spans (rare) are replayed row by row here. */
  bool any_zero = false;
  for (const SpanOut& sp : spans) any_zero = any_zero || sp.zero != 0;
  if (any_zero) {
    NEED(e->sp_members, (nd + 1ull) * sizeof(SpanMember));
    HIPCHK(span_members(u_recs, nd, c, ng + nr, t_cpu, t, e->sp_members.as<SpanMember>(), (uint32_t)nd, e->sp_count.as<uint32_t>(), st));
    HIPCHK(hipMemcpyAsync(&e->h_ctl->n_out, e->sp_count.p, 4, hipMemcpyDeviceToHost, st));
    HIPCHK(hipStreamSynchronize(st));
    const uint32_t n_members = e->h_ctl->n_out;
    std::vector<SpanMember> members(n_members);
    if (n_members) HIPCHK(hipMemcpyAsync(members.data(), e->sp_members.p, n_members * sizeof(SpanMember), hipMemcpyDeviceToHost, st));
    HIPCHK(hipStreamSynchronize(st));
    std::sort(members.begin(), members.end(), [](const SpanMember& a, const SpanMember& b) { return a.row < b.row; });
    std::unordered_map<uint32_t, size_t> by_slot;
    for (size_t k = 0; k < spans.size(); ++k)
      if (spans[k].zero) by_slot[spans[k].zero] = k;
    std::vector<uint8_t> started(spans.size(), 0);
    for (const SpanMember& m : members) {
      const auto it = by_slot.find(m.slot);
      if (it == by_slot.end()) continue;
      SpanOut& sp = spans[it->second];
      if (!started[it->second]) { started[it->second] = 1; sp.start = m.ts; }
      if (m.ts < sp.start || sp.start == 0) sp.start = m.ts;
    }
  }

  /* logEvents order (:313-319) */
  std::map<std::pair<int64_t, int64_t>, std::unordered_map<int64_t, size_t>> streams;
  for (size_t k = 0; k < spans.size(); ++k)
    streams[{(int64_t)spans[k].dev, spans[k].res}].insert({(int64_t)spans[k].ext, k});
  std::vector<ktj_generic_rec> recs;
  recs.reserve(spans.size());
  for (const auto& stream : streams) {
    for (const auto& entry : stream.second) {
      const SpanOut& sp = spans[entry.second];
      ktj_generic_rec r{}; /* createUserGpuSpan (:277-290): no metadata, no flow, no linked activity */
      r.start_ns = sp.start;
      r.end_ns = sp.end;
      r.resource = sp.res;
      r.device = sp.dev;
      r.id = (int32_t)(int64_t)sp.ext;
      r.name_id = sp.name;
      r.schema_id = KTJ_NONE;
      r.type = KTJ_TYPE_GPU_USER_ANNOTATION;
      recs.push_back(r);
    }
  }
  NEED(e->synth_recs, recs.size() * sizeof(ktj_generic_rec) + 16);
  HIPCHK(hipMemcpyAsync(e->synth_recs.p, recs.data(), recs.size() * sizeof(ktj_generic_rec), hipMemcpyHostToDevice, st));
  HIPCHK(hipStreamSynchronize(st));
  HIPCHK(decode_generic(e->synth_recs.as<ktj_generic_rec>(), recs.size(), c, first_row, sc, ctx, nullptr, st));
  e->n_spans = recs.size();
  return KTJ_OK;
}


/* What every engine needs before its first record — a stream, its events, the pinned buffers of the
 * hand-over, the input arena — and what its first pass allocates (the pool of working buffers and
 * the document, while they are small) costs several times what a trace of a few records takes on
 * the GPU.  ktj_destroy leaves one such set per device behind for the next ktj_create, which takes
 * it whole; a second engine alive at the same time makes its own.  Nothing of an engine that saw a
 * HIP error is kept.  Device and pinned memory that is kept: at most KTJ_KIT_DEVICE_BYTES_MAX of
 * working and document memory, the input arena, the small pinned buffers; it is held until the
 * process ends. */
struct Kit {
  bool full = false;
  hipStream_t stream = nullptr;
  hipEvent_t ev[EV_COUNT] = {};
  hipEvent_t ev_d2h[2] = {};
  hipEvent_t ev_file_stage[2] = {};
  hipEvent_t ev_stage_big[2 * KTJ_STAGE_THREADS_MAX] = {};
  void* pinned_small = nullptr; size_t pinned_small_cap = 0; char* pinned_small_dev = nullptr;
  HostCtl* h_ctl = nullptr; HostCtl* h_ctl_dev = nullptr;
  char* pinned_out = nullptr; size_t pinned_out_cap = 0;
  char* file_stage[2] = {nullptr, nullptr}; size_t file_stage_cap[2] = {0, 0};
  char* stage_small = nullptr; char* stage_small_dev = nullptr;
  char* stage_big = nullptr; size_t stage_big_chunks = 0;
  DevBuf d_scalars, pool, out, arena_mem;
};
std::mutex g_kit_mutex;
std::map<int, Kit*>& kits() { static auto* m = new std::map<int, Kit*>(); return *m; } /* never destroyed: the runtime may be gone by then */

/* the engine's device is current */
bool take_kit(ktj_engine* e) {
  std::lock_guard<std::mutex> lock(g_kit_mutex);
  auto it = kits().find(e->device);
  if (it == kits().end() || !it->second->full) return false;
  Kit& k = *it->second;
  e->stream = k.stream;
  memcpy(e->ev, k.ev, sizeof k.ev); memcpy(e->ev_d2h, k.ev_d2h, sizeof k.ev_d2h);
  memcpy(e->ev_file_stage, k.ev_file_stage, sizeof k.ev_file_stage);
  memcpy(e->ev_stage_big, k.ev_stage_big, sizeof k.ev_stage_big);
  e->pinned_small = k.pinned_small; e->pinned_small_cap = k.pinned_small_cap; e->pinned_small_dev = k.pinned_small_dev;
  e->h_ctl = k.h_ctl; e->h_ctl_dev = k.h_ctl_dev;
  e->pinned_out = k.pinned_out; e->pinned_out_cap = k.pinned_out_cap;
  for (int i = 0; i < 2; ++i) { e->file_stage[i] = k.file_stage[i]; e->file_stage_cap[i] = k.file_stage_cap[i]; }
  e->stage_small = k.stage_small; e->stage_small_dev = k.stage_small_dev;
  e->stage_big = k.stage_big; e->stage_big_chunks = k.stage_big_chunks;
  e->d_scalars = std::move(k.d_scalars); e->pool = std::move(k.pool); e->out = std::move(k.out);
  e->input_arena.mem = std::move(k.arena_mem);
  k = Kit();
  return true;
}

/* the engine's device is current and its stream is idle; whatever is not taken stays with the engine */
void give_kit(ktj_engine* e) {
  if (e->hip_failed || !e->stream || !e->h_ctl || !e->pinned_small || !e->stage_small || !e->d_scalars.own) return;
  if (e->pinned_small_cap > KTJ_KIT_PINNED_BYTES_MAX) return; /* grown for an unusually long header: not worth holding */
  for (auto& ev : e->ev) if (!ev) return;
  for (auto& ev : e->ev_d2h) if (!ev) return;
  std::lock_guard<std::mutex> lock(g_kit_mutex);
  Kit* slot = nullptr;
  try {
    Kit*& entry = kits()[e->device];
    if (!entry) entry = new Kit();
    slot = entry;
  } catch (...) { return; }
  if (slot->full) return;
  Kit& k = *slot;
  k.stream = e->stream; e->stream = nullptr;
  memcpy(k.ev, e->ev, sizeof k.ev); memset(e->ev, 0, sizeof e->ev);
  memcpy(k.ev_d2h, e->ev_d2h, sizeof k.ev_d2h); memset(e->ev_d2h, 0, sizeof e->ev_d2h);
  memcpy(k.ev_file_stage, e->ev_file_stage, sizeof k.ev_file_stage); memset(e->ev_file_stage, 0, sizeof e->ev_file_stage);
  memcpy(k.ev_stage_big, e->ev_stage_big, sizeof k.ev_stage_big); memset(e->ev_stage_big, 0, sizeof e->ev_stage_big);
  k.pinned_small = e->pinned_small; k.pinned_small_cap = e->pinned_small_cap; k.pinned_small_dev = e->pinned_small_dev;
  e->pinned_small = nullptr;
  k.h_ctl = e->h_ctl; k.h_ctl_dev = e->h_ctl_dev; e->h_ctl = nullptr;
  if (e->pinned_out_cap <= KTJ_KIT_PINNED_BYTES_MAX) { k.pinned_out = e->pinned_out; k.pinned_out_cap = e->pinned_out_cap; e->pinned_out = nullptr; }
  for (int i = 0; i < 2; ++i)
    if (e->file_stage_cap[i] <= KTJ_KIT_PINNED_BYTES_MAX) { k.file_stage[i] = e->file_stage[i]; k.file_stage_cap[i] = e->file_stage_cap[i]; e->file_stage[i] = nullptr; }
  k.stage_small = e->stage_small; k.stage_small_dev = e->stage_small_dev; e->stage_small = nullptr;
  k.stage_big = e->stage_big; k.stage_big_chunks = e->stage_big_chunks; e->stage_big = nullptr;
  k.d_scalars = std::move(e->d_scalars);
  if (e->pool.own_cap + e->out.own_cap <= KTJ_KIT_DEVICE_BYTES_MAX) {
    /* back from whatever they were lent (the pool never is; the document may sit in a caller's buffer) */
    e->pool.p = e->pool.own; e->pool.cap = e->pool.own_cap;
    e->out.p = e->out.own; e->out.cap = e->out.own_cap;
    k.pool = std::move(e->pool);
    k.out = std::move(e->out);
  }
  k.arena_mem = std::move(e->input_arena.mem);
  k.full = true;
}

}  // namespace

extern "C" {

const char* ktj_version(void) { return "ktj 0.1 (gfx950)"; }

int ktj_create(ktj_engine** out, const char* out_path, int64_t base_time_ns, int hip_device, uint32_t flags) {
  if (!out) return KTJ_ERR_ARG;
  *out = nullptr;
  ktj_engine* e = new (std::nothrow) ktj_engine();
  if (!e) return KTJ_ERR_NOMEM;
  e->out_path = (out_path && out_path[0]) ? out_path : default_file_name();
  e->tmp_path = e->out_path + ".tmp";
  e->base_time_ns = base_time_ns;
  e->device = hip_device;
  e->flags = flags;
  e->sort_mode = (flags & KTJ_CREATE_PAIR_SORT) ? 1 : 0;
  e->clock.scale = 1.0;
  *out = e; /* from here on errors are reported through the handle */
  if (!(flags & KTJ_CREATE_NO_FILE)) { /* openTraceFile, output_json.cpp:485-493 */
    e->sink = fopen(e->tmp_path.c_str(), "w");
    if (!e->sink) { e->bad_sink = true; e->last_error = "Failed to open '" + e->out_path + "': " + strerror(errno); }
  }
  HIPCHK(hipSetDevice(hip_device));
  if (!take_kit(e)) {
    HIPCHK(hipStreamCreate(&e->stream));
    for (auto& ev : e->ev) HIPCHK(hipEventCreate(&ev));
    for (auto& ev : e->ev_d2h) HIPCHK(hipEventCreate(&ev));
    HIPCHK(e->d_scalars.ensure(sizeof(Scalars)));
    HIPCHK(hipHostMalloc(&e->pinned_small, KTJ_PINNED_SMALL_BYTES, hipHostMallocDefault));
    e->pinned_small_cap = KTJ_PINNED_SMALL_BYTES;
    void* p = nullptr;
    HIPCHK(hipHostMalloc(&p, sizeof(HostCtl), hipHostMallocDefault));
    e->h_ctl = static_cast<HostCtl*>(p);
    void* d = nullptr;
    HIPCHK(hipHostGetDevicePointer(&d, e->h_ctl, 0));
    e->h_ctl_dev = static_cast<HostCtl*>(d);
    HIPCHK(hipHostGetDevicePointer(&d, e->pinned_small, 0));
    e->pinned_small_dev = static_cast<char*>(d);
    p = nullptr;
    HIPCHK(hipHostMalloc(&p, KTJ_STAGE_SMALL_BYTES, hipHostMallocDefault));
    e->stage_small = static_cast<char*>(p);
    HIPCHK(hipHostGetDevicePointer(&d, e->stage_small, 0));
    e->stage_small_dev = static_cast<char*>(d);
    HIPCHK(e->input_arena.mem.ensure(KTJ_INPUT_ARENA_BYTES, false));
  }
  memset(e->h_ctl, 0, sizeof(HostCtl));
  { /* this device's copy of the static scratch array (ktj_process_noalloc) */
    void* p = nullptr;
    size_t bytes = 0;
    HIPCHK(scratch_address(hip_device, &p, &bytes));
    e->arena = static_cast<char*>(p);
    e->arena_cap = bytes;
  }
  return KTJ_OK;
}

void ktj_destroy(ktj_engine* e) {
  if (!e) return;
  (void)hipSetDevice(e->device);
  if (e->stream) (void)hipStreamSynchronize(e->stream);
  give_kit(e); /* what the next engine on this device can start from; the rest is freed here */
  /* device buffers free themselves when the engine is deleted below */
  if (e->pinned_small) (void)hipHostFree(e->pinned_small);
  if (e->h_ctl) (void)hipHostFree(e->h_ctl);
  if (e->pinned_out) (void)hipHostFree(e->pinned_out);
  if (e->stage_small) (void)hipHostFree(e->stage_small);
  if (e->stage_big) (void)hipHostFree(e->stage_big);
  for (auto& p : e->file_stage) if (p) (void)hipHostFree(p);
  for (auto& ev : e->ev_file_stage) if (ev) (void)hipEventDestroy(ev);
  for (auto& ev : e->ev_stage_big) if (ev) (void)hipEventDestroy(ev);
  for (auto& ev : e->ev) if (ev) (void)hipEventDestroy(ev);
  for (auto& ev : e->ev_d2h) if (ev) (void)hipEventDestroy(ev);
  if (e->stream) (void)hipStreamDestroy(e->stream);
  if (e->sink) { fclose(e->sink); remove(e->tmp_path.c_str()); }
  delete e;
}

const char* ktj_last_error(const ktj_engine* e) { return e ? e->last_error.c_str() : "null engine"; }

int ktj_trace_start(ktj_engine* e, const char* const* meta_kv, size_t n_kv, const char* device_properties) {
  if (!e || (n_kv && !meta_kv)) return KTJ_ERR_ARG;
  if (e->bad_sink) return KTJ_OK;
  e->txt_header.clear();
  append_trace_start(e->txt_header, meta_kv, n_kv, device_properties, e->base_time_ns, (e->flags & KTJ_CREATE_DISPLAY_NS) != 0);
  e->started = true;
  e->processed = false;
  return KTJ_OK;
}

int ktj_intern_strings(ktj_engine* e, const char* blob, const uint64_t* offsets, size_t n, uint32_t* first_id) {
  if (!e || (n && (!blob || !offsets))) return KTJ_ERR_ARG;
  if (first_id) *first_id = (uint32_t)e->n_strings;
  if (e->bad_sink || n == 0) return KTJ_OK;
  if (e->n_strings + n >= KTJ_NONE) return KTJ_ERR_LIMIT;
  HIPCHK(hipSetDevice(e->device));
  const uint64_t src0 = offsets[0], nbytes = offsets[n] - offsets[0];
  std::vector<uint64_t> abs_off(n + 1);
  for (size_t i = 0; i <= n; ++i) {
    if (offsets[i] < src0 || (i && offsets[i] < offsets[i - 1])) return KTJ_ERR_ARG;
    abs_off[i] = e->blob_bytes + (offsets[i] - src0);
  }
  { const int rc = append_from_host(e, e->str_blob, blob + src0, nbytes); if (rc != KTJ_OK) return rc; }
  {
    /* entry n_strings already equals blob_bytes */
    const int rc = e->n_strings == 0 ? append_from_host(e, e->str_off, abs_off.data(), (n + 1) * 8)
                                     : append_from_host(e, e->str_off, abs_off.data() + 1, n * 8);
    if (rc != KTJ_OK) return rc;
  }
  e->n_strings += n;
  e->blob_bytes += nbytes;
  e->processed = false;
  return KTJ_OK;
}

int ktj_register_schema(ktj_engine* e, const ktj_field* f, size_t n_fields, uint32_t* schema_id) {
  if (!e || (n_fields && !f)) return KTJ_ERR_ARG;
  if (n_fields > KTJ_MAX_SCHEMA_FIELDS) return KTJ_ERR_LIMIT;
  int depth = 0;
  for (size_t i = 0; i < n_fields; ++i) {
    const uint16_t t = f[i].type;
    if (t > KTJ_F_UNSUPPORTED) return KTJ_ERR_ARG;
    const bool no_slots = t == KTJ_F_DICT_BEGIN || t == KTJ_F_DICT_END || t == KTJ_F_UNSUPPORTED;
    const bool array = t == KTJ_F_I64_ARRAY || t == KTJ_F_STR_ARRAY;
    if (no_slots ? f[i].count != 0 : array ? false : f[i].count != 1) return KTJ_ERR_ARG; /* arrays may be empty */
    if ((t == KTJ_F_DICT_BEGIN || t == KTJ_F_UNSUPPORTED) && f[i].key_id == KTJ_NONE) return KTJ_ERR_ARG;
    if (t == KTJ_F_DICT_BEGIN) ++depth;
    if (t == KTJ_F_DICT_END && --depth < 0) return KTJ_ERR_ARG;
  }
  if (depth != 0) return KTJ_ERR_ARG; /* every dict is closed */
  if (n_fields && f[0].type == KTJ_F_COLLECTIVE) e->coll_schemas = true;
  ktj_schema_desc d;
  d.first_field = (uint32_t)e->fields.size();
  d.n_fields = (uint32_t)n_fields;
  e->fields.insert(e->fields.end(), f, f + n_fields);
  if (schema_id) *schema_id = (uint32_t)e->schemas.size();
  e->schemas.push_back(d);
  e->schemas_dirty = true;
  e->processed = false;
  return KTJ_OK;
}

int ktj_add_collective(ktj_engine* e, const ktj_collective_meta* meta, uint32_t* index) {
  if (!e || !meta) return KTJ_ERR_ARG;
  if (e->collectives.size() >= KTJ_MAX_COLLECTIVES) return KTJ_ERR_LIMIT; /* the join tables keep 1 + index in 29 bits */
  if (index) *index = (uint32_t)e->collectives.size();
  e->collectives.push_back(make_collective(*meta));
  e->coll_dirty = true;
  e->processed = false;
  return KTJ_OK;
}

int ktj_submit_args(ktj_engine* e, const uint64_t* slots, size_t n_slots, uint64_t* first_slot) {
  if (!e || (n_slots && !slots)) return KTJ_ERR_ARG;
  if (first_slot) *first_slot = e->n_args;
  if (e->bad_sink || n_slots == 0) return KTJ_OK;
  HIPCHK(hipSetDevice(e->device));
  { const int rc = append_from_host(e, e->args, slots, n_slots * 8); if (rc != KTJ_OK) return rc; }
  e->n_args += n_slots;
  e->processed = false;
  return KTJ_OK;
}

int ktj_set_api_table(ktj_engine* e, const uint32_t* cid_name_ids, size_t n_cids, const uint32_t* flow_start_cids,
                      size_t n_flow_start, uint32_t malloc_cid) {
  if (!e || (n_cids && !cid_name_ids) || (n_flow_start && !flow_start_cids)) return KTJ_ERR_ARG;
  e->cid_names.assign(cid_name_ids, cid_name_ids + n_cids);
  e->flow_bits.assign((n_cids + 31) / 32 + 1, 0u);
  for (size_t i = 0; i < n_flow_start; ++i)
    if (flow_start_cids[i] < n_cids) e->flow_bits[flow_start_cids[i] >> 5] |= 1u << (flow_start_cids[i] & 31u);
  e->malloc_cid = malloc_cid;
  e->api_dirty = true;
  e->processed = false;
  return KTJ_OK;
}

int ktj_set_clock_model(ktj_engine* e, const ktj_clock_model* m) {
  if (!e || !m) return KTJ_ERR_ARG;
  if (m->runtime_mode > KTJ_CLOCK_OFFSET || m->device_mode > KTJ_CLOCK_OFFSET) return KTJ_ERR_ARG;
  e->clock = *m;
  e->processed = false;
  return KTJ_OK;
}

int ktj_set_window(ktj_engine* e, int64_t start_ns, int64_t end_ns) {
  if (!e) return KTJ_ERR_ARG;
  e->win_start = start_ns;
  e->win_end = end_ns;
  e->processed = false;
  return KTJ_OK;
}

static RecordSet* record_set(ktj_engine* e, int rec_class, size_t* rec_size) {
  switch (rec_class) {
    case KTJ_REC_GENERIC: *rec_size = sizeof(ktj_generic_rec); return &e->generic;
    case KTJ_REC_RUNTIME: *rec_size = sizeof(ktj_runtime_rec); return &e->runtime;
    case KTJ_REC_DEVICE: *rec_size = sizeof(ktj_device_rec); return &e->devrows;
    case KTJ_REC_EXTCORR: *rec_size = sizeof(ktj_extcorr_rec); return &e->extcorr;
    case KTJ_REC_USERCORR: *rec_size = sizeof(ktj_extcorr_rec); return &e->usercorr;
    default: return nullptr;
  }
}

static int flush_sdk_api_rows(ktj_engine* e);
/* rows of ktj_submit_sdk_api_record that wait on the host arrived before anything submitted now */
static bool class_has_buffered_sdk_rows(int rec_class) {
  return rec_class == KTJ_REC_RUNTIME || rec_class == KTJ_REC_EXTCORR || rec_class == KTJ_REC_USERCORR;
}

int ktj_submit_records(ktj_engine* e, int rec_class, const void* packed, size_t n_records) {
  if (!e || (n_records && !packed)) return KTJ_ERR_ARG;
  size_t rs = 0;
  RecordSet* set = record_set(e, rec_class, &rs);
  if (!set) return KTJ_ERR_ARG;
  if (e->bad_sink || n_records == 0) return KTJ_OK;
  if (class_has_buffered_sdk_rows(rec_class)) {
    const int flushed = flush_sdk_api_rows(e);
    if (flushed != KTJ_OK) return flushed;
  }
  if (set->external) return KTJ_ERR_STATE;
  HIPCHK(hipSetDevice(e->device));
  { const int rc = append_from_host(e, set->owned, packed, n_records * rs); if (rc != KTJ_OK) return rc; }
  set->n += n_records;
  if (rec_class == KTJ_REC_GENERIC || rec_class == KTJ_REC_RUNTIME || rec_class == KTJ_REC_DEVICE) e->activities_begun = true;
  e->processed = false;
  return KTJ_OK;
}

int ktj_host_alloc(ktj_engine* e, size_t n_bytes, void** host_ptr) {
  if (!e || !host_ptr) return KTJ_ERR_ARG;
  *host_ptr = nullptr;
  HIPCHK(hipSetDevice(e->device));
  void* p = nullptr;
  const hipError_t rc = hipHostMalloc(&p, n_bytes ? n_bytes : 16, hipHostMallocDefault);
  if (rc != hipSuccess) { e->last_error = std::string("hipHostMalloc: ") + hipGetErrorString(rc); return KTJ_ERR_NOMEM; }
  *host_ptr = p;
  return KTJ_OK;
}

int ktj_host_free(ktj_engine* e, void* host_ptr) {
  if (!e) return KTJ_ERR_ARG;
  if (!host_ptr) return KTJ_OK;
  HIPCHK(hipSetDevice(e->device));
  HIPCHK(hipHostFree(host_ptr));
  return KTJ_OK;
}

int ktj_submit_records_device(ktj_engine* e, int rec_class, const void* device_ptr, size_t n_records) {
  if (!e || (n_records && !device_ptr)) return KTJ_ERR_ARG;
  size_t rs = 0;
  RecordSet* set = record_set(e, rec_class, &rs);
  if (!set) return KTJ_ERR_ARG;
  if (((uintptr_t)device_ptr & 15u) != 0) return KTJ_ERR_ARG; /* kernels read 16-byte lanes */
  if (e->bad_sink) return KTJ_OK;
  if (class_has_buffered_sdk_rows(rec_class)) {
    const int flushed = flush_sdk_api_rows(e);
    if (flushed != KTJ_OK) return flushed;
  }
  if (set->owned.bytes != 0) return KTJ_ERR_STATE;
  set->external = n_records ? device_ptr : nullptr;
  set->n = n_records;
  if (n_records && (rec_class == KTJ_REC_GENERIC || rec_class == KTJ_REC_RUNTIME || rec_class == KTJ_REC_DEVICE)) e->activities_begun = true;
  e->processed = false;
  return KTJ_OK;
}

/* ---- rocprofiler-sdk buffer records (include/ktj_rocprofiler.h) ---- */

int ktj_set_sdk_agents(ktj_engine* e, const uint64_t* agent_handles, const int32_t* device_ids, size_t n) {
  if (!e || (n && (!agent_handles || !device_ids))) return KTJ_ERR_ARG;
  e->sdk_agents.clear();
  for (size_t i = 0; i < n; ++i) e->sdk_agents[agent_handles[i]] = device_ids[i];
  return KTJ_OK;
}

int ktj_set_sdk_kernel_names(ktj_engine* e, const uint64_t* kernel_ids, const uint32_t* name_ids, size_t n,
                             uint32_t unknown_name_id) {
  if (!e || (n && (!kernel_ids || !name_ids))) return KTJ_ERR_ARG;
  for (size_t i = 0; i < n; ++i) e->sdk_kernel_names[kernel_ids[i]] = name_ids[i];
  e->sdk_unknown_name = unknown_name_id;
  return KTJ_OK;
}

/* RocprofLogger::buffer_callback (libkineto/src/RocprofLogger.cpp:681-749): the fields of a
 * rocprofAsyncRow (src/RocLogger.h:216-240) from a kernel-dispatch or memory-copy record. */
int ktj_submit_sdk_buffer(ktj_engine* e, void* const* headers, size_t num_headers, uint64_t* n_rows) {
  if (n_rows) *n_rows = 0;
  if (!e || (num_headers && !headers)) return KTJ_ERR_ARG;
  std::vector<ktj_device_rec>& rows = e->sdk_rows;
  rows.clear();
  rows.reserve(num_headers);
  auto device_of = [e](uint64_t agent_handle) {
    const auto it = e->sdk_agents.find(agent_handle);
    return it != e->sdk_agents.end() ? it->second : -1;
  };
  for (size_t i = 0; i < num_headers; ++i) {
    const rocprofiler_record_header_t* h = static_cast<const rocprofiler_record_header_t*>(headers[i]);
    if (!h || h->category != ROCPROFILER_BUFFER_CATEGORY_TRACING || !h->payload) continue;
    ktj_device_rec r{};
    if (h->kind == ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH) {
      const auto& rec = *static_cast<const rocprofiler_buffer_tracing_kernel_dispatch_record_t*>(h->payload);
      const auto name = e->sdk_kernel_names.find(rec.dispatch_info.kernel_id);
      r.id = rec.correlation_id.internal;
      r.begin = rec.start_timestamp;
      r.end = rec.end_timestamp;
      r.domain = KTJ_DOM_KERNEL_DISPATCH;
      r.op = static_cast<uint32_t>(rec.operation);
      r.device = device_of(rec.dispatch_info.agent_id.handle);
      r.name_id = name != e->sdk_kernel_names.end() ? name->second : e->sdk_unknown_name;
      r.queue = rec.dispatch_info.queue_id.handle;
    } else if (h->kind == ROCPROFILER_BUFFER_TRACING_MEMORY_COPY) {
      const auto& rec = *static_cast<const rocprofiler_buffer_tracing_memory_copy_record_t*>(h->payload);
      r.id = rec.correlation_id.internal;
      r.begin = rec.start_timestamp;
      r.end = rec.end_timestamp;
      r.domain = KTJ_DOM_MEMORY_COPY;
      r.op = static_cast<uint32_t>(rec.operation);
      r.device = device_of(rec.dst_agent_id.handle);
      r.name_id = KTJ_NONE; /* the row's name is empty; the copy direction names the activity */
      r.queue = 0;
    } else {
      continue;
    }
    rows.push_back(r);
  }
  if (n_rows) *n_rows = rows.size();
  return ktj_submit_records(e, KTJ_REC_DEVICE, rows.data(), rows.size());
}

/* Runtime rows and correlation pairs that ktj_submit_sdk_api_record collected go to the device.  The
 * vectors are taken out first: the submit calls below flush whatever is buffered before they append. */
static int flush_sdk_api_rows(ktj_engine* e) {
  if (e->sdk_api_rows.empty() && e->sdk_api_ext.empty() && e->sdk_api_user.empty()) return KTJ_OK;
  std::vector<ktj_runtime_rec> rows; rows.swap(e->sdk_api_rows);
  std::vector<ktj_extcorr_rec> ext, user; ext.swap(e->sdk_api_ext); user.swap(e->sdk_api_user);
  int rc = KTJ_OK;
  if (!rows.empty()) rc = ktj_submit_records(e, KTJ_REC_RUNTIME, rows.data(), rows.size());
  if (rc == KTJ_OK && !ext.empty()) rc = ktj_submit_records(e, KTJ_REC_EXTCORR, ext.data(), ext.size());
  if (rc == KTJ_OK && !user.empty()) rc = ktj_submit_records(e, KTJ_REC_USERCORR, user.data(), user.size());
  if (rc != KTJ_OK) { /* nothing is lost: what a later flush finds is what this one could not place */
    e->sdk_api_rows.swap(rows); e->sdk_api_ext.swap(ext); e->sdk_api_user.swap(user);
  } else { /* keep the capacity for the next batch */
    rows.clear(); e->sdk_api_rows.swap(rows);
  }
  return rc;
}

int ktj_flush(ktj_engine* e) {
  if (!e) return KTJ_ERR_ARG;
  if (e->bad_sink) return KTJ_OK;
  return flush_sdk_api_rows(e);
}

#define KTJ_SDK_API_BATCH 65536u
int ktj_submit_sdk_api_record(ktj_engine* e, const void* record, uint64_t begin, uint64_t end, uint32_t pid, uint32_t tid,
                              const uint64_t* external_id, const uint64_t* user_external_id) {
  if (!e || !record) return KTJ_ERR_ARG;
  if (e->bad_sink) return KTJ_OK;
  const auto& rec = *static_cast<const rocprofiler_callback_tracing_record_t*>(record);
  if (rec.kind != ROCPROFILER_CALLBACK_TRACING_HIP_RUNTIME_API || !rec.payload) return KTJ_OK; /* RocprofLogger.cpp:567 */
  const auto& data = *static_cast<const rocprofiler_callback_tracing_hip_api_data_t*>(rec.payload);
  ktj_runtime_rec row;
  sdk_api::runtime_row(static_cast<uint32_t>(rec.operation), rec.correlation_id.internal, data.args, begin, end, pid, tid, &row);
  e->sdk_api_rows.push_back(row);
  if (external_id) e->sdk_api_ext.push_back(ktj_extcorr_rec{rec.correlation_id.internal, *external_id});
  if (user_external_id) e->sdk_api_user.push_back(ktj_extcorr_rec{rec.correlation_id.internal, *user_external_id});
  e->activities_begun = true;
  e->processed = false;
  return e->sdk_api_rows.size() >= KTJ_SDK_API_BATCH ? flush_sdk_api_rows(e) : KTJ_OK;
}

int ktj_begin_activities(ktj_engine* e) {
  if (!e) return KTJ_ERR_ARG;
  e->activities_begun = true;
  return KTJ_OK;
}

int ktj_submit_info(ktj_engine* e, int info_kind, const void* info) {
  if (!e || !info) return KTJ_ERR_ARG;
  if (e->bad_sink) return KTJ_OK;
  std::string& txt = e->activities_begun ? e->txt_after : e->txt_before;
  switch (info_kind) {
    case KTJ_INFO_DEVICE: append_device_info(txt, *static_cast<const ktj_device_info*>(info), e->base_time_ns); break;
    case KTJ_INFO_RESOURCE: append_resource_info(txt, *static_cast<const ktj_resource_info*>(info), e->base_time_ns); break;
    case KTJ_INFO_OVERHEAD: append_overhead_info(txt, *static_cast<const ktj_overhead_info*>(info), e->base_time_ns); break;
    case KTJ_INFO_SPAN: append_trace_span(txt, *static_cast<const ktj_trace_span*>(info), e->base_time_ns); break;
    default: return KTJ_ERR_ARG;
  }
  e->processed = false;
  return KTJ_OK;
}

/* One pass of the whole path.  out_device == nullptr: the document goes into the engine's own
 * buffer and working memory is allocated as needed (ktj_process).  Otherwise (ktj_process_noalloc,
 * e->noalloc set by the caller): the document goes into the caller's buffer of out_cap bytes and
 * every working buffer is a piece of the scratch array. */
static int process_pass(ktj_engine* e, int64_t end_time_ns, void* out_device, uint64_t out_cap) {
  HIPCHK(hipSetDevice(e->device));
  hipStream_t st = e->stream;
  { const int rc = put_pending_pieces(e); if (rc != KTJ_OK) return rc; }
  e->arena_used = 0;
  e->processed = false;
  e->total_bytes = 0;
  if (e->noalloc) e->schemas_dirty = e->api_dirty = e->coll_dirty = true; /* small tables live in the scratch array too */
  const uint64_t ng = e->generic.n, nr = e->runtime.n, nd = e->devrows.n, nx = e->extcorr.n, nu = e->usercorr.n;
  uint64_t N = ng + nr + nd; /* grows by the synthesised GPU user-annotation spans, at most one per device row */
  const uint64_t max_spans = nu ? nd : 0;
  if (N + max_spans >= 0xFFFFFFF0ull) { e->last_error = "more than 2^32 - 16 records"; return KTJ_ERR_LIMIT; }
  e->N = N;
  e->n_spans = 0;
  e->host_copy_valid = false;
  const uint64_t Na = N + max_spans ? N + max_spans : 1;

  /* small tables */
  if (e->schemas_dirty) {
    int rc = upload_small(e, e->d_fields, e->fields.data(), e->fields.size() * sizeof(ktj_field));
    if (rc) return rc;
    rc = upload_small(e, e->d_schemas, e->schemas.data(), e->schemas.size() * sizeof(ktj_schema_desc));
    if (rc) return rc;
    e->schemas_dirty = false;
  }
  if (e->api_dirty) {
    int rc = upload_small(e, e->d_cid_names, e->cid_names.data(), e->cid_names.size() * 4);
    if (rc) return rc;
    if (e->flow_bits.empty()) e->flow_bits.assign(1, 0u);
    rc = upload_small(e, e->d_flow_bits, e->flow_bits.data(), e->flow_bits.size() * 4);
    if (rc) return rc;
    e->api_dirty = false;
  }

  /* working memory */
  const uint32_t ns = (uint32_t)e->n_strings;
  if (nx >= 0x7FFFFFFFull || nr >= 0x7FFFFFFFull) { e->last_error = "more than 2^31 - 2 records of one class"; return KTJ_ERR_LIMIT; }
  /* capacities for the hash mode (load <= 2/3); the direct mode uses a prefix of the same buffers */
  const uint32_t cap_full = pow2_at_least((nr + nd) + (nr + nd) / 2);
  const uint32_t cap_narrow = pow2_at_least((nx + nr) + (nx + nr) / 2), cap_cpu = pow2_at_least(2 * ng);
  e->pool_used = 0;
  for (int phase = e->noalloc ? 1 : 0; phase < 2; ++phase) { /* 0: add the sizes up and size the pool; 1: hand the buffers out */
  e->measuring = phase == 0;
  e->pool_need = 0;
  NEED(e->d_name_len, (ns + 1) * 4ull); NEED(e->d_arg_len, (ns + 1) * 4ull);
  NEED(e->d_sflags, (ns + 1) * 4ull);
  NEED(e->d_name_off, (ns + 2) * 8ull); NEED(e->d_arg_off, (ns + 2) * 8ull);
  NEED(e->d_name_blob, e->blob_bytes * 2 + 8ull * ns + 16); NEED(e->d_arg_blob, e->blob_bytes + 16);
  NEED(e->c_ts, Na * 8); NEED(e->c_dur, Na * 8); NEED(e->c_corr, Na * 8);
  NEED(e->c_dev, Na * 8); NEED(e->c_res, Na * 8); NEED(e->c_meta, Na * 4);
  NEED(e->c_ext, Na * 4);
  NEED(e->t_full, (cap_full + 1ull) * 8); NEED(e->t_narrow, (cap_narrow + 1ull) * 8);
  NEED(e->t_cpu, (cap_cpu + 1ull) * 8);
  NEED(e->f_first, (cap_full + 1ull) * 4); NEED(e->f_stream_src, (cap_full + 1ull) * 4);
  NEED(e->f_pay, (cap_full + 1ull) * sizeof(FullPay));
  NEED(e->f_has_runtime, (cap_full / 32 + 2ull) * 4);
  NEED(e->n_ext_src, (cap_narrow + 1ull) * 4); NEED(e->n_kern_src, (cap_narrow + 1ull) * 4);
  NEED(e->n_copy_src, (cap_narrow + 1ull) * 4); NEED(e->n_pay, (cap_narrow + 1ull) * sizeof(NarrowPay));
  NEED(e->slot_f, nr * 4 + 16); NEED(e->slot_n, nr * 4 + 16);
  NEED(e->dev_link, nd * sizeof(DevLink) + 16);
  NEED(e->dev_brief, nd * sizeof(DevBrief) + 16);
  NEED(e->q_keys, (KTJ_QUEUE_CAP + 1ull) * 8); NEED(e->q_stream, (KTJ_QUEUE_CAP + 1ull) * 8);
  NEED(e->q_amb, (KTJ_QUEUE_CAP + 1ull) * 4);
  NEED(e->dn_hash, (KTJ_DENSE_CAP + 1ull) * 8); NEED(e->dn_first, (KTJ_DENSE_CAP + 1ull) * 4);
  NEED(e->dn_dev, (KTJ_DENSE_CAP + 1ull) * 4); NEED(e->dn_key, (KTJ_DENSE_CAP + 1ull) * 8);
  NEED(e->dn_rank, (KTJ_DENSE_CAP + 1ull) * 4);
  NEED(e->s_dev_k, (KTJ_SET_CAP + 1ull) * 8); NEED(e->s_dev_r, (KTJ_SET_CAP + 1ull) * 4);
  NEED(e->s_res_k, (KTJ_SET_CAP + 1ull) * 8); NEED(e->s_res_r, (KTJ_SET_CAP + 1ull) * 4);
  NEED(e->keys_a, Na * 8); NEED(e->keys_b, Na * 8);
  NEED(e->vals_a, Na * 4); NEED(e->vals_b, Na * 4);
  NEED(e->range_parts, (decode_blocks(ng) + 2 * decode_blocks(nr) + decode_blocks(nd) + 1) * sizeof(KeyRange));
  NEED(e->hist, radix_tmp_elems(Na) * 4);
  {
    uint64_t m = scan_tmp_elems(radix_tmp_elems(Na));
    const uint64_t m2 = scan_tmp_elems(Na), m3 = scan_tmp_elems(ns + 1ull);
    if (m2 > m) m = m2;
    if (m3 > m) m = m3;
    NEED(e->scan_tmp, m * 8);
  }
  NEED(e->mat, Na * sizeof(MatRow)); NEED(e->len, Na * 4); NEED(e->len_sorted, Na * 4); NEED(e->kind_sorted, Na + 16);
  NEED(e->offs, (Na + 1) * 8);
  if (e->measuring) {
    e->measuring = false;
    if (e->pool.cap < e->pool_need + 4096) HIPCHK(e->pool.ensure(e->pool_need + 4096));
  }
  }

  Scalars* sc = e->d_scalars.as<Scalars>();
  Columns c;
  c.ts = e->c_ts.as<int64_t>(); c.dur = e->c_dur.as<int64_t>(); c.corr = e->c_corr.as<uint64_t>();
  c.dev = e->c_dev.as<int64_t>(); c.res = e->c_res.as<int64_t>(); c.meta = e->c_meta.as<uint32_t>();
  c.ext = e->c_ext.as<int32_t>();
  const ktj_generic_rec* g_recs = static_cast<const ktj_generic_rec*>(e->generic.ptr());
  const ktj_runtime_rec* r_recs = static_cast<const ktj_runtime_rec*>(e->runtime.ptr());
  const ktj_device_rec* d_recs = static_cast<const ktj_device_rec*>(e->devrows.ptr());
  const ktj_extcorr_rec* x_recs = static_cast<const ktj_extcorr_rec*>(e->extcorr.ptr());

  /* an event on the stream costs the GPU a microsecond or two between two kernels: a trace of a few
   * records can do without the ten that separate the stages (KTJ_CREATE_NO_STAGE_TIMES) */
  const bool stage_times = !(e->flags & KTJ_CREATE_NO_STAGE_TIMES);
  HIPCHK(hipEventRecord(e->ev[EV_START], st));
  HIPCHK(init_scalars(sc, st));

  /* ---- stage 0: dictionary ---- */
  EmitCtx ctx;
  ctx.dict.name_blob = e->d_name_blob.as<char>(); ctx.dict.name_off = e->d_name_off.as<uint64_t>();
  ctx.dict.arg_blob = e->d_arg_blob.as<char>(); ctx.dict.arg_off = e->d_arg_off.as<uint64_t>();
  ctx.dict.raw_blob = e->str_blob.buf.as<char>(); ctx.dict.raw_off = e->str_off.buf.as<uint64_t>();
  ctx.dict.flags = e->d_sflags.as<uint32_t>(); ctx.dict.n = ns;
  ctx.fields = e->d_fields.as<ktj_field>(); ctx.schemas = e->d_schemas.as<ktj_schema_desc>();
  ctx.n_schemas = (uint32_t)e->schemas.size();
  ctx.args = e->args.buf.as<uint64_t>(); ctx.n_args = e->n_args;
  ctx.base_time_ns = e->base_time_ns;
  ctx.create_flags = e->flags;
  /* collective metadata is looked at only if both entries and a schema that refers to them exist */
  const uint32_t n_coll = e->coll_schemas ? (uint32_t)e->collectives.size() : 0u;
  if (n_coll && e->coll_dirty) {
    std::string blob;
    std::vector<uint64_t> off(e->collectives.size() + 1, 0);
    for (size_t k = 0; k < e->collectives.size(); ++k) { blob += e->collectives[k].args; off[k + 1] = blob.size(); }
    blob.append(16, '\0'); /* string copies load whole aligned words */
    int rc = upload_small(e, e->d_coll_blob, blob.data(), blob.size());
    if (rc == KTJ_OK) rc = upload_small(e, e->d_coll_off, off.data(), off.size() * 8);
    if (rc != KTJ_OK) return rc;
    e->coll_dirty = false;
  }
  ctx.coll_blob = e->d_coll_blob.as<char>(); ctx.coll_off = e->d_coll_off.as<uint64_t>(); ctx.n_coll = n_coll;
  uint32_t* cpu_row = nullptr; /* last CPU op per id: only where something is read from that op */
  if (n_coll || max_spans) {
    NEED(e->cpu_row, (cap_cpu + 1ull) * 4);
    cpu_row = e->cpu_row.as<uint32_t>();
    HIPCHK(fill_u32(cpu_row, 0, cap_cpu + 1ull, st));
  }
  if (n_coll) NEED(e->d_coll_first, 2ull * n_coll * 4);
  if (ns) {
    HIPCHK(dict_measure(e->str_blob.buf.as<char>(), e->str_off.buf.as<uint64_t>(), ns, e->d_name_len.as<uint32_t>(),
                        e->d_arg_len.as<uint32_t>(), e->d_sflags.as<uint32_t>(), st));
    HIPCHK(scan_u32_to_u64(e->d_name_len.as<uint32_t>(), e->d_name_off.as<uint64_t>(), ns, e->scan_tmp.as<uint64_t>(), st));
    HIPCHK(scan_u32_to_u64(e->d_arg_len.as<uint32_t>(), e->d_arg_off.as<uint64_t>(), ns, e->scan_tmp.as<uint64_t>(), st));
    HIPCHK(dict_write(e->str_blob.buf.as<char>(), e->str_off.buf.as<uint64_t>(), ns, e->d_name_off.as<uint64_t>(),
                      e->d_arg_off.as<uint64_t>(), e->d_sflags.as<uint32_t>(), e->d_name_blob.as<char>(),
                      e->d_arg_blob.as<char>(), st));
  }
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_DICT], st));

  /* ---- stage 1: decode ---- */
  KeyRange* parts = e->range_parts.as<KeyRange>(); /* [generic | runtime | runtime narrowed | device] */
  /* stage 2a, clock conversion and window filter, happens inside the runtime and device decode */
  ClockDev clk;
  clk.t0_approx = e->clock.t0_approx; clk.t0 = e->clock.t0;
  memcpy(&clk.scale_bits, &e->clock.scale, 8);
  clk.async_offset = e->clock.async_offset; clk.runtime_mode = e->clock.runtime_mode; clk.device_mode = e->clock.device_mode;
  HIPCHK(decode_generic(g_recs, ng, c, 0, sc, ctx, parts, st));
  HIPCHK(decode_runtime(r_recs, nr, c, ng, parts + decode_blocks(ng), parts + decode_blocks(ng) + decode_blocks(nr), clk,
                        e->win_start, e->win_end, sc, st));
  HIPCHK(decode_device(d_recs, nd, c, ng + nr, e->dev_brief.as<DevBrief>(), parts + decode_blocks(ng) + 2 * decode_blocks(nr), clk,
                       e->win_start, e->win_end, sc, st));
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_DECODE], st));
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_CONVERT], st));

  /* ---- stage 2b: joins ---- */
  Table tf{e->t_full.as<uint64_t>(), cap_full - 1, 0u, &sc->plan.ctl[KTJ_TBL_FULL]};
  Table tn{e->t_narrow.as<uint64_t>(), cap_narrow - 1, 0u, &sc->plan.ctl[KTJ_TBL_NARROW]};
  Table t_cpu{e->t_cpu.as<uint64_t>(), cap_cpu - 1, 1u, &sc->plan.ctl[KTJ_TBL_CPU]};
  FullCols fc{e->f_has_runtime.as<uint32_t>(), e->f_first.as<uint32_t>(), e->f_stream_src.as<uint32_t>(), e->f_pay.as<FullPay>()};
  NarrowCols nc{e->n_ext_src.as<uint32_t>(), e->n_kern_src.as<uint32_t>(), e->n_copy_src.as<uint32_t>(), e->n_pay.as<NarrowPay>()};
  HIPCHK(plan_tables(parts, ng, nr, nd, x_recs, nx, cap_full, cap_narrow, cap_cpu, (e->flags & KTJ_CREATE_HASH_JOIN) != 0, sc, st));
  HIPCHK(clear_tables(tf, fc, tn, nc, t_cpu, st));
  StreamTables stt{e->q_keys.as<uint64_t>(), e->q_stream.as<uint64_t>(), e->q_amb.as<uint32_t>(), e->dn_hash.as<uint64_t>(),
                   e->dn_first.as<uint32_t>(), e->dn_dev.as<int32_t>(), e->dn_key.as<uint64_t>(), e->dn_rank.as<uint32_t>()};
  SortSets sets{e->s_dev_k.as<uint64_t>(), e->s_dev_r.as<uint32_t>(), e->s_res_k.as<uint64_t>(), e->s_res_r.as<uint32_t>()};
  {
    FillJobs f;
    f.count = 0;
    f.add(stt.q_keys, KTJ_EMPTY_KEY, KTJ_QUEUE_CAP + 1ull, 8); f.add(stt.q_stream, 0, KTJ_QUEUE_CAP + 1ull, 8);
    f.add(stt.q_amb, 0, KTJ_QUEUE_CAP + 1ull, 4);
    f.add(stt.d_hash, KTJ_EMPTY_KEY, KTJ_DENSE_CAP + 1ull, 8); f.add(stt.d_first, 0xFFFFFFFFu, KTJ_DENSE_CAP + 1ull, 4);
    f.add(stt.d_rank, 0, KTJ_DENSE_CAP + 1ull, 4);
    f.add(sets.dev_keys, KTJ_EMPTY_KEY, KTJ_SET_CAP + 1ull, 8); f.add(sets.res_keys, KTJ_EMPTY_KEY, KTJ_SET_CAP + 1ull, 8);
    HIPCHK(fill_many(f, st));
  }
  ApiTable api{e->d_cid_names.as<uint32_t>(), (uint32_t)e->cid_names.size(), e->d_flow_bits.as<uint32_t>(), e->malloc_cid};
  MatRow* mat = e->mat.as<MatRow>();
  HIPCHK(build_cpu_ids(g_recs, ng, t_cpu, cpu_row, sc, st));
  HIPCHK(build_extcorr(x_recs, nx, tn, nc, t_cpu, cpu_row, g_recs, ctx, sc, st));
  HIPCHK(join_runtime_rows(r_recs, nr, c, ng, api, tf, fc, tn, nc, e->slot_f.as<uint32_t>(), e->slot_n.as<uint32_t>(), ctx, mat,
                           e->len.as<uint32_t>(), sc, st));
  HIPCHK(republish_runtime_rows(r_recs, nr, c, ng, fc, nc, e->slot_f.as<uint32_t>(), e->slot_n.as<uint32_t>(), sc, st));
  HIPCHK(link_device_rows(nd, c, ng + nr, tf, fc, tn, nc, e->dev_link.as<DevLink>(), sc, st));
  HIPCHK(backfill_streams(e->dev_brief.as<DevBrief>(), nd, c, ng + nr, stt, sc, st));
  if (max_spans) {
    const int rc = synthesise_user_spans(e, c, ctx, t_cpu, cpu_row, sc, N);
    if (rc != KTJ_OK) return rc;
    N += e->n_spans;
    e->N = N;
  }
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_JOIN], st));

  /* ---- stage 3: canonical order ---- */
  HIPCHK(collect_distinct(c, N, sets, sc, st));
  HIPCHK(rank_distinct(sets, sc, st));
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_SORT_A], st));
  HIPCHK(publish(sc, nullptr, nullptr, 0, &e->h_ctl_dev->scalars, nullptr, nullptr, st));
  if (!out_device && !e->noalloc && e->out.cap == 0) {
    /* An engine's first pass has no document buffer yet, and how long the document is comes out of
     * the scan.  A first guess is allocated here, while the GPU is busy with the join: per row the
     * fixed text of an event and one string of average length, at most 2 KB.  If that turns out too
     * small (or cannot be had) the buffer is allocated where its size is known, as in later passes. */
    const uint64_t avg_string = e->n_strings ? e->blob_bytes / e->n_strings : 0;
    const uint64_t per_row = KTJ_GUESS_BYTES_PER_ROW + avg_string < 2048 ? KTJ_GUESS_BYTES_PER_ROW + avg_string : 2048;
    if (e->out.ensure(N * per_row + (1u << 20), false) != hipSuccess) (void)hipGetLastError();
  }
  HIPCHK(hipStreamSynchronize(st));
  e->scalars = e->h_ctl->scalars;
  const unsigned distinct_overflow = e->scalars.error & (KTJ_DEVERR_DISTINCT_DEVICES | KTJ_DEVERR_DISTINCT_RESOURCES);
  if (e->scalars.error & ~distinct_overflow) {
    e->last_error = limit_text(e->scalars.error);
    return KTJ_ERR_LIMIT;
  }
  uint32_t ts_bits = 0, res_bits = 0, key_bits = 0, rank_bits = 0;
  if (e->scalars.n_valid) {
    ts_bits = (uint32_t)bits_for(e->scalars.ts_max_biased - e->scalars.ts_min_biased);
    res_bits = (uint32_t)bits_for(e->scalars.n_res_ranks ? e->scalars.n_res_ranks - 1 : 0);
    const uint32_t dev_bits = (uint32_t)bits_for(e->scalars.n_dev_ranks ? e->scalars.n_dev_ranks - 1 : 0);
    key_bits = ts_bits + res_bits + dev_bits;
    rank_bits = res_bits + dev_bits;
  }
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_SORT_B], st));
  {
    uint64_t* ka = e->keys_a.as<uint64_t>(); uint32_t* va = e->vals_a.as<uint32_t>();
    uint64_t* kb = e->keys_b.as<uint64_t>(); uint32_t* vb = e->vals_b.as<uint32_t>();
    uint32_t* hist = e->hist.as<uint32_t>(); uint64_t* scan_tmp = e->scan_tmp.as<uint64_t>();
    /* one more stable sort on top of the order so far: keys made from the rows in that order,
     * into the pair of buffers that does not hold it */
    auto sort_again = [&](auto make, uint32_t bits) -> int {
      const uint32_t* order = e->perm;
      if (order == va) { HIPCHK(make(order, kb, vb)); HIPCHK(radix_sort(kb, vb, ka, va, N, bits, hist, scan_tmp, &e->sorted_keys, &e->perm, st)); }
      else { HIPCHK(make(order, ka, va)); HIPCHK(radix_sort(ka, va, kb, vb, N, bits, hist, scan_tmp, &e->sorted_keys, &e->perm, st)); }
      return KTJ_OK;
    };
    if (distinct_overflow) {
      /* too many distinct deviceId or resourceId values for ranks: timestamp, then resourceId, then
       * deviceId, each on the raw values, then dropped rows to the back */
      HIPCHK(clear_error_bits(sc, distinct_overflow, st));
      HIPCHK(make_ts_keys(c, N, sc, ka, va, st));
      HIPCHK(radix_sort(ka, va, kb, vb, N, ts_bits, hist, scan_tmp, &e->sorted_keys, &e->perm, st));
      int rc = sort_again([&](const uint32_t* o, uint64_t* k, uint32_t* v) { return make_column_keys(c.res, c.meta, o, N, 0, k, v, st); }, 64);
      if (rc == KTJ_OK) rc = sort_again([&](const uint32_t* o, uint64_t* k, uint32_t* v) { return make_column_keys(c.dev, c.meta, o, N, 0, k, v, st); }, 64);
      if (rc == KTJ_OK) rc = sort_again([&](const uint32_t* o, uint64_t* k, uint32_t* v) { return make_column_keys(c.dev, c.meta, o, N, 1, k, v, st); }, 1);
      if (rc != KTJ_OK) return rc;
    } else if (key_bits <= 62 && e->sort_mode != 1 && sort_packed_fits(N, key_bits)) {
      HIPCHK(sort_packed(c, N, sets, sc, ts_bits, res_bits, key_bits, ka, kb, va, hist, scan_tmp, st));
      e->perm = va;
      e->sorted_keys = nullptr;
    } else if (key_bits <= 62) {
      HIPCHK(make_keys(c, N, sets, sc, ts_bits, res_bits, key_bits, ka, va, st));
      HIPCHK(radix_sort(ka, va, kb, vb, N, key_bits + 1, hist, scan_tmp, &e->sorted_keys, &e->perm, st));
    } else {
      /* timestamp span too wide for one composite key: stable sort by timestamp, then by ranks
       * (at most 2 x 12 bits) */
      HIPCHK(make_ts_keys(c, N, sc, ka, va, st));
      HIPCHK(radix_sort(ka, va, kb, vb, N, ts_bits, hist, scan_tmp, &e->sorted_keys, &e->perm, st));
      const int rc = sort_again([&](const uint32_t* o, uint64_t* k, uint32_t* v) { return make_rank_keys(c, o, N, sets, res_bits, rank_bits, k, v, st); },
                                rank_bits + 1);
      if (rc != KTJ_OK) return rc;
    }
  }
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_SORT], st));

  /* ---- stage 4a: joined rows + lengths ---- */
  const uint32_t* sync_first = nullptr;
  if (e->scalars.n_sync_typed != 0) { /* known since the read-back before the sort */
    NEED(e->sync_keys, (KTJ_SYNC_CAP + 1ull) * 8); NEED(e->sync_pos, (KTJ_SYNC_CAP + 1ull) * 4);
    NEED(e->sync_first, ng * 4 + 16);
    HIPCHK(stream_sync_first(e->perm, e->scalars.n_valid, g_recs, ng, c.dev, ctx.dict, e->sync_keys.as<uint64_t>(),
                             e->sync_pos.as<uint32_t>(), e->sync_first.as<uint32_t>(), sc, st));
    sync_first = e->sync_first.as<uint32_t>();
  }
  HIPCHK(mat_generic_rows(g_recs, ng, 0, ctx, sync_first, mat, e->len.as<uint32_t>(), sc, st));
  HIPCHK(mat_generic_rows(e->synth_recs.as<ktj_generic_rec>(), e->n_spans, ng + nr + nd, ctx, nullptr, mat, e->len.as<uint32_t>(),
                          sc, st));
  HIPCHK(mat_device_rows(d_recs, nd, c, ng + nr, e->dev_link.as<DevLink>(), ctx, mat, e->len.as<uint32_t>(), sc, st));
  HIPCHK(gather_len(e->perm, e->len.as<uint32_t>(), N, e->len_sorted.as<uint32_t>(), e->kind_sorted.as<uint8_t>(), st));
  if (n_coll) HIPCHK(collective_first(mat, e->perm, e->scalars.n_valid, n_coll, e->d_coll_first.as<uint32_t>(), st));
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_SIZE], st));

  /* ---- scan ---- */
  HIPCHK(scan_u32_to_u64(e->len_sorted.as<uint32_t>(), e->offs.as<uint64_t>(), N, e->scan_tmp.as<uint64_t>(), st));
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_SCAN], st));
  uint64_t act_bytes = 0;
  e->coll_first.assign(2ull * n_coll, 0xFFFFFFFFu);
  const bool list_fits = 2ull * n_coll * 4 <= e->pinned_small_cap; /* through the engine's pinned buffer when it fits */
  if (n_coll && !list_fits && e->noalloc) {
    e->last_error = "ktj_process_noalloc: too many collective entries for the pinned staging buffer";
    return KTJ_ERR_LIMIT;
  }
  HIPCHK(publish(sc, e->offs.as<uint64_t>() + N, e->d_coll_first.as<uint32_t>(), list_fits ? 2u * n_coll : 0u, &e->h_ctl_dev->scalars,
                 &e->h_ctl_dev->act_bytes, reinterpret_cast<uint32_t*>(e->pinned_small_dev), st));
  if (n_coll && !list_fits) HIPCHK(hipMemcpyAsync(e->coll_first.data(), e->d_coll_first.p, 2ull * n_coll * 4, hipMemcpyDeviceToHost, st));
  HIPCHK(hipStreamSynchronize(st));
  if (n_coll && list_fits) memcpy(e->coll_first.data(), e->pinned_small, 2ull * n_coll * 4);
  act_bytes = e->h_ctl->act_bytes;
  e->scalars = e->h_ctl->scalars;
  if (e->scalars.error) {
    e->last_error = limit_text(e->scalars.error);
    return KTJ_ERR_LIMIT;
  }
  std::string distributed_info;
  if (n_coll) { /* the uses in emission order: one per entry and backend is enough, later ones repeat it */
    std::vector<std::pair<uint32_t, uint32_t>> firsts; /* (position, 2 * index + hccl) */
    for (uint32_t k = 0; k < 2u * n_coll; ++k)
      if (e->coll_first[k] != 0xFFFFFFFFu) firsts.emplace_back(e->coll_first[k], k);
    std::sort(firsts.begin(), firsts.end());
    std::vector<CollectiveUse> uses;
    for (const auto& f : firsts) uses.push_back(CollectiveUse{f.second >> 1, (f.second & 1u) != 0});
    distributed_info = distributed_info_text(e->collectives, uses);
  }

  /* ---- emit ---- */
  std::string prefix = e->txt_header + e->txt_before;
  std::string suffix = e->txt_after;
  append_trace_end(suffix, end_time_ns, e->base_time_ns, e->out_path, distributed_info);
  e->prefix_len = prefix.size();
  e->act_bytes = act_bytes;
  e->total_bytes = prefix.size() + act_bytes + suffix.size();
  if (out_device) { /* the caller's buffer: whole 16-byte blocks are stored, so a little room past the end is needed */
    if (e->total_bytes + 64 > out_cap) {
      e->last_error = "ktj_process_noalloc: the document has " + std::to_string(e->total_bytes) + " bytes and needs an output buffer of " +
                      std::to_string(e->total_bytes + 64);
      return KTJ_ERR_LIMIT;
    }
    e->out.borrow(out_device, out_cap);
  } else NEED(e->out, e->total_bytes + 64);
  const size_t small = prefix.size() + suffix.size() + 64; /* each piece starts where its place in the document does, modulo 16 */
  if (small > e->pinned_small_cap && e->noalloc) {
    e->last_error = "ktj_process_noalloc: header and footer text of " + std::to_string(small) + " bytes exceeds the pinned staging buffer";
    return KTJ_ERR_LIMIT;
  }
  if (small > e->pinned_small_cap) {
    if (e->pinned_small) HIPCHK(hipHostFree(e->pinned_small));
    e->pinned_small = nullptr;
    e->pinned_small_cap = 0;
    HIPCHK(hipHostMalloc(&e->pinned_small, small * 2 + 4096, hipHostMallocDefault));
    e->pinned_small_cap = small * 2 + 4096;
    void* d = nullptr;
    HIPCHK(hipHostGetDevicePointer(&d, e->pinned_small, 0));
    e->pinned_small_dev = static_cast<char*>(d);
  }
  {
    char* dst_a = e->out.as<char>();
    char* dst_b = dst_a + prefix.size() + act_bytes;
    const size_t at_a = (size_t)(((uintptr_t)dst_a - (uintptr_t)e->pinned_small_dev) & 15u);
    const size_t after_a = (at_a + prefix.size() + 15u) & ~(size_t)15u;
    const size_t at_b = after_a + (size_t)(((uintptr_t)dst_b - (uintptr_t)(e->pinned_small_dev + after_a)) & 15u);
    memcpy(static_cast<char*>(e->pinned_small) + at_a, prefix.data(), prefix.size());
    memcpy(static_cast<char*>(e->pinned_small) + at_b, suffix.data(), suffix.size());
    HIPCHK(put_text(e->pinned_small_dev + at_a, dst_a, prefix.size(), e->pinned_small_dev + at_b, dst_b, suffix.size(), st));
  }
  const uint32_t tile = emit_tile_bytes(act_bytes, e->scalars.n_valid);
  NEED(e->tile_start, (emit_tile_count(e->prefix_len, act_bytes, tile) + 2) * 4);
  if (stage_times) HIPCHK(hipEventRecord(e->ev[EV_EMIT_START], st));
  {
    if (e->flags & KTJ_CREATE_TILE_EMIT)
      HIPCHK(emit(mat, e->perm, e->offs.as<uint64_t>(), N, ctx, e->out.as<char>(), e->prefix_len, act_bytes, tile,
                  e->tile_start.as<uint32_t>(), st));
    else
      HIPCHK(emit_direct(mat, e->perm, e->offs.as<uint64_t>(), e->kind_sorted.as<uint8_t>(), e->scalars.n_valid, act_bytes, ctx,
                         e->out.as<char>(), e->prefix_len, st));
  }
  HIPCHK(hipEventRecord(e->ev[EV_EMIT], st));
  HIPCHK(hipStreamSynchronize(st));

  /* ---- statistics ---- */
  ktj_stats& s = e->stats;
  memset(&s, 0, sizeof s);
  s.n_generic = ng; s.n_runtime = nr; s.n_device = nd; s.n_extcorr = nx;
  s.n_emitted = e->scalars.n_valid;
  s.out_of_range_events = e->scalars.out_of_range;
  s.gpu_and_cpu_op_out_of_order = e->scalars.out_of_order;
  s.n_flow_events = e->scalars.n_flow;
  s.n_linked = e->scalars.n_linked;
  s.n_blank_names = e->scalars.n_blank_names;
  s.output_bytes = e->total_bytes;
  s.activity_bytes = act_bytes;
  /* stage time = elapsed between the events that bracket it; the two host read-backs (after the
   * distinct-value ranking and after the scan) are excluded from the per-stage figures but are
   * part of KTJ_STAGE_TOTAL_GPU */
  struct { int stage, from, to; } spans[] = {
      {KTJ_STAGE_DICT, EV_START, EV_DICT},       {KTJ_STAGE_DECODE, EV_DICT, EV_DECODE},
      {KTJ_STAGE_DECODE, EV_DECODE, EV_CONVERT}, {KTJ_STAGE_JOIN, EV_CONVERT, EV_JOIN},
      {KTJ_STAGE_SORT, EV_JOIN, EV_SORT_A},      {KTJ_STAGE_SORT, EV_SORT_B, EV_SORT},
      {KTJ_STAGE_SIZE, EV_SORT, EV_SIZE},        {KTJ_STAGE_SCAN, EV_SIZE, EV_SCAN},
      {KTJ_STAGE_EMIT, EV_EMIT_START, EV_EMIT}};
  for (const auto& sp : spans) {
    if (!stage_times) break;
    float ms = 0;
    HIPCHK(hipEventElapsedTime(&ms, e->ev[sp.from], e->ev[sp.to]));
    s.stage_ms[sp.stage] += ms;
  }
  {
    float ms = 0;
    HIPCHK(hipEventElapsedTime(&ms, e->ev[EV_START], e->ev[EV_EMIT]));
    s.stage_ms[KTJ_STAGE_TOTAL_GPU] = ms;
  }
  const uint64_t raw_in = ng * sizeof(ktj_generic_rec) + nr * sizeof(ktj_runtime_rec) + nd * sizeof(ktj_device_rec);
  s.stage_bytes[KTJ_STAGE_DICT] = e->blob_bytes * 3;
  /* clock conversion and window filter run inside the decode kernels on values that are in registers
   * there: their bytes (two timestamps in, two out) are bytes of the decode stage already */
  s.stage_bytes[KTJ_STAGE_DECODE] = raw_in + N * 48;
  s.stage_bytes[KTJ_STAGE_CONVERT] = 0;
  s.stage_bytes[KTJ_STAGE_JOIN] = nx * 12 + ng * 12 + nr * 12 + (nr + nd) * 12 * 2 +
                                   nr * (sizeof(ktj_runtime_rec) + 48 + sizeof(MatRow) + 4); /* incl. the runtime rows' joined rows */
  s.stage_bytes[KTJ_STAGE_SORT] = N * 56;
  s.stage_bytes[KTJ_STAGE_SIZE] = (ng * sizeof(ktj_generic_rec) + nd * sizeof(ktj_device_rec)) + (ng + nd) * 48 +
                                   (ng + nd) * (sizeof(MatRow) + 4) + N * 8;
  s.stage_bytes[KTJ_STAGE_SCAN] = N * 12;
  s.stage_bytes[KTJ_STAGE_EMIT] = e->scalars.n_valid * (sizeof(MatRow) + 12) + act_bytes;
  e->processed = true;
  return KTJ_OK;
}

int ktj_process(ktj_engine* e, int64_t end_time_ns) {
  if (!e) return KTJ_ERR_ARG;
  if (e->bad_sink) return KTJ_OK;
  const int flushed = flush_sdk_api_rows(e);
  if (flushed != KTJ_OK) return flushed;
  e->noalloc = false;
  return process_pass(e, end_time_ns, nullptr, 0);
}

/* The pass with no allocation in it: working memory is this GPU's copy of the static scratch
 * array, the document goes to the caller's buffer, small tables and read-backs go through the
 * pinned buffers that ktj_create allocated. */
int ktj_process_noalloc(ktj_engine* e, int64_t end_time_ns, void* out_device, uint64_t out_capacity, uint64_t* n_bytes) {
  if (n_bytes) *n_bytes = 0;
  if (!e || !out_device || ((uintptr_t)out_device & 15u) != 0) return KTJ_ERR_ARG;
  if (e->bad_sink) return KTJ_OK;
  if (!e->arena) { e->last_error = "ktj_process_noalloc: no scratch array on this device"; return KTJ_ERR_STATE; }
  if (!e->sdk_api_rows.empty() || !e->sdk_api_ext.empty() || !e->sdk_api_user.empty()) {
    e->last_error = "ktj_process_noalloc: rows of ktj_submit_sdk_api_record are still buffered on the host (call ktj_flush first: it may allocate)";
    return KTJ_ERR_STATE;
  }
  if (e->usercorr.n != 0) {
    e->last_error = "ktj_process_noalloc: user-domain correlation records (GPU user annotations) are not supported here";
    return KTJ_ERR_LIMIT;
  }
  e->noalloc = true;
  const int rc = process_pass(e, end_time_ns, out_device, out_capacity);
  e->noalloc = false;
  /* The small tables of this pass sit in the scratch array, which every engine on this GPU shares:
   * whatever the pass returned, the next allocating pass must upload them into its own buffers again. */
  e->schemas_dirty = e->api_dirty = e->coll_dirty = true;
  if (n_bytes) *n_bytes = e->total_bytes; /* on KTJ_ERR_LIMIT for a short output buffer: the size that is needed */
  return rc;
}

int ktj_output_device(ktj_engine* e, const void** device_ptr, uint64_t* n_bytes) {
  if (!e || !device_ptr || !n_bytes) return KTJ_ERR_ARG;
  if (!e->processed) return KTJ_ERR_STATE;
  *device_ptr = e->out.p;
  *n_bytes = e->total_bytes;
  return KTJ_OK;
}

int ktj_output_host(ktj_engine* e, const char** host_ptr, uint64_t* n_bytes) {
  if (!e || !host_ptr || !n_bytes) return KTJ_ERR_ARG;
  if (!e->processed) return KTJ_ERR_STATE;
  HIPCHK(hipSetDevice(e->device));
  if (!e->host_copy_valid) {
    if (e->total_bytes > e->pinned_out_cap) {
      if (e->pinned_out) HIPCHK(hipHostFree(e->pinned_out));
      e->pinned_out = nullptr; e->pinned_out_cap = 0;
      void* p = nullptr;
      HIPCHK(hipHostMalloc(&p, e->total_bytes + 4096, hipHostMallocDefault));
      e->pinned_out = static_cast<char*>(p);
      e->pinned_out_cap = e->total_bytes + 4096;
    }
    HIPCHK(hipEventRecord(e->ev_d2h[0], e->stream));
    HIPCHK(hipMemcpyAsync(e->pinned_out, e->out.p, e->total_bytes, hipMemcpyDeviceToHost, e->stream));
    HIPCHK(hipEventRecord(e->ev_d2h[1], e->stream));
    HIPCHK(hipStreamSynchronize(e->stream));
    float ms = 0;
    HIPCHK(hipEventElapsedTime(&ms, e->ev_d2h[0], e->ev_d2h[1]));
    e->stats.stage_ms[KTJ_STAGE_D2H] = ms;
    e->stats.stage_bytes[KTJ_STAGE_D2H] = e->total_bytes;
    e->host_copy_valid = true;
  }
  *host_ptr = e->pinned_out;
  *n_bytes = e->total_bytes;
  return KTJ_OK;
}

/* The file sink streams the document from HBM through two small pinned buffers: the copy of one
 * chunk runs while the previous one is written.  One pinned buffer for the whole document would
 * cost more than the copy and the write together: its pages are mapped for the CPU one fault at a
 * time when write() first reads them (0.9 s for 1.6 GB, against 0.03 s for the copy and 0.15 s for
 * the write into the page cache). */
#define KTJ_FILE_STAGE_BYTES (16ull << 20)
static int stream_document_to_file(ktj_engine* e, int fd, float* copy_wait_ms) {
  const uint64_t n = e->total_bytes;
  const uint64_t n_chunks = (n + KTJ_FILE_STAGE_BYTES - 1) / KTJ_FILE_STAGE_BYTES;
  for (uint64_t k = 0; k < 2 && k < n_chunks; ++k) { /* small documents take one small buffer */
    const size_t need = (size_t)((std::min<uint64_t>(KTJ_FILE_STAGE_BYTES, n) + 65535) & ~65535ull);
    if (e->file_stage_cap[k] < need) {
      if (e->file_stage[k]) HIPCHK(hipHostFree(e->file_stage[k]));
      e->file_stage[k] = nullptr; e->file_stage_cap[k] = 0;
      void* p = nullptr;
      HIPCHK(hipHostMalloc(&p, need, hipHostMallocDefault));
      e->file_stage[k] = static_cast<char*>(p);
      e->file_stage_cap[k] = need;
    }
    if (!e->ev_file_stage[k]) HIPCHK(hipEventCreateWithFlags(&e->ev_file_stage[k], hipEventDisableTiming));
  }
  auto chunk_len = [n](uint64_t c) { return std::min<uint64_t>(KTJ_FILE_STAGE_BYTES, n - c * KTJ_FILE_STAGE_BYTES); };
  auto start_copy = [e, &chunk_len](uint64_t c) -> hipError_t {
    hipError_t rc = hipMemcpyAsync(e->file_stage[c & 1], static_cast<const char*>(e->out.p) + c * KTJ_FILE_STAGE_BYTES,
                                   chunk_len(c), hipMemcpyDeviceToHost, e->stream);
    return rc != hipSuccess ? rc : hipEventRecord(e->ev_file_stage[c & 1], e->stream);
  };
  double waited = 0;
  if (n_chunks) HIPCHK(start_copy(0));
  for (uint64_t c = 0; c < n_chunks; ++c) {
    /* the other buffer is free: its chunk (c - 1) has been written */
    if (c + 1 < n_chunks) HIPCHK(start_copy(c + 1));
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    HIPCHK(hipEventSynchronize(e->ev_file_stage[c & 1]));
    clock_gettime(CLOCK_MONOTONIC, &t1);
    waited += (t1.tv_sec - t0.tv_sec) * 1e3 + (t1.tv_nsec - t0.tv_nsec) * 1e-6;
    const char* src = e->file_stage[c & 1];
    uint64_t left = chunk_len(c);
    while (left) {
      const ssize_t w = write(fd, src, left);
      if (w < 0 && errno == EINTR) continue;
      if (w <= 0) { (void)hipStreamSynchronize(e->stream); return KTJ_ERR_IO; }
      src += w; left -= (uint64_t)w;
    }
  }
  if (copy_wait_ms) *copy_wait_ms = (float)waited;
  return KTJ_OK;
}

int ktj_finalize(ktj_engine* e, int64_t end_time_ns, uint64_t* bytes_written) {
  if (!e) return KTJ_ERR_ARG;
  if (bytes_written) *bytes_written = 0;
  if (e->bad_sink) { /* output_json.cpp:1067-1070 */
    e->last_error = "Failed to write to log file!";
    return KTJ_ERR_IO;
  }
  int rc = ktj_process(e, end_time_ns);
  if (rc != KTJ_OK) return rc;
  if (e->flags & KTJ_CREATE_NO_FILE) {
    if (bytes_written) *bytes_written = e->total_bytes;
    return KTJ_OK;
  }
  HIPCHK(hipSetDevice(e->device));
  const uint64_t n = e->total_bytes;
  struct timespec t0, t1;
  clock_gettime(CLOCK_MONOTONIC, &t0);
  if (!e->sink) return KTJ_ERR_STATE;
  float copy_wait_ms = 0;
  rc = fflush(e->sink) == 0 ? stream_document_to_file(e, fileno(e->sink), &copy_wait_ms) : KTJ_ERR_IO;
  const int crc = fclose(e->sink);
  e->sink = nullptr;
  if (rc == KTJ_ERR_IO || (rc == KTJ_OK && crc != 0)) { e->last_error = "short write to " + e->tmp_path; return KTJ_ERR_IO; }
  if (rc != KTJ_OK) return rc;
  e->stats.stage_ms[KTJ_STAGE_D2H] = copy_wait_ms; /* time the writer waited for copies */
  e->stats.stage_bytes[KTJ_STAGE_D2H] = n;
  remove(e->out_path.c_str()); /* output_json.cpp:1100-1107 */
  if (rename(e->tmp_path.c_str(), e->out_path.c_str()) != 0) {
    e->last_error = "Failed to rename " + e->tmp_path + " to " + e->out_path + ": " + strerror(errno);
    return KTJ_ERR_IO;
  }
  clock_gettime(CLOCK_MONOTONIC, &t1);
  e->stats.stage_ms[KTJ_STAGE_FILE] = (float)((t1.tv_sec - t0.tv_sec) * 1e3 + (t1.tv_nsec - t0.tv_nsec) * 1e-6);
  e->stats.stage_bytes[KTJ_STAGE_FILE] = n;
  if (bytes_written) *bytes_written = n;
  return KTJ_OK;
}

int ktj_get_stats(ktj_engine* e, ktj_stats* out) {
  if (!e || !out) return KTJ_ERR_ARG;
  *out = e->stats;
  return KTJ_OK;
}

void ktj_debug_force_sort_passes(int on) { sort_packed_force_passes(on != 0); }

int ktj_debug_copy_reference(ktj_engine* e, uint64_t n_bytes, float* ms) {
  if (!e || !ms) return KTJ_ERR_ARG;
  HIPCHK(hipSetDevice(e->device));
  DevBuf a, b;
  HIPCHK(a.ensure(n_bytes));
  HIPCHK(b.ensure(n_bytes));
  HIPCHK(hipMemsetAsync(a.p, 1, n_bytes, e->stream));
  HIPCHK(copy_reference(a.p, b.p, n_bytes, e->stream)); /* warm-up */
  HIPCHK(hipEventRecord(e->ev_d2h[0], e->stream));
  HIPCHK(copy_reference(a.p, b.p, n_bytes, e->stream));
  HIPCHK(hipEventRecord(e->ev_d2h[1], e->stream));
  HIPCHK(hipStreamSynchronize(e->stream));
  HIPCHK(hipEventElapsedTime(ms, e->ev_d2h[0], e->ev_d2h[1]));
  a.release();
  b.release();
  return KTJ_OK;
}

int ktj_debug_fetch(ktj_engine* e, int what, void* dst, uint64_t cap, uint64_t* n_bytes) {
  if (!e || !n_bytes) return KTJ_ERR_ARG;
  if (!e->processed) return KTJ_ERR_STATE;
  const void* src = nullptr;
  uint64_t n = 0;
  const uint64_t N = e->N;
  switch (what) {
    case KTJ_DBG_COL_TS: src = e->c_ts.p; n = N * 8; break;
    case KTJ_DBG_COL_DUR: src = e->c_dur.p; n = N * 8; break;
    case KTJ_DBG_COL_DEV: src = e->c_dev.p; n = N * 8; break;
    case KTJ_DBG_COL_RES: src = e->c_res.p; n = N * 8; break;
    case KTJ_DBG_COL_META: src = e->c_meta.p; n = N * 4; break;
    case KTJ_DBG_COL_EXT: src = e->c_ext.p; n = N * 4; break;
    case KTJ_DBG_PERM: src = e->perm; n = N * 4; break;
    case KTJ_DBG_LEN: src = e->len_sorted.p; n = N * 4; break;
    case KTJ_DBG_OFFS: src = e->offs.p; n = (N + 1) * 8; break;
    case KTJ_DBG_MAT: src = e->mat.p; n = N * sizeof(MatRow); break;
    case KTJ_DBG_SORT_KEYS:
      if (!e->sorted_keys) { e->last_error = "the sorted keys exist only in an engine created with KTJ_CREATE_PAIR_SORT"; return KTJ_ERR_STATE; }
      src = e->sorted_keys; n = N * 8; break;
    case KTJ_DBG_NAME_VIEW: src = e->d_name_blob.p; n = e->blob_bytes * 2 + 8ull * e->n_strings; break;
    case KTJ_DBG_NAME_OFF: src = e->d_name_off.p; n = (e->n_strings + 1) * 8; break;
    case KTJ_DBG_ARG_VIEW: src = e->d_arg_blob.p; n = e->blob_bytes; break;
    case KTJ_DBG_ARG_OFF: src = e->d_arg_off.p; n = (e->n_strings + 1) * 8; break;
    default: return KTJ_ERR_ARG;
  }
  *n_bytes = n;
  if (dst && src && n) {
    HIPCHK(hipSetDevice(e->device));
    HIPCHK(hipMemcpy(dst, src, n < cap ? n : cap, hipMemcpyDeviceToHost));
  }
  return KTJ_OK;
}

}  // extern "C"
