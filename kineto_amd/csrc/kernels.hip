/*
 * kernels.hip — HIP kernels of the trace post-processing engine, written for gfx950 (CDNA4):
 * 64-wide wavefronts, ballot/popcount based ranking, LDS-staged tiles, 16-byte lanes.
 *
 * Nothing here is a dense contraction, so there is no MFMA; every kernel is bound by HBM (or,
 * for the hash joins, by random 64-byte sector access).  Stage by stage:
 *   0  dictionary   strings → name view (logger's name pipeline) and arg view (sanitised)
 *   1  decode       packed activity records → columns, through LDS so that global reads are
 *                   lane-consecutive 16-byte loads
 *   2  convert/join clock model, window filter, external-correlation join, runtime↔device join,
 *                   stream back-fill with dense per-device stream indices
 *   3  order        dense ranks of (device, resource), 64-bit composite keys, stable LSD radix sort
 *   4  size/emit    exact byte length per activity, device-wide exclusive scan, output-partitioned
 *                   tiles formatted in LDS and flushed with aligned 16-byte stores
 */
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <mutex>

#include "gpu_stages.h"

namespace ktj {
namespace gpu {

#define KTJ_NOSLOT 0xFFFFFFFFu
#define KTJ_BLOCK 256

/* ------------------------------------------------------------------------------------------ */
/* helpers                                                                                      */
/* ------------------------------------------------------------------------------------------ */
__device__ __forceinline__ uint64_t hash64(uint64_t x) {
  x ^= x >> 33; x *= 0xff51afd7ed558ccdULL; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ULL; x ^= x >> 33;
  return x;
}
__device__ __forceinline__ uint32_t lane_id() { return threadIdx.x & 63u; }
/* Values that a pass streams through once — a row's own columns and records, the rows it writes —
 * are loaded and stored past the L2's usual replacement: what the cache is for in these passes are
 * the table lines that rows reach at random. */
template <typename T> __device__ __forceinline__ T load_once(const T* p) { return __builtin_nontemporal_load(p); }
template <typename T> __device__ __forceinline__ void store_once(T* p, T v) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ uint64_t lanemask_lt() { return (1ULL << lane_id()) - 1ULL; }

/* Returns the slot holding `key`, inserting it if absent; KTJ_NOSLOT when no free slot lies within
 * KTJ_TABLE_PROBES slots of the key's home slot (a table that is at most half full never gets
 * there; one that is close to full does at once, so that an input with far too many distinct keys
 * costs a bounded number of probes per row and is reported instead of crawling). */
__device__ uint32_t table_insert(uint64_t* keys, uint32_t mask, uint64_t key) {
  if (key == KTJ_EMPTY_KEY) { keys[mask + 1u] = 0; return mask + 1u; }
  uint32_t slot = (uint32_t)hash64(key) & mask;
  for (uint32_t probe = 0; probe <= mask && probe < KTJ_TABLE_PROBES; ++probe) {
    uint64_t cur = keys[slot];
    if (cur == key) return slot;
    if (cur == KTJ_EMPTY_KEY) {
      unsigned long long prev = atomicCAS((unsigned long long*)&keys[slot], (unsigned long long)KTJ_EMPTY_KEY,
                                          (unsigned long long)key);
      if (prev == KTJ_EMPTY_KEY || prev == key) return slot;
    }
    slot = (slot + 1u) & mask;
  }
  return KTJ_NOSLOT;
}
/* table_insert for a table with a documented limit on its distinct keys: the key that would be
 * number `limit` + 1 is refused (KTJ_NOSLOT), whatever room the table still has, so that a trace is
 * accepted or refused by the count the limit names and not by how its keys happen to hash. */
__device__ uint32_t table_insert_counted(uint64_t* keys, uint32_t mask, uint64_t key, unsigned int* count, uint32_t limit) {
  if (key == KTJ_EMPTY_KEY) {
    if (atomicExch((unsigned long long*)&keys[mask + 1u], 0ULL) != 0ULL && atomicAdd(count, 1u) >= limit) return KTJ_NOSLOT;
    return mask + 1u;
  }
  uint32_t slot = (uint32_t)hash64(key) & mask;
  for (uint32_t probe = 0; probe <= mask && probe < KTJ_TABLE_PROBES; ++probe) {
    uint64_t cur = keys[slot];
    if (cur == key) return slot;
    if (cur == KTJ_EMPTY_KEY) {
      if (*(volatile unsigned int*)count >= limit) return KTJ_NOSLOT; /* full by count: take no further slot */
      unsigned long long prev = atomicCAS((unsigned long long*)&keys[slot], (unsigned long long)KTJ_EMPTY_KEY,
                                          (unsigned long long)key);
      if (prev == KTJ_EMPTY_KEY) return atomicAdd(count, 1u) >= limit ? KTJ_NOSLOT : slot;
      if (prev == key) return slot;
    }
    slot = (slot + 1u) & mask;
  }
  return KTJ_NOSLOT;
}
__device__ uint32_t table_find(const uint64_t* keys, uint32_t mask, uint64_t key) {
  if (key == KTJ_EMPTY_KEY) return keys[mask + 1u] == 0 ? mask + 1u : KTJ_NOSLOT;
  uint32_t slot = (uint32_t)hash64(key) & mask;
  for (uint32_t probe = 0; probe <= mask && probe < KTJ_TABLE_PROBES; ++probe) {
    uint64_t cur = keys[slot];
    if (cur == key) return slot;
    if (cur == KTJ_EMPTY_KEY) return KTJ_NOSLOT;
    slot = (slot + 1u) & mask;
  }
  return KTJ_NOSLOT;
}

/* Join tables (Table).  Direct mode: slot = key - base.  Hash mode: slots are grouped in runs of
 * sixteen; a key lives at position (key + rotation) & 15 of a run, where the rotation and the
 * probe sequence over runs (double hashing) depend only on the remaining key bits.  Sixteen
 * consecutive ids therefore share one run, while strided or clustered ids still spread like under
 * a full hash and a collision costs one probe in another run rather than a walk through a full one. */
struct ProbeSeq {
  uint32_t run, step, low;
  __device__ __forceinline__ ProbeSeq(uint64_t key) {
    const uint64_t h = hash64(key >> 4);
    run = (uint32_t)h;
    step = (uint32_t)(h >> 32) | 1u; /* odd: visits every run of a power-of-two table */
    low = ((uint32_t)key + (uint32_t)((h * 0x9E3779B97F4A7C15ULL) >> 60)) & 15u; /* ids sharing low bits still use all positions */
  }
  __device__ __forceinline__ uint32_t slot(uint32_t mask) const { return ((run << 4) | low) & mask; }
  __device__ __forceinline__ void next() { run += step; }
};
/* Returns the slot of `key`, inserting it if absent; KTJ_NOSLOT when the table is full (hash
 * mode) or the key lies outside the planned range (direct mode; cannot happen for keys that were
 * part of the range computation). */
__device__ uint32_t slot_insert(const Table& t, uint64_t key) {
  if (t.ctl->direct) {
    if (t.keyed_direct && key == KTJ_EMPTY_KEY) { t.keys[t.mask + 1u] = 0; return t.mask + 1u; }
    const uint64_t idx = key - t.ctl->base;
    if (idx > t.ctl->span) return KTJ_NOSLOT;
    if (t.keyed_direct && t.keys[idx] != key) t.keys[idx] = key; /* every writer stores the same value */
    return (uint32_t)idx;
  }
  if (key == KTJ_EMPTY_KEY) { t.keys[t.mask + 1u] = 0; return t.mask + 1u; }
  ProbeSeq p(key);
  for (uint32_t probe = 0; probe <= (t.mask >> 4); ++probe, p.next()) {
    const uint32_t slot = p.slot(t.mask);
    uint64_t cur = t.keys[slot];
    if (cur == key) return slot;
    if (cur == KTJ_EMPTY_KEY) {
      unsigned long long prev = atomicCAS((unsigned long long*)&t.keys[slot], (unsigned long long)KTJ_EMPTY_KEY,
                                          (unsigned long long)key);
      if (prev == KTJ_EMPTY_KEY || prev == key) return slot;
    }
  }
  return KTJ_NOSLOT;
}
/* In direct mode without stored keys every id inside the range has a slot; one that was never
 * inserted reads as empty per-slot values. */
__device__ uint32_t slot_find(const Table& t, uint64_t key) {
  if (t.ctl->direct) {
    if (t.keyed_direct && key == KTJ_EMPTY_KEY) return t.keys[t.mask + 1u] == 0 ? t.mask + 1u : KTJ_NOSLOT;
    const uint64_t idx = key - t.ctl->base;
    if (idx > t.ctl->span) return KTJ_NOSLOT;
    if (t.keyed_direct && t.keys[idx] != key) return KTJ_NOSLOT;
    return (uint32_t)idx;
  }
  if (key == KTJ_EMPTY_KEY) return t.keys[t.mask + 1u] == 0 ? t.mask + 1u : KTJ_NOSLOT;
  ProbeSeq p(key);
  for (uint32_t probe = 0; probe <= (t.mask >> 4); ++probe, p.next()) {
    const uint32_t slot = p.slot(t.mask);
    uint64_t cur = t.keys[slot];
    if (cur == key) return slot;
    if (cur == KTJ_EMPTY_KEY) return KTJ_NOSLOT;
  }
  return KTJ_NOSLOT;
}

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
/* Sums a per-thread count over the workgroup and adds it to a global counter with one atomic per
 * workgroup (a single hot address serialises atomics in L2, so they must be rare).  Must be
 * reached by every thread of the workgroup.  block_add_to: a counter of its own address, for counts
 * that are zero in nearly every workgroup; block_add: one of the sharded counters of Scalars. */
__device__ __forceinline__ uint32_t block_sum(uint32_t mine) { /* the sum, in thread 0 */
  __shared__ uint32_t partial[KTJ_BLOCK >> 6];
  const uint32_t w = wave_sum_u32(mine);
  __syncthreads();
  if (lane_id() == 0) partial[threadIdx.x >> 6] = w;
  __syncthreads();
  uint32_t t = 0;
  if (threadIdx.x == 0)
    for (uint32_t k = 0; k < (blockDim.x >> 6); ++k) t += partial[k];
  return t;
}
__device__ __forceinline__ void block_add_to(unsigned long long* counter, uint32_t mine) {
  const uint32_t t = block_sum(mine);
  if (threadIdx.x == 0 && t) atomicAdd(counter, (unsigned long long)t);
}
__device__ __forceinline__ void block_add(Scalars* sc, int which, uint32_t mine) {
  const uint32_t t = block_sum(mine);
  if (threadIdx.x == 0 && t) atomicAdd(&sc->shard[blockIdx.x & (KTJ_COUNTER_SHARDS - 1u)][which], (unsigned long long)t);
}
/* grid-stride kernels: enough workgroups to fill 256 CUs several times over */
#define KTJ_MAX_GRID 4096u

__global__ void k_fill_u64(uint64_t* p, uint64_t v, uint64_t n) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
__global__ void k_fill_u32(uint32_t* p, uint32_t v, uint64_t n) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
__global__ void k_init_scalars(Scalars* s) {
  if (blockIdx.x == 0)
    for (uint32_t c = threadIdx.x; c < KTJ_COUNTER_SHARDS; c += blockDim.x)
      for (int k = 0; k < 16; ++k) s->shard[c][k] = 0;
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    s->ts_min_biased = ~0ULL; s->ts_max_biased = 0;
    s->out_of_range = 0; s->out_of_order = 0; s->n_flow = 0; s->n_linked = 0; s->n_blank_names = 0; s->n_valid = 0;
    s->n_unresolved = 0; s->n_sync_typed = 0; s->n_device_orphans = 0; s->error = 0; s->have_stream_src = 0; s->n_dev_ranks = 0; s->n_res_ranks = 0; s->n_dense = 0; s->runtime_ids_repeat = 0;
    s->n_queues = 0; s->n_sync_rows = 0; s->ext_ids_repeat = 0;
    for (int k = 0; k < 3; ++k) {
      s->plan.range[k].lo = ~0ULL; s->plan.range[k].hi = 0;
      s->plan.ctl[k].base = 0; s->plan.ctl[k].span = 0; s->plan.ctl[k].direct = 0; s->plan.ctl[k].pad = 0;
    }
  }
}

static inline unsigned grid_for(uint64_t n, unsigned per_block) { return (unsigned)((n + per_block - 1) / per_block); }
static inline unsigned grid_stride_for(uint64_t n, unsigned per_block) {
  const uint64_t g = (n + per_block - 1) / per_block;
  return (unsigned)(g < KTJ_MAX_GRID ? g : KTJ_MAX_GRID);
}
#define KTJ_LAUNCH_CHECK() hipGetLastError()

hipError_t fill_u64(uint64_t* p, uint64_t v, uint64_t n, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_fill_u64, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, p, v, n);
  return KTJ_LAUNCH_CHECK();
}
hipError_t fill_u32(uint32_t* p, uint32_t v, uint64_t n, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_fill_u32, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, p, v, n);
  return KTJ_LAUNCH_CHECK();
}
/* several fills in one launch (blockIdx.y picks the job): a small trace pays per launch, not per byte */
__global__ void k_fill_many(FillJobs jobs) {
  const uint32_t j = blockIdx.y;
  const uint64_t n = jobs.n[j], v = jobs.value[j];
  if (jobs.bytes_each[j] == 8) {
    uint64_t* p = static_cast<uint64_t*>(jobs.p[j]);
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) p[i] = v;
  } else {
    uint32_t* p = static_cast<uint32_t*>(jobs.p[j]);
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) p[i] = (uint32_t)v;
  }
}
hipError_t fill_many(const FillJobs& jobs, hipStream_t st) {
  if (jobs.count == 0) return hipSuccess;
  uint64_t most = 1;
  for (uint32_t j = 0; j < jobs.count; ++j) most = jobs.n[j] > most ? jobs.n[j] : most;
  hipLaunchKernelGGL(k_fill_many, dim3(grid_stride_for(most, KTJ_BLOCK * 4), jobs.count), dim3(KTJ_BLOCK), 0, st, jobs);
  return KTJ_LAUNCH_CHECK();
}
hipError_t init_scalars(Scalars* s, hipStream_t st) {
  static_assert((KTJ_COUNTER_SHARDS & (KTJ_COUNTER_SHARDS - 1u)) == 0, "a workgroup's copy is its index modulo the number of copies");
  hipLaunchKernelGGL(k_init_scalars, dim3(1), dim3(64), 0, st, s);
  return KTJ_LAUNCH_CHECK();
}

/* ------------------------------------------------------------------------------------------ */
/* static scratch array: the working memory of ktj_process_noalloc.  Every GPU the library runs  */
/* on holds its own copy, at its own address, until the process ends.  In host code the array's  */
/* name is only a handle for hipGetSymbolAddress; everything else uses the looked-up address.    */
/* ------------------------------------------------------------------------------------------ */
static __device__ __align__(256) unsigned char scratch[KTJ_NOALLOC_SCRATCH_BYTES];
#define KTJ_MAX_DEVICES 64
static void* g_scratch_ptr[KTJ_MAX_DEVICES];
static std::mutex g_scratch_lock;

hipError_t scratch_address(int device, void** ptr, size_t* bytes) {
  *ptr = nullptr;
  *bytes = 0;
  if (device < 0 || device >= KTJ_MAX_DEVICES) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    const hipError_t rc = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (rc != hipSuccess) return rc;
    g_scratch_ptr[device] = p;
  }
  *ptr = g_scratch_ptr[device];
  *bytes = KTJ_NOALLOC_SCRATCH_BYTES;
  return hipSuccess;
}

/* ------------------------------------------------------------------------------------------ */
/* exclusive scan: per-block sums → scan of the sums (one block) → per-block scan               */
/* ------------------------------------------------------------------------------------------ */
#define SCAN_ITEMS 8
#define SCAN_TILE (KTJ_BLOCK * SCAN_ITEMS)

#define SCAN_MAX_WAVES 16 /* workgroups of up to 1024 lanes */
/* a lane's SCAN_ITEMS consecutive values: two 16-byte loads where the whole run is inside the input
 * (the inputs are 16-byte aligned device buffers), single values at the end */
__device__ __forceinline__ void scan_load_items(const uint32_t* in, uint64_t n, uint64_t base, uint32_t (&v)[SCAN_ITEMS]) {
  static_assert(SCAN_ITEMS == 8, "two uint4 per lane");
  if (base + SCAN_ITEMS <= n) {
    const uint4 a = *reinterpret_cast<const uint4*>(in + base), b = *reinterpret_cast<const uint4*>(in + base + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    for (int k = 0; k < SCAN_ITEMS; ++k) v[k] = base + k < n ? in[base + k] : 0u;
  }
}
__device__ __forceinline__ uint64_t block_exclusive_scan_u64(uint64_t v, uint64_t* lds_wave /* SCAN_MAX_WAVES */, uint64_t* total) {
  /* inclusive scan inside the wave */
  unsigned long long x = v;
  for (int o = 1; o < 64; o <<= 1) {
    const unsigned long long y = __shfl_up(x, (unsigned)o);
    if ((int)lane_id() >= o) x += y;
  }
  const uint32_t w = threadIdx.x >> 6;
  if (lane_id() == 63) lds_wave[w] = x;
  __syncthreads();
  uint64_t base = 0, tot = 0;
  for (uint32_t k = 0; k < (blockDim.x >> 6); ++k) {
    const uint64_t s = lds_wave[k];
    if (k < w) base += s;
    tot += s;
  }
  __syncthreads();
  *total = tot;
  return base + x - v;
}

__global__ void k_scan_sums(const uint32_t* in, uint64_t n, uint64_t* sums) {
  __shared__ uint64_t lds_wave[SCAN_MAX_WAVES];
  const uint64_t base = (uint64_t)blockIdx.x * SCAN_TILE + (uint64_t)threadIdx.x * SCAN_ITEMS;
  uint32_t v[SCAN_ITEMS];
  scan_load_items(in, n, base, v);
  uint64_t s = 0;
  for (int k = 0; k < SCAN_ITEMS; ++k) s += v[k];
  uint64_t tot;
  block_exclusive_scan_u64(s, lds_wave, &tot);
  if (threadIdx.x == 0) sums[blockIdx.x] = tot;
}
/* one block: sums[0..m) → exclusive prefix in place, grand total → sums[m] */
__global__ void k_scan_of_sums(uint64_t* sums, uint64_t m) {
  __shared__ uint64_t lds_wave[SCAN_MAX_WAVES];
  uint64_t carry = 0;
  for (uint64_t base = 0; base < m; base += blockDim.x) {
    const uint64_t i = base + threadIdx.x;
    const uint64_t v = i < m ? sums[i] : 0;
    uint64_t tot;
    const uint64_t ex = block_exclusive_scan_u64(v, lds_wave, &tot);
    if (i < m) sums[i] = carry + ex;
    carry += tot;
  }
  if (threadIdx.x == 0) sums[m] = carry;
}
template <typename OutT>
__global__ void k_scan_final(const uint32_t* in, uint64_t n, const uint64_t* sums, uint64_t m, OutT* out,
                             bool write_total) {
  __shared__ uint64_t lds_wave[SCAN_MAX_WAVES];
  const uint64_t base = (uint64_t)blockIdx.x * SCAN_TILE + (uint64_t)threadIdx.x * SCAN_ITEMS;
  uint32_t v[SCAN_ITEMS];
  scan_load_items(in, n, base, v);
  uint64_t s = 0;
  for (int k = 0; k < SCAN_ITEMS; ++k) s += v[k];
  uint64_t tot;
  uint64_t ex = block_exclusive_scan_u64(s, lds_wave, &tot) + sums[blockIdx.x];
  if (base + SCAN_ITEMS <= n) { /* the lane's run as 16-byte stores (the outputs are 16-byte aligned device buffers) */
    OutT r[SCAN_ITEMS];
    for (int k = 0; k < SCAN_ITEMS; ++k) { r[k] = (OutT)ex; ex += v[k]; }
    constexpr int PER = 16 / sizeof(OutT);
    typedef OutT vec __attribute__((ext_vector_type(PER)));
    vec* dst = reinterpret_cast<vec*>(out + base);
    for (int q = 0; q < SCAN_ITEMS / PER; ++q) {
      vec x;
      for (int j = 0; j < PER; ++j) x[j] = r[q * PER + j];
      dst[q] = x;
    }
  } else {
    for (int k = 0; k < SCAN_ITEMS; ++k) {
      if (base + k < n) out[base + k] = (OutT)ex;
      ex += v[k];
    }
  }
  if (write_total && blockIdx.x == 0 && threadIdx.x == 0) out[n] = (OutT)sums[m];
}

/* small inputs (one tile of SCAN_SMALL_THREADS lanes): the whole scan in one workgroup and one pass.
 * More tiles in one workgroup measured slower than the three launches over many workgroups. */
#define SCAN_SMALL_THREADS 1024u
#define SCAN_SMALL_MAX (SCAN_SMALL_THREADS * SCAN_ITEMS)
template <typename OutT>
__global__ void __launch_bounds__(SCAN_SMALL_THREADS) k_scan_small(const uint32_t* in, uint64_t n, OutT* out, bool write_total) {
  __shared__ uint64_t wave_sum[SCAN_SMALL_THREADS >> 6];
  const uint64_t base = (uint64_t)threadIdx.x * SCAN_ITEMS;
  uint32_t v[SCAN_ITEMS];
  uint64_t s = 0;
#pragma unroll
  for (int k = 0; k < SCAN_ITEMS; ++k) { v[k] = base + k < n ? in[base + k] : 0u; s += v[k]; }
  unsigned long long x = s; /* inclusive scan inside the wavefront, then over the wavefronts' sums */
  for (int o = 1; o < 64; o <<= 1) {
    const unsigned long long y = __shfl_up(x, (unsigned)o);
    if ((int)lane_id() >= o) x += y;
  }
  const uint32_t w = threadIdx.x >> 6;
  if (lane_id() == 63) wave_sum[w] = x;
  __syncthreads();
  uint64_t before = 0, tot = 0;
  for (uint32_t k = 0; k < (SCAN_SMALL_THREADS >> 6); ++k) {
    const uint64_t t = wave_sum[k];
    if (k < w) before += t;
    tot += t;
  }
  uint64_t ex = before + x - s;
#pragma unroll
  for (int k = 0; k < SCAN_ITEMS; ++k) { /* a lane reads and writes its own items only: in place is fine */
    if (base + k < n) out[base + k] = (OutT)ex;
    ex += v[k];
  }
  if (write_total && threadIdx.x == 0) out[n] = (OutT)tot;
}

uint64_t scan_tmp_elems(uint64_t n) { return (n + SCAN_TILE - 1) / SCAN_TILE + 2; }

hipError_t scan_u32_to_u64(const uint32_t* in, uint64_t* out, uint64_t n, uint64_t* tmp, hipStream_t st) {
  const uint64_t m = (n + SCAN_TILE - 1) / SCAN_TILE;
  if (n <= SCAN_SMALL_MAX) {
    hipLaunchKernelGGL(HIP_KERNEL_NAME(k_scan_small<uint64_t>), dim3(1), dim3(SCAN_SMALL_THREADS), 0, st, in, n, out, true);
    return KTJ_LAUNCH_CHECK();
  }
  if (m > 0) hipLaunchKernelGGL(k_scan_sums, dim3((unsigned)m), dim3(KTJ_BLOCK), 0, st, in, n, tmp);
  hipLaunchKernelGGL(k_scan_of_sums, dim3(1), dim3(m > KTJ_BLOCK ? 1024 : KTJ_BLOCK), 0, st, tmp, m);
  if (m > 0)
    hipLaunchKernelGGL(HIP_KERNEL_NAME(k_scan_final<uint64_t>), dim3((unsigned)m), dim3(KTJ_BLOCK), 0, st, in, n,
                       (const uint64_t*)tmp, m, out, true);
  else
    hipLaunchKernelGGL(k_fill_u64, dim3(1), dim3(64), 0, st, out, (uint64_t)0, (uint64_t)1);
  return KTJ_LAUNCH_CHECK();
}
hipError_t scan_u32_inplace(uint32_t* data, uint64_t n, uint64_t* tmp, hipStream_t st) {
  const uint64_t m = (n + SCAN_TILE - 1) / SCAN_TILE;
  if (m == 0) return hipSuccess;
  if (n <= SCAN_SMALL_MAX) {
    hipLaunchKernelGGL(HIP_KERNEL_NAME(k_scan_small<uint32_t>), dim3(1), dim3(SCAN_SMALL_THREADS), 0, st, (const uint32_t*)data, n, data, false);
    return KTJ_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(k_scan_sums, dim3((unsigned)m), dim3(KTJ_BLOCK), 0, st, (const uint32_t*)data, n, tmp);
  hipLaunchKernelGGL(k_scan_of_sums, dim3(1), dim3(m > KTJ_BLOCK ? 1024 : KTJ_BLOCK), 0, st, tmp, m);
  /* every block reads its tile completely before writing it, and tiles do not overlap */
  hipLaunchKernelGGL(HIP_KERNEL_NAME(k_scan_final<uint32_t>), dim3((unsigned)m), dim3(KTJ_BLOCK), 0, st,
                     (const uint32_t*)data, n, (const uint64_t*)tmp, m, data, false);
  return KTJ_LAUNCH_CHECK();
}

/* ------------------------------------------------------------------------------------------ */
/* stage 0: dictionary.  One wavefront per string.                                              */
/*   arg view  = sanitizeStrForJSON            (libkineto/src/output_json.cpp:72-78)            */
/*   name view = "kernel"→"Kernel", sanitize, non-printable → "unknown", quote escaping         */
/*                                             (output_json.cpp:946-949, 86-112)                */
/* ------------------------------------------------------------------------------------------ */
__global__ void k_dict_measure(const char* blob, const uint64_t* off, uint32_t n, uint32_t* name_len,
                               uint32_t* arg_len, uint32_t* flags) {
  const uint32_t id = blockIdx.x * (KTJ_BLOCK >> 6) + (threadIdx.x >> 6);
  if (id >= n) return;
  const char* p = blob + off[id];
  const uint64_t len = off[id + 1] - off[id];
  uint32_t nl = 0, q = 0, bad = 0, nonblank = 0;
  for (uint64_t k = lane_id(); k < len; k += 64) {
    const unsigned char c = (unsigned char)p[k];
    if (c == '\n') { ++nl; continue; }
    if (c == '"') ++q;
    if (c < 0x20 || c > 0x7e) ++bad;
    if (!(c == ' ' || c == '\t' || c == '\v' || c == '\f' || c == '\r')) ++nonblank;
  }
  nl = wave_sum_u32(nl); q = wave_sum_u32(q); bad = wave_sum_u32(bad); nonblank = wave_sum_u32(nonblank);
  if (lane_id() == 0) {
    const bool is_kernel = len == 6 && p[0] == 'k' && p[1] == 'e' && p[2] == 'r' && p[3] == 'n' && p[4] == 'e' && p[5] == 'l';
    uint32_t f = 0;
    uint32_t nlen;
    if (is_kernel) { f |= KTJ_SF_NAME_KERNEL; nlen = 6; }
    else if (bad) { f |= KTJ_SF_NAME_UNKNOWN; nlen = 7; }
    else nlen = (uint32_t)len - nl + q;
    if (nonblank == 0) f |= KTJ_SF_ARG_BLANK;
    if (len == 11) {
      const char* want = "Stream Sync";
      bool same = true;
      for (int k = 0; k < 11; ++k) same = same && p[k] == want[k];
      if (same) f |= KTJ_SF_STREAM_SYNC;
    }
    name_len[id] = nlen;
    arg_len[id] = (uint32_t)len - nl;
    flags[id] = f;
  }
}

__global__ void k_dict_write(const char* blob, const uint64_t* off, uint32_t n, const uint64_t* name_off,
                             const uint64_t* arg_off, const uint32_t* flags, char* name_blob, char* arg_blob) {
  const uint32_t id = blockIdx.x * (KTJ_BLOCK >> 6) + (threadIdx.x >> 6);
  if (id >= n) return;
  const char* p = blob + off[id];
  const uint64_t len = off[id + 1] - off[id];
  const uint32_t f = flags[id];
  char* an = arg_blob + arg_off[id];
  char* nn = name_blob + name_off[id];
  const bool literal_name = (f & (KTJ_SF_NAME_KERNEL | KTJ_SF_NAME_UNKNOWN)) != 0;
  if (literal_name) {
    const char* lit = (f & KTJ_SF_NAME_KERNEL) ? "Kernel" : "unknown";
    const uint32_t ll = (f & KTJ_SF_NAME_KERNEL) ? 6u : 7u;
    if (lane_id() < ll) nn[lane_id()] = lit[lane_id()];
  }
  uint64_t aw = 0, nw = 0; /* bytes written so far (wave-uniform) */
  const uint64_t lt = lanemask_lt();
  for (uint64_t base = 0; base < len; base += 64) {
    const uint64_t k = base + lane_id();
    const bool in = k < len;
    unsigned char c = in ? (unsigned char)p[k] : 0;
    const bool keep = in && c != '\n';
    if (c == '\\') c = '/';
    const bool isq = keep && c == '"';
    const uint64_t km = __ballot(keep ? 1 : 0);
    const uint64_t qm = __ballot(isq ? 1 : 0);
    const uint32_t kpos = (uint32_t)__popcll(km & lt);
    if (keep) {
      an[aw + kpos] = (char)c;
      if (!literal_name) {
        const uint64_t np = nw + kpos + (uint32_t)__popcll(qm & lt);
        if (isq) { nn[np] = '\\'; nn[np + 1] = '"'; }
        else nn[np] = (char)c;
      }
    }
    aw += (uint32_t)__popcll(km);
    nw += (uint32_t)__popcll(km) + (uint32_t)__popcll(qm);
  }
}

hipError_t dict_measure(const char* blob, const uint64_t* off, uint32_t n, uint32_t* name_len, uint32_t* arg_len,
                        uint32_t* flags, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_dict_measure, dim3(grid_for(n, KTJ_BLOCK >> 6)), dim3(KTJ_BLOCK), 0, st, blob, off, n,
                     name_len, arg_len, flags);
  return KTJ_LAUNCH_CHECK();
}
hipError_t dict_write(const char* blob, const uint64_t* off, uint32_t n, const uint64_t* name_off,
                      const uint64_t* arg_off, const uint32_t* flags, char* name_blob, char* arg_blob, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_dict_write, dim3(grid_for(n, KTJ_BLOCK >> 6)), dim3(KTJ_BLOCK), 0, st, blob, off, n, name_off,
                     arg_off, flags, name_blob, arg_blob);
  return KTJ_LAUNCH_CHECK();
}

/* ------------------------------------------------------------------------------------------ */
/* stage 1: decode.  A workgroup pulls 256 packed records into LDS with lane-consecutive 16-byte */
/* loads (fully coalesced), then each lane unpacks its own record into the columns.              */
/* ------------------------------------------------------------------------------------------ */
template <typename Rec>
__device__ __forceinline__ const Rec* stage_records(const Rec* recs, uint64_t n, uint4* stage, uint32_t* n_here) {
  constexpr uint32_t U = sizeof(Rec) / 16;
  const uint64_t base = (uint64_t)blockIdx.x * KTJ_BLOCK;
  const uint32_t cnt = (uint32_t)((n - base) < KTJ_BLOCK ? (n - base) : KTJ_BLOCK);
  const uint4* g = reinterpret_cast<const uint4*>(recs + base);
  for (uint32_t i = threadIdx.x; i < cnt * U; i += KTJ_BLOCK) stage[i] = g[i];
  __syncthreads();
  *n_here = cnt;
  return reinterpret_cast<const Rec*>(stage);
}

/* Smallest and largest key of the workgroup's rows into part[blockIdx.x] (empty: lo > hi).  The
 * join tables are planned from these ranges; collecting them here saves a pass over the ids.
 * Must be reached by every thread of the workgroup. */
__device__ __forceinline__ void block_key_range(bool has, uint64_t key, KeyRange* part) {
  __shared__ unsigned long long s_lo[KTJ_BLOCK >> 6], s_hi[KTJ_BLOCK >> 6];
  unsigned long long lo = has ? key : ~0ULL, hi = has ? key : 0ULL;
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned long long l2 = __shfl_xor(lo, o), h2 = __shfl_xor(hi, o);
    lo = l2 < lo ? l2 : lo;
    hi = h2 > hi ? h2 : hi;
  }
  __syncthreads();
  if (lane_id() == 0) { s_lo[threadIdx.x >> 6] = lo; s_hi[threadIdx.x >> 6] = hi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (uint32_t k = 1; k < (blockDim.x >> 6); ++k) { lo = s_lo[k] < lo ? s_lo[k] : lo; hi = s_hi[k] > hi ? s_hi[k] : hi; }
    KeyRange r;
    r.lo = lo; r.hi = hi;
    part[blockIdx.x] = r;
  }
}
__global__ void k_decode_generic(const ktj_generic_rec* recs, uint64_t n, Columns c, uint64_t first, Scalars* sc,
                                 EmitCtx ctx, KeyRange* id_range) {
  __shared__ uint4 stage[KTJ_BLOCK * sizeof(ktj_generic_rec) / 16];
  uint32_t cnt;
  const ktj_generic_rec* l = stage_records(recs, n, stage, &cnt);
  /* rows that may need a Stream Sync row of their own are rare: the extra passes run only if any */
  const bool sync_typed = threadIdx.x < cnt && l[threadIdx.x].type == KTJ_TYPE_CUDA_SYNC;
  if (__syncthreads_or(sync_typed ? 1 : 0)) block_add(sc, KTJ_CNT_SYNC_TYPED, sync_typed ? 1u : 0u);
  if (id_range) block_key_range(threadIdx.x < cnt, threadIdx.x < cnt ? (uint64_t)(int64_t)l[threadIdx.x].id : 0, id_range);
  if (threadIdx.x >= cnt) return;
  const ktj_generic_rec g = l[threadIdx.x];
  const uint64_t a = first + (uint64_t)blockIdx.x * KTJ_BLOCK + threadIdx.x;
  c.ts[a] = g.start_ns;
  c.dur[a] = g.end_ns - g.start_ns;               /* GenericTraceActivity.h:65-67 */
  c.corr[a] = (uint64_t)(int64_t)g.id;
  c.dev[a] = generic_device(g, ctx.args, ctx.n_args);
  c.res[a] = g.resource;
  c.meta[a] = (generic_record_prints(g, ctx) ? KTJ_M_VALID : 0u) | (KTJ_CLASS_GENERIC << KTJ_M_CLASS_SHIFT);
  c.ext[a] = 0;
}
/* The runtime and device kernels also convert the clock and apply the capture window (stage 2a:
 * RocprofActivityApi.cpp:166-175, ApproximateClock.cpp:83-90, RocprofActivity.h:42-47 and 122-127,
 * GenericActivityProfiler.cpp:329-340), so that timestamp and duration are written once. */
__global__ void k_decode_runtime(const ktj_runtime_rec* recs, uint64_t n, Columns c, uint64_t first, KeyRange* id_range,
                                 KeyRange* narrow_range, ClockDev clk, int64_t win_start, int64_t win_end, Scalars* sc) {
  __shared__ uint4 stage[KTJ_BLOCK * sizeof(ktj_runtime_rec) / 16];
  uint32_t cnt;
  const ktj_runtime_rec* l = stage_records(recs, n, stage, &cnt);
  {
    const bool has = threadIdx.x < cnt;
    const uint64_t id = has ? l[threadIdx.x].id : 0;
    block_key_range(has, id, id_range);
    block_key_range(has, narrow_corr_key(id), narrow_range);
  }
  uint32_t oor = 0;
  if (threadIdx.x < cnt) {
  const ktj_runtime_rec* r = &l[threadIdx.x];
  const uint64_t a = first + (uint64_t)blockIdx.x * KTJ_BLOCK + threadIdx.x;
  uint64_t b = r->begin, e = r->end;
  convert_range(clk, clk.runtime_mode, &b, &e);
  const int64_t ts = (int64_t)b, dur = (int64_t)(e - b);   /* RocprofActivity.h:42-47 */
  oor = out_of_range(ts, dur, win_start, win_end) ? 1u : 0u;
  c.ts[a] = ts;
  c.dur[a] = dur;
  c.corr[a] = r->id;
  c.dev[a] = (int64_t)r->pid;
  c.res[a] = (int64_t)r->tid;
  const uint32_t kind = r->kind <= KTJ_RT_MALLOC ? r->kind : KTJ_RT_DEFAULT;
  const uint64_t stream = kind == KTJ_RT_KERNEL ? r->u.kernel.stream : (kind == KTJ_RT_COPY ? r->u.copy.stream : 0);
  c.meta[a] = (KTJ_CLASS_RUNTIME << KTJ_M_CLASS_SHIFT) | (kind << KTJ_M_KIND_SHIFT) | (stream != 0 ? KTJ_M_HAS_STREAM : 0u) |
              (oor ? 0u : KTJ_M_VALID);
  c.ext[a] = 0;
  }
  block_add(sc, KTJ_CNT_OUT_OF_RANGE, oor);
}
__global__ void k_decode_device(const ktj_device_rec* recs, uint64_t n, Columns c, uint64_t first, DevBrief* brief,
                                KeyRange* id_range, ClockDev clk, int64_t win_start, int64_t win_end, Scalars* sc) {
  __shared__ uint4 stage[KTJ_BLOCK * sizeof(ktj_device_rec) / 16];
  uint32_t cnt;
  const ktj_device_rec* l = stage_records(recs, n, stage, &cnt);
  block_key_range(threadIdx.x < cnt, threadIdx.x < cnt ? l[threadIdx.x].id : 0, id_range);
  uint32_t oor = 0;
  if (threadIdx.x < cnt) {
  const ktj_device_rec* d = &l[threadIdx.x];
  const uint64_t a = first + (uint64_t)blockIdx.x * KTJ_BLOCK + threadIdx.x;
  const uint32_t dom = device_row_domain(d->domain);
  uint64_t b = d->begin, e = d->end;
  convert_range(clk, clk.device_mode, &b, &e);
  int64_t ts, dur;
  device_times(dom, b, e, &ts, &dur);
  oor = out_of_range(ts, dur, win_start, win_end) ? 1u : 0u;
  c.ts[a] = ts;
  c.dur[a] = dur;
  c.corr[a] = d->id;
  c.dev[a] = (int64_t)d->device;
  c.res[a] = device_row_stream(dom, d->stream);
  c.meta[a] = (KTJ_CLASS_DEVICE << KTJ_M_CLASS_SHIFT) | (dom << KTJ_M_KIND_SHIFT) | (oor ? 0u : KTJ_M_VALID);
  c.ext[a] = 0;
  DevBrief br;
  br.queue = d->queue; br.device = d->device; br.domain = dom;
  brief[a - first] = br;
  }
  block_add(sc, KTJ_CNT_OUT_OF_RANGE, oor);
}

uint64_t decode_blocks(uint64_t n) { return grid_for(n, KTJ_BLOCK); }
hipError_t decode_generic(const ktj_generic_rec* r, uint64_t n, Columns c, uint64_t first, Scalars* sc, EmitCtx ctx,
                          KeyRange* id_range, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_decode_generic, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, r, n, c, first, sc, ctx, id_range);
  return KTJ_LAUNCH_CHECK();
}
hipError_t decode_runtime(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first, KeyRange* id_range,
                          KeyRange* narrow_range, ClockDev clk, int64_t win_start, int64_t win_end, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_decode_runtime, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, r, n, c, first, id_range,
                     narrow_range, clk, win_start, win_end, sc);
  return KTJ_LAUNCH_CHECK();
}
hipError_t decode_device(const ktj_device_rec* r, uint64_t n, Columns c, uint64_t first, DevBrief* brief, KeyRange* id_range,
                         ClockDev clk, int64_t win_start, int64_t win_end, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_decode_device, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, r, n, c, first, brief, id_range,
                     clk, win_start, win_end, sc);
  return KTJ_LAUNCH_CHECK();
}

/* ------------------------------------------------------------------------------------------ */
/* stage 2b: joins.  "Last writer wins" of the reference's sequential map updates becomes        */
/* atomicMax over the source row index; "first seen" becomes atomicMin over the arrival index.   */
/* What a device row takes over from "its" runtime row is then published into the table slot by  */
/* the winning row, so that a device row needs one slot of each table and no other row.          */
/* ------------------------------------------------------------------------------------------ */
__device__ __forceinline__ void flag_error(Scalars* sc, unsigned bit) { atomicOr(&sc->error, bit); }

/* min / max of p[i * stride] (optionally int-narrowed) into *out: one atomic pair per workgroup */
__global__ void k_key_range(const uint64_t* p, uint32_t stride, uint64_t n, int narrow, KeyRange* out) {
  __shared__ unsigned long long s_lo[KTJ_BLOCK >> 6], s_hi[KTJ_BLOCK >> 6];
  unsigned long long lo = ~0ULL, hi = 0;
  const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i0 = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i0 < n; i0 += 4 * step) {
    uint64_t k[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) { const uint64_t i = i0 + u * step; k[u] = i < n ? p[i * stride] : p[i0 * stride]; }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint64_t v = narrow ? narrow_corr_key(k[u]) : k[u];
      lo = v < lo ? v : lo;
      hi = v > hi ? v : hi;
    }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned long long l2 = __shfl_xor(lo, o), h2 = __shfl_xor(hi, o);
    lo = l2 < lo ? l2 : lo;
    hi = h2 > hi ? h2 : hi;
  }
  if (lane_id() == 0) { s_lo[threadIdx.x >> 6] = lo; s_hi[threadIdx.x >> 6] = hi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (uint32_t k = 1; k < (blockDim.x >> 6); ++k) { lo = s_lo[k] < lo ? s_lo[k] : lo; hi = s_hi[k] > hi ? s_hi[k] : hi; }
    if (lo <= hi) { atomicMin(&out->lo, lo); atomicMax(&out->hi, hi); }
  }
}
/* the per-workgroup ranges of the decode kernels into the plan's ranges: MERGE_SPLIT workgroups per job */
#define MERGE_SPLIT 16u
struct RangeJobs {
  const KeyRange* src[4];
  uint64_t n[4];
  uint32_t dst[4]; /* KTJ_TBL_* */
};
__global__ void k_merge_ranges(RangeJobs jobs, Scalars* sc) {
  __shared__ unsigned long long s_lo[1024 >> 6], s_hi[1024 >> 6];
  const uint32_t job = blockIdx.x / MERGE_SPLIT, part = blockIdx.x % MERGE_SPLIT;
  const KeyRange* src = jobs.src[job];
  const uint64_t n = jobs.n[job];
  unsigned long long lo = ~0ULL, hi = 0;
  for (uint64_t i = (uint64_t)part * blockDim.x + threadIdx.x; i < n; i += (uint64_t)MERGE_SPLIT * blockDim.x) {
    const KeyRange r = src[i];
    if (r.lo <= r.hi) { lo = r.lo < lo ? r.lo : lo; hi = r.hi > hi ? r.hi : hi; }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned long long l2 = __shfl_xor(lo, o), h2 = __shfl_xor(hi, o);
    lo = l2 < lo ? l2 : lo;
    hi = h2 > hi ? h2 : hi;
  }
  if (lane_id() == 0) { s_lo[threadIdx.x >> 6] = lo; s_hi[threadIdx.x >> 6] = hi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (uint32_t k = 1; k < (blockDim.x >> 6); ++k) { lo = s_lo[k] < lo ? s_lo[k] : lo; hi = s_hi[k] > hi ? s_hi[k] : hi; }
    KeyRange* out = &sc->plan.range[jobs.dst[job]];
    if (lo <= hi) { atomicMin(&out->lo, lo); atomicMax(&out->hi, hi); }
  }
}
__global__ void k_plan_tables(Scalars* sc, uint32_t cap_full, uint32_t cap_narrow, uint32_t cap_cpu, int force_hash) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  const uint32_t cap[3] = {cap_full, cap_narrow, cap_cpu};
  for (int k = 0; k < 3; ++k) {
    const KeyRange r = sc->plan.range[k];
    TableCtl c;
    c.base = 0; c.span = 0; c.direct = 0; c.pad = 0;
    /* the reserved key never takes part in direct addressing (it has its own slot) */
    if (!force_hash && r.lo <= r.hi && r.hi - r.lo < (unsigned long long)cap[k]) { c.base = r.lo; c.span = r.hi - r.lo; c.direct = 1; }
    sc->plan.ctl[k] = c;
  }
}
/* frees what can be reached: the planned span in direct mode, the whole table otherwise */
__device__ __forceinline__ uint64_t table_extent(const Table& t) {
  return t.ctl->direct ? t.ctl->span + 1ull : (uint64_t)t.mask + 1ull;
}
__device__ __forceinline__ void clear_keys(const Table& t) {
  if (t.ctl->direct && !t.keyed_direct) return; /* keys are not used at all */
  const uint64_t n = table_extent(t);
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) t.keys[i] = KTJ_EMPTY_KEY;
  if (blockIdx.x == 0 && threadIdx.x == 0) t.keys[t.mask + 1ull] = KTJ_EMPTY_KEY;
}
__device__ __forceinline__ void clear_full(const Table& t, const FullCols& c) {
  const uint64_t n = table_extent(t);
  /* the payload is not cleared: every runtime row writes all of its slot's payload, and a slot
   * without a runtime row (its bit in has_runtime is clear) is never read */
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i <= n; i += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t k = i < n ? i : t.mask + 1ull; /* the last iteration clears the reserved slot */
    c.first[k] = 0xFFFFFFFFu; c.stream_src[k] = 0;
  }
  /* the bitmap: whole words up to the extent, and the word of the reserved slot */
  const uint64_t words = (n + 31) / 32;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i <= words; i += (uint64_t)gridDim.x * blockDim.x)
    c.has_runtime[i < words ? i : (t.mask + 1ull) / 32] = 0;
}
__device__ __forceinline__ void clear_narrow(const Table& t, const NarrowCols& c) {
  const uint64_t n = table_extent(t);
  NarrowPay z; z.ext_val = 0; z.info = 0; z.pay[0] = z.pay[1] = z.pay[2] = 0;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i <= n; i += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t k = i < n ? i : t.mask + 1ull;
    c.ext_src[k] = 0; c.kern_src[k] = 0; c.copy_src[k] = 0; c.pay[k] = z;
  }
}

/* all five in one launch: blockIdx.y picks the part */
__global__ void k_clear_tables(Table tf, FullCols fc, Table tn, NarrowCols nc, Table cpu) {
  switch (blockIdx.y) {
    case 0: clear_keys(tf); break;
    case 1: clear_keys(tn); break;
    case 2: clear_keys(cpu); break;
    case 3: clear_full(tf, fc); break;
    default: clear_narrow(tn, nc); break;
  }
}

hipError_t plan_tables(const KeyRange* parts, uint64_t n_generic, uint64_t n_runtime, uint64_t n_device,
                       const ktj_extcorr_rec* e, uint64_t n_ext, uint32_t cap_full, uint32_t cap_narrow, uint32_t cap_cpu,
                       bool force_hash, Scalars* sc, hipStream_t st) {
  const dim3 b(KTJ_BLOCK);
  /* parts: [generic ids | runtime ids | runtime ids narrowed | device ids], decode_blocks() entries each */
  const uint64_t bg = decode_blocks(n_generic), br = decode_blocks(n_runtime), bd = decode_blocks(n_device);
  RangeJobs jobs;
  uint32_t n_jobs = 0;
  auto job = [&](const KeyRange* src, uint64_t n, uint32_t dst) { if (n) { jobs.src[n_jobs] = src; jobs.n[n_jobs] = n; jobs.dst[n_jobs] = dst; ++n_jobs; } };
  job(parts, bg, KTJ_TBL_CPU);
  job(parts + bg, br, KTJ_TBL_FULL);
  job(parts + bg + br, br, KTJ_TBL_NARROW);
  job(parts + bg + 2 * br, bd, KTJ_TBL_FULL);
  for (uint32_t k = n_jobs; k < 4; ++k) { jobs.src[k] = nullptr; jobs.n[k] = 0; jobs.dst[k] = 0; }
  if (n_jobs) hipLaunchKernelGGL(k_merge_ranges, dim3(n_jobs * MERGE_SPLIT), dim3(256), 0, st, jobs, sc);
  if (n_ext)
    hipLaunchKernelGGL(k_key_range, dim3(n_ext < 512ull * KTJ_BLOCK * 4 ? grid_for(n_ext, KTJ_BLOCK * 4) : 512u), b, 0, st, reinterpret_cast<const uint64_t*>(e), 2u,
                       n_ext, 0, &sc->plan.range[KTJ_TBL_NARROW]);
  hipLaunchKernelGGL(k_plan_tables, dim3(1), dim3(64), 0, st, sc, cap_full, cap_narrow, cap_cpu, force_hash ? 1 : 0);
  return KTJ_LAUNCH_CHECK();
}
hipError_t clear_tables(Table tf, FullCols fc, Table tn, NarrowCols nc, Table cpu, hipStream_t st) {
  uint64_t most = (uint64_t)tf.mask + 1;
  if ((uint64_t)tn.mask + 1 > most) most = (uint64_t)tn.mask + 1;
  if ((uint64_t)cpu.mask + 1 > most) most = (uint64_t)cpu.mask + 1;
  hipLaunchKernelGGL(k_clear_tables, dim3(grid_stride_for(most, KTJ_BLOCK * 4), 5), dim3(KTJ_BLOCK), 0, st, tf, fc, tn, nc, cpu);
  return KTJ_LAUNCH_CHECK();
}

/* What linkedActivity() (GenericActivityProfiler.cpp:397-408) finds for an external id: the slot's
 * "External id" value and link flags, or zeros when no CPU op has the id. */
__device__ __forceinline__ void resolved_external(uint64_t ext_id, const Table& cpu, const uint32_t* cpu_row, const ktj_generic_rec* g,
                                                  const EmitCtx& ctx, int32_t* ext_val, uint32_t* info) {
  *ext_val = 0;
  *info = 0;
  const uint32_t cs = slot_find(cpu, ext_id);
  if (cs == KTJ_NOSLOT) return;
  *ext_val = (int32_t)(int64_t)ext_id;
  *info = KTJ_NP_LINKED;
  if (cpu_row) { /* the linked op is the last record with that id (activityMap_, GenericActivityProfiler.cpp:262) */
    const uint32_t row = cpu_row[cs];
    if (row) *info |= collective_for_linked(g[row - 1], ctx) << KTJ_NP_COLL_SHIFT;
  }
}
/* cpuCorrelationMap_[correlation] = externalId: RocmActivityProfiler.cpp:135-148.  The last record of
 * a correlation id stays (atomicMax over the record index).  Every record resolves its external id
 * against the CPU-op ids at once and writes the result into the slot: that is final when no two
 * records share a correlation id, which the returning atomicMax tells; only otherwise
 * k_resolve_external lets the winners write again.  The CPU-op ids are in their table already, the
 * table was cleared, and the runtime rows come later. */
__global__ void k_build_extcorr(const ktj_extcorr_rec* e, uint64_t n, Table tn, NarrowCols nc, Table cpu, const uint32_t* cpu_row,
                                const ktj_generic_rec* g, EmitCtx ctx, Scalars* sc) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  bool repeats = false;
  if (i < n) {
    ktj_extcorr_rec rec;
    rec.correlation = load_once(&e[i].correlation);
    rec.external_id = load_once(&e[i].external_id);
    const uint32_t slot = slot_insert(tn, rec.correlation);
    if (slot == KTJ_NOSLOT) flag_error(sc, KTJ_DEVERR_TABLE_FULL);
    else {
      repeats = atomicMax(&nc.ext_src[slot], (uint32_t)i + 1u) != 0u;
      int32_t ext_val;
      uint32_t info;
      resolved_external(rec.external_id, cpu, cpu_row, g, ctx, &ext_val, &info);
      if (info != 0) { nc.pay[slot].ext_val = ext_val; nc.pay[slot].info = info; }
    }
  }
  /* one store per workgroup at most: every lane storing the same flag would queue up in L2 */
  if (__syncthreads_or(repeats ? 1 : 0) && threadIdx.x == 0) sc->ext_ids_repeat = 1;
}
/* activityMap_[act->correlationId()] = act: GenericActivityProfiler.cpp:262 */
/* cpu_row (optional): per slot, 1 + index of the last record with that id, for the traces whose
 * CPU ops hand collective metadata to the kernels linked to them */
__global__ void k_build_cpu_ids(const ktj_generic_rec* g, uint64_t n, Table cpu, uint32_t* cpu_row, Scalars* sc) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t slot = slot_insert(cpu, (uint64_t)(int64_t)load_once(&g[i].id));
  if (slot == KTJ_NOSLOT) { flag_error(sc, KTJ_DEVERR_TABLE_FULL); return; }
  if (cpu_row) atomicMax(&cpu_row[slot], (uint32_t)i + 1u);
}
/* Only when external-correlation records share a correlation id: the record that won the slot
 * writes what it resolved again, zeros included, over whatever the other records of the id left. */
__global__ void k_resolve_external(const ktj_extcorr_rec* e, uint64_t n, Table tn, NarrowCols nc, Table cpu,
                                   const uint32_t* cpu_row, const ktj_generic_rec* g, EmitCtx ctx, const Scalars* sc) {
  if (sc->ext_ids_repeat == 0) return;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    const ktj_extcorr_rec rec = e[i];
    const uint32_t slot = slot_find(tn, rec.correlation);
    if (slot == KTJ_NOSLOT || nc.ext_src[slot] != (uint32_t)i + 1u) continue;
    int32_t ext_val;
    uint32_t info;
    resolved_external(rec.external_id, cpu, cpu_row, g, ctx, &ext_val, &info);
    nc.pay[slot].ext_val = ext_val;
    nc.pay[slot].info = info;
  }
}
__device__ __forceinline__ bool is_async_op(uint32_t domain) { return domain != KTJ_DOM_MEMSET; }

/* One pass over the device rows with one slot of each table:
 *  - "External id" (output_json.cpp:871-874) from the narrow slot,
 *  - checkTimestampOrder (GenericActivityProfiler.cpp:363-395) against the first row of the id,
 *  - the stream of the correlation-matched runtime row (RocmStreamQueue.h:56-75, first pass),
 *  - the size or grid/block the launching row hands over (RocprofActivity_inl.h:161-180).
 * The first row of an id is its first runtime row wherever one exists (runtime rows arrive before
 * device rows), which a bitmap tells, and the slot's payload holds that row's timestamp, so the
 * array of first rows is only touched for ids that no runtime row has: in-window device rows take part in "first seen" there and are
 * checked afterwards by k_device_orphans.  Rows outside the window still take a stream from the
 * slot (slots with a stream come from runtime rows and exist already). */
__global__ void k_link_device(uint64_t n, Columns c, uint64_t first_device, Table tf, FullCols fc, Table tn, NarrowCols nc,
                              DevLink* link, Scalars* sc) {
  uint32_t n_linked = 0, n_bad = 0, n_unresolved = 0, n_orphans = 0;
  const bool have_stream_src = sc->have_stream_src != 0;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t a = first_device + i;
    /* all reads first (the row's columns, then one slot of each table), all writes after them:
     * the round trips overlap instead of queueing behind each other */
    const uint64_t id = load_once(&c.corr[a]);
    const uint32_t meta = load_once(&c.meta[a]);
    int64_t res = load_once(&c.res[a]);
    const int64_t t2 = load_once(&c.ts[a]);
    const uint32_t domain = (meta & KTJ_M_KIND_MASK) >> KTJ_M_KIND_SHIFT;
    const bool valid = (meta & KTJ_M_VALID) != 0;
    const uint32_t sn = slot_find(tn, narrow_corr_key(id));
    const uint32_t sf = valid ? slot_insert(tf, id) : slot_find(tf, id);
    NarrowPay np;
    np.ext_val = 0; np.info = 0; np.pay[0] = np.pay[1] = np.pay[2] = 0;
    FullPay fp;
    fp.first_ts = 0; fp.stream = 0;
    uint32_t runtime_bits = 0;
    if (sn != KTJ_NOSLOT) np = nc.pay[sn];
    if (sf != KTJ_NOSLOT) {
      fp = fc.pay[sf];
      runtime_bits = fc.has_runtime[sf >> 5];
      if (!((runtime_bits >> (sf & 31u)) & 1u)) { fp.first_ts = 0; fp.stream = 0; } /* no runtime row wrote this slot in this pass */
    }
    DevLink l;
    l.p[0] = l.p[1] = l.p[2] = 0; l.flags = 0; l.coll = 0;
    if (sn != KTJ_NOSLOT) {
      if ((np.info & KTJ_NP_LINKED) && valid) ++n_linked;
      if (domain != KTJ_DOM_MEMSET && (np.info & KTJ_NP_KIND_MASK) != 0) {
        l.flags = np.info & KTJ_NP_KIND_MASK;
        l.p[0] = np.pay[0]; l.p[1] = np.pay[1]; l.p[2] = np.pay[2];
      }
      l.coll = np.info >> KTJ_NP_COLL_SHIFT;
    }
    store_once(&c.ext[a], np.ext_val);
    if (valid && sf == KTJ_NOSLOT) flag_error(sc, KTJ_DEVERR_TABLE_FULL);
    if (sf != KTJ_NOSLOT) {
      if (valid) {
        if ((runtime_bits >> (sf & 31u)) & 1u) { /* act1 = the first runtime row, act2 = this row */
          const int64_t t1 = fp.first_ts;
          if (t2 != 0 && t1 > t2) ++n_bad;
        } else {
          if (fc.first[sf] > (uint32_t)a) atomicMin(&fc.first[sf], (uint32_t)a);
          l.flags |= KTJ_DL_ORPHAN;
          ++n_orphans;
        }
      }
      if (have_stream_src && is_async_op(domain) && res == 0 && fp.stream != 0) { res = (int64_t)fp.stream; c.res[a] = res; }
    }
    {
      typedef unsigned int v4u __attribute__((ext_vector_type(4)));
      static_assert(sizeof(DevLink) == 32, "two 16-byte stores");
      const v4u* lv = reinterpret_cast<const v4u*>(&l);
      v4u* dst = reinterpret_cast<v4u*>(&link[i]);
      store_once(&dst[0], lv[0]);
      store_once(&dst[1], lv[1]);
    }
    if (is_async_op(domain) && res == 0) ++n_unresolved;
  }
  block_add(sc, KTJ_CNT_LINKED, n_linked);
  block_add(sc, KTJ_CNT_OUT_OF_ORDER, n_bad);
  block_add_to(&sc->n_unresolved, n_unresolved);
  block_add_to(&sc->n_device_orphans, n_orphans);
}
/* Only when some in-window device row has an id that no runtime row has: such a row is checked
 * against the first device row of its id (act1 = this row, act2 = the first one). */
__global__ void k_device_orphans(uint64_t n, Columns c, uint64_t first_device, Table tf, FullCols fc, const DevLink* link,
                                 Scalars* sc) {
  if (sc->n_device_orphans == 0) return;
  uint32_t n_bad = 0;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    if (!(link[i].flags & KTJ_DL_ORPHAN)) continue;
    const uint64_t a = first_device + i;
    const uint32_t sf = slot_find(tf, c.corr[a]);
    if (sf == KTJ_NOSLOT) continue;
    const uint64_t f = fc.first[sf];
    if (f != a && f != 0xFFFFFFFFull) {
      const int64_t t1 = c.ts[a], t2 = c.ts[f];
      if (t2 != 0 && t1 > t2) ++n_bad;
    }
  }
  block_add(sc, KTJ_CNT_OUT_OF_ORDER, n_bad);
}

hipError_t build_cpu_ids(const ktj_generic_rec* g, uint64_t n, Table cpu, uint32_t* cpu_row, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_build_cpu_ids, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, g, n, cpu, cpu_row, sc);
  return KTJ_LAUNCH_CHECK();
}
/* after build_cpu_ids: the external ids are resolved against that table as the records pass */
hipError_t build_extcorr(const ktj_extcorr_rec* e, uint64_t n, Table tn, NarrowCols nc, Table cpu, const uint32_t* cpu_row,
                         const ktj_generic_rec* g, EmitCtx ctx, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_build_extcorr, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, e, n, tn, nc, cpu, cpu_row, g, ctx, sc);
  hipLaunchKernelGGL(k_resolve_external, dim3(grid_stride_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, e, n, tn, nc, cpu, cpu_row, g,
                     ctx, (const Scalars*)sc);
  return KTJ_LAUNCH_CHECK();
}
hipError_t link_device_rows(uint64_t n, Columns c, uint64_t first_device, Table tf, FullCols fc, Table tn, NarrowCols nc,
                            DevLink* link, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_link_device, dim3(grid_stride_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, n, c, first_device, tf, fc, tn,
                     nc, link, sc);
  hipLaunchKernelGGL(k_device_orphans, dim3(grid_stride_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, n, c, first_device, tf, fc,
                     (const DevLink*)link, sc);
  return KTJ_LAUNCH_CHECK();
}

/* ---- GPU user annotations: GenericActivityProfiler.cpp:277-327, 423-433 ---- */
/* userCorrelationMap_[correlation] = externalId, the last record of an id stays */
__global__ void k_build_usercorr(const ktj_extcorr_rec* u, uint64_t n, SpanTables t, Scalars* sc) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t slot = table_insert(t.u_keys, t.u_mask, u[i].correlation);
  if (slot == KTJ_NOSLOT) { flag_error(sc, KTJ_DEVERR_TABLE_FULL); return; }
  atomicMax(&t.u_src[slot], (uint32_t)i + 1u);
}
__device__ __forceinline__ uint64_t span_hash(int64_t device, int64_t resource, uint64_t ext) {
  uint64_t h = hash64(ext ^ hash64((uint64_t)resource + 0x9E3779B97F4A7C15ULL) ^ hash64((uint64_t)device * 0xC2B2AE3D27D4EB4FULL + 1ULL));
  return h == KTJ_EMPTY_KEY ? 0x5bd1e995ULL : h;
}
/* the annotation a device row belongs to: its id and the slot of that id in the CPU-op table */
__device__ __forceinline__ bool span_of_row(const ktj_extcorr_rec* u, const SpanTables& t, const Table& cpu, uint64_t corr,
                                            uint64_t* ext, uint32_t* cpu_slot) {
  const uint32_t us = table_find(t.u_keys, t.u_mask, corr);
  if (us == KTJ_NOSLOT || t.u_src[us] == 0) return false;
  *ext = u[t.u_src[us] - 1u].external_id;
  *cpu_slot = slot_find(cpu, *ext);
  return *cpu_slot != KTJ_NOSLOT;
}
/* insertOrExtendEvent for every in-window device row: extent of the span, its first row */
__global__ void k_span_extend(const ktj_extcorr_rec* u, uint64_t n, Columns c, uint64_t first_device, Table cpu, SpanTables t,
                              Scalars* sc) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint64_t a = first_device + i;
  if (!(c.meta[a] & KTJ_M_VALID)) return;
  uint64_t ext; uint32_t cs;
  if (!span_of_row(u, t, cpu, c.corr[a], &ext, &cs)) return;
  const uint32_t slot = table_insert(t.hash, t.mask, span_hash(c.dev[a], c.res[a], ext));
  if (slot == KTJ_NOSLOT) { flag_error(sc, KTJ_DEVERR_TABLE_FULL); return; }
  const int64_t ts = c.ts[a];
  atomicMin(&t.first[slot], (uint32_t)i);
  atomicMin((unsigned long long*)&t.lo[slot], (unsigned long long)((uint64_t)ts ^ 0x8000000000000000ULL));
  atomicMax((unsigned long long*)&t.hi[slot], (unsigned long long)((uint64_t)(ts + c.dur[a]) ^ 0x8000000000000000ULL));
  if (ts == 0) t.zero[slot] = 1u;
}
/* createUserGpuSpan: the first row of a span names it (single writer per slot) */
__global__ void k_span_owner(const ktj_extcorr_rec* u, const ktj_generic_rec* g, uint64_t n, Columns c, uint64_t first_device,
                             Table cpu, const uint32_t* cpu_row, SpanTables t) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint64_t a = first_device + i;
  if (!(c.meta[a] & KTJ_M_VALID)) return;
  uint64_t ext; uint32_t cs;
  if (!span_of_row(u, t, cpu, c.corr[a], &ext, &cs)) return;
  const uint32_t slot = table_find(t.hash, t.mask, span_hash(c.dev[a], c.res[a], ext));
  if (slot == KTJ_NOSLOT || t.first[slot] != (uint32_t)i) return;
  t.dev[slot] = (int32_t)c.dev[a]; t.res[slot] = c.res[a]; t.ext[slot] = ext;
  const uint32_t row = cpu_row[cs]; /* the annotation is the last record with that id */
  t.name[slot] = row ? g[row - 1u].name_id : KTJ_NONE;
}
__global__ void k_span_compact(SpanTables t, SpanOut* out, uint32_t* n_out) {
  const uint64_t s = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (s > (uint64_t)t.mask + 1u || t.hash[s] == KTJ_EMPTY_KEY || t.first[s] == 0xFFFFFFFFu) return;
  SpanOut o;
  o.res = t.res[s]; o.ext = t.ext[s];
  o.start = (int64_t)(t.lo[s] ^ 0x8000000000000000ULL); o.end = (int64_t)(t.hi[s] ^ 0x8000000000000000ULL);
  o.dev = t.dev[s]; o.name = t.name[s]; o.first = t.first[s]; o.zero = t.zero[s] ? (uint32_t)s + 1u : 0u;
  out[atomicAdd(n_out, 1u)] = o;
}
/* rows of the spans whose start needs the sequential rule (a row at time 0), for the host */
__global__ void k_span_members(const ktj_extcorr_rec* u, uint64_t n, Columns c, uint64_t first_device, Table cpu,
                               SpanTables t, SpanMember* out, uint32_t cap_out, uint32_t* n_out) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint64_t a = first_device + i;
  if (!(c.meta[a] & KTJ_M_VALID)) return;
  uint64_t ext; uint32_t cs;
  if (!span_of_row(u, t, cpu, c.corr[a], &ext, &cs)) return;
  const uint32_t slot = table_find(t.hash, t.mask, span_hash(c.dev[a], c.res[a], ext));
  if (slot == KTJ_NOSLOT || t.zero[slot] == 0) return;
  const uint32_t k = atomicAdd(n_out, 1u);
  if (k < cap_out) { SpanMember m; m.slot = slot + 1u; m.row = (uint32_t)i; m.ts = c.ts[a]; out[k] = m; }
}
hipError_t build_usercorr(const ktj_extcorr_rec* u, uint64_t n, SpanTables t, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_build_usercorr, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, u, n, t, sc);
  return KTJ_LAUNCH_CHECK();
}
hipError_t group_spans(const ktj_extcorr_rec* u, const ktj_generic_rec* g, uint64_t n_device, Columns c, uint64_t first_device,
                       Table cpu, const uint32_t* cpu_row, SpanTables t, SpanOut* out, uint32_t* n_out, Scalars* sc,
                       hipStream_t st) {
  hipError_t e = fill_u32(n_out, 0, 1, st);
  if (e != hipSuccess || n_device == 0) return e;
  const dim3 grid(grid_for(n_device, KTJ_BLOCK)), block(KTJ_BLOCK);
  hipLaunchKernelGGL(k_span_extend, grid, block, 0, st, u, n_device, c, first_device, cpu, t, sc);
  hipLaunchKernelGGL(k_span_owner, grid, block, 0, st, u, g, n_device, c, first_device, cpu, cpu_row, t);
  hipLaunchKernelGGL(k_span_compact, dim3(grid_for((uint64_t)t.mask + 2u, KTJ_BLOCK)), block, 0, st, t, out, n_out);
  return KTJ_LAUNCH_CHECK();
}
hipError_t span_members(const ktj_extcorr_rec* u, uint64_t n_device, Columns c, uint64_t first_device, Table cpu,
                        SpanTables t, SpanMember* out, uint32_t cap_out, uint32_t* n_out, hipStream_t st) {
  hipError_t e = fill_u32(n_out, 0, 1, st);
  if (e != hipSuccess || n_device == 0) return e;
  hipLaunchKernelGGL(k_span_members, dim3(grid_for(n_device, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, u, n_device, c, first_device,
                     cpu, t, out, cap_out, n_out);
  return KTJ_LAUNCH_CHECK();
}

/* ---- stream back-fill: libkineto/src/RocmStreamQueue.h:42-136 (its first pass, the stream of
 * the correlation-matched runtime row, is part of k_link_device) ---- */
/* pass 2a: queue → stream, ambiguous when one queue shows two different streams.  Passes 2a/2b
 * have no effect when the first pass left no row without a stream (the usual case: every device
 * row has a launching runtime row), and return at once then. */
__global__ void k_queue_build(const DevBrief* d, uint64_t n, Columns c, uint64_t first_device, StreamTables t,
                              Scalars* sc) {
  if (sc->have_stream_src == 0 || sc->n_unresolved == 0) return;
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint64_t stream = (uint64_t)c.res[first_device + i];
  const uint64_t queue = d[i].queue;
  if (!is_async_op(d[i].domain) || stream == 0 || queue == 0) return;
  const uint32_t slot = table_insert_counted(t.q_keys, KTJ_QUEUE_CAP - 1u, queue, &sc->n_queues, KTJ_MAX_QUEUES);
  if (slot == KTJ_NOSLOT) { flag_error(sc, KTJ_DEVERR_QUEUES); return; }
  unsigned long long cur = t.q_stream[slot];
  if (cur == 0) cur = atomicCAS((unsigned long long*)&t.q_stream[slot], 0ULL, (unsigned long long)stream);
  if (cur != 0 && cur != stream) t.q_amb[slot] = 1u;
}
/* pass 2b: rows still without a stream take their queue's stream */
__global__ void k_queue_fill(const DevBrief* d, uint64_t n, Columns c, uint64_t first_device, StreamTables t,
                             const Scalars* sc) {
  if (sc->have_stream_src == 0 || sc->n_unresolved == 0) return;
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint64_t a = first_device + i;
  if (!is_async_op(d[i].domain) || c.res[a] != 0) return;
  const uint32_t slot = table_find(t.q_keys, KTJ_QUEUE_CAP - 1u, d[i].queue);
  if (slot == KTJ_NOSLOT || t.q_amb[slot] != 0 || t.q_stream[slot] == 0) return;
  c.res[a] = (int64_t)t.q_stream[slot];
}
__device__ __forceinline__ bool dense_key(const DevBrief& d, uint64_t stream, uint64_t* key) {
  if (!is_async_op(d.domain)) return false;
  if (stream != 0) *key = stream;
  else if (d.queue != 0) *key = d.queue | (1ULL << 63);
  else return false;
  return true;
}
__device__ __forceinline__ uint64_t dense_hash(int32_t device, uint64_t key) {
  uint64_t h = hash64(key ^ hash64((uint64_t)(int64_t)device + 0x9E3779B97F4A7C15ULL));
  return h == KTJ_EMPTY_KEY ? 0x5bd1e995ULL : h;
}
/* pass 3a: first arrival index per (device, stream key).  Millions of rows share a few hundred
 * pairs, so each workgroup first reduces its rows in an LDS table and touches the global table
 * once per pair. */
#define DENSE_LOCAL_SLOTS 1024u
__global__ void k_dense_first(const DevBrief* d, uint64_t n, Columns c, uint64_t first_device, StreamTables t,
                              Scalars* sc) {
  __shared__ unsigned long long l_key[DENSE_LOCAL_SLOTS];
  __shared__ unsigned long long l_pair_key[DENSE_LOCAL_SLOTS];
  __shared__ int32_t l_pair_dev[DENSE_LOCAL_SLOTS];
  __shared__ uint32_t l_min[DENSE_LOCAL_SLOTS];
  if (sc->have_stream_src == 0) return;
  for (uint32_t k = threadIdx.x; k < DENSE_LOCAL_SLOTS; k += blockDim.x) { l_key[k] = KTJ_EMPTY_KEY; l_min[k] = 0xFFFFFFFFu; }
  __syncthreads();
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    uint64_t key;
    const DevBrief b = d[i];
    if (!dense_key(b, (uint64_t)c.res[first_device + i], &key)) continue;
    const uint64_t h = dense_hash(b.device, key);
    uint32_t slot = (uint32_t)(h >> 20) & (DENSE_LOCAL_SLOTS - 1u);
    bool placed = false;
    for (uint32_t probe = 0; probe < 16 && !placed; ++probe) {
      unsigned long long cur = l_key[slot];
      if (cur == KTJ_EMPTY_KEY) {
        cur = atomicCAS(&l_key[slot], (unsigned long long)KTJ_EMPTY_KEY, (unsigned long long)h);
        /* the pair itself, for the table entry: every row of the pair would write the same two values
         * (two pairs with one hash are told apart when the rows read the table back) */
        if (cur == KTJ_EMPTY_KEY) { l_pair_dev[slot] = b.device; l_pair_key[slot] = key; }
      }
      if (cur == KTJ_EMPTY_KEY || cur == h) { atomicMin(&l_min[slot], (uint32_t)i); placed = true; }
      else slot = (slot + 1u) & (DENSE_LOCAL_SLOTS - 1u);
    }
    if (!placed) { /* local table crowded: straight to the global one */
      const uint32_t g = table_insert(t.d_hash, KTJ_DENSE_CAP - 1u, h);
      if (g == KTJ_NOSLOT) flag_error(sc, KTJ_DEVERR_STREAMS);
      else {
        if (t.d_first[g] > (uint32_t)i) atomicMin(&t.d_first[g], (uint32_t)i);
        t.d_dev[g] = b.device; t.d_key[g] = key;
      }
    }
  }
  __syncthreads();
  for (uint32_t k = threadIdx.x; k < DENSE_LOCAL_SLOTS; k += blockDim.x) {
    const unsigned long long h = l_key[k];
    if (h == KTJ_EMPTY_KEY) continue;
    const uint32_t g = table_insert(t.d_hash, KTJ_DENSE_CAP - 1u, h);
    if (g == KTJ_NOSLOT) { flag_error(sc, KTJ_DEVERR_STREAMS); continue; }
    if (t.d_first[g] > l_min[k]) atomicMin(&t.d_first[g], l_min[k]);
    t.d_dev[g] = l_pair_dev[k]; t.d_key[g] = l_pair_key[k];
  }
}
/* pass 3b (one workgroup): index = 1 + number of pairs of the same device seen earlier */
#define KTJ_DENSE_MAX KTJ_MAX_STREAM_PAIRS
__global__ void k_dense_rank(StreamTables t, Scalars* sc) {
  __shared__ uint32_t slots[KTJ_DENSE_MAX];
  __shared__ uint32_t count;
  if (sc->have_stream_src == 0) return;
  if (threadIdx.x == 0) count = 0;
  __syncthreads();
  for (uint32_t s = threadIdx.x; s <= KTJ_DENSE_CAP; s += blockDim.x) {
    if (t.d_hash[s] != KTJ_EMPTY_KEY && t.d_first[s] != 0xFFFFFFFFu) {
      const uint32_t k = atomicAdd(&count, 1u);
      if (k < KTJ_DENSE_MAX) slots[k] = s;
    }
  }
  __syncthreads();
  const uint32_t m = count;
  if (m > KTJ_DENSE_MAX) { if (threadIdx.x == 0) flag_error(sc, KTJ_DEVERR_STREAMS); return; }
  if (threadIdx.x == 0) sc->n_dense = m;
  for (uint32_t k = threadIdx.x; k < m; k += blockDim.x) {
    const uint32_t s = slots[k];
    const int32_t dev = t.d_dev[s];
    const uint32_t first = t.d_first[s];
    uint32_t rank = 1;
    for (uint32_t j = 0; j < m; ++j) {
      const uint32_t o = slots[j];
      if (t.d_dev[o] == dev && t.d_first[o] < first) ++rank;
    }
    t.d_rank[s] = rank;
  }
}
/* pass 3c: resourceId() = stream != 0 ? stream : queue (RocprofActivity.h:100-102) */
__global__ void k_dense_assign(const DevBrief* d, uint64_t n, Columns c, uint64_t first_device, StreamTables t,
                               Scalars* sc) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint64_t a = first_device + i;
  const DevBrief b = d[i];
  if (!is_async_op(b.domain)) return;
  uint64_t stream = (uint64_t)c.res[a];
  if (sc->have_stream_src != 0) {
    uint64_t key;
    if (dense_key(b, stream, &key)) {
      const uint32_t slot = table_find(t.d_hash, KTJ_DENSE_CAP - 1u, dense_hash(b.device, key));
      if (slot == KTJ_NOSLOT || t.d_dev[slot] != b.device || t.d_key[slot] != key) {
        flag_error(sc, KTJ_DEVERR_HASH_COLLISION);
      } else stream = t.d_rank[slot];
    }
  }
  c.res[a] = (int64_t)(stream != 0 ? stream : b.queue);
}

hipError_t backfill_streams(const DevBrief* d, uint64_t n, Columns c, uint64_t first_device, StreamTables t,
                            Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  const dim3 g(grid_for(n, KTJ_BLOCK)), b(KTJ_BLOCK);
  hipLaunchKernelGGL(k_queue_build, g, b, 0, st, d, n, c, first_device, t, sc);
  hipLaunchKernelGGL(k_queue_fill, g, b, 0, st, d, n, c, first_device, t, (const Scalars*)sc);
  hipLaunchKernelGGL(k_dense_first, dim3(grid_stride_for(n, KTJ_BLOCK * 8)), b, 0, st, d, n, c, first_device, t, sc);
  hipLaunchKernelGGL(k_dense_rank, dim3(1), dim3(1024), 0, st, t, sc);
  hipLaunchKernelGGL(k_dense_assign, g, b, 0, st, d, n, c, first_device, t, sc);
  return KTJ_LAUNCH_CHECK();
}

/* ------------------------------------------------------------------------------------------ */
/* stage 3: canonical order = stable sort by (deviceId, resourceId, timestamp), signed            */
/* ------------------------------------------------------------------------------------------ */
/* Workgroup-local set in LDS in front of the global set: a value reaches the global table once
 * per workgroup instead of once per row.  (All rows share a handful of device/resource ids, and
 * millions of probes of the same few global slots serialise in L2.)  Returns true when the
 * caller is the first in its workgroup to see the key, or when the local set is full. */
#define LOCAL_SET_SLOTS 1024u
__device__ __forceinline__ bool local_set_first(unsigned long long* lds, uint64_t key) {
  const uint32_t h = ((uint32_t)key ^ ((uint32_t)(key >> 32) * 0x9E3779B1u)) * 0x85EBCA6Bu;
  uint32_t slot = h >> 22; /* 10 bits */
  for (uint32_t probe = 0; probe < 16; ++probe) {
    const unsigned long long cur = lds[slot];
    if (cur == key) return false;
    if (cur == KTJ_EMPTY_KEY) {
      const unsigned long long prev = atomicCAS(&lds[slot], (unsigned long long)KTJ_EMPTY_KEY, (unsigned long long)key);
      if (prev == KTJ_EMPTY_KEY) return true;
      if (prev == key) return false;
    }
    slot = (slot + 1u) & (LOCAL_SET_SLOTS - 1u);
  }
  return true;
}
/* a wavefront's rows mostly share one value: only one lane of those that hold the value of the
 * first active lane goes on to probe, and lanes with another value probe for themselves */
__device__ __forceinline__ bool wave_representative(uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  const uint64_t first = ((uint64_t)hi << 32) | lo;
  const uint64_t same = __ballot(v == first); /* never empty: the first active lane is in it */
  return v != first || (uint32_t)__builtin_ctzll(same) == lane_id();
}
#define COLLECT_ROWS 4
__global__ void k_collect_distinct(Columns c, uint64_t n, SortSets s, Scalars* sc) {
  __shared__ uint64_t red_min[KTJ_BLOCK >> 6], red_max[KTJ_BLOCK >> 6];
  __shared__ unsigned long long seen_dev[LOCAL_SET_SLOTS], seen_res[LOCAL_SET_SLOTS];
  for (uint32_t k = threadIdx.x; k < LOCAL_SET_SLOTS; k += blockDim.x) { seen_dev[k] = KTJ_EMPTY_KEY; seen_res[k] = KTJ_EMPTY_KEY; }
  __syncthreads();
  uint64_t mn = ~0ULL, mx = 0ULL;
  uint32_t n_valid = 0;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t a0 = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; a0 < n; a0 += stride * COLLECT_ROWS) {
    uint32_t meta[COLLECT_ROWS];
    uint64_t dev[COLLECT_ROWS], res[COLLECT_ROWS], ts[COLLECT_ROWS];
#pragma unroll
    for (int r = 0; r < COLLECT_ROWS; ++r) { /* all loads of the group in flight together */
      const uint64_t a = a0 + (uint64_t)r * stride;
      const bool in = a < n;
      meta[r] = in ? c.meta[a] : 0u;
      dev[r] = in ? (uint64_t)c.dev[a] : 0;
      res[r] = in ? (uint64_t)c.res[a] : 0;
      ts[r] = in ? (uint64_t)c.ts[a] : 0;
    }
#pragma unroll
    for (int r = 0; r < COLLECT_ROWS; ++r) {
      if (!(meta[r] & KTJ_M_VALID)) continue;
      if (wave_representative(dev[r]) && (dev[r] == KTJ_EMPTY_KEY || local_set_first(seen_dev, dev[r]))) {
        if (table_insert(s.dev_keys, KTJ_SET_CAP - 1u, dev[r]) == KTJ_NOSLOT) flag_error(sc, KTJ_DEVERR_DISTINCT_DEVICES);
      }
      if (wave_representative(res[r]) && (res[r] == KTJ_EMPTY_KEY || local_set_first(seen_res, res[r]))) {
        if (table_insert(s.res_keys, KTJ_SET_CAP - 1u, res[r]) == KTJ_NOSLOT) flag_error(sc, KTJ_DEVERR_DISTINCT_RESOURCES);
      }
      const uint64_t tb = ts[r] ^ 0x8000000000000000ULL;
      mn = tb < mn ? tb : mn;
      mx = tb > mx ? tb : mx;
      ++n_valid;
    }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const uint64_t on = __shfl_xor((unsigned long long)mn, o), ox = __shfl_xor((unsigned long long)mx, o);
    mn = on < mn ? on : mn;
    mx = ox > mx ? ox : mx;
  }
  if (lane_id() == 0) { red_min[threadIdx.x >> 6] = mn; red_max[threadIdx.x >> 6] = mx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (uint32_t k = 1; k < (blockDim.x >> 6); ++k) {
      mn = red_min[k] < mn ? red_min[k] : mn;
      mx = red_max[k] > mx ? red_max[k] : mx;
    }
    if (mn <= mx) { /* (reading the current range first, to skip the atomics, costs more than they do) */
      atomicMin(&sc->ts_min_biased, (unsigned long long)mn);
      atomicMax(&sc->ts_max_biased, (unsigned long long)mx);
    }
  }
  block_add(sc, KTJ_CNT_VALID, n_valid);
}
/* one workgroup per set: rank of each distinct value = number of smaller values (signed) */
__global__ void k_rank_distinct(SortSets s, Scalars* sc) {
  __shared__ int64_t vals[KTJ_SET_MAX];
  __shared__ uint32_t slots[KTJ_SET_MAX];
  __shared__ uint32_t count;
  uint64_t* keys = blockIdx.x == 0 ? s.dev_keys : s.res_keys;
  uint32_t* rank = blockIdx.x == 0 ? s.dev_rank : s.res_rank;
  if (threadIdx.x == 0) count = 0;
  __syncthreads();
  for (uint32_t k = threadIdx.x; k <= KTJ_SET_CAP; k += blockDim.x) {
    bool occupied = k < KTJ_SET_CAP ? keys[k] != KTJ_EMPTY_KEY : keys[k] == 0;
    if (occupied) {
      const uint32_t j = atomicAdd(&count, 1u);
      if (j < KTJ_SET_MAX) { slots[j] = k; vals[j] = k < KTJ_SET_CAP ? (int64_t)keys[k] : (int64_t)-1; }
    }
  }
  __syncthreads();
  const uint32_t m = count;
  if (m > KTJ_SET_MAX) {
    if (threadIdx.x == 0) flag_error(sc, blockIdx.x == 0 ? KTJ_DEVERR_DISTINCT_DEVICES : KTJ_DEVERR_DISTINCT_RESOURCES);
    return;
  }
  if (threadIdx.x == 0) { if (blockIdx.x == 0) sc->n_dev_ranks = m; else sc->n_res_ranks = m; }
  for (uint32_t k = threadIdx.x; k < m; k += blockDim.x) {
    const int64_t v = vals[k];
    uint32_t r = 0;
    for (uint32_t j = 0; j < m; ++j) r += vals[j] < v ? 1u : 0u;
    rank[slots[k]] = r;
  }
}
/* Rank of a value through its set.  The rows of a wavefront mostly share one value: then a single
 * lookup with a wavefront-uniform key (which the compiler can keep on the scalar unit) serves all
 * lanes. */
__device__ __forceinline__ uint64_t set_rank(const uint64_t* keys, const uint32_t* rank, uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  const uint64_t first = ((uint64_t)hi << 32) | lo;
  if (__ballot(v != first) == 0) {
    const uint32_t slot = table_find(keys, KTJ_SET_CAP - 1u, first);
    return slot != KTJ_NOSLOT ? rank[slot] : 0;
  }
  const uint32_t slot = table_find(keys, KTJ_SET_CAP - 1u, v);
  return slot != KTJ_NOSLOT ? rank[slot] : 0;
}
/* The same for a thread that looks up one row after the other: rows that follow each other in a
 * record buffer mostly belong to one stream or thread, so the last wavefront-wide value and its rank
 * are kept, and a lookup (two dependent loads at least) is only made when the value changes.  A
 * lane's memo is a (value, rank) pair that it took part in looking up, or nothing. */
struct RankMemo { uint64_t key; uint32_t rank; bool have; };
__device__ __forceinline__ uint64_t set_rank_memo(const uint64_t* keys, const uint32_t* rank, uint64_t v, RankMemo& m) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  const uint64_t first = ((uint64_t)hi << 32) | lo;
  if (__ballot(v != first) == 0) {
    if (m.have && m.key == first) return m.rank;
    const uint32_t slot = table_find(keys, KTJ_SET_CAP - 1u, first);
    m.key = first; m.rank = slot != KTJ_NOSLOT ? rank[slot] : 0; m.have = true;
    return m.rank;
  }
  const uint32_t slot = table_find(keys, KTJ_SET_CAP - 1u, v);
  return slot != KTJ_NOSLOT ? rank[slot] : 0;
}
__global__ void k_make_keys(Columns c, uint64_t n, SortSets s, const Scalars* sc, uint32_t ts_bits, uint32_t res_bits,
                            uint32_t key_bits, uint64_t* keys, uint32_t* vals) {
  const uint64_t a = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (a >= n) return;
  uint64_t key = key_bits >= 64 ? ~0ULL : (1ULL << key_bits); /* dropped rows sort behind everything */
  if (c.meta[a] & KTJ_M_VALID) {
    const uint64_t rd = set_rank(s.dev_keys, s.dev_rank, (uint64_t)c.dev[a]);
    const uint64_t rr = set_rank(s.res_keys, s.res_rank, (uint64_t)c.res[a]);
    const uint64_t rel = ((uint64_t)c.ts[a] ^ 0x8000000000000000ULL) - sc->ts_min_biased;
    uint64_t hi = (rd << res_bits) | rr;
    key = ts_bits >= 64 ? rel : ((hi << ts_bits) | rel);
  }
  keys[a] = key;
  vals[a] = (uint32_t)a;
}

/* Wide timestamp spans (a row at time 0 next to rows at wall-clock time) do not fit one 64-bit
 * composite key.  The order is then built in two stable sorts: by timestamp, then by the
 * (device, resource) ranks of the rows in that order. */
__global__ void k_make_ts_keys(Columns c, uint64_t n, const Scalars* sc, uint64_t* keys, uint32_t* vals) {
  const uint64_t a = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (a >= n) return;
  keys[a] = (c.meta[a] & KTJ_M_VALID) ? (((uint64_t)c.ts[a] ^ 0x8000000000000000ULL) - sc->ts_min_biased) : 0;
  vals[a] = (uint32_t)a;
}
__global__ void k_make_rank_keys(Columns c, const uint32_t* order, uint64_t n, SortSets s, uint32_t res_bits,
                                 uint32_t rank_bits, uint64_t* keys, uint32_t* vals) {
  const uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n) return;
  const uint32_t a = order[p];
  uint64_t key = 1ULL << rank_bits; /* dropped rows sort behind everything */
  if (c.meta[a] & KTJ_M_VALID) {
    const uint64_t rd = set_rank(s.dev_keys, s.dev_rank, (uint64_t)c.dev[a]);
    const uint64_t rr = set_rank(s.res_keys, s.res_rank, (uint64_t)c.res[a]);
    key = (rd << res_bits) | rr;
  }
  keys[p] = key;
  vals[p] = a;
}
/* Traces with more distinct deviceId or resourceId values than the rank sets hold are ordered by
 * the raw values: one more stable sort per column (sign-biased 64-bit keys), and a last one that
 * moves the dropped rows behind the kept ones. */
__global__ void k_make_column_keys(const int64_t* column, const uint32_t* meta, const uint32_t* order, uint64_t n, int validity,
                                   uint64_t* keys, uint32_t* vals) {
  const uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n) return;
  const uint32_t a = order[p];
  const bool valid = (meta[a] & KTJ_M_VALID) != 0;
  keys[p] = validity ? (valid ? 0ull : 1ull) : (valid ? ((uint64_t)column[a] ^ 0x8000000000000000ULL) : 0ull);
  vals[p] = a;
}
hipError_t make_column_keys(const int64_t* column, const uint32_t* meta, const uint32_t* order, uint64_t n, int validity,
                            uint64_t* keys, uint32_t* vals, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_make_column_keys, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, column, meta, order, n, validity,
                     keys, vals);
  return KTJ_LAUNCH_CHECK();
}
__global__ void k_clear_error_bits(Scalars* sc, unsigned int bits) { sc->error &= ~bits; }
hipError_t clear_error_bits(Scalars* sc, unsigned int bits, hipStream_t st) {
  hipLaunchKernelGGL(k_clear_error_bits, dim3(1), dim3(1), 0, st, sc, bits);
  return KTJ_LAUNCH_CHECK();
}
hipError_t make_ts_keys(Columns c, uint64_t n, const Scalars* sc, uint64_t* keys, uint32_t* vals, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_make_ts_keys, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, c, n, sc, keys, vals);
  return KTJ_LAUNCH_CHECK();
}
hipError_t make_rank_keys(Columns c, const uint32_t* order, uint64_t n, SortSets s, uint32_t res_bits, uint32_t rank_bits,
                          uint64_t* keys, uint32_t* vals, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_make_rank_keys, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, c, order, n, s, res_bits,
                     rank_bits, keys, vals);
  return KTJ_LAUNCH_CHECK();
}

hipError_t collect_distinct(Columns c, uint64_t n, SortSets s, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  /* few, fat workgroups: each one pays for its own local set once (few rows: one group each) */
  /* at most four workgroups per CU: every workgroup pays for its local sets and its atomics at the
   * end once, and a thousand of them keep enough loads in flight (4096: 0.23 ms for 22 M rows,
   * 1024: 0.17 ms) */
  unsigned g = grid_stride_for(n, n < (1u << 20) ? KTJ_BLOCK * COLLECT_ROWS : KTJ_BLOCK * 16);
  if (g > 1024u) g = 1024u;
  hipLaunchKernelGGL(k_collect_distinct, dim3(g), dim3(KTJ_BLOCK), 0, st, c, n, s, sc);
  return KTJ_LAUNCH_CHECK();
}
hipError_t rank_distinct(SortSets s, Scalars* sc, hipStream_t st) {
  hipLaunchKernelGGL(k_rank_distinct, dim3(2), dim3(1024), 0, st, s, sc);
  return KTJ_LAUNCH_CHECK();
}
hipError_t make_keys(Columns c, uint64_t n, SortSets s, const Scalars* sc, uint32_t ts_bits, uint32_t res_bits,
                     uint32_t key_bits, uint64_t* keys, uint32_t* vals, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_make_keys, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, c, n, s, sc, ts_bits,
                     res_bits, key_bits, keys, vals);
  return KTJ_LAUNCH_CHECK();
}

/* ---- stable LSD radix sort, 8 bits per pass ----
 * A workgroup owns a tile of 4096 consecutive keys, one quarter per wavefront.  Ranks within the
 * tile come from wavefront match (ballots) plus per-wavefront running counts; the tile is then
 * laid out in LDS in digit order and written from there, so that neighbouring lanes store
 * neighbouring elements of a digit's run (whole lines instead of single 8-byte stores). */
#define RADIX_ITEMS 16
#define RADIX_TILE (KTJ_BLOCK * RADIX_ITEMS)
#define RADIX_WAVES (KTJ_BLOCK >> 6)
#define RADIX_WAVE_KEYS (64 * RADIX_ITEMS)

__global__ void __launch_bounds__(KTJ_BLOCK)
k_radix_hist(const uint64_t* keys, uint64_t n, uint32_t shift, uint32_t* hist, uint32_t n_blocks) {
  __shared__ uint32_t h[256];
  h[threadIdx.x] = 0;
  __syncthreads();
  const uint64_t base = (uint64_t)blockIdx.x * RADIX_TILE;
  for (int r = 0; r < RADIX_ITEMS; ++r) {
    const uint64_t i = base + (uint64_t)r * KTJ_BLOCK + threadIdx.x;
    if (i < n) atomicAdd(&h[(uint32_t)(keys[i] >> shift) & 0xFFu], 1u);
  }
  __syncthreads();
  hist[(uint64_t)threadIdx.x * n_blocks + blockIdx.x] = h[threadIdx.x]; /* digit-major */
}
__global__ void __launch_bounds__(KTJ_BLOCK)
k_radix_scatter(const uint64_t* keys_in, const uint32_t* vals_in, uint64_t* keys_out, uint32_t* vals_out, uint64_t n,
                uint32_t shift, const uint32_t* hist_scanned, uint32_t n_blocks) {
  __shared__ uint64_t s_key[RADIX_TILE];
  __shared__ uint32_t s_val[RADIX_TILE];
  __shared__ uint32_t wave_run[RADIX_WAVES][256]; /* count per (wavefront, digit), then its start inside the digit's run */
  __shared__ uint32_t digit_start[256];           /* start of the digit's run inside the tile     */
  __shared__ uint32_t base_of[256];               /* global offset of this tile's run per digit   */
  __shared__ uint32_t wave_tot[RADIX_WAVES];
  base_of[threadIdx.x] = hist_scanned[(uint64_t)threadIdx.x * n_blocks + blockIdx.x];
  for (int k = 0; k < RADIX_WAVES; ++k) wave_run[k][threadIdx.x] = 0;
  __syncthreads();
  const uint32_t w = threadIdx.x >> 6, lane = lane_id();
  const uint64_t lt = lanemask_lt();
  const uint64_t tile_base = (uint64_t)blockIdx.x * RADIX_TILE;
  const uint64_t chunk = tile_base + (uint64_t)w * RADIX_WAVE_KEYS;
  /* my_run: this wavefront's running counts; accessed as LDS (a plain pointer to the row would
   * turn into flat accesses), re-read every round because other lanes of the wavefront update it */
  typedef volatile __attribute__((address_space(3))) uint32_t* lds_counts;
  lds_counts my_run = (lds_counts)&wave_run[w][0];
  uint64_t key[RADIX_ITEMS];
  uint32_t val[RADIX_ITEMS], rank[RADIX_ITEMS];
#pragma unroll
  for (int r = 0; r < RADIX_ITEMS; ++r) {
    const uint64_t i = chunk + (uint64_t)r * 64u + lane;
    const bool valid = i < n;
    key[r] = valid ? keys_in[i] : ~0ULL;
    val[r] = valid ? vals_in[i] : 0u;
  }
#pragma unroll
  for (int r = 0; r < RADIX_ITEMS; ++r) {
    const bool valid = chunk + (uint64_t)r * 64u + lane < n;
    const uint32_t digit = (uint32_t)(key[r] >> shift) & 0xFFu;
    /* lanes of this wavefront holding the same digit */
    uint64_t peers = __ballot(valid ? 1 : 0);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const uint64_t bal = __ballot((digit >> b) & 1u);
      peers &= ((digit >> b) & 1u) ? bal : ~bal;
    }
    const uint32_t rank_in_wave = (uint32_t)__popcll(peers & lt);
    const uint32_t before = my_run[digit];   /* same digit in earlier rounds of this wavefront */
    rank[r] = before + rank_in_wave;
    if (valid && rank_in_wave == 0) my_run[digit] = before + (uint32_t)__popcll(peers);
  }
  __syncthreads();
  {
    /* per digit: wavefront counts -> starts inside the digit's run; digit totals -> exclusive scan */
    uint32_t tot = 0;
    for (int k = 0; k < RADIX_WAVES; ++k) { const uint32_t cnt = wave_run[k][threadIdx.x]; wave_run[k][threadIdx.x] = tot; tot += cnt; }
    uint32_t inc = tot;
    for (int o = 1; o < 64; o <<= 1) { const uint32_t t = __shfl_up(inc, o); if (lane >= (uint32_t)o) inc += t; }
    if (lane == 63) wave_tot[w] = inc;
    __syncthreads();
    uint32_t add = 0;
    for (uint32_t k = 0; k < w; ++k) add += wave_tot[k];
    digit_start[threadIdx.x] = add + inc - tot;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < RADIX_ITEMS; ++r) {
    if (chunk + (uint64_t)r * 64u + lane < n) {
      const uint32_t digit = (uint32_t)(key[r] >> shift) & 0xFFu;
      const uint32_t p = digit_start[digit] + wave_run[w][digit] + rank[r];
      s_key[p] = key[r];
      s_val[p] = val[r];
    }
  }
  __syncthreads();
  const uint32_t cnt = (uint32_t)(n - tile_base < RADIX_TILE ? n - tile_base : RADIX_TILE);
  for (uint32_t p = threadIdx.x; p < cnt; p += KTJ_BLOCK) {
    const uint64_t k = s_key[p];
    const uint32_t digit = (uint32_t)(k >> shift) & 0xFFu;
    const uint64_t dst = (uint64_t)base_of[digit] + (p - digit_start[digit]);
    keys_out[dst] = k;
    vals_out[dst] = s_val[p];
  }
}

/* counts per (digit, tile) plus the digits' totals; below SORTP_SMALL_N keys the packed sort's tiles are 512 keys */
#define SORTP_SMALL_N (1ull << 19)
#define SORTP_STREAM_N (1ull << 24)
uint64_t radix_tmp_elems(uint64_t n) {
  const uint64_t tiles = n < SORTP_SMALL_N ? (n + 511) / 512 : (n + RADIX_TILE - 1) / RADIX_TILE;
  return 256ull * tiles + 256;
}

hipError_t radix_sort(uint64_t* keys_a, uint32_t* vals_a, uint64_t* keys_b, uint32_t* vals_b, uint64_t n,
                      uint32_t bits, uint32_t* hist, uint64_t* scan_tmp, uint64_t** res_keys, uint32_t** res_vals,
                      hipStream_t st) {
  *res_keys = keys_a;
  *res_vals = vals_a;
  if (n == 0) return hipSuccess;
  const uint32_t n_blocks = (uint32_t)((n + RADIX_TILE - 1) / RADIX_TILE);
  uint64_t* ki = keys_a; uint32_t* vi = vals_a; uint64_t* ko = keys_b; uint32_t* vo = vals_b;
  for (uint32_t shift = 0; shift < bits; shift += 8) {
    hipLaunchKernelGGL(k_radix_hist, dim3(n_blocks), dim3(KTJ_BLOCK), 0, st, (const uint64_t*)ki, n, shift, hist, n_blocks);
    hipError_t e = scan_u32_inplace(hist, 256ull * n_blocks, scan_tmp, st);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(k_radix_scatter, dim3(n_blocks), dim3(KTJ_BLOCK), 0, st, (const uint64_t*)ki, (const uint32_t*)vi,
                       ko, vo, n, shift, (const uint32_t*)hist, n_blocks);
    uint64_t* tk = ki; ki = ko; ko = tk;
    uint32_t* tv = vi; vi = vo; vo = tv;
  }
  *res_keys = ki;
  *res_vals = vi;
  return KTJ_LAUNCH_CHECK();
}

/* ---- the same sort on single 64-bit words ----
 * When the composite key and the arrival index fit one word, the sort moves 8 bytes per row and
 * pass instead of 12 and needs no separate index array.  The first pass reads the full keys
 * (arrival index = position) and consumes their lowest digit, so the words it writes hold only
 * the remaining key bits above the index: word = (key >> BITS) << idx_bits | index.  Later passes
 * take their digit from the word; the last one writes the bare indices.  The per-tile digit
 * counts of the first pass come from the kernel that builds the keys. */
enum { SORTP_KEYS_TO_WORDS = 0, SORTP_WORDS_TO_WORDS = 1, SORTP_WORDS_TO_PERM = 2, SORTP_KEYS_TO_PERM = 3 };
template <int BITS, int THREADS, int ITEMS_> struct SortP {
  static constexpr int NB = 1 << BITS;
  static constexpr int WAVES = THREADS / 64;
  static constexpr int ITEMS = ITEMS_; /* keys per thread: 16, or 2 where a trace has too few keys to fill the GPU with tiles of 4096 */
  static constexpr int TILE = THREADS * ITEMS;
  static constexpr int WAVE_KEYS = 64 * ITEMS;
  static_assert(NB % THREADS == 0 || THREADS % NB == 0, "digits and threads must divide");
};

template <int BITS, int THREADS, int ITEMS>
__global__ void __launch_bounds__(THREADS)
k_sortp_make_keys(Columns c, uint64_t n, SortSets s, const Scalars* sc, uint32_t ts_bits, uint32_t res_bits, uint32_t key_bits,
                  uint64_t* keys, uint32_t* hist, uint32_t n_blocks) {
  using P = SortP<BITS, THREADS, ITEMS>;
  __shared__ uint32_t h[P::NB];
  for (int d = threadIdx.x; d < P::NB; d += THREADS) h[d] = 0;
  __syncthreads();
  const uint64_t base = (uint64_t)blockIdx.x * P::TILE;
  const uint64_t ts_min = sc->ts_min_biased;
  constexpr int G = ITEMS < 4 ? ITEMS : 4; /* rows per thread whose loads are in flight together */
  RankMemo memo_dev{0, 0, false}, memo_res{0, 0, false};
  for (int r0 = 0; r0 < P::ITEMS; r0 += G) {
    uint32_t meta[G];
    uint64_t dev[G], res[G], ts[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const uint64_t a = base + (uint64_t)(r0 + g) * THREADS + threadIdx.x;
      const bool in = a < n;
      meta[g] = in ? c.meta[a] : 0u;
      dev[g] = in ? (uint64_t)c.dev[a] : 0;
      res[g] = in ? (uint64_t)c.res[a] : 0;
      ts[g] = in ? (uint64_t)c.ts[a] : 0;
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const uint64_t a = base + (uint64_t)(r0 + g) * THREADS + threadIdx.x;
      if (a >= n) continue;
      uint64_t key = 1ULL << key_bits; /* dropped rows sort behind everything */
      if (meta[g] & KTJ_M_VALID) {
        const uint64_t rd = set_rank_memo(s.dev_keys, s.dev_rank, dev[g], memo_dev);
        const uint64_t rr = set_rank_memo(s.res_keys, s.res_rank, res[g], memo_res);
        const uint64_t rel = (ts[g] ^ 0x8000000000000000ULL) - ts_min;
        key = ((((rd << res_bits) | rr)) << ts_bits) | rel;
      }
      keys[a] = key;
      atomicAdd(&h[(uint32_t)key & (P::NB - 1u)], 1u);
    }
  }
  __syncthreads();
  if (hist != nullptr)
    for (int d = threadIdx.x; d < P::NB; d += THREADS) hist[(uint64_t)d * n_blocks + blockIdx.x] = h[d]; /* digit-major */
}
template <int BITS, int THREADS, int ITEMS>
__global__ void __launch_bounds__(THREADS)
k_sortp_hist(const uint64_t* words, uint64_t n, uint32_t shift, uint32_t* hist, uint32_t n_blocks) {
  using P = SortP<BITS, THREADS, ITEMS>;
  __shared__ uint32_t h[P::NB];
  for (int d = threadIdx.x; d < P::NB; d += THREADS) h[d] = 0;
  __syncthreads();
  const uint64_t base = (uint64_t)blockIdx.x * P::TILE;
#pragma unroll
  for (int r = 0; r < P::ITEMS; ++r) {
    const uint64_t i = base + (uint64_t)r * THREADS + threadIdx.x;
    if (i < n) atomicAdd(&h[(uint32_t)(words[i] >> shift) & (P::NB - 1u)], 1u);
  }
  __syncthreads();
  for (int d = threadIdx.x; d < P::NB; d += THREADS) hist[(uint64_t)d * n_blocks + blockIdx.x] = h[d];
}
/* The per-tile digit counts (digit-major: hist[d * n_blocks + tile]) become, for every digit, the
 * running count over the tiles before each tile, and the digit's total goes to totals[d]: workgroup
 * d scans row d, every thread a contiguous piece of it.  One launch; the digits' own offsets (a scan
 * over 256 totals) are left to every scatter workgroup. */
template <int THREADS>
__global__ void __launch_bounds__(THREADS)
k_sortp_scan_digits(uint32_t* hist, uint32_t n_blocks, uint32_t* totals) {
  __shared__ uint32_t wave_tot[THREADS / 64];
  uint32_t* row = hist + (uint64_t)blockIdx.x * n_blocks;
  const uint32_t per = (n_blocks + THREADS - 1) / THREADS;
  const uint32_t lo = threadIdx.x * per < n_blocks ? threadIdx.x * per : n_blocks;
  const uint32_t hi = lo + per < n_blocks ? lo + per : n_blocks;
  uint32_t sum = 0;
  for (uint32_t t = lo; t < hi; ++t) sum += row[t];
  uint32_t inc = sum;
  const uint32_t lane = lane_id(), w = threadIdx.x >> 6;
  for (int o = 1; o < 64; o <<= 1) { const uint32_t v = __shfl_up(inc, o); if (lane >= (uint32_t)o) inc += v; }
  if (lane == 63) wave_tot[w] = inc;
  __syncthreads();
  uint32_t run = inc - sum;
  uint32_t all = 0;
  for (uint32_t k = 0; k < THREADS / 64; ++k) { if (k < w) run += wave_tot[k]; all += wave_tot[k]; }
  for (uint32_t t = lo; t < hi; ++t) { const uint32_t c = row[t]; row[t] = run; run += c; }
  if (threadIdx.x == 0) totals[blockIdx.x] = all;
}

template <int BITS, int THREADS, int ITEMS, int MODE>
__global__ void __launch_bounds__(THREADS)
k_sortp_scatter(const uint64_t* in, uint64_t* words_out, uint32_t* perm_out, uint64_t n, uint32_t shift, uint32_t idx_bits,
                const uint32_t* hist_scanned, const uint32_t* totals, uint32_t n_blocks) {
  using P = SortP<BITS, THREADS, ITEMS>;
  constexpr bool FROM_KEYS = MODE == SORTP_KEYS_TO_WORDS || MODE == SORTP_KEYS_TO_PERM;
  constexpr bool TO_PERM = MODE == SORTP_WORDS_TO_PERM || MODE == SORTP_KEYS_TO_PERM;
  __shared__ uint64_t s_word[P::TILE];
  __shared__ uint16_t s_digit[FROM_KEYS ? P::TILE : 1]; /* the first pass's digit is no longer part of the word */
  __shared__ uint32_t wave_run[P::WAVES][P::NB]; /* count per (wavefront, digit), then its start inside the digit's run */
  __shared__ uint32_t digit_start[P::NB];        /* start of the digit's run inside the tile     */
  __shared__ uint32_t base_of[P::NB];            /* global offset of this tile's run per digit   */
  __shared__ uint32_t wave_tot[P::WAVES];
  const uint32_t w = threadIdx.x >> 6, lane = lane_id();
  {
    /* where a digit's run begins in the output: the totals of the digits before it, scanned here by
     * every workgroup (256 values), plus the count of that digit in the tiles before this one */
    static_assert(P::NB <= THREADS, "a thread scans one digit's total");
    uint32_t tot = 0;
    if (hist_scanned != nullptr && (int)threadIdx.x < P::NB) tot = totals[threadIdx.x];
    uint32_t inc = tot;
    for (int o = 1; o < 64; o <<= 1) { const uint32_t v = __shfl_up(inc, o); if (lane >= (uint32_t)o) inc += v; }
    if (lane == 63) wave_tot[w] = inc;
    __syncthreads();
    uint32_t digit_base = inc - tot;
    for (uint32_t k = 0; k < w; ++k) digit_base += wave_tot[k];
    if ((int)threadIdx.x < P::NB) {
      const int d = (int)threadIdx.x;
      base_of[d] = hist_scanned != nullptr ? digit_base + hist_scanned[(uint64_t)d * n_blocks + blockIdx.x] : 0u;
      for (int k = 0; k < P::WAVES; ++k) wave_run[k][d] = 0;
    }
  }
  __syncthreads();
  const uint64_t lt = lanemask_lt();
  const uint64_t tile_base = (uint64_t)blockIdx.x * P::TILE;
  const uint64_t chunk = tile_base + (uint64_t)w * P::WAVE_KEYS;
  /* my_run: this wavefront's running counts; accessed as LDS (a plain pointer to the row would
   * turn into flat accesses), re-read every round because other lanes of the wavefront update it */
  typedef volatile __attribute__((address_space(3))) uint32_t* lds_counts;
  lds_counts my_run = (lds_counts)&wave_run[w][0];
  uint64_t word[P::ITEMS];
  uint32_t rank[P::ITEMS];
  uint16_t dig[P::ITEMS];
  /* this pass is the last to read the words: where they are more than the last-level cache keeps
   * between the count and the scatter anyway, they are loaded past the L2's usual replacement
   * (config 3, 22 M words: 1.20 -> 1.11 ms for the sort; at 11 M words the hint costs 2 %) */
  if (n > SORTP_STREAM_N) {
#pragma unroll
    for (int r = 0; r < P::ITEMS; ++r) {
      const uint64_t i = chunk + (uint64_t)r * 64u + lane;
      word[r] = i < n ? load_once(&in[i]) : ~0ULL;
    }
  } else {
#pragma unroll
    for (int r = 0; r < P::ITEMS; ++r) {
      const uint64_t i = chunk + (uint64_t)r * 64u + lane;
      word[r] = i < n ? in[i] : ~0ULL;
    }
  }
#pragma unroll
  for (int r = 0; r < P::ITEMS; ++r) {
    const uint64_t i = chunk + (uint64_t)r * 64u + lane;
    const bool valid = i < n;
    uint32_t digit;
    if (FROM_KEYS) {
      digit = (uint32_t)word[r] & (P::NB - 1u);
      word[r] = (MODE == SORTP_KEYS_TO_PERM) ? i : ((((word[r] >> BITS)) << idx_bits) | i);
    } else {
      digit = (uint32_t)(word[r] >> shift) & (P::NB - 1u);
    }
    dig[r] = (uint16_t)digit;
    /* lanes of this wavefront holding the same digit */
    uint64_t peers = __ballot(valid ? 1 : 0);
#pragma unroll
    for (int b = 0; b < BITS; ++b) {
      const uint64_t bal = __ballot((digit >> b) & 1u);
      peers &= ((digit >> b) & 1u) ? bal : ~bal;
    }
    const uint32_t rank_in_wave = (uint32_t)__popcll(peers & lt);
    const uint32_t before = my_run[digit];   /* same digit in earlier rounds of this wavefront */
    rank[r] = before + rank_in_wave;
    if (valid && rank_in_wave == 0) my_run[digit] = before + (uint32_t)__popcll(peers);
  }
  __syncthreads();
  {
    /* per digit: wavefront counts -> starts inside the digit's run; digit totals -> exclusive scan.
     * A thread owns K consecutive digits (or none, where there are more threads than digits). */
    constexpr int K = P::NB >= THREADS ? P::NB / THREADS : 1;
    const bool owner = (int)threadIdx.x * K < P::NB;
    uint32_t tot[K], sum = 0;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      uint32_t t = 0;
      if (owner) {
        const int d = (int)threadIdx.x * K + j;
        for (int k = 0; k < P::WAVES; ++k) { const uint32_t cnt = wave_run[k][d]; wave_run[k][d] = t; t += cnt; }
      }
      tot[j] = t;
      sum += t;
    }
    uint32_t inc = sum;
    for (int o = 1; o < 64; o <<= 1) { const uint32_t t = __shfl_up(inc, o); if (lane >= (uint32_t)o) inc += t; }
    if (lane == 63) wave_tot[w] = inc;
    __syncthreads();
    uint32_t start = inc - sum;
    for (uint32_t k = 0; k < w; ++k) start += wave_tot[k];
    if (owner) {
#pragma unroll
      for (int j = 0; j < K; ++j) { digit_start[(int)threadIdx.x * K + j] = start; start += tot[j]; }
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < P::ITEMS; ++r) {
    if (chunk + (uint64_t)r * 64u + lane < n) {
      const uint32_t digit = dig[r];
      const uint32_t p = digit_start[digit] + wave_run[w][digit] + rank[r];
      s_word[p] = word[r];
      if (FROM_KEYS) s_digit[p] = dig[r];
    }
  }
  __syncthreads();
  const uint32_t cnt = (uint32_t)(n - tile_base < (uint64_t)P::TILE ? n - tile_base : (uint64_t)P::TILE);
  const uint64_t idx_mask = idx_bits >= 64 ? ~0ULL : ((1ULL << idx_bits) - 1ULL);
  for (uint32_t p = threadIdx.x; p < cnt; p += THREADS) {
    const uint64_t v = s_word[p];
    const uint32_t digit = FROM_KEYS ? (uint32_t)s_digit[p] : ((uint32_t)(v >> shift) & (P::NB - 1u));
    /* a single tile (no counts given): the tile's order is the output's */
    const uint64_t dst = hist_scanned != nullptr ? (uint64_t)base_of[digit] + (p - digit_start[digit]) : (uint64_t)p;
    if (TO_PERM) perm_out[dst] = (uint32_t)(v & idx_mask);
    else words_out[dst] = v;
  }
}

/* A trace of one tile: keys, every pass and the permutation in one launch of one workgroup (six
 * launches of a few microseconds each otherwise).  Keys and arrival indices stay in registers and
 * LDS between the passes; a pass ranks the keys as k_sortp_scatter does (ballots among the lanes of
 * a wavefront, running counts per wavefront and digit) and puts them in LDS in the new order, from
 * where every thread takes the keys of its positions for the next pass. */
template <int BITS, int THREADS, int ITEMS>
__global__ void __launch_bounds__(THREADS)
k_sortp_single(Columns c, uint32_t n, SortSets s, const Scalars* sc, uint32_t ts_bits, uint32_t res_bits, uint32_t key_bits,
               uint32_t* perm_out) {
  using P = SortP<BITS, THREADS, ITEMS>;
  __shared__ uint64_t s_key[P::TILE];
  __shared__ uint16_t s_idx[P::TILE];
  __shared__ uint32_t wave_run[P::WAVES][P::NB];
  __shared__ uint32_t digit_start[P::NB];
  __shared__ uint32_t wave_tot[P::WAVES];
  static_assert(P::TILE <= 65536, "arrival indices are kept as 16 bits");
  static_assert(P::NB == THREADS, "a thread owns one digit");
  const uint32_t w = threadIdx.x >> 6, lane = lane_id();
  const uint64_t lt = lanemask_lt();
  const uint32_t chunk = w * P::WAVE_KEYS;
  typedef volatile __attribute__((address_space(3))) uint32_t* lds_counts;
  lds_counts my_run = (lds_counts)&wave_run[w][0];
  uint64_t key[P::ITEMS];
  uint16_t idx[P::ITEMS];
  uint32_t rank[P::ITEMS];
  uint16_t dig[P::ITEMS];
  const uint64_t ts_min = sc->ts_min_biased;
#pragma unroll
  for (int r = 0; r < P::ITEMS; ++r) {
    const uint32_t a = chunk + (uint32_t)r * 64u + lane;
    uint64_t k = 1ULL << key_bits; /* dropped rows sort behind everything */
    if (a < n && (c.meta[a] & KTJ_M_VALID)) {
      const uint64_t rd = set_rank(s.dev_keys, s.dev_rank, (uint64_t)c.dev[a]);
      const uint64_t rr = set_rank(s.res_keys, s.res_rank, (uint64_t)c.res[a]);
      const uint64_t rel = ((uint64_t)c.ts[a] ^ 0x8000000000000000ULL) - ts_min;
      k = ((((rd << res_bits) | rr)) << ts_bits) | rel;
    }
    key[r] = k;
    idx[r] = (uint16_t)a;
  }
  const uint32_t passes = (key_bits + 1u + BITS - 1u) / BITS;
  for (uint32_t pass = 0; pass < passes; ++pass) {
    const uint32_t shift = pass * BITS;
    wave_run[0][threadIdx.x] = 0;
#pragma unroll
    for (int k = 1; k < P::WAVES; ++k) wave_run[k][threadIdx.x] = 0;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < P::ITEMS; ++r) {
      const bool valid = chunk + (uint32_t)r * 64u + lane < n;
      const uint32_t digit = (uint32_t)(key[r] >> shift) & (P::NB - 1u);
      dig[r] = (uint16_t)digit;
      uint64_t peers = __ballot(valid ? 1 : 0);
#pragma unroll
      for (int b = 0; b < BITS; ++b) {
        const uint64_t bal = __ballot((digit >> b) & 1u);
        peers &= ((digit >> b) & 1u) ? bal : ~bal;
      }
      const uint32_t rank_in_wave = (uint32_t)__popcll(peers & lt);
      const uint32_t before = my_run[digit];
      rank[r] = before + rank_in_wave;
      if (valid && rank_in_wave == 0) my_run[digit] = before + (uint32_t)__popcll(peers);
    }
    __syncthreads();
    {
      /* thread d: the wavefronts' counts of digit d become their starts inside the digit's run, the
       * digit's total goes into the scan that gives the run's start inside the tile */
      const int d = (int)threadIdx.x;
      uint32_t t = 0;
#pragma unroll
      for (int k = 0; k < P::WAVES; ++k) { const uint32_t cnt = wave_run[k][d]; wave_run[k][d] = t; t += cnt; }
      uint32_t inc = t;
      for (int o = 1; o < 64; o <<= 1) { const uint32_t v = __shfl_up(inc, o); if (lane >= (uint32_t)o) inc += v; }
      if (lane == 63) wave_tot[w] = inc;
      __syncthreads();
      uint32_t start = inc - t;
      for (uint32_t k = 0; k < w; ++k) start += wave_tot[k];
      digit_start[d] = start;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < P::ITEMS; ++r) {
      if (chunk + (uint32_t)r * 64u + lane < n) {
        const uint32_t digit = dig[r];
        const uint32_t p = digit_start[digit] + wave_run[w][digit] + rank[r];
        s_key[p] = key[r];
        s_idx[p] = idx[r];
      }
    }
    __syncthreads();
    if (pass + 1 == passes) break;
#pragma unroll
    for (int r = 0; r < P::ITEMS; ++r) {
      const uint32_t a = chunk + (uint32_t)r * 64u + lane;
      if (a < n) { key[r] = s_key[a]; idx[r] = s_idx[a]; }
    }
    __syncthreads();
  }
  for (uint32_t p = threadIdx.x; p < n; p += THREADS) perm_out[p] = s_idx[p];
}

template <int BITS, int THREADS, int ITEMS>
static hipError_t sort_packed_t(Columns c, uint64_t n, SortSets s, const Scalars* sc, uint32_t ts_bits, uint32_t res_bits,
                                uint32_t key_bits, uint32_t idx_bits, uint64_t* buf_a, uint64_t* buf_b, uint32_t* perm,
                                uint32_t* hist, uint64_t* scan_tmp, hipStream_t st) {
  using P = SortP<BITS, THREADS, ITEMS>;
  const uint32_t n_blocks = (uint32_t)((n + P::TILE - 1) / P::TILE);
  const uint32_t total_bits = key_bits + 1u;
  const uint32_t passes = (total_bits + BITS - 1) / BITS;
  const dim3 g(n_blocks), b(THREADS);
  /* one tile: a pass needs no counts from other tiles, so no count and scan launches */
  const bool single = n_blocks == 1;
  uint32_t* counts = single ? nullptr : hist;
  /* the digits' totals live behind the counts (radix_tmp_elems leaves 256 spare entries) */
  uint32_t* totals = hist + (uint64_t)P::NB * n_blocks;
  static_assert(P::NB <= 256, "room for the totals behind the counts");
  (void)scan_tmp;
  hipLaunchKernelGGL((k_sortp_make_keys<BITS, THREADS, ITEMS>), g, b, 0, st, c, n, s, sc, ts_bits, res_bits, key_bits, buf_a, counts, n_blocks);
  if (!single) hipLaunchKernelGGL((k_sortp_scan_digits<THREADS>), dim3(P::NB), b, 0, st, hist, n_blocks, totals);
  if (passes == 1) {
    hipLaunchKernelGGL((k_sortp_scatter<BITS, THREADS, ITEMS, SORTP_KEYS_TO_PERM>), g, b, 0, st, (const uint64_t*)buf_a, buf_b, perm, n,
                       0u, idx_bits, (const uint32_t*)counts, (const uint32_t*)totals, n_blocks);
    return KTJ_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL((k_sortp_scatter<BITS, THREADS, ITEMS, SORTP_KEYS_TO_WORDS>), g, b, 0, st, (const uint64_t*)buf_a, buf_b, perm, n,
                     0u, idx_bits, (const uint32_t*)counts, (const uint32_t*)totals, n_blocks);
  uint64_t* in = buf_b; uint64_t* out = buf_a;
  for (uint32_t p = 1; p < passes; ++p) {
    const uint32_t shift = idx_bits + (p - 1u) * BITS;
    if (!single) {
      hipLaunchKernelGGL((k_sortp_hist<BITS, THREADS, ITEMS>), g, b, 0, st, (const uint64_t*)in, n, shift, hist, n_blocks);
      hipLaunchKernelGGL((k_sortp_scan_digits<THREADS>), dim3(P::NB), b, 0, st, hist, n_blocks, totals);
    }
    if (p + 1 == passes)
      hipLaunchKernelGGL((k_sortp_scatter<BITS, THREADS, ITEMS, SORTP_WORDS_TO_PERM>), g, b, 0, st, (const uint64_t*)in, out, perm, n,
                         shift, idx_bits, (const uint32_t*)counts, (const uint32_t*)totals, n_blocks);
    else
      hipLaunchKernelGGL((k_sortp_scatter<BITS, THREADS, ITEMS, SORTP_WORDS_TO_WORDS>), g, b, 0, st, (const uint64_t*)in, out, perm, n,
                         shift, idx_bits, (const uint32_t*)counts, (const uint32_t*)totals, n_blocks);
    uint64_t* t = in; in = out; out = t;
  }
  return KTJ_LAUNCH_CHECK();
}
#define SORTP_BITS 8
#define SORTP_THREADS 256
/* tests: the one-launch sort of a single tile switched off, so that such a trace takes the passes of a large one */
static bool g_sortp_no_single = false;
void sort_packed_force_passes(bool on) { g_sortp_no_single = on; }
bool sort_packed_fits(uint64_t n, uint32_t key_bits) {
  const uint32_t total_bits = key_bits + 1u;
  const uint32_t idx_bits = (uint32_t)(64 - __builtin_clzll(n > 1 ? n - 1 : 1));
  return (total_bits > SORTP_BITS ? total_bits - SORTP_BITS : 0u) + idx_bits <= 64u;
}
hipError_t sort_packed(Columns c, uint64_t n, SortSets s, const Scalars* sc, uint32_t ts_bits, uint32_t res_bits,
                       uint32_t key_bits, uint64_t* buf_a, uint64_t* buf_b, uint32_t* perm, uint32_t* hist, uint64_t* scan_tmp,
                       hipStream_t st) {
  if (n == 0) return hipSuccess;
  const uint32_t idx_bits = (uint32_t)(64 - __builtin_clzll(n > 1 ? n - 1 : 1));
  if (n <= (uint64_t)SORTP_THREADS * 16u && !g_sortp_no_single) {
    hipLaunchKernelGGL((k_sortp_single<SORTP_BITS, SORTP_THREADS, 16>), dim3(1), dim3(SORTP_THREADS), 0, st, c, (uint32_t)n, s, sc, ts_bits,
                       res_bits, key_bits, perm);
    return KTJ_LAUNCH_CHECK();
  }
  /* a few thousand keys are one tile; up to SORTP_SMALL_N keys, tiles of 512 spread over the GPU
   * finish a pass sooner than the few 4096-key tiles would (30 000 keys: 76 against 130 us for the
   * sort, 330 000 keys: 113 against 155 us; from a million keys on the large tiles win) */
  if (n > (uint64_t)SORTP_THREADS * 16u && n < SORTP_SMALL_N)
    return sort_packed_t<SORTP_BITS, SORTP_THREADS, 2>(c, n, s, sc, ts_bits, res_bits, key_bits, idx_bits, buf_a, buf_b, perm, hist,
                                                       scan_tmp, st);
  return sort_packed_t<SORTP_BITS, SORTP_THREADS, 16>(c, n, s, sc, ts_bits, res_bits, key_bits, idx_bits, buf_a, buf_b, perm, hist,
                                                      scan_tmp, st);
}

/* ------------------------------------------------------------------------------------------ */
/* stage 4a: joined rows and exact byte lengths, arrival order                                  */
/* ------------------------------------------------------------------------------------------ */
__device__ __forceinline__ void store_row(MatRow* dst, const MatRow& m) {
  const uint4* s = reinterpret_cast<const uint4*>(&m);
  uint4* d = reinterpret_cast<uint4*>(dst);
  for (int k = 0; k < (int)(sizeof(MatRow) / 16); ++k) d[k] = s[k];
}
/* Packed rows between global memory and LDS: a lane that loads or stores its own 64- or 96-byte
 * row touches a cache line (or two) of its own with every 16-byte access, 64 lines per
 * instruction; moved by the workgroup with lane-consecutive 16-byte accesses the same bytes are
 * whole lines.  `rows` is the workgroup's first row, `cnt` its number of rows; the callers put
 * the barriers.  Records are read once and joined rows written once: both go past the L2's usual
 * replacement (config 3: join stage 2.51 -> 2.26 ms). */
template <typename T>
__device__ __forceinline__ void rows_global_to_lds(const T* rows, uint32_t cnt, uint4* lds) {
  typedef unsigned int v4u __attribute__((ext_vector_type(4)));
  const v4u* g = reinterpret_cast<const v4u*>(rows);
  v4u* l = reinterpret_cast<v4u*>(lds);
  for (uint32_t k = threadIdx.x; k < cnt * (uint32_t)(sizeof(T) / 16); k += blockDim.x) l[k] = load_once(&g[k]);
}
template <typename T>
__device__ __forceinline__ void rows_lds_to_global(T* rows, uint32_t cnt, const uint4* lds) {
  typedef unsigned int v4u __attribute__((ext_vector_type(4)));
  v4u* g = reinterpret_cast<v4u*>(rows);
  const v4u* l = reinterpret_cast<const v4u*>(lds);
  for (uint32_t k = threadIdx.x; k < cnt * (uint32_t)(sizeof(T) / 16); k += blockDim.x) store_once(&g[k], l[k]);
}
template <typename T>
__device__ __forceinline__ T row_from_lds(const uint4* lds) {
  T r;
  uint4* d = reinterpret_cast<uint4*>(&r);
#pragma unroll
  for (int k = 0; k < (int)(sizeof(T) / 16); ++k) d[k] = lds[threadIdx.x * (sizeof(T) / 16) + k];
  return r;
}
template <typename T>
__device__ __forceinline__ void row_to_lds(const T& r, uint4* lds) {
  const uint4* s = reinterpret_cast<const uint4*>(&r);
#pragma unroll
  for (int k = 0; k < (int)(sizeof(T) / 16); ++k) lds[threadIdx.x * (sizeof(T) / 16) + k] = s[k];
}
/* exact byte length in the low 30 bits, tail kind (see tail_kind) in the top two */
__device__ __forceinline__ uint32_t row_length(const MatRow& m, const EmitCtx& ctx, Scalars* sc) {
  if (!(m.meta & KTJ_M_VALID)) return 0;
  CountWriter cw;
  format_activity(cw, m, ctx);
  if (cw.n >= (1ull << 30)) { flag_error(sc, KTJ_DEVERR_RECORD_TOO_LONG); return 0; }
  return (uint32_t)cw.n | (tail_kind(m, has_args(m, ctx)) << 30);
}
struct RowStats { uint32_t n_flow = 0, n_blank = 0; };
__device__ __forceinline__ void count_row_stats(const MatRow& m, const EmitCtx& ctx, RowStats* rs) {
  if (!(m.meta & KTJ_M_VALID)) return;
  if (m.meta & KTJ_M_FLOW) ++rs->n_flow;
  if (!(m.meta & KTJ_M_NAME_BUILTIN) && m.name_id < ctx.dict.n && (ctx.dict.flags[m.name_id] & KTJ_SF_NAME_UNKNOWN))
    ++rs->n_blank;
}
__device__ __forceinline__ void flush_row_stats(const RowStats& rs, Scalars* sc) {
  block_add(sc, KTJ_CNT_FLOW, rs.n_flow);
  block_add(sc, KTJ_CNT_BLANK_NAMES, rs.n_blank);
}

/* Stream Sync rows (output_json.cpp:913-943): which activity is the first of its (device, row) key
 * in emission order.  Pass a: smallest sorted position per key; pass b: the activity at that
 * position is marked.  Both run over the sorted positions of generic rows only when the stream
 * holds CUDA_SYNC activities at all. */
__device__ __forceinline__ bool is_stream_sync(const ktj_generic_rec& g, const DictViews& d) {
  return g.type == KTJ_TYPE_CUDA_SYNC && g.name_id < d.n && (d.flags[g.name_id] & KTJ_SF_STREAM_SYNC);
}
__global__ void k_sync_first_a(const uint32_t* perm, uint64_t n_sorted, const ktj_generic_rec* g, uint64_t n_generic,
                               const int64_t* dev, DictViews d, uint64_t* keys, uint32_t* first_pos, Scalars* sc) {
  const uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n_sorted) return;
  const uint64_t a = perm[p];
  if (a >= n_generic || !is_stream_sync(g[a], d)) return;
  const uint32_t slot = table_insert_counted(keys, KTJ_SYNC_CAP - 1u, stream_sync_key(dev[a], g[a].resource), &sc->n_sync_rows,
                                             KTJ_MAX_SYNC_ROWS);
  if (slot == KTJ_NOSLOT) { flag_error(sc, KTJ_DEVERR_SYNC_ROWS); return; }
  atomicMin(&first_pos[slot], (uint32_t)p);
}
__global__ void k_sync_first_b(const uint32_t* perm, uint64_t n_sorted, const ktj_generic_rec* g, uint64_t n_generic,
                               const int64_t* dev, DictViews d, const uint64_t* keys, const uint32_t* first_pos, uint32_t* is_first) {
  const uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n_sorted) return;
  const uint64_t a = perm[p];
  if (a >= n_generic) return;
  uint32_t first = 0;
  if (is_stream_sync(g[a], d)) {
    const uint32_t slot = table_find(keys, KTJ_SYNC_CAP - 1u, stream_sync_key(dev[a], g[a].resource));
    first = slot != KTJ_NOSLOT && first_pos[slot] == (uint32_t)p;
  }
  is_first[a] = first;
}
hipError_t stream_sync_first(const uint32_t* perm, uint64_t n_sorted, const ktj_generic_rec* g, uint64_t n_generic,
                             const int64_t* dev, DictViews d, uint64_t* keys, uint32_t* first_pos, uint32_t* is_first, Scalars* sc,
                             hipStream_t st) {
  if (n_sorted == 0 || n_generic == 0) return hipSuccess;
  hipError_t e = fill_u64(keys, KTJ_EMPTY_KEY, KTJ_SYNC_CAP + 1ull, st);
  if (e != hipSuccess) return e;
  e = fill_u32(first_pos, 0xFFFFFFFFu, KTJ_SYNC_CAP + 1ull, st);
  if (e != hipSuccess) return e;
  e = fill_u32(is_first, 0u, n_generic, st);
  if (e != hipSuccess) return e;
  const dim3 grid(grid_for(n_sorted, KTJ_BLOCK)), b(KTJ_BLOCK);
  hipLaunchKernelGGL(k_sync_first_a, grid, b, 0, st, perm, n_sorted, g, n_generic, dev, d, keys, first_pos, sc);
  hipLaunchKernelGGL(k_sync_first_b, grid, b, 0, st, perm, n_sorted, g, n_generic, dev, d, (const uint64_t*)keys,
                     (const uint32_t*)first_pos, is_first);
  return KTJ_LAUNCH_CHECK();
}

__global__ void k_mat_generic(const ktj_generic_rec* g, uint64_t n, uint64_t first, EmitCtx ctx, const uint32_t* sync_first,
                              MatRow* mat, uint32_t* len, Scalars* sc) {
  static_assert(sizeof(MatRow) >= sizeof(ktj_generic_rec), "the staging area holds the records, then the joined rows");
  __shared__ uint4 stage[KTJ_BLOCK * sizeof(MatRow) / 16];
  RowStats rs;
  for (uint64_t base = (uint64_t)blockIdx.x * blockDim.x; base < n; base += (uint64_t)gridDim.x * blockDim.x) {
    const uint32_t cnt = (uint32_t)(n - base < blockDim.x ? n - base : blockDim.x);
    __syncthreads(); /* the previous round's rows have left the staging area */
    rows_global_to_lds(g + base, cnt, stage);
    __syncthreads();
    const uint64_t i = base + threadIdx.x;
    const bool active = threadIdx.x < cnt;
    MatRow m;
    if (active) {
      const ktj_generic_rec rec = row_from_lds<ktj_generic_rec>(stage);
      m = mat_generic(rec, generic_device(rec, ctx.args, ctx.n_args));
      if (!generic_record_prints(rec, ctx)) m.meta &= ~KTJ_M_VALID;
      attach_own_collective(m, rec, ctx);
      mark_stream_sync(m, ctx, sync_first != nullptr && sync_first[i] != 0);
      len[first + i] = row_length(m, ctx, sc);
      count_row_stats(m, ctx, &rs);
    }
    __syncthreads(); /* every lane has taken its record */
    if (active) row_to_lds(m, stage);
    __syncthreads();
    rows_lds_to_global(mat + first + base, cnt, stage);
  }
  flush_row_stats(rs, sc);
}
/* The pass over the runtime rows.
 * full table : correlation id → stream_src = last runtime row that carries a stream
 *              (RocmStreamQueue.h:47-54), first = first arrival index seen, for checkTimestampOrder
 *              (GenericActivityProfiler.cpp:363-395)
 * narrow table: int-narrowed id → kern_src = last in-window kernel row, copy_src = last in-window
 *              copy/malloc row (thread_local correlationToGrid/Block/Size,
 *              RocprofActivity_inl.h:28-30, 221-223, 245, 267)
 * Every row writes what device rows take over from it (timestamp, stream, grid/block or size)
 * into the payload of its slots straight away.  That is final when no two runtime rows share a
 * slot, which the returning atomicMin on `first` tells; only otherwise k_runtime_winners finds
 * the winning row of each slot field and k_republish_runtime lets the winners write again.  The
 * "External id" was resolved before this pass, so the joined row and its length are produced here
 * too.  The slots are remembered per row for those two passes. */
__device__ __forceinline__ bool runtime_rows_share_slots(const Scalars* sc) {
  /* ids beyond 31 bits may coincide after narrowing without sharing a slot of the full table */
  const KeyRange r = sc->plan.range[KTJ_TBL_FULL];
  return sc->runtime_ids_repeat != 0 || (r.lo <= r.hi && r.hi >= 0x80000000ULL);
}
/* Sets the slot's bit in a bitmap and tells whether it was set before.  All lanes of the wavefront
 * call it (active = the lane has a slot).  Rows that arrive in id order put up to 32 neighbouring
 * lanes on one word, so the lanes are grouped by word (up to BITMAP_GROUPS groups, found with
 * ballots; 64 consecutive slots lie in two or three words) and the lowest lane of each group sets
 * all of its group's bits in one atomic; the groups' atomics leave in a single instruction.  Lanes
 * beyond the last group set their own bit.  Two lanes of the wavefront with the same slot are
 * reported as "set before" for every lane of their group (callers only ask whether any slot is
 * shared). */
#define BITMAP_GROUPS 4
__device__ __forceinline__ uint32_t wave_or_u32(uint32_t v) {
  for (int o = 32; o > 0; o >>= 1) v |= (uint32_t)__shfl_xor((int)v, o);
  return v;
}
__device__ __forceinline__ bool bitmap_test_and_set(uint32_t* bitmap, uint32_t slot, bool active) {
  const uint32_t word = slot >> 5, bit = active ? 1u << (slot & 31u) : 0u;
  uint64_t todo = __ballot(active);
  if (!todo) return false;
  int leader = (int)lane_id();   /* lanes outside every group lead themselves */
  uint32_t bits = bit;
  bool twice = false;
  for (int g = 0; g < BITMAP_GROUPS && todo; ++g) {
    const int l = __ffsll((unsigned long long)todo) - 1;
    const uint32_t w = (uint32_t)__shfl((int)word, l);
    const bool in = ((todo >> lane_id()) & 1ull) != 0 && word == w;
    const uint64_t m = __ballot(in);
    const uint32_t all = wave_or_u32(in ? bit : 0u);
    if (in) { leader = l; bits = all; twice = (uint32_t)__popc(all) != (uint32_t)__popcll(m); }
    todo &= ~m;
  }
  uint32_t old = 0;
  if (active && leader == (int)lane_id()) old = atomicOr(&bitmap[word], bits);
  old = (uint32_t)__shfl((int)old, leader);
  return active && (twice || (old & bit) != 0);
}
#define JOIN_ROWS 4
#define JOIN_SMALL_ROWS (1u << 18)
#ifndef KX_JOIN_ATTR
#define KX_JOIN_ATTR
#endif
__global__ void KX_JOIN_ATTR k_join_runtime(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first_runtime, ApiTable api, Table tf,
                               FullCols fc, Table tn, NarrowCols nc, uint32_t* slot_f, uint32_t* slot_n, EmitCtx ctx, MatRow* mat,
                               uint32_t* len, Scalars* sc, int rounds) {
  RowStats rs;
  uint32_t n_linked = 0;
  bool any_carries_stream = false, any_repeats = false;
  /* a workgroup takes `rounds` consecutive groups of blockDim.x rows: the per-workgroup counters
   * at the end (one atomic each on a hot address) are paid once for all of them */
  static_assert(sizeof(MatRow) == sizeof(ktj_runtime_rec), "the staging area holds the records, then the joined rows");
  __shared__ uint4 stage[KTJ_BLOCK * sizeof(ktj_runtime_rec) / 16];
  for (int round = 0; round < rounds; ++round) {
    const uint64_t base = ((uint64_t)blockIdx.x * rounds + round) * blockDim.x;
    if (base >= n) break;
    const uint32_t cnt = (uint32_t)(n - base < blockDim.x ? n - base : blockDim.x);
    __syncthreads(); /* the previous round's rows have left the staging area */
    rows_global_to_lds(r + base, cnt, stage);
    __syncthreads();
    const uint64_t i = base + threadIdx.x;
    bool carries_stream = false;
    uint32_t sf = KTJ_NOSLOT;
    /* everything the row reads from its own record and columns is requested up front, so that the
     * table accesses below (each a round trip of its own) overlap with it */
    const uint64_t a = first_runtime + (i < n ? i : 0);
    /* the lane's record stays in LDS and is read field by field; the joined row takes its place */
    uint4* my_slot = &stage[threadIdx.x * (sizeof(ktj_runtime_rec) / 16)];
    const ktj_runtime_rec& rec = *reinterpret_cast<const ktj_runtime_rec*>(my_slot);
    uint64_t id = 0;
    uint32_t meta = 0;
    int64_t ts = 0, dur = 0;
    if (i < n) {
      id = load_once(&c.corr[a]);
      meta = load_once(&c.meta[a]);
      ts = load_once(&c.ts[a]);
      dur = load_once(&c.dur[a]);
      sf = slot_insert(tf, id);
    }
    const uint32_t kind = (meta & KTJ_M_KIND_MASK) >> KTJ_M_KIND_SHIFT;
    const bool valid = (meta & KTJ_M_VALID) != 0;
    const bool publishes = valid && kind != KTJ_RT_DEFAULT;
    /* every slot that carries an external id exists already (k_build_extcorr ran before) */
    uint32_t sn = KTJ_NOSLOT;
    if (i < n) sn = publishes ? slot_insert(tn, narrow_corr_key(id)) : slot_find(tn, narrow_corr_key(id));
    int32_t ext = 0;
    uint32_t np_info = 0;
    if (sn != KTJ_NOSLOT) { ext = nc.pay[sn].ext_val; np_info = nc.pay[sn].info; }
    const bool repeats = bitmap_test_and_set(fc.has_runtime, sf, sf != KTJ_NOSLOT);
    if (i < n) {
      carries_stream = (meta & KTJ_M_HAS_STREAM) != 0;
      store_once(&slot_f[i], sf);
      if (sf == KTJ_NOSLOT) flag_error(sc, KTJ_DEVERR_TABLE_FULL);
      else {
        FullPay fp;
        fp.first_ts = ts;
        fp.stream = 0;
        if (carries_stream) fp.stream = rec.kind == KTJ_RT_KERNEL ? rec.u.kernel.stream : rec.u.copy.stream;
        fc.pay[sf] = fp;
      }
      if (publishes) {
        if (sn == KTJ_NOSLOT) flag_error(sc, KTJ_DEVERR_TABLE_FULL);
        else {
          NarrowPay* np = &nc.pay[sn];
          if (kind == KTJ_RT_KERNEL) {
            pack_grid(rec, np->pay);
            np->info = (np_info & ~KTJ_NP_KIND_MASK) | KTJ_DL_HAS_GRID;
          } else {
            np->pay[0] = rec.kind == KTJ_RT_COPY ? rec.u.copy.size : rec.u.malloc_.size;
            np->info = (np_info & ~KTJ_NP_KIND_MASK) | KTJ_DL_HAS_SIZE;
          }
        }
      }
      store_once(&slot_n[i], sn);
      if ((np_info & KTJ_NP_LINKED) && valid) ++n_linked;
      store_once(&c.ext[a], ext);
      const bool known = rec.cid < api.n_cids;
      const uint32_t name = known ? api.cid_name_ids[rec.cid] : KTJ_NONE;
      const bool fstart = known && ((api.flow_start_bits[rec.cid >> 5] >> (rec.cid & 31u)) & 1u);
      MatRow* m = reinterpret_cast<MatRow*>(my_slot);
      *m = mat_runtime(rec, ts, dur, valid, ext, name, fstart, rec.cid == api.malloc_cid);
      store_once(&len[a], row_length(*m, ctx, sc));
      count_row_stats(*m, ctx, &rs);
    }
    __syncthreads(); /* the joined rows go out the way the records came in */
    rows_lds_to_global(mat + first_runtime + base, cnt, stage);
    any_carries_stream |= carries_stream;
    any_repeats |= repeats;
  }
  /* one store per workgroup at most: every lane storing the same flag would queue up in L2 */
  const int any_stream = __syncthreads_or(any_carries_stream ? 1 : 0);
  const int any_repeat = __syncthreads_or(any_repeats ? 1 : 0);
  if (threadIdx.x == 0) {
    if (any_stream) sc->have_stream_src = 1;
    if (any_repeat) sc->runtime_ids_repeat = 1;
  }
  flush_row_stats(rs, sc);
  block_add(sc, KTJ_CNT_LINKED, n_linked);
}
/* Only when runtime rows share slots: which row of a slot the device rows take each value from
 * (the last row that carries a stream; the last in-window kernel launch; the last in-window copy
 * or allocation), by atomicMax over row indices.  k_republish_runtime reads the winners. */
__global__ void k_runtime_winners(uint64_t n, Columns c, uint64_t first, FullCols fc, NarrowCols nc, const uint32_t* slot_f,
                                  const uint32_t* slot_n, const Scalars* sc) {
  if (!runtime_rows_share_slots(sc)) return;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    const uint32_t meta = c.meta[first + i];
    const uint32_t kind = (meta & KTJ_M_KIND_MASK) >> KTJ_M_KIND_SHIFT;
    const uint32_t sf = slot_f[i], sn = slot_n[i];
    if (sf != KTJ_NOSLOT) {
      atomicMin(&fc.first[sf], (uint32_t)(first + i));
      if (meta & KTJ_M_HAS_STREAM) atomicMax(&fc.stream_src[sf], (uint32_t)i + 1u);
    }
    if (sn != KTJ_NOSLOT && (meta & KTJ_M_VALID) && kind != KTJ_RT_DEFAULT)
      atomicMax(kind == KTJ_RT_KERNEL ? &nc.kern_src[sn] : &nc.copy_src[sn], (uint32_t)i + 1u);
  }
}
/* Only when runtime rows share slots: the row that won a slot field writes the payload again, and
 * every row is checked against the first row of its id (checkTimestampOrder with the roles
 * swapped).  Where no two runtime rows share a slot each row is the first of its id and what it
 * wrote in k_join_runtime stands. */
__global__ void k_republish_runtime(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first, FullCols fc, NarrowCols nc,
                                    const uint32_t* slot_f, const uint32_t* slot_n, Scalars* sc) {
  if (!runtime_rows_share_slots(sc)) return;
  uint32_t n_bad = 0;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t a = first + i;
    const ktj_runtime_rec rec = r[i];
    const int64_t ts = c.ts[a];
    const uint32_t sf = slot_f[i], sn = slot_n[i];
    if (sf != KTJ_NOSLOT) {
      const uint64_t f = fc.first[sf];
      if (f == a) fc.pay[sf].first_ts = ts;
      else if (f != 0xFFFFFFFFull) { /* an earlier runtime row has this id */
        const int64_t t1 = c.ts[f];
        if (ts != 0 && t1 > ts) ++n_bad;
      }
      const uint32_t stream_src = fc.stream_src[sf];
      if (stream_src == (uint32_t)i + 1u)
        fc.pay[sf].stream = rec.kind == KTJ_RT_KERNEL ? rec.u.kernel.stream : rec.u.copy.stream;
      else if (stream_src == 0) fc.pay[sf].stream = 0; /* no row of this id carries one */
    }
    if (sn != KTJ_NOSLOT) {
      NarrowPay* np = &nc.pay[sn];
      const uint32_t copy_src = nc.copy_src[sn]; /* final: the pass above has ended */
      if (copy_src == (uint32_t)i + 1u) {
        np->pay[0] = rec.kind == KTJ_RT_COPY ? rec.u.copy.size : rec.u.malloc_.size;
        np->info = (np->info & ~KTJ_NP_KIND_MASK) | KTJ_DL_HAS_SIZE;
      } else if (copy_src == 0 && nc.kern_src[sn] == (uint32_t)i + 1u) {
        pack_grid(rec, np->pay);
        np->info = (np->info & ~KTJ_NP_KIND_MASK) | KTJ_DL_HAS_GRID;
      }
    }
  }
  block_add(sc, KTJ_CNT_OUT_OF_ORDER, n_bad);
}
__global__ void k_mat_device(const ktj_device_rec* d, uint64_t n, Columns c, uint64_t first, const DevLink* link,
                             EmitCtx ctx, MatRow* mat, uint32_t* len, Scalars* sc) {
  __shared__ uint4 stage[KTJ_BLOCK * sizeof(MatRow) / 16]; /* the records, then the joined rows */
  RowStats rs;
  for (uint64_t base = (uint64_t)blockIdx.x * blockDim.x; base < n; base += (uint64_t)gridDim.x * blockDim.x) {
    const uint32_t cnt = (uint32_t)(n - base < blockDim.x ? n - base : blockDim.x);
    __syncthreads(); /* the previous round's rows have left the staging area */
    rows_global_to_lds(d + base, cnt, stage);
    __syncthreads();
    const uint64_t i = base + threadIdx.x, a = first + i;
    const bool active = threadIdx.x < cnt;
    MatRow m;
    if (active) {
      const ktj_device_rec rec = row_from_lds<ktj_device_rec>(stage);
      DevLink l;
      {
        typedef unsigned int v4u __attribute__((ext_vector_type(4)));
        const v4u* src = reinterpret_cast<const v4u*>(&link[i]);
        v4u* lv = reinterpret_cast<v4u*>(&l);
        lv[0] = load_once(&src[0]);
        lv[1] = load_once(&src[1]);
      }
      m = mat_device_v(rec, load_once(&c.ts[a]), load_once(&c.dur[a]), load_once(&c.res[a]),
                       (load_once(&c.meta[a]) & KTJ_M_VALID) != 0, load_once(&c.ext[a]),
                       (l.flags & KTJ_DL_HAS_GRID) != 0, l.p[0], l.p[1], l.p[2], (l.flags & KTJ_DL_HAS_SIZE) != 0, l.p[0], l.coll);
      store_once(&len[a], row_length(m, ctx, sc));
      count_row_stats(m, ctx, &rs);
    }
    __syncthreads(); /* every lane has taken its record */
    if (active) row_to_lds(m, stage);
    __syncthreads();
    rows_lds_to_global(mat + first + base, cnt, stage);
  }
  flush_row_stats(rs, sc);
}
/* Collective metadata: the first activity, in emission order, that prints each entry, per
 * backend (first[2k] nccl, first[2k + 1] hccl).  The host replays appendCollectiveMetadata's
 * bookkeeping (output_json.cpp:799-835) over these.  Runs only for traces that carry any. */
__global__ void k_collective_first(const MatRow* mat, const uint32_t* perm, uint64_t n_rows, uint32_t n_coll, uint32_t* first) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_rows) return;
  const MatRow* m = &mat[perm[i]];
  const uint32_t meta = m->meta;
  const uint32_t cls = (meta & KTJ_M_CLASS_MASK) >> KTJ_M_CLASS_SHIFT;
  uint32_t k = 0;
  if (cls == KTJ_CLASS_GENERIC) k = (uint32_t)m->p[1];
  else if (cls == KTJ_CLASS_DEVICE && (meta & KTJ_M_TYPE_MASK) == KTJ_TYPE_CONCURRENT_KERNEL) k = (uint32_t)m->p[4];
  if (k == 0 || k > n_coll) return;
  const uint32_t hccl = cls == KTJ_CLASS_GENERIC && (meta & KTJ_M_TYPE_MASK) == KTJ_TYPE_MTIA_CCP_EVENTS ? 1u : 0u;
  atomicMin(&first[2u * (k - 1u) + hccl], (uint32_t)i);
}
hipError_t collective_first(const MatRow* mat, const uint32_t* perm, uint64_t n_rows, uint32_t n_coll, uint32_t* first,
                            hipStream_t st) {
  hipError_t e = fill_u32(first, 0xFFFFFFFFu, 2ull * n_coll, st);
  if (e != hipSuccess || n_rows == 0) return e;
  hipLaunchKernelGGL(k_collective_first, dim3(grid_for(n_rows, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, mat, perm, n_rows, n_coll,
                     first);
  return KTJ_LAUNCH_CHECK();
}
/* lengths and tail kinds in emission order (the size pass leaves both in one word per arrival index) */
__global__ void k_gather_len(const uint32_t* perm, const uint32_t* len, uint64_t n, uint32_t* len_sorted, uint8_t* kind_sorted) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t v = len[load_once(&perm[i])];
  store_once(&len_sorted[i], v & 0x3FFFFFFFu);
  kind_sorted[i] = (uint8_t)(v >> 30);
}

hipError_t mat_generic_rows(const ktj_generic_rec* g, uint64_t n, uint64_t first, EmitCtx ctx, const uint32_t* sync_first,
                            MatRow* mat, uint32_t* len, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_mat_generic, dim3(grid_stride_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, g, n, first, ctx, sync_first,
                     mat, len, sc);
  return KTJ_LAUNCH_CHECK();
}
hipError_t join_runtime_rows(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first, ApiTable api, Table tf, FullCols fc,
                             Table tn, NarrowCols nc, uint32_t* slot_f, uint32_t* slot_n, EmitCtx ctx, MatRow* mat,
                             uint32_t* len, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  /* few rows: one group per workgroup, so that the launch is as wide and as short as it can be */
  const int rounds = n < JOIN_SMALL_ROWS ? 1 : JOIN_ROWS;
  hipLaunchKernelGGL(k_join_runtime, dim3(grid_for(n, KTJ_BLOCK * rounds)), dim3(KTJ_BLOCK), 0, st, r, n, c, first, api, tf, fc, tn, nc,
                     slot_f, slot_n, ctx, mat, len, sc, rounds);
  return KTJ_LAUNCH_CHECK();
}
hipError_t republish_runtime_rows(const ktj_runtime_rec* r, uint64_t n, Columns c, uint64_t first, FullCols fc, NarrowCols nc,
                                  const uint32_t* slot_f, const uint32_t* slot_n, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_runtime_winners, dim3(grid_stride_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, n, c, first, fc, nc, slot_f,
                     slot_n, (const Scalars*)sc);
  hipLaunchKernelGGL(k_republish_runtime, dim3(grid_stride_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, r, n, c, first, fc, nc,
                     slot_f, slot_n, sc);
  return KTJ_LAUNCH_CHECK();
}
hipError_t mat_device_rows(const ktj_device_rec* d, uint64_t n, Columns c, uint64_t first, const DevLink* link,
                           EmitCtx ctx, MatRow* mat, uint32_t* len, Scalars* sc, hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_mat_device, dim3(grid_stride_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, d, n, c, first, link, ctx,
                     mat, len, sc);
  return KTJ_LAUNCH_CHECK();
}
hipError_t gather_len(const uint32_t* perm, const uint32_t* len, uint64_t n, uint32_t* len_sorted, uint8_t* kind_sorted,
                      hipStream_t st) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(k_gather_len, dim3(grid_for(n, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, perm, len, n, len_sorted, kind_sorted);
  return KTJ_LAUNCH_CHECK();
}

/* ------------------------------------------------------------------------------------------ */
/* stage 4b: emit.  Workgroup k owns the output bytes [k*T, (k+1)*T) of the whole document      */
/* (clipped to the activity section), so every global store is an aligned 16-byte store.  The    */
/* first activity of every tile is found once by k_tile_starts (binary search in the offsets);   */
/* the emit workgroup formats one activity per lane into LDS through a 64-bit accumulator        */
/* (literals are immediates, digits are packed arithmetically, no per-byte loads), with clipping */
/* (an activity straddling a tile boundary is formatted by both tiles), copies dictionary        */
/* strings with whole wavefronts, and flushes the tile.  T is chosen by the host so that a tile  */
/* holds about as many activities as the workgroup has lanes.                                    */
/* ------------------------------------------------------------------------------------------ */
#define EMIT_THREADS 128
#define EMIT_MAX_JOBS 512

__global__ void k_tile_starts(const uint64_t* offs, uint64_t n, uint64_t prefix_len, uint32_t tile, uint64_t first_tile,
                              uint32_t n_tiles, uint32_t* start) {
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t > n_tiles) return;
  if (t == n_tiles) { start[t] = (uint32_t)n; return; }
  const uint64_t t0 = (first_tile + t) * (uint64_t)tile;
  const uint64_t lo = (t0 > prefix_len ? t0 : prefix_len) - prefix_len;
  uint64_t a = 0, b = n; /* first record with offs[r + 1] > lo */
  while (a < b) { const uint64_t m = (a + b) >> 1; if (offs[m + 1] > lo) b = m; else a = m + 1; }
  start[t] = (uint32_t)a;
}

__global__ void __launch_bounds__(EMIT_THREADS)
k_emit(const MatRow* mat, const uint32_t* perm, const uint64_t* offs, uint64_t n, EmitCtx ctx, char* out,
       uint64_t prefix_len, uint64_t act_bytes, uint32_t tile, uint64_t first_tile, const uint32_t* start) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* buf = smem;                                                   /* tile bytes */
  CopyJob* jobs = reinterpret_cast<CopyJob*>(smem + tile);            /* EMIT_MAX_JOBS */
  uint32_t* n_jobs = reinterpret_cast<uint32_t*>(smem + tile + EMIT_MAX_JOBS * sizeof(CopyJob));

  const uint64_t t0 = (first_tile + blockIdx.x) * (uint64_t)tile;     /* absolute, multiple of the tile size */
  const uint64_t abs_lo = t0 > prefix_len ? t0 : prefix_len;
  const uint64_t abs_end = prefix_len + act_bytes;
  const uint64_t abs_hi = t0 + tile < abs_end ? t0 + tile : abs_end;
  if (abs_lo >= abs_hi) return;
  const int32_t lo = (int32_t)(abs_lo - t0), hi = (int32_t)(abs_hi - t0); /* tile-local */

  const uint64_t r0 = start[blockIdx.x];
  uint64_t r1 = start[blockIdx.x + 1];
  if (r1 < n && offs[r1] + prefix_len < abs_hi) ++r1;                  /* the straddler at the upper edge */

  if (threadIdx.x == 0) *n_jobs = 0;
  {
    uint4* z = reinterpret_cast<uint4*>(buf);
    const uint4 zero = make_uint4(0, 0, 0, 0);
    for (uint32_t k = threadIdx.x; k < tile / 16u; k += EMIT_THREADS) z[k] = zero;
  }
  __syncthreads();
  for (uint64_t r = r0 + threadIdx.x; r < r1; r += EMIT_THREADS) {
    const uint64_t o = offs[r];
    if (offs[r + 1] == o) continue; /* dropped or empty */
    const MatRow m = mat[perm[r]];
    TileWriter w;
    w.buf = buf; w.size = tile;
    w.jobs = jobs; w.n_jobs = n_jobs; w.max_jobs = EMIT_MAX_JOBS;
    w.begin((int32_t)((int64_t)(o + prefix_len) - (int64_t)t0));
    format_activity(w, m, ctx);
    w.end();
  }
  __syncthreads();
  {
    /* string copies: one job per 16-lane group; aligned 8-byte words in the middle (two aligned
     * global loads funnel-shifted into one aligned LDS store), single bytes at both ends */
    const uint32_t nj = *n_jobs < EMIT_MAX_JOBS ? *n_jobs : EMIT_MAX_JOBS;
    const uint32_t group = threadIdx.x >> 4, gl = threadIdx.x & 15u;
    for (uint32_t j = group; j < nj; j += (EMIT_THREADS >> 4)) {
      const CopyJob job = jobs[j];
      uint32_t headb = (8u - ((uint32_t)job.dst & 7u)) & 7u;
      if (headb > job.len) headb = job.len;
      if (gl < headb) buf[job.dst + (int32_t)gl] = job.src[gl];
      const uint32_t words = (job.len - headb) >> 3;
      const uintptr_t sa = (uintptr_t)(job.src + headb);
      const uint32_t sh = (uint32_t)(sa & 7u) * 8u;
      const uint64_t* sp = reinterpret_cast<const uint64_t*>(sa & ~(uintptr_t)7);
      uint64_t* dp = reinterpret_cast<uint64_t*>(buf + job.dst + (int32_t)headb);
      for (uint32_t k = gl; k < words; k += 16u) {
        uint64_t v = sp[k];
        if (sh) v = (v >> sh) | (sp[k + 1] << (64u - sh));
        dp[k] = v;
      }
      const uint32_t done = headb + words * 8u;
      if (gl < job.len - done) buf[job.dst + (int32_t)(done + gl)] = job.src[done + gl];
    }
  }
  __syncthreads();
  /* flush: unaligned head bytes (first tile only), 16-byte body, tail bytes */
  char* g = out + abs_lo;
  const char* s = buf + lo;
  const uint32_t nbytes = (uint32_t)(hi - lo);
  uint32_t pre = (uint32_t)((16u - (uint32_t)((uintptr_t)g & 15u)) & 15u);
  if (pre > nbytes) pre = nbytes;
  for (uint32_t k = threadIdx.x; k < pre; k += EMIT_THREADS) g[k] = s[k];
  const uint32_t body = (nbytes - pre) / 16u;
  {
    uint4* gv = reinterpret_cast<uint4*>(g + pre);
    const uint4* sv = reinterpret_cast<const uint4*>(s + pre);
    for (uint32_t k = threadIdx.x; k < body; k += EMIT_THREADS) gv[k] = sv[k];
  }
  for (uint32_t k = pre + body * 16u + threadIdx.x; k < nbytes; k += EMIT_THREADS) g[k] = s[k];
}

/* Direct variant: one lane per activity; blocks of 16 bytes, aligned in the document (see
 * BlockWriter for who writes the blocks that two activities share).  Finished blocks wait in the
 * lane's stage in LDS, one 128-byte line of the document and the beginning of the next, and a line
 * leaves when it is complete (a line written in pieces some microseconds apart leaves the L2 cache
 * once per piece): at the points where the whole wavefront meets — after the head of the event,
 * after its args if some lane's stage is full by then, and after the flow event — the four lanes
 * of a quad store each other's blocks, 64 contiguous bytes per quad and instruction, and in between
 * a lane whose stage is nearly full stores its line itself (BlockWriter::relief).  Lanes without an activity stay until the end
 * for the quads' sake.  The document's prefix and suffix are already in place when this kernel
 * runs; the first and the last activity merge with them. */
__global__ void __launch_bounds__(KTJ_BLOCK) __attribute__((amdgpu_waves_per_eu(3)))
k_emit_direct(const MatRow* mat, const uint32_t* perm, const uint64_t* offs, const uint8_t* kind_sorted, uint64_t n_rows,
              EmitCtx ctx, char* out, uint64_t prefix_len) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint64_t o = 0;
  uint32_t row = 0;
  bool active = i < n_rows;
  /* A wavefront that has just started comes first on its SIMD until the loads of its joined row are
   * on their way (two dependent loads with a few instructions between them, which would otherwise
   * queue behind the formatting of the two older wavefronts): config 3 4.70 -> 4.61 ms, config 4
   * 2.12 -> 2.07 ms.  Priority 1, 2 or 3: the same.  Kept up until the name is copied, lowered in
   * steps, lowered behind the branch below or before the row's loads: slower or no gain; a
   * scheduling barrier in place of the priority: no gain. */
  __builtin_amdgcn_s_setprio(3);
  if (active) { row = perm[i]; o = offs[i]; active = offs[i + 1] != o; } /* one wait for both */
  MatRow m;
  BlockWriter w;
  w.stage_init((uint32_t)threadIdx.x * (KTJ_STAGE_BLOCKS * 16u));
  ActivityParts<BlockWriter> parts;
  if (active) {
    m = mat[row];
    __builtin_amdgcn_s_setprio(0); /* (a wavefront without any activity keeps it: it ends at once) */
    w.begin(out, prefix_len + o, i ? kind_sorted[i - 1] : 0u, i == 0);
    w.stage_follow();
    format_head(w, m, ctx, parts);
  }
  w.flush(false);
  if (active) format_args(w, m, ctx, parts);
  w.flush_if_full();
  if (active) {
    format_flow(w, m, ctx, parts);
    w.end(i + 1 == n_rows);
  }
  w.flush(true);
}
hipError_t emit_direct(const MatRow* mat, const uint32_t* perm, const uint64_t* offs, const uint8_t* kind_sorted,
                       uint64_t n_rows, uint64_t act_bytes, EmitCtx ctx, char* out, uint64_t prefix_len, hipStream_t st) {
  if (n_rows == 0) return hipSuccess;
  (void)act_bytes;
  const size_t stage_lds = (size_t)KTJ_BLOCK * KTJ_STAGE_BLOCKS * 16u;
  hipLaunchKernelGGL(k_emit_direct, dim3(grid_for(n_rows, KTJ_BLOCK)), dim3(KTJ_BLOCK), stage_lds, st, mat, perm, offs,
                     kind_sorted, n_rows, ctx, out, prefix_len);
  return KTJ_LAUNCH_CHECK();
}

/* What the host needs during a pass goes straight into its pinned memory, and the text it made
 * (header, infos, footer) comes straight out of it: one small kernel each instead of one copy
 * engine transfer per value. */
__global__ void k_publish(Scalars* sc, const uint64_t* total, const uint32_t* list, uint32_t n_list, Scalars* h_sc,
                          uint64_t* h_total, uint32_t* h_list) {
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x, stride = gridDim.x * blockDim.x;
  if (blockIdx.x == 0) {
    /* the sharded counters: their sums so far into the fields the host reads (written, not added:
     * a pass publishes twice) */
    if (threadIdx.x < KTJ_CNT_COUNT) {
      unsigned long long sum = 0;
      for (uint32_t k = 0; k < KTJ_COUNTER_SHARDS; ++k) sum += sc->shard[k][threadIdx.x];
      switch (threadIdx.x) {
        case KTJ_CNT_OUT_OF_RANGE: sc->out_of_range = sum; break;
        case KTJ_CNT_OUT_OF_ORDER: sc->out_of_order = sum; break;
        case KTJ_CNT_FLOW: sc->n_flow = sum; break;
        case KTJ_CNT_LINKED: sc->n_linked = sum; break;
        case KTJ_CNT_BLANK_NAMES: sc->n_blank_names = sum; break;
        case KTJ_CNT_VALID: sc->n_valid = sum; break;
        default: sc->n_sync_typed = sum; break;
      }
    }
    __syncthreads();
    constexpr uint32_t head_words = (uint32_t)(offsetof(Scalars, shard) / 4);
    const uint32_t* src = reinterpret_cast<const uint32_t*>(sc);
    uint32_t* dst = reinterpret_cast<uint32_t*>(h_sc);
    for (uint32_t k = threadIdx.x; k < head_words; k += blockDim.x) dst[k] = src[k];
  }
  for (uint32_t k = t; k < n_list; k += stride) h_list[k] = list[k];
  if (t == 0 && total != nullptr) *h_total = *total;
  __threadfence_system();
}
hipError_t publish(Scalars* sc, const uint64_t* total, const uint32_t* list, uint32_t n_list, Scalars* h_sc,
                   uint64_t* h_total, uint32_t* h_list, hipStream_t st) {
  static_assert(KTJ_CNT_COUNT == 7, "k_publish names every sharded counter");
  hipLaunchKernelGGL(k_publish, dim3(n_list > 4096 ? 16 : 1), dim3(KTJ_BLOCK), 0, st, sc, total, list, n_list, h_sc, h_total, h_list);
  return KTJ_LAUNCH_CHECK();
}
/* two pieces of text, each to its place; source and destination of a piece agree modulo 16 */
__global__ void k_put_text(const char* src_a, char* dst_a, uint64_t n_a, const char* src_b, char* dst_b, uint64_t n_b) {
  const char* src = blockIdx.y ? src_b : src_a;
  char* dst = blockIdx.y ? dst_b : dst_a;
  const uint64_t n = blockIdx.y ? n_b : n_a;
  uint64_t head = (16u - (uint32_t)((uintptr_t)dst & 15u)) & 15u;
  if (head > n) head = n;
  const uint64_t body = (n - head) >> 4, tail = (n - head) & 15u;
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  if (t < head) dst[t] = src[t];
  const uint4* sv = reinterpret_cast<const uint4*>(src + head);
  uint4* dv = reinterpret_cast<uint4*>(dst + head);
  for (uint64_t k = t; k < body; k += stride) dv[k] = sv[k];
  if (t < tail) dst[head + body * 16u + t] = src[head + body * 16u + t];
}
hipError_t put_text(const char* src_a, char* dst_a, uint64_t n_a, const char* src_b, char* dst_b, uint64_t n_b, hipStream_t st) {
  if ((((uintptr_t)src_a ^ (uintptr_t)dst_a) & 15u) || (((uintptr_t)src_b ^ (uintptr_t)dst_b) & 15u)) return hipErrorInvalidValue;
  const uint64_t most = n_a > n_b ? n_a : n_b;
  if (most == 0) return hipSuccess;
  hipLaunchKernelGGL(k_put_text, dim3(grid_stride_for((most >> 4) + 1, KTJ_BLOCK), 2), dim3(KTJ_BLOCK), 0, st, src_a, dst_a, n_a, src_b,
                     dst_b, n_b);
  return KTJ_LAUNCH_CHECK();
}

/* up to KTJ_MAX_PIECES pieces of page-locked host memory, each to its place in device memory (the
 * small submissions an engine has gathered); source and destination of a piece agree modulo 16 */
__global__ void k_put_pieces(PieceJobs jobs) {
  const char* src = jobs.src[blockIdx.y];
  char* dst = jobs.dst[blockIdx.y];
  const uint64_t n = jobs.n[blockIdx.y];
  uint64_t head = (16u - (uint32_t)((uintptr_t)dst & 15u)) & 15u;
  if (head > n) head = n;
  const uint64_t body = (n - head) >> 4, tail = (n - head) & 15u;
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  if (t < head) dst[t] = src[t];
  const uint4* sv = reinterpret_cast<const uint4*>(src + head);
  uint4* dv = reinterpret_cast<uint4*>(dst + head);
  for (uint64_t k = t; k < body; k += stride) dv[k] = sv[k];
  if (t < tail) dst[head + body * 16u + t] = src[head + body * 16u + t];
}
hipError_t put_pieces(const PieceJobs& jobs, hipStream_t st) {
  if (jobs.count == 0) return hipSuccess;
  if (jobs.count > KTJ_MAX_PIECES) return hipErrorInvalidValue;
  uint64_t most = 0;
  for (uint32_t k = 0; k < jobs.count; ++k) {
    if (((uintptr_t)jobs.src[k] ^ (uintptr_t)jobs.dst[k]) & 15u) return hipErrorInvalidValue;
    if (jobs.n[k] > most) most = jobs.n[k];
  }
  hipLaunchKernelGGL(k_put_pieces, dim3(grid_stride_for((most >> 4) + 1, KTJ_BLOCK), jobs.count), dim3(KTJ_BLOCK), 0, st, jobs);
  return KTJ_LAUNCH_CHECK();
}

/* plain 16-byte-per-lane copy of known size: the yardstick for the HBM counters */
__global__ void k_copy_reference(const uint4* src, uint4* dst, uint64_t n16) {
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * blockDim.x) dst[i] = src[i];
}
hipError_t copy_reference(const void* src, void* dst, uint64_t bytes, hipStream_t st) {
  const uint64_t n16 = bytes / 16;
  if (n16 == 0) return hipSuccess;
  hipLaunchKernelGGL(k_copy_reference, dim3(grid_stride_for(n16, KTJ_BLOCK * 4)), dim3(KTJ_BLOCK), 0, st,
                     static_cast<const uint4*>(src), static_cast<uint4*>(dst), n16);
  return KTJ_LAUNCH_CHECK();
}

uint32_t emit_tile_bytes(uint64_t act_bytes, uint64_t n_rows) {
  /* about 0.85 activities per lane, in steps of 4 KiB, between 8 and 40 KiB */
  const uint64_t avg = n_rows ? act_bytes / n_rows : 512;
  uint64_t t = (avg * EMIT_THREADS * 85 / 100 + 4095) / 4096 * 4096;
  if (t < 8192) t = 8192;
  if (t > 40960) t = 40960;
  return (uint32_t)t;
}
uint64_t emit_tile_count(uint64_t prefix_len, uint64_t act_bytes, uint32_t tile) {
  if (act_bytes == 0) return 0;
  return (prefix_len + act_bytes - 1) / tile - prefix_len / tile + 1;
}

hipError_t emit(const MatRow* mat, const uint32_t* perm, const uint64_t* offs, uint64_t n, EmitCtx ctx, char* out,
                uint64_t prefix_len, uint64_t act_bytes, uint32_t tile, uint32_t* tile_start, hipStream_t st) {
  if (act_bytes == 0) return hipSuccess;
  const uint64_t first_tile = prefix_len / tile;
  const uint32_t tiles = (uint32_t)emit_tile_count(prefix_len, act_bytes, tile);
  hipLaunchKernelGGL(k_tile_starts, dim3(grid_for((uint64_t)tiles + 1, KTJ_BLOCK)), dim3(KTJ_BLOCK), 0, st, offs, n,
                     prefix_len, tile, first_tile, tiles, tile_start);
  const size_t lds = (size_t)tile + EMIT_MAX_JOBS * sizeof(CopyJob) + 16;
  hipLaunchKernelGGL(k_emit, dim3(tiles), dim3(EMIT_THREADS), lds, st, mat, perm, offs, n, ctx, out, prefix_len,
                     act_bytes, tile, first_tile, (const uint32_t*)tile_start);
  return KTJ_LAUNCH_CHECK();
}

}  // namespace gpu
}  // namespace ktj
