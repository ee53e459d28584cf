/*
 * synth.c — deterministic generator of the five synthetic record streams the engine is measured
 * and checked on.  Integer arithmetic only (counter-based splitmix64 RNG, fixed-point log2/exp2
 * for the Zipf and lognormal shapes), so the same parameters give the same bytes on any machine.
 *
 * The record shapes mirror what libkineto's ROCm backend would hand to its post-processing stage
 * (libkineto/src/RocLogger.h:82-240 rows, libkineto/include/GenericTraceActivity.h CPU ops); the
 * mix of each configuration follows the benchmark description (kernel/memcpy/memset mix, graph
 * launches with fan-out, orphans, string-heavy kernel names with typed args).
 */
#include "ktj_stream.h"

#include <stdlib.h>
#include <string.h>

typedef unsigned __int128 u128;

/* ------------------------------------------------------------------------------------------ */
/* RNG                                                                                          */
/* ------------------------------------------------------------------------------------------ */
static inline uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ULL;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}
/* value of random variable `var` for item `i` under `seed` */
static inline uint64_t rnd(uint64_t seed, uint64_t var, uint64_t i) {
  return mix64(mix64(seed ^ (var * 0xD6E8FEB86659FD93ULL)) + i * 0xA0761D6478BD642FULL);
}

/* ------------------------------------------------------------------------------------------ */
/* fixed point                                                                                  */
/* ------------------------------------------------------------------------------------------ */
/* 2^(2^-i) in Q62, i = 1..32 */
static const uint64_t kExp2Frac[32] = {
    0x5a827999fcef3242ULL, 0x4c1bf828c6dc54b8ULL, 0x45cae0f1f545eb73ULL, 0x42d561b3e6243d8aULL,
    0x4166c34c5615d0ecULL, 0x40b268f9de0183baULL, 0x4058f6a7ecccd5b6ULL, 0x402c6be96af2fb58ULL,
    0x4016321b687027a8ULL, 0x400b18178ba33b14ULL, 0x40058bce410147e8ULL, 0x4002c5d7bff71dafULL,
    0x400162e807ee7e5bULL, 0x4000b1730df6a524ULL, 0x400058b9497b8152ULL, 0x40002c5c955dd701ULL,
    0x4000162e46d6f26cULL, 0x40000b1722757b1bULL, 0x4000058b90fd3e0cULL, 0x400002c5c86f3f26ULL,
    0x40000162e433c79bULL, 0x400000b17218edd0ULL, 0x40000058b90c3968ULL, 0x4000002c5c860d54ULL,
    0x400000162e4302d2ULL, 0x4000000b17218073ULL, 0x400000058b90bffcULL, 0x40000002c5c85fefULL,
    0x4000000162e42ff3ULL, 0x40000000b17217f9ULL, 0x4000000058b90bfcULL, 0x400000002c5c85feULL};

/* 2^f for f in [0,1) given as Q32; result in Q62 (in [2^62, 2^63)) */
static uint64_t exp2_frac_q62(uint32_t f_q32) {
  uint64_t r = 1ULL << 62;
  for (int i = 1; i <= 32; ++i) {
    if (f_q32 & (1u << (32 - i))) r = (uint64_t)(((u128)r * kExp2Frac[i - 1]) >> 62);
  }
  return r;
}

/* log2(k) in Q32 for k >= 1 */
static uint64_t log2_q32(uint64_t k) {
  int n = 63 - __builtin_clzll(k);
  u128 y = (u128)k << (63 - n); /* Q63 in [1,2) */
  uint64_t frac = 0;
  for (int i = 0; i < 32; ++i) {
    y = (y * y) >> 63; /* Q63 in [1,4) */
    frac <<= 1;
    if (y >> 64) {
      frac |= 1;
      y >>= 1;
    }
  }
  return ((uint64_t)n << 32) | frac;
}

/* median * 2^(e) for signed exponent e in Q32, clamped to [1, 2^40] */
static uint64_t scale_exp2(uint64_t median, int64_t e_q32) {
  int64_t ip = e_q32 >> 32; /* floor */
  uint32_t fp = (uint32_t)(e_q32 & 0xFFFFFFFFu);
  uint64_t m = exp2_frac_q62(fp); /* Q62 */
  u128 v = (u128)median * m;      /* Q62 */
  int sh = 62 - (int)ip;
  uint64_t r;
  if (sh >= 127) r = 0;
  else if (sh <= 0) r = 1ULL << 40;
  else {
    u128 q = v >> sh;
    r = q > ((u128)1 << 40) ? (1ULL << 40) : (uint64_t)q;
  }
  return r < 1 ? 1 : r;
}

/* lognormal-shaped sample: median * exp(sigma * z), z ~ sum of 12 uniforms (Irwin–Hall) */
static uint64_t lognormal(uint64_t seed, uint64_t var, uint64_t i, uint64_t median, uint32_t sigma_q16) {
  int64_t s = 0;
  uint64_t a = rnd(seed, var, i), b = rnd(seed, var + 0x5151, i), c = rnd(seed, var + 0xA2A2, i);
  for (int k = 0; k < 4; ++k) {
    s += (int64_t)((a >> (16 * k)) & 0xFFFF) + (int64_t)((b >> (16 * k)) & 0xFFFF) +
         (int64_t)((c >> (16 * k)) & 0xFFFF);
  }
  int64_t z_q16 = s - 393210;                 /* mean 12*32767.5, std 65536 */
  int64_t e = z_q16 * 94548;                  /* * 65536/ln2  → Q32 */
  e = (e * (int64_t)sigma_q16) >> 16;
  return scale_exp2(median, e);
}

/* ------------------------------------------------------------------------------------------ */
/* Zipf sampler over n items with exponent s (Q16)                                              */
/* ------------------------------------------------------------------------------------------ */
typedef struct zipf_t {
  uint64_t* cdf;
  uint32_t n;
} zipf_t;

static int zipf_init(zipf_t* z, uint32_t n, uint32_t s_q16) {
  z->cdf = (uint64_t*)malloc(sizeof(uint64_t) * n);
  z->n = n;
  if (!z->cdf) return -1;
  uint64_t acc = 0;
  for (uint32_t k = 1; k <= n; ++k) {
    uint64_t x = (uint64_t)(((u128)log2_q32(k) * s_q16) >> 16); /* s*log2(k), Q32 */
    uint64_t ip = x >> 32;
    uint32_t fp = (uint32_t)x;
    uint64_t w; /* 2^-x in Q48 */
    if (fp == 0) w = ip >= 48 ? 0 : (1ULL << 48) >> ip;
    else {
      uint64_t m = exp2_frac_q62((uint32_t)(0u - fp)); /* 2^(1-f) Q62 */
      uint64_t sh = ip + 1 + 14;
      w = sh >= 64 ? 0 : m >> sh;
    }
    if (w == 0) w = 1;
    acc += w;
    z->cdf[k - 1] = acc;
  }
  return 0;
}
static uint32_t zipf_sample(const zipf_t* z, uint64_t r) {
  uint64_t u = r % z->cdf[z->n - 1];
  uint32_t lo = 0, hi = z->n - 1;
  while (lo < hi) {
    uint32_t mid = (lo + hi) >> 1;
    if (z->cdf[mid] > u) hi = mid; else lo = mid + 1;
  }
  return lo;
}

/* ------------------------------------------------------------------------------------------ */
/* growable buffers                                                                             */
/* ------------------------------------------------------------------------------------------ */
typedef struct buf_t {
  char* p;
  size_t n, cap;
} buf_t;
static int buf_put(buf_t* b, const void* src, size_t n) {
  if (b->n + n > b->cap) {
    size_t nc = b->cap ? b->cap * 2 : 4096;
    while (nc < b->n + n) nc *= 2;
    char* np = (char*)realloc(b->p, nc);
    if (!np) return -1;
    b->p = np;
    b->cap = nc;
  }
  memcpy(b->p + b->n, src, n);
  b->n += n;
  return 0;
}

typedef struct gen_t {
  ktj_stream s;
  buf_t blob;  /* strings */
  buf_t off;   /* uint64 offsets */
  buf_t fields;
  buf_t schemas;
  uint64_t seed;
  buf_t owned; /* void* pointers released by ktj_synth_free */
  char* host_kv[2];
  char* host_val;
  char* trace_name;
  const char* meta_ptrs[2];
} gen_t;

static void* own(gen_t* g, void* p) {
  if (p) buf_put(&g->owned, &p, sizeof p);
  return p;
}

static uint32_t next_string_id(const gen_t* g) { return (uint32_t)(g->off.n / 8 - 1); }

static uint32_t add_string(gen_t* g, const char* p, size_t n) {
  uint32_t id = next_string_id(g);
  buf_put(&g->blob, p, n);
  uint64_t e = g->blob.n;
  buf_put(&g->off, &e, 8);
  return id;
}
static uint32_t add_cstr(gen_t* g, const char* s) { return add_string(g, s, strlen(s)); }

static uint32_t add_schema(gen_t* g, const ktj_field* f, uint32_t n) {
  ktj_schema_desc d;
  d.first_field = (uint32_t)(g->fields.n / sizeof(ktj_field));
  d.n_fields = n;
  buf_put(&g->fields, f, sizeof(ktj_field) * n);
  uint32_t id = (uint32_t)(g->schemas.n / sizeof(ktj_schema_desc));
  buf_put(&g->schemas, &d, sizeof d);
  return id;
}

/* ------------------------------------------------------------------------------------------ */
/* vocabularies                                                                                 */
/* ------------------------------------------------------------------------------------------ */
static const char kIdentChars[] = "abcdefghijklmnopqrstuvwxyzABCDEFGHIJKLMNOPQRSTUVWXYZ0123456789_";

/* ASCII identifier of 8..120 chars */
static uint32_t add_identifier(gen_t* g, uint64_t var, uint64_t i) {
  char tmp[128];
  uint32_t len = 8 + (uint32_t)(rnd(g->seed, var, i) % 113);
  for (uint32_t k = 0; k < len; ++k) {
    uint64_t r = rnd(g->seed, var + 1 + k, i);
    tmp[k] = k == 0 ? kIdentChars[r % 52] : kIdentChars[r % 63];
  }
  return add_string(g, tmp, len);
}

static const char* const kCpuOps[] = {
    "aten::mm", "aten::addmm", "aten::linear", "aten::conv2d", "aten::_convolution",
    "aten::cudnn_convolution", "aten::batch_norm", "aten::native_batch_norm", "aten::relu",
    "aten::relu_", "aten::add", "aten::add_", "aten::mul", "aten::empty", "aten::empty_like",
    "aten::zeros", "aten::copy_", "aten::to", "aten::_to_copy", "aten::softmax", "aten::_softmax",
    "aten::layer_norm", "aten::native_layer_norm", "aten::matmul", "aten::bmm", "aten::transpose",
    "aten::view", "aten::reshape", "aten::dropout", "aten::gelu", "aten::embedding",
    "aten::scaled_dot_product_attention", "autograd::engine::evaluate_function: AddmmBackward0",
    "AddmmBackward0", "Optimizer.step#AdamW.step", "aten::_foreach_add_", "aten::sum", "aten::mean",
    "aten::cat", "aten::slice", "aten::select", "aten::index", "aten::clone", "aten::contiguous",
    "aten::fill_", "aten::zero_", "aten::div", "aten::sqrt", "aten::addcmul_", "aten::addcdiv_",
    "aten::lerp_", "ProfilerStep#3", "enumerate(DataLoader)#_SingleProcessDataLoaderIter.__next__",
    "aten::max_pool2d", "aten::adaptive_avg_pool2d", "aten::flatten", "aten::log_softmax",
    "aten::nll_loss", "aten::cross_entropy_loss", "torch::autograd::AccumulateGrad", "aten::detach",
    "aten::item", "aten::_local_scalar_dense", "record_param_comms_like"};
#define N_CPU_OPS (sizeof(kCpuOps) / sizeof(kCpuOps[0]))

/* templated C++ symbol of `target` bytes with quotes, backslashes, angle brackets */
static const char* const kSymPieces[] = {
    "at::native::", "(anonymous namespace)::", "vectorized_elementwise_kernel<4, ",
    "at::native::BinaryFunctor<float, float, float, ", "std::array<char*, 3>", "c10::BFloat16",
    "cutlass::gemm::kernel::Gemm<", "ck::tensor_operation::device::DeviceGemm_Xdl_CShuffle<",
    "ck::Sequence<1, 256, 1>, ", "float const*", "unsigned int", "TensorInfo<long, unsigned int>",
    "at::detail::Array<char*, 2>", "rocprim::detail::block_reduce_kernel<", "__half2", ">, ",
    "> >", "<true>", "(int, float*, ", "hipcub::Sum", "OffsetCalculator<2, unsigned int, false>",
    "Foo<\"lit\", 'c'>", "path\\to\\header.h", "\"quoted arg\"", "a\\b", "<<<", ">>>",
    "operator()<", "lambda(int)#1}", "{lambda(float)#2", "void ", "const&, ", "&&", "::operator<<",
    "std::integral_constant<bool, true>", "TileShape<128, 256, 64>", "MFMA_F32_32x32x8F16"};
#define N_SYM_PIECES (sizeof(kSymPieces) / sizeof(kSymPieces[0]))

static uint32_t add_symbol(gen_t* g, uint64_t var, uint64_t i, uint32_t min_len, uint32_t max_len) {
  char tmp[4096];
  uint32_t target = min_len + (uint32_t)(rnd(g->seed, var, i) % (max_len - min_len + 1));
  uint32_t n = 0, k = 0;
  memcpy(tmp, "void ", 5);
  n = 5;
  while (n < target) {
    const char* pc = kSymPieces[rnd(g->seed, var + 1 + k, i) % N_SYM_PIECES];
    ++k;
    uint32_t l = (uint32_t)strlen(pc);
    if (n + l > target) {
      /* fill the rest with identifier characters */
      while (n < target) {
        tmp[n] = kIdentChars[rnd(g->seed, var + 7777 + n, i) % 63];
        ++n;
      }
      break;
    }
    memcpy(tmp + n, pc, l);
    n += l;
  }
  uint64_t r = rnd(g->seed, var + 999983, i);
  if (r % 1000 == 0 || i == 7) tmp[n / 2] = (char)(1 + (r >> 20) % 31); /* control byte (may be \n) */
  if ((r >> 32) % 50 == 0) tmp[n / 3] = '\n';                           /* newline: deleted    */
  if ((r >> 40) % 400 == 0) tmp[n / 4] = (char)0xC3;                    /* non-ASCII byte       */
  return add_string(g, tmp, n);
}

/* ------------------------------------------------------------------------------------------ */
/* common pieces                                                                                */
/* ------------------------------------------------------------------------------------------ */
enum { CID_LAUNCH = 0, CID_MEMCPY_ASYNC, CID_MEMSET_ASYNC, CID_GRAPH_LAUNCH, CID_MALLOC, CID_FREE,
       CID_STREAM_SYNC, CID_MODULE_LAUNCH, N_CIDS };
static const char* const kCidNames[N_CIDS] = {
    "hipLaunchKernel", "hipMemcpyAsync", "hipMemsetAsync", "hipGraphLaunch", "hipMalloc", "hipFree",
    "hipStreamSynchronize", "hipModuleLaunchKernel"};

#define PID 4242u
#define STREAM_HANDLE(k) (0x7f3a10000000ULL + (uint64_t)(k) * 0x1000ULL)

typedef struct common_t {
  uint32_t cpu_name0;     /* first id of CPU-op names */
  uint32_t cpu_schema;
  uint32_t kern_name0;    /* first id of kernel-name vocabulary */
  uint32_t n_kern_names;
  uint32_t fill_name;     /* fill kernel */
} common_t;

static char* dupstr(const char* s) {
  size_t n = strlen(s) + 1;
  char* p = (char*)malloc(n);
  if (p) memcpy(p, s, n);
  return p;
}

static void add_infos(gen_t* g, uint32_t n_threads, uint32_t n_streams, uint64_t n_cpu, uint64_t n_dev,
                      int with_overhead) {
  ktj_stream* s = &g->s;
  int64_t t = s->window_start_ns;
  /* resource infos in std::map<(device,id)> order: GPU 0 streams, then host threads */
  uint64_t nres = n_streams + n_threads;
  ktj_resource_info* ri = (ktj_resource_info*)own(g, calloc(nres ? nres : 1, sizeof *ri));
  uint64_t k = 0;
  for (uint32_t i = 0; i < n_streams; ++i, ++k) {
    char nm[64];
    int n = 0;
    /* fmt::format("stream {} {}", id, "") */
    char dig[24];
    int nd = 0;
    uint32_t v = i + 1;
    do { dig[nd++] = (char)('0' + v % 10); v /= 10; } while (v);
    memcpy(nm, "stream ", 7); n = 7;
    while (nd) nm[n++] = dig[--nd];
    nm[n++] = ' ';
    nm[n] = 0;
    ri[k].id = i + 1;
    ri[k].sort_index = i + 1;
    ri[k].device_id = 0;
    ri[k].name = (const char*)own(g, dupstr(nm));
    ri[k].host_thread = 0;
    ri[k].time_ns = t;
  }
  for (uint32_t i = 0; i < n_threads; ++i, ++k) {
    ri[k].id = PID + 1 + i;
    ri[k].sort_index = PID + 1 + i;
    ri[k].device_id = PID;
    ri[k].name = i == 0 ? "pt_main_thread" : (i == 1 ? "pt_autograd_0" : "pt_data_\"worker\"\\0");
    ri[k].host_thread = 1;
    ri[k].time_ns = t;
  }
  s->resource_infos = ri;
  s->n_resource_infos = nres;

  static const char* const kGpuLabels[16] = {"GPU 0", "GPU 1", "GPU 2", "GPU 3", "GPU 4", "GPU 5",
      "GPU 6", "GPU 7", "GPU 8", "GPU 9", "GPU 10", "GPU 11", "GPU 12", "GPU 13", "GPU 14", "GPU 15"};
  ktj_device_info* di = (ktj_device_info*)own(g, calloc(17, sizeof *di));
  di[0].id = PID; di[0].sort_index = PID; di[0].name = "python"; di[0].label = "CPU"; di[0].time_ns = t;
  for (int gpu = 0; gpu < 16; ++gpu) {
    di[1 + gpu].id = gpu;
    di[1 + gpu].sort_index = gpu + 5000000;
    di[1 + gpu].name = "python";
    di[1 + gpu].label = kGpuLabels[gpu];
    di[1 + gpu].time_ns = t;
  }
  s->device_infos = di;
  s->n_device_infos = 17;

  if (with_overhead) {
    ktj_overhead_info* oi = (ktj_overhead_info*)own(g, calloc(1, sizeof *oi));
    oi->name = "Instrumentation \"overhead\"";
    oi->time_ns = t;
    s->overhead_infos = oi;
    s->n_overhead_infos = 1;
  }

  ktj_trace_span* sp = (ktj_trace_span*)own(g, calloc(2, sizeof *sp));
  sp[0].start_ns = s->window_start_ns; sp[0].end_ns = s->window_end_ns;
  sp[0].op_count = (int32_t)n_cpu; sp[0].iteration = 0; sp[0].name = "PyTorch Profiler"; sp[0].prefix = "";
  sp[1].start_ns = s->window_start_ns + 1500; sp[1].end_ns = s->window_end_ns - 2500;
  sp[1].op_count = (int32_t)n_dev; sp[1].iteration = 0; sp[1].name = "PyTorch Profiler"; sp[1].prefix = "GPU: ";
  s->spans = sp;
  s->n_spans = n_cpu ? 2 : 1;
  if (!n_cpu) { sp[0] = sp[1]; }
}

static void add_common(gen_t* g, common_t* c, uint32_t n_kernel_names, int symbols) {
  /* runtime API names */
  uint32_t* cidn = (uint32_t*)own(g, malloc(sizeof(uint32_t) * N_CIDS));
  for (int i = 0; i < N_CIDS; ++i) cidn[i] = add_cstr(g, kCidNames[i]);
  g->s.cid_name_ids = cidn;
  g->s.n_cids = N_CIDS;
  static const uint32_t kFlowStart[] = {CID_LAUNCH, CID_MEMCPY_ASYNC, CID_GRAPH_LAUNCH, CID_MALLOC,
                                        CID_FREE, CID_MODULE_LAUNCH};
  g->s.flow_start_cids = kFlowStart;
  g->s.n_flow_start = sizeof(kFlowStart) / sizeof(kFlowStart[0]);
  g->s.malloc_cid = CID_MALLOC;

  c->cpu_name0 = next_string_id(g);
  for (size_t i = 0; i < N_CPU_OPS; ++i) add_cstr(g, kCpuOps[i]);

  /* CPU-op args in the order libstdc++'s unordered_map iterates this key set after inserting
   * "Sequence number", "Fwd thread id", "Record function id", "Ev Idx" */
  ktj_field f[4];
  f[0].key_id = add_cstr(g, "Ev Idx"); f[0].type = KTJ_F_I64; f[0].count = 1;
  f[1].key_id = add_cstr(g, "Record function id"); f[1].type = KTJ_F_U64; f[1].count = 1;
  f[2].key_id = add_cstr(g, "Fwd thread id"); f[2].type = KTJ_F_U64; f[2].count = 1;
  f[3].key_id = add_cstr(g, "Sequence number"); f[3].type = KTJ_F_I64; f[3].count = 1;
  c->cpu_schema = add_schema(g, f, 4);

  c->fill_name = add_cstr(g, "__amd_rocclr_fillBufferAligned.kd");
  c->kern_name0 = next_string_id(g);
  c->n_kern_names = n_kernel_names;
  for (uint32_t i = 0; i < n_kernel_names; ++i) {
    if (symbols) add_symbol(g, 0x5000, i, 200, 2048);
    else if (i == 3) add_cstr(g, "kernel");           /* exercises the "kernel"→"Kernel" rename */
    else if (i == 11) add_cstr(g, "void f<\"q\", a\\b>(int)\n");
    else if (i == 17) add_string(g, "bad\x01name", 8);
    else add_identifier(g, 0x4000, i);
  }
}

static void fill_cpu_op(gen_t* g, const common_t* c, ktj_generic_rec* r, uint64_t* args, uint64_t i,
                        int64_t start, int64_t dur, uint32_t tid, int32_t id) {
  memset(r, 0, sizeof *r);
  r->start_ns = start;
  r->end_ns = start + dur;
  r->resource = tid;
  r->id = id;
  r->device = (int32_t)PID;
  r->name_id = c->cpu_name0 + (uint32_t)(rnd(g->seed, 0x61, i) % N_CPU_OPS);
  r->type = KTJ_TYPE_CPU_OP;
  r->schema_id = c->cpu_schema;
  r->args_off = i * 4;
  args[i * 4 + 0] = (uint64_t)(int64_t)(i * 3 + 17);                 /* Ev Idx */
  args[i * 4 + 1] = 0;                                               /* Record function id */
  args[i * 4 + 2] = (rnd(g->seed, 0x62, i) % 7 == 0) ? 1 : 0;        /* Fwd thread id */
  args[i * 4 + 3] = (rnd(g->seed, 0x63, i) % 5 == 0) ? (uint64_t)-1LL : i; /* Sequence number */
}

static void fill_launch(gen_t* g, ktj_runtime_rec* r, uint64_t i, uint64_t corr, uint64_t begin,
                        uint64_t end, uint32_t tid, uint32_t stream_k) {
  memset(r, 0, sizeof *r);
  r->id = corr; r->begin = begin; r->end = end;
  r->cid = (rnd(g->seed, 0x70, i) % 16 == 0) ? CID_MODULE_LAUNCH : CID_LAUNCH;
  r->pid = PID; r->tid = tid; r->kind = KTJ_RT_KERNEL;
  uint64_t q = rnd(g->seed, 0x71, i);
  r->u.kernel.grid[0] = 1u << (q % 14);
  r->u.kernel.grid[1] = 1 + (uint32_t)((q >> 8) % 4);
  r->u.kernel.grid[2] = 1;
  r->u.kernel.workgroup[0] = 64u << ((q >> 16) % 4);
  r->u.kernel.workgroup[1] = 1;
  r->u.kernel.workgroup[2] = 1;
  r->u.kernel.group_segment_size = ((q >> 24) % 9) * 8192;
  r->u.kernel.stream = STREAM_HANDLE(stream_k);
  r->u.kernel.kernel_name_id = KTJ_NONE;
}

static void fill_kernel_row(ktj_device_rec* d, uint64_t corr, uint64_t begin, uint64_t end,
                            uint32_t name_id, uint64_t queue) {
  memset(d, 0, sizeof *d);
  d->id = corr; d->begin = begin; d->end = end;
  d->domain = KTJ_DOM_KERNEL_DISPATCH; d->op = 0; d->device = 0;
  d->name_id = name_id; d->queue = queue; d->stream = 0;
}

/* inverse of the clock model, good enough to land raw ticks near the wanted wall time */
static uint64_t to_raw(const ktj_clock_model* m, int64_t wall) {
  return m->t0_approx + (uint64_t)(wall - m->t0);
}

/* ------------------------------------------------------------------------------------------ */
/* configurations 1–3: CPU op → launch → device op, joined 1:1 (k launches per CPU op)          */
/* ------------------------------------------------------------------------------------------ */
static int gen_launch_chain(gen_t* g, uint32_t config, uint64_t N) {
  ktj_stream* s = &g->s;
  common_t c;
  const uint32_t n_streams = config == 1 ? 4 : (config == 2 ? 32 : 128);
  const uint32_t n_threads = config == 3 ? 3 : 2;
  const uint32_t launches_per_op = config == 3 ? 5 : 1;
  const uint32_t n_names = config == 3 ? 5000 : 200;
  const uint32_t zipf_s = config == 3 ? 68813 : 72090; /* 1.05 / 1.1 in Q16 */
  const int64_t B = s->base_time_ns;
  const uint64_t window = 1000000000ULL;
  uint64_t n_cpu = (N + launches_per_op - 1) / launches_per_op;

  s->window_start_ns = B;
  s->window_end_ns = B + (int64_t)window + 500000;
  s->end_time_ns = s->window_end_ns;
  add_common(g, &c, n_names, 0);
  add_infos(g, n_threads, n_streams, n_cpu, N, config == 1);

  ktj_clock_model* m = &s->clock;
  memset(m, 0, sizeof *m);
  m->t0_approx = 1000000007ULL;
  m->t0 = B - 7777;
  m->scale = 1.0;
  if (config == 1) {
    m->runtime_mode = KTJ_CLOCK_IDENTITY;
    m->device_mode = KTJ_CLOCK_OFFSET;
    m->async_offset = 123456789;
  } else if (config == 2) {
    m->runtime_mode = KTJ_CLOCK_CONVERT;
    m->device_mode = KTJ_CLOCK_CONVERT;
    m->scale = 1.000001;
  } else {
    m->runtime_mode = KTJ_CLOCK_CONVERT;
    m->device_mode = KTJ_CLOCK_OFFSET;
    m->scale = 0.999999;
    m->async_offset = -987654321;
  }

  zipf_t z;
  if (zipf_init(&z, n_names, zipf_s)) return -1;

  ktj_generic_rec* cpu = (ktj_generic_rec*)own(g, malloc(sizeof *cpu * (n_cpu ? n_cpu : 1)));
  uint64_t* args = (uint64_t*)own(g, malloc(8 * 4 * (n_cpu ? n_cpu : 1)));
  ktj_runtime_rec* rt = (ktj_runtime_rec*)own(g, malloc(sizeof *rt * (N ? N : 1)));
  ktj_device_rec* dv = (ktj_device_rec*)own(g, malloc(sizeof *dv * (N ? N : 1)));
  ktj_extcorr_rec* ec = (ktj_extcorr_rec*)own(g, malloc(sizeof *ec * (N ? N : 1)));
  uint32_t* stream_of = (uint32_t*)malloc(sizeof(uint32_t) * (N ? N : 1));
  if (!cpu || !args || !rt || !dv || !ec || !stream_of) { free(stream_of); free(z.cdf); return -1; }

  for (uint64_t j = 0; j < n_cpu; ++j) {
    int64_t start;
    if (config == 3) start = B + (int64_t)((u128)j * window / n_cpu);
    else start = B + (int64_t)(rnd(g->seed, 1, j) % window);
    int64_t dur = (int64_t)lognormal(g->seed, 2, j, 20000, 65536);
    uint32_t tid = PID + 1 + (uint32_t)(rnd(g->seed, 3, j) % n_threads);
    fill_cpu_op(g, &c, &cpu[j], args, j, start, dur, tid, (int32_t)(j + 1));
    if (config == 1 && j % 997 == 5) cpu[j].end_ns = cpu[j].start_ns - 3; /* negative duration → 0 */
  }

  for (uint64_t i = 0; i < N; ++i) {
    uint64_t j = i / launches_per_op;
    uint64_t corr = i + 1;
    uint32_t sk = (uint32_t)(rnd(g->seed, 4, i) % n_streams);
    stream_of[i] = sk;
    int64_t op_start = cpu[j].start_ns;
    int64_t op_dur = cpu[j].end_ns > cpu[j].start_ns ? cpu[j].end_ns - cpu[j].start_ns : 1000;
    int64_t l_begin, l_end;
    if (config == 3) {
      /* monotone in i so that each stream's own sequence is time-ordered */
      int64_t slot = (int64_t)(window / N);
      l_begin = B + (int64_t)((u128)i * window / N) + (int64_t)(rnd(g->seed, 5, i) % (uint64_t)(slot > 1 ? slot / 2 : 1));
      l_end = l_begin + 1 + (slot > 4 ? slot / 4 : 1);
    } else {
      l_begin = op_start + op_dur / 4;
      l_end = l_begin + (int64_t)lognormal(g->seed, 6, i, 5000, 65536);
    }
    int64_t d_begin = l_end + (int64_t)lognormal(g->seed, 7, i, 10000, 65536);
    int64_t d_dur = (int64_t)lognormal(g->seed, 8, i, 20000, 65536) + 2;
    if (config == 3) {
      int64_t slot = (int64_t)(window / N);
      d_begin = l_end + 20000; /* constant latency keeps per-stream order */
      d_dur = 2 + (int64_t)(rnd(g->seed, 8, i) % (uint64_t)(slot * n_streams / 2 + 1));
    }
    uint64_t rb = m->runtime_mode == KTJ_CLOCK_CONVERT ? to_raw(m, l_begin) : (uint64_t)l_begin;
    uint64_t re = m->runtime_mode == KTJ_CLOCK_CONVERT ? to_raw(m, l_end) : (uint64_t)l_end;
    uint64_t db = m->device_mode == KTJ_CLOCK_CONVERT ? to_raw(m, d_begin) : (uint64_t)(d_begin - m->async_offset);
    uint64_t de = m->device_mode == KTJ_CLOCK_CONVERT ? to_raw(m, d_begin + d_dur) : (uint64_t)(d_begin + d_dur - m->async_offset);

    uint32_t kind_sel = config == 2 ? (uint32_t)(rnd(g->seed, 9, i) % 10) : 0; /* 0-6 kernel, 7-8 copy, 9 memset */
    uint32_t tid = (uint32_t)cpu[j].resource;
    if (kind_sel <= 6) {
      fill_launch(g, &rt[i], i, corr, rb, re, tid, sk);
      fill_kernel_row(&dv[i], corr, db, de, c.kern_name0 + zipf_sample(&z, rnd(g->seed, 10, i)), 1 + sk);
      if (config == 1 && i % 1013 == 7) dv[i].end = dv[i].begin; /* zero-length: duration −1 → 0 */
    } else if (kind_sel <= 8) {
      ktj_runtime_rec* r = &rt[i];
      memset(r, 0, sizeof *r);
      r->id = corr; r->begin = rb; r->end = re; r->cid = CID_MEMCPY_ASYNC; r->pid = PID; r->tid = tid;
      r->kind = KTJ_RT_COPY;
      uint64_t q = rnd(g->seed, 11, i);
      uint32_t dir = (uint32_t)(q % 3); /* H2D, D2H, D2D */
      r->u.copy.src = 0x7f0000000000ULL + ((q >> 8) & 0xFFFFFF) * 256;
      r->u.copy.dst = (q >> 40) % 97 == 0 ? 0 : 0x7e0000000000ULL + ((q >> 32) & 0xFFFFFF) * 256;
      r->u.copy.size = lognormal(g->seed, 12, i, 65536, 65536);
      r->u.copy.stream = STREAM_HANDLE(sk);
      r->u.copy.copy_kind = dir + 1; /* hipMemcpyHostToDevice=1, DeviceToHost=2, DeviceToDevice=3 */
      ktj_device_rec* d = &dv[i];
      memset(d, 0, sizeof *d);
      d->id = corr; d->begin = db; d->end = de; d->domain = KTJ_DOM_MEMORY_COPY;
      d->op = dir == 0 ? KTJ_COPY_H2D : (dir == 1 ? KTJ_COPY_D2H : KTJ_COPY_D2D);
      d->device = 0; d->name_id = KTJ_NONE; d->queue = 1 + sk; d->stream = 0;
      if (i % 4001 == 9) d->end = d->begin; /* zero raw duration: no bandwidth arg */
    } else {
      ktj_runtime_rec* r = &rt[i];
      memset(r, 0, sizeof *r);
      r->id = corr; r->begin = rb; r->end = re; r->cid = CID_MEMSET_ASYNC; r->pid = PID; r->tid = tid;
      r->kind = KTJ_RT_DEFAULT;
      ktj_memset_rec m; /* the memset view of a device row */
      memset(&m, 0, sizeof m);
      m.id = corr; m.begin = db; m.end = de; m.domain = KTJ_DOM_MEMSET; m.device = 0;
      m.memory_kind = KTJ_MEMKIND_DEVICE; m.channel_type = 1; m.channel_id = 4 + (uint32_t)(sk % 4);
      m.context = 1; m.stream = 1 + (uint32_t)sk;
      m.bytes = lognormal(g->seed, 13, i, 65536, 65536);
      memcpy(&dv[i], &m, sizeof m);
    }
    ec[i].correlation = corr;
    ec[i].external_id = j + 1;
  }

  if (config == 3 && N > 1) {
    /* arrival order: every stream's (time-ordered) buffer is cut into blocks of 4096 records and
     * the blocks of all streams are shuffled */
    const uint32_t BLK = 4096;
    uint64_t* cnt = (uint64_t*)calloc(n_streams + 1, sizeof(uint64_t));
    for (uint64_t i = 0; i < N; ++i) cnt[stream_of[i] + 1]++;
    for (uint32_t k = 0; k < n_streams; ++k) cnt[k + 1] += cnt[k];
    uint64_t* by_stream = (uint64_t*)malloc(sizeof(uint64_t) * N);
    uint64_t* fillp = (uint64_t*)malloc(sizeof(uint64_t) * n_streams);
    for (uint32_t k = 0; k < n_streams; ++k) fillp[k] = cnt[k];
    for (uint64_t i = 0; i < N; ++i) by_stream[fillp[stream_of[i]]++] = i;
    uint64_t n_blocks = 0;
    for (uint32_t k = 0; k < n_streams; ++k) n_blocks += (cnt[k + 1] - cnt[k] + BLK - 1) / BLK;
    uint64_t* bstart = (uint64_t*)malloc(sizeof(uint64_t) * (n_blocks ? n_blocks : 1));
    uint64_t* bend = (uint64_t*)malloc(sizeof(uint64_t) * (n_blocks ? n_blocks : 1));
    uint64_t nb = 0;
    for (uint32_t k = 0; k < n_streams; ++k)
      for (uint64_t p = cnt[k]; p < cnt[k + 1]; p += BLK) {
        bstart[nb] = p;
        bend[nb] = p + BLK < cnt[k + 1] ? p + BLK : cnt[k + 1];
        ++nb;
      }
    for (uint64_t b = nb; b > 1; --b) { /* Fisher–Yates */
      uint64_t o = rnd(g->seed, 20, b) % b;
      uint64_t t0 = bstart[b - 1], t1 = bend[b - 1];
      bstart[b - 1] = bstart[o]; bend[b - 1] = bend[o];
      bstart[o] = t0; bend[o] = t1;
    }
    ktj_runtime_rec* rt2 = (ktj_runtime_rec*)malloc(sizeof *rt2 * N);
    ktj_device_rec* dv2 = (ktj_device_rec*)malloc(sizeof *dv2 * N);
    if (!rt2 || !dv2 || !by_stream || !bstart || !bend) return -1;
    uint64_t w = 0;
    for (uint64_t b = 0; b < nb; ++b)
      for (uint64_t p = bstart[b]; p < bend[b]; ++p, ++w) {
        rt2[w] = rt[by_stream[p]];
        dv2[w] = dv[by_stream[p]];
      }
    memcpy(rt, rt2, sizeof *rt * N);
    memcpy(dv, dv2, sizeof *dv * N);
    free(rt2); free(dv2); free(cnt); free(by_stream); free(fillp); free(bstart); free(bend);
  }
  free(stream_of);
  free(z.cdf);

  s->generic = cpu; s->n_generic = n_cpu;
  s->args = args; s->n_args = n_cpu * 4;
  s->runtime = rt; s->n_runtime = N;
  s->device = dv; s->n_device = N;
  s->extcorr = ec; s->n_extcorr = N;
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* configuration 4: graph launches with fan-out, orphans both ways                              */
/* ------------------------------------------------------------------------------------------ */
static int gen_graph(gen_t* g, uint64_t N) {
  ktj_stream* s = &g->s;
  common_t c;
  const int64_t B = s->base_time_ns;
  const uint64_t window = 1000000000ULL;
  uint64_t G = N / 550;
  if (G < 2) G = 2;
  uint32_t* fan = (uint32_t*)malloc(sizeof(uint32_t) * G);
  if (!fan) return -1;
  uint64_t n_k = 0;
  for (uint64_t q = 0; q < G; ++q) {
    fan[q] = 100 + (uint32_t)(rnd(g->seed, 30, q) % 901);
    n_k += fan[q];
  }
  uint64_t n_orph_dev = n_k / 20;
  uint64_t n_orph_rt = G / 20 + 1;
  uint64_t n_dev = n_k + n_orph_dev;
  uint64_t n_rt = G + n_orph_rt;

  s->window_start_ns = B + 1000;
  s->window_end_ns = B + (int64_t)window;
  s->end_time_ns = s->window_end_ns;
  add_common(g, &c, 1000, 0);
  /* streams seen: 8 queue-keyed rows for graph kernels + 4 for orphans → 12 dense indices */
  add_infos(g, 2, 12, G, n_dev, 0);

  ktj_clock_model* m = &s->clock;
  memset(m, 0, sizeof *m);
  m->t0_approx = 5; m->t0 = B; m->scale = 1.0;
  m->runtime_mode = KTJ_CLOCK_IDENTITY;
  m->device_mode = KTJ_CLOCK_OFFSET;
  m->async_offset = 0;

  zipf_t z;
  if (zipf_init(&z, 1000, 68813)) return -1;
  ktj_generic_rec* cpu = (ktj_generic_rec*)own(g, malloc(sizeof *cpu * G));
  uint64_t* args = (uint64_t*)own(g, malloc(8 * 4 * G));
  ktj_runtime_rec* rt = (ktj_runtime_rec*)own(g, malloc(sizeof *rt * n_rt));
  ktj_device_rec* dv = (ktj_device_rec*)own(g, malloc(sizeof *dv * n_dev));
  ktj_extcorr_rec* ec = (ktj_extcorr_rec*)own(g, malloc(sizeof *ec * G));
  if (!cpu || !args || !rt || !dv || !ec) return -1;

  uint64_t w = 0;
  for (uint64_t q = 0; q < G; ++q) {
    uint64_t corr = 1000 + q;
    int64_t start = B + 2000 + (int64_t)((u128)q * (window - 60000000ULL) / G);
    uint32_t tid = PID + 1 + (uint32_t)(q & 1);
    fill_cpu_op(g, &c, &cpu[q], args, q, start, 40000, tid, (int32_t)(q + 1));
    ktj_runtime_rec* r = &rt[q];
    memset(r, 0, sizeof *r);
    r->id = corr; r->begin = (uint64_t)(start + 5000); r->end = (uint64_t)(start + 30000);
    r->cid = CID_GRAPH_LAUNCH; r->pid = PID; r->tid = tid; r->kind = KTJ_RT_DEFAULT;
    ec[q].correlation = corr;
    ec[q].external_id = q + 1;
    int64_t t = start + 35000;
    for (uint32_t k = 0; k < fan[q]; ++k, ++w) {
      int64_t d = 500 + (int64_t)(rnd(g->seed, 31, w) % 4000);
      fill_kernel_row(&dv[w], corr, (uint64_t)t, (uint64_t)(t + d),
                      c.kern_name0 + zipf_sample(&z, rnd(g->seed, 32, w)), 1 + (q % 8));
      t += d + 200;
    }
  }
  for (uint64_t o = 0; o < n_orph_dev; ++o, ++w) {
    int64_t t = B + (int64_t)(rnd(g->seed, 33, o) % (window + 20000000ULL)); /* some beyond the window */
    fill_kernel_row(&dv[w], 2000000000ULL + o * 3, (uint64_t)t, (uint64_t)(t + 1500),
                    c.kern_name0 + zipf_sample(&z, rnd(g->seed, 34, o)), 100 + (o % 4));
    if (o % 7 == 0) dv[w].id = 0; /* correlation 0: no flow event */
  }
  for (uint64_t o = 0; o < n_orph_rt; ++o) {
    ktj_runtime_rec* r = &rt[G + o];
    memset(r, 0, sizeof *r);
    int64_t t = B + 3000 + (int64_t)(rnd(g->seed, 35, o) % (window - 1000000ULL));
    r->id = 3000000000ULL + o; r->begin = (uint64_t)t; r->end = (uint64_t)(t + 7000);
    r->cid = (o & 1) ? CID_STREAM_SYNC : CID_GRAPH_LAUNCH; r->pid = PID; r->tid = PID + 1; r->kind = KTJ_RT_DEFAULT;
    if (o % 5 == 4) { r->cid = CID_MALLOC; r->kind = KTJ_RT_MALLOC; r->u.malloc_.ptr = 0x7f1200000000ULL + o * 4096; r->u.malloc_.size = 4096 * (o + 1); }
    if (o % 5 == 3) { r->cid = CID_FREE; r->kind = KTJ_RT_MALLOC; r->u.malloc_.ptr = 0x7f1200000000ULL + o * 4096; r->u.malloc_.size = 0; }
  }
  free(fan);
  free(z.cdf);
  s->generic = cpu; s->n_generic = G;
  s->args = args; s->n_args = G * 4;
  s->runtime = rt; s->n_runtime = n_rt;
  s->device = dv; s->n_device = n_dev;
  s->extcorr = ec; s->n_extcorr = G;
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* configuration 5: string-heavy generic kernel activities with typed args                      */
/* ------------------------------------------------------------------------------------------ */
static int gen_strings(gen_t* g, uint64_t N) {
  ktj_stream* s = &g->s;
  common_t c;
  const int64_t B = s->base_time_ns;
  const uint64_t window = 1000000000ULL;
  s->window_start_ns = B;
  s->window_end_ns = B + (int64_t)window + 1000000000LL;
  s->end_time_ns = s->window_end_ns;
  add_common(g, &c, 2000, 1);
  add_infos(g, 0, 16, 0, N, 0);
  memset(&s->clock, 0, sizeof s->clock);
  s->clock.scale = 1.0;

  /* emission order of libstdc++'s unordered_map for keys inserted as grid, block,
   * registers per thread, shared memory, occupancy */
  ktj_field f[5];
  f[0].key_id = add_cstr(g, "occupancy"); f[0].type = KTJ_F_F64; f[0].count = 1;
  f[1].key_id = add_cstr(g, "registers per thread"); f[1].type = KTJ_F_U64; f[1].count = 1;
  f[2].key_id = add_cstr(g, "block"); f[2].type = KTJ_F_I64_ARRAY; f[2].count = 3;
  f[3].key_id = add_cstr(g, "shared memory"); f[3].type = KTJ_F_I64; f[3].count = 1;
  f[4].key_id = add_cstr(g, "grid"); f[4].type = KTJ_F_I64_ARRAY; f[4].count = 3;
  uint32_t schema = add_schema(g, f, 5);

  zipf_t z;
  if (zipf_init(&z, 2000, 68813)) return -1;
  ktj_generic_rec* rec = (ktj_generic_rec*)own(g, malloc(sizeof *rec * (N ? N : 1)));
  uint64_t* args = (uint64_t*)own(g, malloc(8 * 9 * (N ? N : 1)));
  if (!rec || !args) return -1;
  for (uint64_t i = 0; i < N; ++i) {
    ktj_generic_rec* r = &rec[i];
    memset(r, 0, sizeof *r);
    r->start_ns = B + (int64_t)(rnd(g->seed, 40, i) % window);
    r->end_ns = r->start_ns + (int64_t)lognormal(g->seed, 41, i, 20000, 65536);
    r->resource = 1 + (int64_t)(rnd(g->seed, 42, i) % 16);
    r->id = (int32_t)(i + 1);
    r->device = 0;
    r->name_id = c.kern_name0 + zipf_sample(&z, rnd(g->seed, 43, i));
    r->flow_id = (uint32_t)(i + 1);
    r->flow_type = KTJ_LINK_ASYNC_CPU_GPU;
    r->flags = 0;
    r->type = KTJ_TYPE_CONCURRENT_KERNEL;
    r->schema_id = schema;
    r->args_off = i * 9;
    uint64_t q = rnd(g->seed, 44, i);
    uint64_t* a = &args[i * 9];
    double occ;
    switch (q % 4) {
      case 0: occ = (double)((q >> 8) % 1000001) / 1000000.0; break;
      case 1: occ = (double)((q >> 8) % 65) / (double)(40 + 8 * ((q >> 20) % 4)); if (occ > 1.0) occ = 1.0; break;
      case 2: occ = (double)((q >> 8) % 4096) / 1099511627776.0; break;
      default: occ = (double)(1 + (q >> 8) % 2048) / 2048.0; break;
    }
    memcpy(&a[0], &occ, 8);
    a[1] = 16 + (q >> 32) % 240;                   /* registers per thread 16–255 */
    a[2] = 64u << ((q >> 40) % 5); a[3] = 1 + (q >> 44) % 2; a[4] = 1; /* block */
    a[5] = ((q >> 48) % 161) * 1024;               /* shared memory 0–160 KiB */
    a[6] = 1 + (rnd(g->seed, 45, i) % 65535); a[7] = 1 + (q >> 56) % 8; a[8] = 1; /* grid */
  }
  free(z.cdf);
  s->generic = rec; s->n_generic = N;
  s->args = args; s->n_args = N * 9;
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
ktj_stream* ktj_synth_generate(const ktj_synth_params* p) {
  if (!p || p->config < 1 || p->config > 5) return NULL;
  gen_t* g = (gen_t*)calloc(1, sizeof *g);
  if (!g) return NULL;
  static const uint64_t kSeeds[6] = {0, 0x4B310001, 0x4B310002, 0x4B310003, 0x4B310004, 0x4B310005};
  static const uint64_t kFull[6] = {0, 10000, 1000000, 10000000, 11000000, 5000000};
  g->seed = kSeeds[p->config];
  {
    uint64_t zero = 0;
    if (buf_put(&g->off, &zero, 8)) { free(g); return NULL; }
  }
  uint64_t N = p->n_device ? p->n_device : kFull[p->config];
  ktj_stream* s = &g->s;
  s->base_time_ns = p->base_time_ns;
  g->trace_name = dupstr(p->trace_name ? p->trace_name : "synthetic.json");
  s->trace_name = g->trace_name;
  s->device_properties = "";
  if (p->host_name) {
    size_t n = strlen(p->host_name);
    g->host_val = (char*)malloc(n + 3);
    g->host_val[0] = '"';
    memcpy(g->host_val + 1, p->host_name, n);
    g->host_val[n + 1] = '"';
    g->host_val[n + 2] = 0;
    g->meta_ptrs[0] = "host_name";
    g->meta_ptrs[1] = g->host_val;
    s->meta_kv = g->meta_ptrs;
    s->n_meta = 1;
  }
  int rc;
  if (p->config <= 3) rc = gen_launch_chain(g, p->config, N);
  else if (p->config == 4) rc = gen_graph(g, N);
  else rc = gen_strings(g, N);
  if (rc) { ktj_synth_free(s); return NULL; }
  s->str_blob = g->blob.p;
  s->str_off = (const uint64_t*)g->off.p;
  s->n_strings = g->off.n / 8 - 1;
  s->fields = (const ktj_field*)g->fields.p;
  s->n_fields = g->fields.n / sizeof(ktj_field);
  s->schemas = (const ktj_schema_desc*)g->schemas.p;
  s->n_schemas = g->schemas.n / sizeof(ktj_schema_desc);
  return s;
}

void ktj_synth_free(ktj_stream* s) {
  if (!s) return;
  gen_t* g = (gen_t*)s; /* ktj_stream is the first member */
  void** o = (void**)g->owned.p;
  for (size_t i = 0; i < g->owned.n / sizeof(void*); ++i) free(o[i]);
  free(g->owned.p);
  free(g->blob.p); free(g->off.p); free(g->fields.p); free(g->schemas.p);
  free(g->host_val); free(g->trace_name);
  free(g);
}
