/*
 * sdk_ref_driver.cpp — TEST INFRASTRUCTURE ONLY.
 *
 * Runs the reference's own RocprofLogger callbacks (libkineto/src/RocprofLogger.cpp:561-679
 * api_callback, :681-749 buffer_callback) on records built in memory, without a profiling
 * session, and prints the rocprof*Row objects they produce.  The reference translation unit is
 * compiled where it lies (this file includes it, so that the file-local global context and the
 * private callbacks are reachable; built with -fno-access-control) and linked against the
 * rocprofiler-sdk of this image; nothing of either is copied.
 *
 * A separate executable, never loaded into a test process: the translation unit defines
 * rocprofiler_configure, which a process that initialises HIP would hand to the SDK.
 *
 * stdin (binary, little endian):
 *   u32 mode                       1 = buffer records, 2 = HIP runtime API records, 3 = activity wrappers,
 *                                  4 = stream back-fill, then activity wrappers
 * mode 1:
 *   u64 n_rows, ktj_device_rec rows[n_rows], u64 agent_base, u64 kernel_base, u32 unknown_name_id,
 *   u32 noise, u64 n_agents, {u64 handle, i64 device}[n_agents], u64 n_kernels,
 *   {u64 kernel_id, u64 name_id}[n_kernels]
 *   The SDK records are built by tests/host_sim/sdk_records.cpp from the rows, as in the tests.
 * mode 2:
 *   u64 n_records, {u32 operation, u32 pad, u64 correlation_id, u8 args[sizeof(rocprofiler_hip_api_args_t)]}[n]
 *   Each record goes through api_callback twice (enter, exit).  Pointer-typed arguments should point
 *   into [KTJ_ARG_ARENA, KTJ_ARG_ARENA + 16 MiB): the driver maps zero pages there, because the SDK's
 *   argument iterator follows pointers when it renders them.
 * mode 3:
 *   u64 n_runtime, ktj_runtime_rec rows[n_runtime], u64 n_device, ktj_device_rec rows[n_device],
 *   u64 n_names, {u32 length, bytes}[n_names]      (the device rows' name_id indexes these)
 *   The rows become rocprofRow / rocprofKernelRow / rocprofCopyRow / rocprofMallocRow and rocprofAsyncRow
 *   objects and are wrapped in the reference's RuntimeActivity<T> and GpuActivity
 *   (libkineto/src/RocprofActivity.h:37-162, RocprofActivity_inl.h), runtime rows first, in the order
 *   given: what each wrapper reports through ITraceActivity (and the args text of metadataJson(),
 *   which also passes grid, block and size from a runtime row to the device rows of its id) is printed.
 *   Mode 4 first runs the reference's detail::backfillAsyncStreams (RocmStreamQueue.h:42-136) over the
 *   rows, as RocprofActivityApi::processActivities does (RocprofActivityApi.cpp:134-142).
 * stdout: one text line per row the logger holds afterwards; in mode 2 the row's line is followed by
 * an "args" line with the SDK's own rendering of every argument (name=text), which is what the
 * reference keeps of dst, src and ptr.
 */
#include "RocprofLogger.cpp"  // NOLINT: the reference's translation unit, found through -I$(REF)/libkineto/src
#include "RocprofActivity.h"  // NOLINT: the reference's activity wrappers (header-only)
#include "RocmStreamQueue.h"  // NOLINT: the reference's stream back-fill (header-only)

#include <sys/mman.h>

#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include <rocprofiler-sdk/hip/api_args.h>

#include "../../include/ktj.h"

extern "C" {
void* ktjsim_sdk_buffer_create(const ktj_device_rec* rows, uint64_t n, uint64_t agent_base, uint64_t kernel_base,
                               uint32_t unknown_name_id, int noise);
void* const* ktjsim_sdk_buffer_headers(void* buf);
uint64_t ktjsim_sdk_buffer_count(void* buf);
}

namespace {

template <typename T> T rd() {
  T v;
  if (fread(&v, sizeof v, 1, stdin) != 1) { fprintf(stderr, "sdk_ref_driver: short input\n"); exit(2); }
  return v;
}

void print_rows() {
  for (const rocprofBase* b : RocprofLogger::singleton().rows_) {
    switch (b->type) {
      case ROCTRACER_ACTIVITY_ASYNC: {
        const auto* r = static_cast<const rocprofAsyncRow*>(b);
        printf("async id=%" PRIu64 " begin=%" PRIu64 " end=%" PRIu64 " domain=%u kind=%u op=%u device=%d queue=%" PRIu64
               " stream=%" PRIu64 " name=%s\n",
               r->id, r->begin, r->end, r->domain, r->kind, r->op, r->device, r->queue, r->stream, r->kernelName.c_str());
        break;
      }
      case ROCTRACER_ACTIVITY_KERNEL: {
        const auto* r = static_cast<const rocprofKernelRow*>(b);
        printf("kernel id=%" PRIu64 " domain=%u cid=%u grid=%u,%u,%u workgroup=%u,%u,%u gss=%zu stream=%" PRIu64
               " faddr=%" PRIu64 " function=%" PRIu64 "\n",
               r->id, r->domain, r->cid, r->gridX, r->gridY, r->gridZ, r->workgroupX, r->workgroupY, r->workgroupZ,
               r->groupSegmentSize, (uint64_t)(uintptr_t)r->stream, (uint64_t)(uintptr_t)r->functionAddr,
               (uint64_t)(uintptr_t)r->function);
        break;
      }
      case ROCTRACER_ACTIVITY_COPY: {
        const auto* r = static_cast<const rocprofCopyRow*>(b);
        /* src and dst hold the address of the SDK's rendering of the argument (RocprofLogger.cpp:52-58,
         * 611-624), which is gone by now: not followed */
        printf("copy id=%" PRIu64 " domain=%u cid=%u size=%zu kind=%d stream=%" PRIu64 "\n", r->id, r->domain, r->cid, r->size,
               (int)r->kind, (uint64_t)(uintptr_t)r->stream);
        break;
      }
      case ROCTRACER_ACTIVITY_MALLOC: {
        const auto* r = static_cast<const rocprofMallocRow*>(b);
        printf("malloc id=%" PRIu64 " domain=%u cid=%u size=%zu\n", r->id, r->domain, r->cid, r->size);
        break;
      }
      case ROCTRACER_ACTIVITY_DEFAULT: {
        const auto* r = static_cast<const rocprofRow*>(b);
        printf("default id=%" PRIu64 " domain=%u cid=%u\n", r->id, r->domain, r->cid);
        break;
      }
      default: printf("other type=%d\n", (int)b->type); break;
    }
  }
}

int run_buffer_records() {
  const uint64_t n = rd<uint64_t>();
  std::vector<ktj_device_rec> rows(n);
  if (n && fread(rows.data(), sizeof(ktj_device_rec), n, stdin) != n) return 2;
  const uint64_t agent_base = rd<uint64_t>(), kernel_base = rd<uint64_t>();
  const uint32_t unknown = rd<uint32_t>(), noise = rd<uint32_t>();
  auto& g = getGlobalContext();
  const uint64_t n_agents = rd<uint64_t>();
  for (uint64_t i = 0; i < n_agents; ++i) {
    const uint64_t handle = rd<uint64_t>();
    const int64_t device = rd<int64_t>();
    rocprofiler_agent_v0_t a;
    std::memset(&a, 0, sizeof a);
    a.id.handle = handle;
    a.logical_node_type_id = (int32_t)device;
    g.agents[handle] = a;
  }
  const uint64_t n_kernels = rd<uint64_t>();
  for (uint64_t i = 0; i < n_kernels; ++i) {
    const uint64_t id = rd<uint64_t>(), name_id = rd<uint64_t>();
    g.kernel_names[id] = "name#" + std::to_string(name_id);
  }
  /* the SDK's numbers for the two record kinds, so that the reader need not know them */
  printf("kinds dispatch=%d copy=%d\n", (int)ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH, (int)ROCPROFILER_BUFFER_TRACING_MEMORY_COPY);
  void* buf = ktjsim_sdk_buffer_create(rows.data(), n, agent_base, kernel_base, unknown, (int)noise);
  auto** headers = reinterpret_cast<rocprofiler_record_header_t**>(const_cast<void**>(ktjsim_sdk_buffer_headers(buf)));
  RocprofLogger::buffer_callback(rocprofiler_context_id_t{0}, rocprofiler_buffer_id_t{0}, headers, ktjsim_sdk_buffer_count(buf),
                                 nullptr, 0);
  print_rows();
  return 0;
}

#define KTJ_ARG_ARENA 0x700000000000ull
int print_arg(rocprofiler_callback_tracing_kind_t, rocprofiler_tracing_operation_t, uint32_t, const void* const, int32_t,
              const char*, const char* arg_name, const char* arg_value_str, int32_t, void*) {
  printf(" %s=%s;", arg_name, arg_value_str);
  return 0;
}

int run_api_records() {
  if (mmap(reinterpret_cast<void*>(KTJ_ARG_ARENA), 16u << 20, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_FIXED,
           -1, 0) == MAP_FAILED) {
    fprintf(stderr, "sdk_ref_driver: cannot map the argument arena\n");
    return 2;
  }
  printf("kind hip_runtime_api=%d\n", (int)ROCPROFILER_CALLBACK_TRACING_HIP_RUNTIME_API);
  const uint64_t n = rd<uint64_t>();
  for (uint64_t i = 0; i < n; ++i) {
    const uint32_t op = rd<uint32_t>();
    (void)rd<uint32_t>();
    const uint64_t corr = rd<uint64_t>();
    rocprofiler_callback_tracing_hip_api_data_t data;
    std::memset(&data, 0, sizeof data);
    data.size = sizeof data;
    if (fread(&data.args, sizeof data.args, 1, stdin) != 1) return 2;
    rocprofiler_callback_tracing_record_t rec;
    std::memset(&rec, 0, sizeof rec);
    rec.correlation_id.internal = corr;
    rec.kind = ROCPROFILER_CALLBACK_TRACING_HIP_RUNTIME_API;
    rec.operation = (rocprofiler_tracing_operation_t)op;
    rec.payload = &data;
    rec.phase = ROCPROFILER_CALLBACK_PHASE_ENTER;
    RocprofLogger::api_callback(rec, nullptr, nullptr);
    rec.phase = ROCPROFILER_CALLBACK_PHASE_EXIT;
    RocprofLogger::api_callback(rec, nullptr, nullptr);
    print_rows();
    RocprofLogger::singleton().rows_.clear();
    printf("args");
    rocprofiler_iterate_callback_tracing_kind_operation_args(rec, print_arg, 1, nullptr);
    printf("\n");
  }
  return 0;
}

template <class A> void print_wrapper(const char* what, uint64_t index, const A& a) {
  printf("%s idx=%" PRIu64 " corr=%" PRId64 " type=%d dev=%" PRId64 " res=%" PRId64 " ts=%" PRId64 " dur=%" PRId64
         " flowstart=%d flowid=%" PRId64 " flowtype=%d name=%s json=%s\n",
         what, index, a.correlationId(), (int)a.type(), a.deviceId(), a.resourceId(), a.timestamp(), a.duration(),
         a.flowStart() ? 1 : 0, a.flowId(), a.flowType(), a.name().c_str(), a.metadataJson().c_str());
}

int run_wrappers(bool backfill) {
  const uint64_t nr = rd<uint64_t>();
  std::vector<ktj_runtime_rec> rt(nr);
  if (nr && fread(rt.data(), sizeof(ktj_runtime_rec), nr, stdin) != nr) return 2;
  const uint64_t nd = rd<uint64_t>();
  std::vector<ktj_device_rec> dev(nd);
  if (nd && fread(dev.data(), sizeof(ktj_device_rec), nd, stdin) != nd) return 2;
  const uint64_t nn = rd<uint64_t>();
  std::vector<std::string> names(nn);
  for (auto& n : names) {
    n.resize(rd<uint32_t>());
    if (!n.empty() && fread(&n[0], 1, n.size(), stdin) != n.size()) return 2;
  }
  /* the operation names, as the reference's tool initialisation takes them from the SDK (RocprofLogger.cpp:346-347) */
  getGlobalContext().name_info = rocprofiler::sdk::get_callback_tracing_names();
  getGlobalContext().buff_name_info = rocprofiler::sdk::get_buffer_tracing_names();
  const uint32_t dom = ROCPROFILER_CALLBACK_TRACING_HIP_RUNTIME_API;
  std::vector<rocprofBase*> rows; /* as RocprofLogger holds them: runtime rows, then device rows */
  for (uint64_t i = 0; i < nr; ++i) {
    const ktj_runtime_rec& r = rt[i];
    switch (r.kind) {
      case KTJ_RT_KERNEL:
        rows.push_back(new rocprofKernelRow(r.id, dom, r.cid, r.pid, r.tid, r.begin, r.end, nullptr, nullptr, r.u.kernel.grid[0],
                                            r.u.kernel.grid[1], r.u.kernel.grid[2], r.u.kernel.workgroup[0], r.u.kernel.workgroup[1],
                                            r.u.kernel.workgroup[2], r.u.kernel.group_segment_size,
                                            reinterpret_cast<hipStream_t>(r.u.kernel.stream)));
        break;
      case KTJ_RT_COPY:
        rows.push_back(new rocprofCopyRow(r.id, dom, r.cid, r.pid, r.tid, r.begin, r.end, reinterpret_cast<const void*>(r.u.copy.src),
                                          reinterpret_cast<const void*>(r.u.copy.dst), r.u.copy.size,
                                          static_cast<hipMemcpyKind>(r.u.copy.copy_kind), reinterpret_cast<hipStream_t>(r.u.copy.stream)));
        break;
      case KTJ_RT_MALLOC:
        rows.push_back(new rocprofMallocRow(r.id, dom, r.cid, r.pid, r.tid, r.begin, r.end,
                                            reinterpret_cast<const void*>(r.u.malloc_.ptr), r.u.malloc_.size));
        break;
      default: rows.push_back(new rocprofRow(r.id, dom, r.cid, r.pid, r.tid, r.begin, r.end)); break;
    }
  }
  for (uint64_t i = 0; i < nd; ++i) {
    const ktj_device_rec& d = dev[i];
    const uint32_t kind = d.domain == KTJ_DOM_MEMORY_COPY ? (uint32_t)ROCPROFILER_BUFFER_TRACING_MEMORY_COPY
                                                          : (uint32_t)ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH;
    auto* row = new rocprofAsyncRow(d.id, kind, kind, d.op, d.device, d.queue, d.begin, d.end,
                                    d.name_id < names.size() ? names[d.name_id] : std::string());
    row->stream = d.stream;
    rows.push_back(row);
  }
  if (backfill) /* RocprofActivityApi.cpp:134-142 with copies and kernels both logged */
    KINETO_NAMESPACE::detail::backfillAsyncStreams(rows, [](const rocprofAsyncRow& a) {
      return a.domain == ROCPROFILER_BUFFER_TRACING_MEMORY_COPY || a.domain == ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH;
    });
  for (uint64_t i = 0; i < rows.size(); ++i) {
    const rocprofBase* b = rows[i];
    switch (b->type) {
      case ROCTRACER_ACTIVITY_KERNEL: print_wrapper("runtime", i, RuntimeActivity<rocprofKernelRow>(static_cast<const rocprofKernelRow*>(b), nullptr)); break;
      case ROCTRACER_ACTIVITY_COPY: print_wrapper("runtime", i, RuntimeActivity<rocprofCopyRow>(static_cast<const rocprofCopyRow*>(b), nullptr)); break;
      case ROCTRACER_ACTIVITY_MALLOC: print_wrapper("runtime", i, RuntimeActivity<rocprofMallocRow>(static_cast<const rocprofMallocRow*>(b), nullptr)); break;
      case ROCTRACER_ACTIVITY_ASYNC: print_wrapper("device", i - nr, GpuActivity(static_cast<const rocprofAsyncRow*>(b), nullptr)); break;
      default: print_wrapper("runtime", i, RuntimeActivity<rocprofRow>(static_cast<const rocprofRow*>(b), nullptr)); break;
    }
  }
  return 0;
}

}  // namespace

int main() {
  const uint32_t mode = rd<uint32_t>();
  int rc = 2;
  if (mode == 1) rc = run_buffer_records();
  else if (mode == 2) rc = run_api_records();
  else if (mode == 3 || mode == 4) rc = run_wrappers(mode == 4);
  fflush(stdout);
  _exit(rc); /* no destructors: the logger's would stop a tracing context that was never created */
}
