/*
 * Test infrastructure, never linked into the product: the reference's own CUDA activity wrappers
 * (libkineto/src/CuptiActivity.h) on records built in memory.
 *
 * The memset device rows of this repository (KTJ_DOM_MEMSET) are shaped like CUpti_ActivityMemset4
 * and print what GpuActivity<CUpti_ActivityMemsetType> prints (CuptiActivity.h:682-719).  This
 * driver includes that header where it lies, against the CUDA 12 / CUPTI headers that the image
 * carries, builds one CUPTI record per packed row, wraps it in the reference's GpuActivity<> and
 * prints what the wrapper reports through ITraceActivity and metadataJson().  No CUPTI or CUDA
 * function is called: the wrappers only read the record.
 *
 * Without arguments.  stdin (binary, little endian):
 *   u64 n, n x ktj_device_rec          rows with domain KTJ_DOM_MEMSET (the ktj_memset_rec view)
 * stdout:
 *   cuda_version <CUDA_VERSION>
 *   memset idx=.. corr=.. type=.. dev=.. res=.. ts=.. dur=.. flowstart=.. flowid=.. flowtype=.. name=.. json=..
 *
 * `cupti_ref_driver log <seed> <reference file> <shim file> [hip device]` (needs a GPU): a seeded set
 * of CUDA activity records of every kind the header wraps, except kernels (whose metadata asks the
 * CUDA runtime for device properties) — runtime and driver API calls, overhead, synchronization,
 * CUDA events, memcpy, peer-to-peer memcpy, memset — some linked to CPU ops, is wrapped in the
 * reference's own classes and logged twice: through the reference's ChromeTraceLogger in
 * (deviceId, resourceId, timestamp) order, and through the GpuChromeTraceLogger shim in arrival order.
 * The caller compares the two files.  Prints the number of activities.
 */
#include <cinttypes>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include <algorithm>
#include <memory>
#include <random>
#include <string>

#include "CuptiActivity.h"
#include "output_json.h"

#include "GpuChromeTraceLogger.h"
#include "ktj.h"

using namespace KINETO_NAMESPACE;

namespace {

template <class T> T rd() {
  T v;
  if (fread(&v, sizeof v, 1, stdin) != 1) { fprintf(stderr, "cupti_ref_driver: short input\n"); exit(2); }
  return v;
}

template <class A> void print_wrapper(const char* what, uint64_t index, const A& a) {
  printf("%s idx=%" PRIu64 " corr=%" PRId64 " type=%d dev=%" PRId64 " res=%" PRId64 " ts=%" PRId64 " dur=%" PRId64
         " flowstart=%d flowid=%" PRId64 " flowtype=%d name=%s json=%s\n",
         what, index, a.correlationId(), (int)a.type(), a.deviceId(), a.resourceId(), a.timestamp(), a.duration(),
         a.flowStart() ? 1 : 0, a.flowId(), a.flowType(), a.name().c_str(), a.metadataJson().c_str());
}

struct RefLogger : public ChromeTraceLogger { /* exposes the protected finalizeTrace(int64_t): no Config object needed */
  using ChromeTraceLogger::ChromeTraceLogger;
  using ChromeTraceLogger::finalizeTrace;
};
struct ShimLogger : public ktj_shim::GpuChromeTraceLogger {
  using GpuChromeTraceLogger::GpuChromeTraceLogger;
  using GpuChromeTraceLogger::finalizeTrace;
};

/* the records live as long as the wrappers that refer to them */
struct Records {
  std::vector<std::unique_ptr<CUpti_ActivityAPI>> api;
  std::vector<std::unique_ptr<CUpti_ActivityOverhead>> overhead;
  std::vector<std::unique_ptr<CUpti_ActivitySynchronization>> sync;
  std::vector<std::unique_ptr<CUpti_ActivityCudaEventType>> event;
  std::vector<std::unique_ptr<CUpti_ActivityMemcpyType>> memcpy_;
  std::vector<std::unique_ptr<CUpti_ActivityMemcpyPtoPType>> p2p;
  std::vector<std::unique_ptr<CUpti_ActivityMemsetType>> memset_;
  std::vector<std::unique_ptr<GenericTraceActivity>> cpu_ops;
  std::vector<std::unique_ptr<ITraceActivity>> wrappers;
};
template <class T> T* zeroed(std::vector<std::unique_ptr<T>>& v) {
  v.emplace_back(new T);
  memset(v.back().get(), 0, sizeof(T));
  return v.back().get();
}

int log_both(unsigned seed, const char* ref_path, const char* shim_path, int hip_device) {
  SET_LOG_SEVERITY_LEVEL(3);
  std::mt19937_64 rng(seed);
  auto pick = [&](uint64_t n) { return (uint64_t)(rng() % n); };
  const int64_t base = ChromeTraceBaseTime::singleton().get();
  Records r;
  TraceSpan span(base, base + 1000000, "cupti");
  for (int k = 0; k < 6; ++k) { /* CPU ops some activities are linked to */
    auto op = std::make_unique<GenericTraceActivity>(span, ActivityType::CPU_OP, "aten::op" + std::to_string(k));
    op->startTime = base + 100 + 50 * k; op->endTime = op->startTime + 40;
    op->id = 700 + k; op->device = 4242; op->resource = 4243 + (k & 1);
    r.cpu_ops.push_back(std::move(op));
  }
  auto linked = [&]() -> const ITraceActivity* { return pick(3) == 0 ? nullptr : r.cpu_ops[pick(r.cpu_ops.size())].get(); };
  const uint32_t runtime_cbids[] = {CUPTI_RUNTIME_TRACE_CBID_cudaLaunchKernel_v7000, CUPTI_RUNTIME_TRACE_CBID_cudaMemcpyAsync_v3020,
                                    CUPTI_RUNTIME_TRACE_CBID_cudaDeviceSynchronize_v3020, CUPTI_RUNTIME_TRACE_CBID_cudaMalloc_v3020,
                                    CUPTI_RUNTIME_TRACE_CBID_cudaGraphLaunch_v10000, CUPTI_RUNTIME_TRACE_CBID_cudaMemset_v3020, 9999};
  const uint32_t driver_cbids[] = {CUPTI_DRIVER_TRACE_CBID_cuLaunchKernel, CUPTI_DRIVER_TRACE_CBID_cuMemcpyHtoDAsync_v2, 9999};
  const int n = 160;
  for (int i = 0; i < n; ++i) {
    const uint64_t start = (uint64_t)base + 1000 + pick(900000), end = start + (pick(5) == 0 ? 0 : pick(50000));
    const uint32_t corr = (uint32_t)(1 + pick(400)), stream = (uint32_t)(7 + pick(3)), ctx = 1, dev = (uint32_t)pick(2);
    switch (pick(9)) {
      case 0: case 1: {
        auto* a = zeroed(r.api);
        a->kind = CUPTI_ACTIVITY_KIND_RUNTIME; a->cbid = runtime_cbids[pick(7)]; a->start = start; a->end = end;
        a->processId = 4242; a->threadId = 77; a->correlationId = corr;
        r.wrappers.emplace_back(new RuntimeActivity(a, linked(), 4243 + (int32_t)pick(2)));
        break;
      }
      case 2: {
        auto* a = zeroed(r.api);
        a->kind = CUPTI_ACTIVITY_KIND_DRIVER; a->cbid = driver_cbids[pick(3)]; a->start = start; a->end = end;
        a->processId = 4242; a->threadId = 77; a->correlationId = corr;
        r.wrappers.emplace_back(new DriverActivity(a, linked(), 4243));
        break;
      }
      case 3: {
        auto* a = zeroed(r.overhead);
        a->kind = CUPTI_ACTIVITY_KIND_OVERHEAD; a->overheadKind = (CUpti_ActivityOverheadKind)(CUPTI_ACTIVITY_OVERHEAD_DRIVER_COMPILER + pick(3));
        a->start = start; a->end = end;
        r.wrappers.emplace_back(new OverheadActivity(a, nullptr, (int32_t)pick(3)));
        break;
      }
      case 4: {
        auto* a = zeroed(r.sync);
        a->kind = CUPTI_ACTIVITY_KIND_SYNCHRONIZATION;
        a->type = (CUpti_ActivitySynchronizationType)(CUPTI_ACTIVITY_SYNCHRONIZATION_TYPE_EVENT_SYNCHRONIZE + pick(4));
        a->start = start; a->end = end; a->correlationId = corr; a->contextId = ctx; a->streamId = stream; a->cudaEventId = (uint32_t)pick(20);
        r.wrappers.emplace_back(new CudaSyncActivity(a, linked(), (int32_t)stream, (int32_t)corr));
        break;
      }
      case 5: {
        auto* a = zeroed(r.event);
        a->kind = CUPTI_ACTIVITY_KIND_CUDA_EVENT; a->correlationId = corr; a->contextId = ctx; a->streamId = stream; a->eventId = (uint32_t)pick(20);
#if CUDA_VERSION >= 12080
        a->deviceTimestamp = start; a->deviceId = dev;
#endif
        r.wrappers.emplace_back(new CudaEventActivity(a, linked()));
        break;
      }
      case 6: {
        auto* a = zeroed(r.memcpy_);
        a->kind = CUPTI_ACTIVITY_KIND_MEMCPY; a->copyKind = (uint8_t)(1 + pick(10)); a->srcKind = (uint8_t)pick(8); a->dstKind = (uint8_t)pick(8);
        a->bytes = pick(1 << 28); a->start = start; a->end = end; a->deviceId = dev; a->contextId = ctx; a->streamId = stream; a->correlationId = corr;
        a->graphId = (uint32_t)pick(3); a->graphNodeId = pick(1000); a->channelID = (uint32_t)pick(8); a->channelType = (CUpti_ChannelType)pick(3);
        r.wrappers.emplace_back(new GpuActivity<CUpti_ActivityMemcpyType>(a, linked()));
        break;
      }
      case 7: {
        auto* a = zeroed(r.p2p);
        a->kind = CUPTI_ACTIVITY_KIND_MEMCPY2; a->copyKind = CUPTI_ACTIVITY_MEMCPY_KIND_PTOP; a->srcKind = 3; a->dstKind = 3;
        a->bytes = pick(1 << 28); a->start = start; a->end = end; a->deviceId = dev; a->contextId = ctx; a->streamId = stream;
        a->srcDeviceId = 0; a->srcContextId = 1; a->dstDeviceId = 1; a->dstContextId = 2; a->correlationId = corr;
        a->graphId = (uint32_t)pick(3); a->graphNodeId = pick(1000); a->channelID = (uint32_t)pick(8); a->channelType = (CUpti_ChannelType)pick(3);
        r.wrappers.emplace_back(new GpuActivity<CUpti_ActivityMemcpyPtoPType>(a, linked()));
        break;
      }
      default: {
        auto* a = zeroed(r.memset_);
        a->kind = CUPTI_ACTIVITY_KIND_MEMSET; a->memoryKind = (uint16_t)pick(9); a->bytes = pick(1 << 24); a->start = start; a->end = end;
        a->deviceId = dev; a->contextId = ctx; a->streamId = stream; a->correlationId = corr;
        a->graphId = (uint32_t)pick(3); a->graphNodeId = pick(1000); a->channelID = (uint32_t)pick(8); a->channelType = (CUpti_ChannelType)pick(3);
        r.wrappers.emplace_back(new GpuActivity<CUpti_ActivityMemsetType>(a, linked()));
        break;
      }
    }
  }
  std::vector<const ITraceActivity*> arrival;
  for (const auto& op : r.cpu_ops) arrival.push_back(op.get());
  for (const auto& w : r.wrappers) arrival.push_back(w.get());
  std::vector<const ITraceActivity*> sorted = arrival;
  std::stable_sort(sorted.begin(), sorted.end(), [](const ITraceActivity* a, const ITraceActivity* b) {
    if (a->deviceId() != b->deviceId()) return a->deviceId() < b->deviceId();
    if (a->resourceId() != b->resourceId()) return a->resourceId() < b->resourceId();
    return a->timestamp() < b->timestamp();
  });
  const int64_t end_time = base + 2000000;
  {
    RefLogger ref(ref_path);
    ref.handleTraceStart({}, "");
    for (const ITraceActivity* a : sorted) ref.handleActivity(*a);
    ref.finalizeTrace(end_time);
  }
  {
    ShimLogger shim(shim_path, hip_device);
    shim.handleTraceStart({}, "");
    for (const ITraceActivity* a : arrival) shim.handleActivity(*a);
    shim.finalizeTrace(end_time);
    if (shim.engineStatus() != 0 || shim.unsupportedActivities() != 0) {
      fprintf(stderr, "cupti_ref_driver: shim status %d, %llu activities not taken\n", shim.engineStatus(),
              (unsigned long long)shim.unsupportedActivities());
      return 3;
    }
  }
  printf("activities %zu\n", arrival.size());
  return 0;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc >= 5 && std::string(argv[1]) == "log")
    return log_both((unsigned)atoi(argv[2]), argv[3], argv[4], argc > 5 ? atoi(argv[5]) : 0);
  /* records carry host-clock nanoseconds already: no TSC conversion (CuptiTimestamp.h:29-51) */
  use_cupti_tsc() = false;
  printf("cuda_version %d\n", (int)CUDA_VERSION);
  const uint64_t n = rd<uint64_t>();
  std::vector<ktj_device_rec> rows(n);
  if (n && fread(rows.data(), sizeof(ktj_device_rec), n, stdin) != n) return 2;
  for (uint64_t i = 0; i < n; ++i) {
    ktj_memset_rec m;
    static_assert(sizeof m == sizeof rows[i], "the memset view is a device row");
    memcpy(&m, &rows[i], sizeof m);
    if (m.domain != KTJ_DOM_MEMSET) { fprintf(stderr, "cupti_ref_driver: row %" PRIu64 " is not a memset row\n", i); return 2; }
    CUpti_ActivityMemsetType rec;
    memset(&rec, 0, sizeof rec);
    rec.kind = CUPTI_ACTIVITY_KIND_MEMSET;
    rec.value = 0;
    rec.bytes = m.bytes;
    rec.start = m.begin;
    rec.end = m.end;
    rec.deviceId = (uint32_t)m.device;
    rec.contextId = m.context;
    rec.streamId = (uint32_t)m.stream;
    rec.correlationId = (uint32_t)m.id;
    rec.memoryKind = m.memory_kind;
    rec.graphNodeId = (uint64_t)m.graph_node_lo | ((uint64_t)m.graph_node_hi << 32);
    rec.graphId = m.graph_id;
    rec.channelID = m.channel_id;
    rec.channelType = (CUpti_ChannelType)m.channel_type;
    print_wrapper("memset", i, GpuActivity<CUpti_ActivityMemsetType>(&rec, nullptr));
  }
  return 0;
}
