/*
 * logger_bench.cpp — the reference's logger benchmark method (benchmarks/json_output_benchmark.cpp:
 * a fixed-seed stream of GenericTraceActivity objects of four kinds, timed from logger construction
 * through handleTraceStart, one handleGenericActivity per activity and finalizeTrace, file
 * included) applied to either logger: the reference's ChromeTraceLogger or the GpuChromeTraceLogger
 * shim, on the same activity objects in the same process.
 *
 * MEASUREMENT / TEST INFRASTRUCTURE ONLY; this repository's own code.
 */
#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <memory>
#include <random>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "Config.h"
#include "GenericTraceActivity.h"
#include "Logger.h"
#include "TraceSpan.h"
#include "output_json.h"

#include "GpuChromeTraceLogger.h"

using namespace libkineto;

namespace {

struct RefLogger : public ChromeTraceLogger {
  using ChromeTraceLogger::ChromeTraceLogger;
  using ChromeTraceLogger::finalizeTrace;
};
struct ShimLogger : public ktj_shim::GpuChromeTraceLogger {
  using GpuChromeTraceLogger::GpuChromeTraceLogger;
  using GpuChromeTraceLogger::finalizeTrace;
};

// name vocabularies of the four kinds (operator names, kernel symbols, copy directions, API names)
const char* const kOps[] = {"aten::convolution", "aten::addmm", "aten::relu_", "aten::native_batch_norm", "aten::add_",
                            "aten::mul", "aten::bmm", "aten::_softmax", "aten::embedding", "aten::native_layer_norm",
                            "aten::gelu", "aten::native_dropout"};
const char* const kKernels[] = {
    "Cijk_Ailk_Bljk_HHS_BH_MT128x64x32_MI32x32x8x1",
    "void at::native::vectorized_elementwise_kernel<4, at::native::FillFunctor<float>, at::detail::Array<char*, 1>>",
    "miopenSp3AsmConv_v30_3_1_gfx9_fp32_f2x3_stride1<float, 128, 6, 7, 3, 3, 5>",
    "void ck::kernel_gemm_xdl_cshuffle_v3<ck::GridwiseGemm_xdl_cshuffle_v3<256, 128, 128, 64, 8, 8>>",
    "Cijk_Alik_Bljk_SB_MT64x32x16_SN_1LDSB0_APM1",
    "void gemv_tn_kernel<float, 128, 16, 2, 4, 6, 7, false>",
    "void at::native::reduce_kernel<512, 1, at::native::ReduceOp<float, at::native::MeanOps<float>>>",
    "void at::native::batch_norm_collect_statistics_kernel<at::native::Var, float, float>"};
const char* const kCopies[] = {"Memcpy HtoD (Pageable -> Device)", "Memcpy DtoH (Device -> Pageable)",
                               "Memcpy DtoD (Device -> Device)"};
const char* const kApis[] = {"hipLaunchKernel", "hipMemcpyAsync", "hipStreamSynchronize", "hipMalloc", "hipFree"};
template <class T, size_t N> constexpr size_t count_of(T (&)[N]) { return N; }

struct Workload {
  TraceSpan span{0, 0, "bench"};
  std::vector<GenericTraceActivity> activities;
  int64_t end_time = 0;
};

// json_output_benchmark.cpp:140-214: kind uniform over four, durations U[1000, 100000] ns, gaps
// U[100, 1000] ns, ids counting from 1, CPU ops on (12345, 67890), the rest on device 0, stream
// i % 8; metadata through addMetadata (rendered text kept by the activity).
std::unique_ptr<Workload> make_workload(uint64_t n, uint32_t seed) {
  auto w = std::make_unique<Workload>();
  const int64_t base = ChromeTraceBaseTime::singleton().get();
  w->span = TraceSpan(base, base + 1000000000LL, "benchTrace");
  w->activities.reserve(n);
  std::mt19937 rng(seed);
  std::uniform_int_distribution<> kind_of(0, 3), duration(1000, 100000), gap(100, 1000);
  int64_t now = base;
  int32_t id = 1;
  for (uint64_t i = 0; i < n; ++i) {
    const int kind = kind_of(rng);
    ActivityType type = ActivityType::CUDA_RUNTIME;
    const char* name = kApis[i % count_of(kApis)];
    if (kind == 0) { type = ActivityType::CPU_OP; name = kOps[i % count_of(kOps)]; }
    else if (kind == 1) { type = ActivityType::CONCURRENT_KERNEL; name = kKernels[i % count_of(kKernels)]; }
    else if (kind == 2) { type = ActivityType::GPU_MEMCPY; name = kCopies[i % count_of(kCopies)]; }
    w->activities.emplace_back(w->span, type, name);
    GenericTraceActivity& a = w->activities.back();
    a.startTime = now;
    a.endTime = now + duration(rng);
    a.id = id++;
    a.device = kind == 0 ? 12345 : 0;
    a.resource = kind == 0 ? 67890 : static_cast<int32_t>(i % 8);
    a.threadId = 67890;
    a.addMetadata("External id", id);
    if (kind == 0) {
      a.addMetadataQuoted("Input Dims", "[[32, 64, 28, 28], [64, 64, 3, 3]]");
      a.addMetadata("Sequence number", static_cast<int64_t>(i));
    } else if (kind == 1) {
      a.addMetadata("grid", 128);
      a.addMetadata("block", 256);
      a.addMetadata("shared memory", 49152);
      a.addMetadata("registers per thread", 32);
    } else if (kind == 2) {
      a.addMetadata("bytes", 1048576);
    }
    now = a.endTime + gap(rng);
  }
  w->end_time = n ? w->activities.back().endTime : w->span.endTime;
  return w;
}

double ms_since(std::chrono::steady_clock::time_point t0) {
  return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
}

}  // namespace

extern "C" {

void* ktj_logger_bench_create(uint64_t n, uint32_t seed) {
  SET_LOG_SEVERITY_LEVEL(3);
  return make_workload(n, seed).release();
}
void ktj_logger_bench_destroy(void* w) { delete static_cast<Workload*>(w); }

// which: 0 = the reference's ChromeTraceLogger, activities in the order they were made (the
//            reference benchmark's own loop);
//        1 = the same logger, activities in (device, resource, start) order: the document the shim
//            must equal byte for byte (sorting is outside the timed region);
//        2 = GpuChromeTraceLogger, one handleGenericActivity call per activity;
//        3 = GpuChromeTraceLogger, one handleActivities call with `threads` packing workers.
// Returns the wall time in ms of one iteration (logger construction to the end of finalizeTrace),
// negative on failure.
double ktj_logger_bench_run(void* workload, int which, const char* path, int hip_device, int threads) {
  const Workload& w = *static_cast<Workload*>(workload);
  std::vector<const GenericTraceActivity*> order;
  if (which == 1) {
    order.reserve(w.activities.size());
    for (const auto& a : w.activities) order.push_back(&a);
    std::stable_sort(order.begin(), order.end(), [](const GenericTraceActivity* x, const GenericTraceActivity* y) {
      return std::make_tuple(x->deviceId(), x->resourceId(), x->timestamp()) <
          std::make_tuple(y->deviceId(), y->resourceId(), y->timestamp());
    });
  }
  std::vector<const ITraceActivity*> all;
  if (which == 3) {
    all.reserve(w.activities.size());
    for (const auto& a : w.activities) all.push_back(&a);
  }
  const std::unordered_map<std::string, std::string> metadata;
  const auto t0 = std::chrono::steady_clock::now();
  if (which == 0 || which == 1) {
    RefLogger logger(path);
    logger.handleTraceStart(metadata, "");
    if (which == 0) for (const auto& a : w.activities) logger.handleGenericActivity(a);
    else for (const GenericTraceActivity* a : order) logger.handleGenericActivity(*a);
    logger.finalizeTrace(w.end_time);
  } else if (which == 2 || which == 3) {
    ShimLogger logger(path, hip_device);
    logger.handleTraceStart(metadata, "");
    if (which == 2) for (const auto& a : w.activities) logger.handleGenericActivity(a);
    else logger.handleActivities(all, static_cast<unsigned>(threads > 0 ? threads : 1));
    logger.finalizeTrace(w.end_time);
    if (logger.engineStatus() != 0) return -1.0;
  } else return -2.0;
  return ms_since(t0);
}

}  // extern "C"
