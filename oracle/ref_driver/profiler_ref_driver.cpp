/*
 * profiler_ref_driver.cpp — TEST INFRASTRUCTURE ONLY.
 *
 * Runs the reference's own post-processing loop — GenericActivityProfiler::processTraceInternal
 * (libkineto/src/GenericActivityProfiler.cpp:141-224) with RocmActivityProfiler's handlers
 * (src/RocmActivityProfiler.cpp:127-208), RocprofActivityApi::processActivities
 * (src/RocprofActivityApi.cpp:103-181) and the real ChromeTraceLogger — on rows, external
 * correlation pairs and CPU ops built in memory, without a profiling session: the rows are put
 * where RocprofLogger keeps them, the profiler's private state that configure()/startTrace()
 * would set is set directly (built with -fno-access-control), and the trace is written to the
 * file named on the command line.  All translation units are the reference's, compiled where
 * they lie (oracle/Makefile); nothing of them is copied.
 *
 * A separate executable (RocprofLogger.cpp defines rocprofiler_configure; see sdk_ref_driver.cpp).
 *
 * argv[1]: output trace file.   stdin (binary, little endian):
 *   i64 window_start_ns, i64 window_end_ns
 *   u64 n_cpu_ops, ktj_generic_rec ops[n]          (CPU ops: name_id, start_ns, end_ns, id, device, resource, type)
 *   u64 n_ext, ktj_extcorr_rec[n]                  (default domain)
 *   u64 n_user, ktj_extcorr_rec[n]                 (user domain)
 *   u64 n_runtime, ktj_runtime_rec[n]; u64 n_device, ktj_device_rec[n]
 *   u64 n_names, {u32 length, bytes}[n]            (name_id of CPU ops and device rows)
 * Device rows' begin/end are taken as final times: RocprofActivityApi adds the offset between
 * its two clocks, sampled while it runs; the driver subtracts its own sample of that offset first,
 * so that what the reference adds back differs from it by the few hundred nanoseconds between the
 * two samples; the caller reads that remainder off the first device event of the trace.
 * stdout: base_time=<ChromeTraceBaseTime>, out_of_range=<n>, out_of_order=<n>
 */
#include "RocprofLogger.cpp"       // NOLINT: the reference's translation unit (its file-local context holds the operation names)
#include "RocprofActivityApi.cpp"  // NOLINT: the reference's translation unit (for getTimeOffset and the private snapshot)

#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <string>
#include <vector>

#include "ActivityBuffers.h"
#include "Config.h"
#include "RocmActivityProfiler.h"
#include "output_json.h"

#include "../../include/ktj.h"

using namespace KINETO_NAMESPACE;

namespace {

template <typename T> T rd() {
  T v;
  if (fread(&v, sizeof v, 1, stdin) != 1) { fprintf(stderr, "profiler_ref_driver: short input\n"); exit(2); }
  return v;
}
template <typename T> std::vector<T> rd_array() {
  const uint64_t n = rd<uint64_t>();
  std::vector<T> v(n);
  if (n && fread(v.data(), sizeof(T), n, stdin) != n) { fprintf(stderr, "profiler_ref_driver: short input\n"); exit(2); }
  return v;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 2) return 2;
  const int64_t win_start = rd<int64_t>(), win_end = rd<int64_t>();
  const auto ops = rd_array<ktj_generic_rec>();
  const auto ext = rd_array<ktj_extcorr_rec>();
  const auto user = rd_array<ktj_extcorr_rec>();
  const auto rt = rd_array<ktj_runtime_rec>();
  const auto dev = rd_array<ktj_device_rec>();
  std::vector<std::string> names(rd<uint64_t>());
  for (auto& n : names) {
    n.resize(rd<uint32_t>());
    if (!n.empty() && fread(&n[0], 1, n.size(), stdin) != n.size()) return 2;
  }
  auto name_of = [&](uint32_t id) { return id < names.size() ? names[id] : std::string(); };

  RocprofLogger& rl = RocprofLogger::singleton();
  getGlobalContext().name_info = rocprofiler::sdk::get_callback_tracing_names();      /* RocprofLogger.cpp:346-347 */
  getGlobalContext().buff_name_info = rocprofiler::sdk::get_buffer_tracing_names();
  const uint32_t dom = ROCPROFILER_CALLBACK_TRACING_HIP_RUNTIME_API;
  for (const auto& r : rt) {
    switch (r.kind) {
      case KTJ_RT_KERNEL:
        rl.rows_.push_back(new rocprofKernelRow(r.id, dom, r.cid, r.pid, r.tid, r.begin, r.end, nullptr, nullptr, r.u.kernel.grid[0],
                                                r.u.kernel.grid[1], r.u.kernel.grid[2], r.u.kernel.workgroup[0], r.u.kernel.workgroup[1],
                                                r.u.kernel.workgroup[2], r.u.kernel.group_segment_size,
                                                reinterpret_cast<hipStream_t>(r.u.kernel.stream)));
        break;
      case KTJ_RT_COPY:
        rl.rows_.push_back(new rocprofCopyRow(r.id, dom, r.cid, r.pid, r.tid, r.begin, r.end, reinterpret_cast<const void*>(r.u.copy.src),
                                              reinterpret_cast<const void*>(r.u.copy.dst), r.u.copy.size,
                                              static_cast<hipMemcpyKind>(r.u.copy.copy_kind),
                                              reinterpret_cast<hipStream_t>(r.u.copy.stream)));
        break;
      case KTJ_RT_MALLOC:
        rl.rows_.push_back(new rocprofMallocRow(r.id, dom, r.cid, r.pid, r.tid, r.begin, r.end,
                                                reinterpret_cast<const void*>(r.u.malloc_.ptr), r.u.malloc_.size));
        break;
      default: rl.rows_.push_back(new rocprofRow(r.id, dom, r.cid, r.pid, r.tid, r.begin, r.end)); break;
    }
  }
  for (const auto& x : ext) rl.externalCorrelations_[RocLogger::CorrelationDomain::Domain0].emplace_back(x.correlation, x.external_id);
  for (const auto& x : user) rl.externalCorrelations_[RocLogger::CorrelationDomain::Domain1].emplace_back(x.correlation, x.external_id);

  RocprofActivityApi& api = RocprofActivityApi::singleton();
  api.activityMaskSnapshot_ = ~0u; /* every activity type was enabled when collection stopped */

  RocmActivityProfiler prof(api, /*cpuOnly=*/false);
  {
    auto cfg = std::make_unique<Config>();
    std::set<ActivityType> all;
    for (int t = 0; t < (int)ActivityType::ENUM_COUNT; ++t) all.insert(static_cast<ActivityType>(t));
    cfg->setSelectedActivityTypes(all);
    prof.derivedConfig_ = std::make_unique<ConfigDerivedState>(*cfg);
    prof.config_ = std::move(cfg);
  }
  prof.captureWindowStartTime_ = win_start;
  prof.captureWindowEndTime_ = win_end;
  prof.traceBuffers_ = std::make_unique<ActivityBuffers>();
  prof.acceptCpuTraces_ = true;

  if (!ops.empty()) {
    auto buf = std::make_unique<CpuTraceBuffer>();
    buf->span = TraceSpan(win_start, win_end, "PyTorch Profiler");
    buf->gpuOpCount = (int)dev.size();
    for (const auto& g : ops) {
      buf->emplace_activity(buf->span, static_cast<ActivityType>(g.type), name_of(g.name_id));
      GenericTraceActivity& a = *buf->activities.back();
      a.startTime = g.start_ns;
      a.endTime = g.end_ns;
      a.id = g.id;
      a.device = g.device;
      a.resource = (int32_t)g.resource;
      a.threadId = (int32_t)g.resource;
    }
    prof.transferCpuTrace(std::move(buf));
  }

  /* as late as possible: what the reference samples inside processActivities then differs from this
   * sample by the time the CPU ops take, not by the start-up of the runtime libraries */
  const int64_t my_offset = getTimeOffset();
  for (const auto& d : dev) {
    const uint32_t kind = d.domain == KTJ_DOM_MEMORY_COPY ? (uint32_t)ROCPROFILER_BUFFER_TRACING_MEMORY_COPY
                                                          : (uint32_t)ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH;
    auto* row = new rocprofAsyncRow(d.id, kind, kind, d.op, d.device, d.queue, d.begin - (uint64_t)my_offset, d.end - (uint64_t)my_offset,
                                    name_of(d.name_id));
    row->stream = d.stream;
    rl.rows_.push_back(row);
  }
  {
    ChromeTraceLogger logger(argv[1]);
    prof.processTraceInternal(logger);
  }
  printf("base_time=%" PRId64 "\nout_of_range=%" PRId64 "\nout_of_order=%" PRId64 "\n",
         (int64_t)ChromeTraceBaseTime::singleton().get(), (int64_t)prof.ecs_.out_of_range_events,
         (int64_t)prof.ecs_.gpu_and_cpu_op_out_of_order);
  fflush(stdout);
  _exit(0); /* no destructors: the loggers' would stop a tracing context that was never created */
}
