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
 * stdin (binary, little endian):
 *   u64 n, n x ktj_device_rec          rows with domain KTJ_DOM_MEMSET (the ktj_memset_rec view)
 * stdout:
 *   cuda_version <CUDA_VERSION>
 *   memset idx=.. corr=.. type=.. dev=.. res=.. ts=.. dur=.. flowstart=.. flowid=.. flowtype=.. name=.. json=..
 */
#include <cinttypes>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "CuptiActivity.h"

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

}  // namespace

int main() {
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
