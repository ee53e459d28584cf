/*
 * GpuChromeTraceLogger — a libkineto::ActivityLogger that hands the trace to the MI355X engine
 * (libktj.so, C ABI of include/ktj.h) instead of formatting it on the CPU.
 *
 * It implements the nine pure virtuals of libkineto/include/output_base.h:37-75 with the
 * behaviour of ChromeTraceLogger (libkineto/src/output_json.h:31-235, output_json.cpp):
 *   - the constructor opens "<traceFileName>.tmp" (output_json.cpp:485-505); with a bad sink
 *     every handler is a silent no-op and finalizeTrace logs one error (:1066-1070);
 *   - no exceptions, no return codes; one producer thread.
 * Activities are borrowed references, so every handler copies the fields it needs into packed
 * records before it returns; nothing of the caller's storage is kept.
 *
 * This file compiles inside the libkineto source tree (it includes libkineto headers) and links
 * against libktj.so only.  Registration, next to the built-in "file" protocol
 * (libkineto/src/ActivityProfilerController.cpp:108-129):
 *
 *   libkineto::api().registerLoggerFactory("gpujson", [](const std::string& url) {
 *     return std::unique_ptr<libkineto::ActivityLogger>(new ktj_shim::GpuChromeTraceLogger(url));
 *   });
 */
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "output_base.h"

#include "ktj.h"

namespace ktj_shim {

class GpuChromeTraceLogger : public libkineto::ActivityLogger {
 public:
  explicit GpuChromeTraceLogger(const std::string& traceFileName, int hipDevice = 0);
  ~GpuChromeTraceLogger() override;
  GpuChromeTraceLogger(const GpuChromeTraceLogger&) = delete;
  GpuChromeTraceLogger& operator=(const GpuChromeTraceLogger&) = delete;

  void handleDeviceInfo(const libkineto::DeviceInfo& info, int64_t time) override;
  void handleResourceInfo(const libkineto::ResourceInfo& info, int64_t time) override;
  void handleOverheadInfo(const OverheadInfo& info, int64_t time) override;
  void handleTraceSpan(const libkineto::TraceSpan& span) override;
  void handleActivity(const libkineto::ITraceActivity& activity) override;
  void handleGenericActivity(const libkineto::GenericTraceActivity& activity) override;
  /* Every activity of a buffering logger's replay loop (libkineto/src/output_membuf.h:91-107) in
   * one call, equivalent to handleActivity() on each in turn; the host-side packing of
   * GenericTraceActivity objects is spread over `threads` workers (0 = one per core). */
  void handleActivities(const std::vector<const libkineto::ITraceActivity*>& activities, unsigned threads = 0);
  void handleTraceStart(const std::unordered_map<std::string, std::string>& metadata,
                        const std::string& device_properties) override;
  void finalizeMemoryTrace(const std::string&, const libkineto::Config&) override;
  void finalizeTrace(const libkineto::Config& config, std::unique_ptr<libkineto::ActivityBuffers> buffers,
                     int64_t endTime) override;

  std::string traceFileName() const { return fileName_; }
  /* activities the engine could not take; every kind is taken at present, so this reads 0 */
  uint64_t unsupportedActivities() const { return unsupported_; }
  /* ktj status of the first failed engine call, 0 if none */
  int engineStatus() const { return status_; }

 protected:
  void finalizeTrace(int64_t endTime); /* output_json.h: protected finalizeTrace(int64_t) */

 private:
  struct Packed;
  static void pack(const libkineto::ITraceActivity& op, uint64_t origin, Packed& out);
  uint32_t intern(const std::string& s);
  void translate(Packed& p);
  uint64_t appendSlots(const Packed& p);
  ktj_generic_rec translated(const Packed& p, size_t i, uint64_t slotBase) const;
  void mergeInOrder(Packed& p);
  void submitRecords(const ktj_generic_rec* records, size_t count);
  void flushStrings();
  void flushRecords();
  bool ok() const { return engine_ != nullptr && status_ == 0; }
  void note(int rc, const char* what);
  void noteFirstActivity();

  ktj_engine* engine_ = nullptr;
  std::string fileName_;
  int status_ = 0;
  bool activitiesBegun_ = false;
  uint64_t unsupported_ = 0;
  uint32_t fragmentSchema_ = KTJ_NONE;
  uint32_t collectiveSchema_ = KTJ_NONE;         /* collective metadata only        */
  uint32_t collectiveFragmentSchema_ = KTJ_NONE; /* collective metadata + fragment  */

  /* strings not yet handed to the engine: blob + offsets, ids are consecutive from nextStringId_ */
  std::unordered_map<std::string, uint32_t> strings_;        /* activity and counter names */
  std::unordered_map<std::string, uint32_t> collectives_;    /* key: the 17 values, each followed by NUL */
  std::unordered_map<std::string, uint32_t> counterSchemas_; /* key: the fields' bytes */
  std::unique_ptr<Packed> staging_;                          /* packer of the single-activity calls */
  std::string pendingBlob_;
  std::vector<uint64_t> pendingOffsets_;
  uint32_t nextStringId_ = 0;
  uint32_t pendingFirstId_ = 0;

  std::vector<ktj_generic_rec> records_; /* packed, flushed in batches */
  std::vector<uint64_t> slots_;
  uint64_t nextSlot_ = 0;
};

}  // namespace ktj_shim
