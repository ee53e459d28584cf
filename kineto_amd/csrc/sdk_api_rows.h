/*
 * sdk_api_rows.h — a rocprofiler-sdk HIP runtime API callback record as one packed runtime row.
 *
 * Replaces the row construction of RocprofLogger::api_callback (libkineto/src/RocprofLogger.cpp:
 * 561-679): which operations give a rocprofKernelRow, rocprofCopyRow, rocprofMallocRow or plain
 * rocprofRow (isKernelApi / isCopyApi / isMallocApi, :165-245) and which call arguments land in
 * which field (extract_kernel_args :84-143, extract_copy_args :47-82, extract_malloc_args :145-163).
 * The reference walks the arguments by name through the SDK's stringifying iterator, once per
 * call; here the same arguments are read straight from the SDK's argument union
 * (rocprofiler-sdk/hip/api_args.h), whose members carry those names, with no iteration and no
 * allocation.  An argument is looked up by its member name and read with the width the
 * reference reads it with, whatever the member's declared type: that keeps the reference's
 * behaviour where the two differ (`sharedMemBytes` is read as 32 bits also where it is a size_t;
 * hipLaunchCooperativeKernel names its block dimensions `blockDimX`, a dim3, of which the
 * reference takes the first word as x and nothing else; its `gridDim` has no counterpart in the
 * reference's list and is not read).
 *
 * Host code only (no HIP call), header-only so that the engine and the CPU-side tests share it.
 */
#ifndef KTJ_SDK_API_ROWS_H_
#define KTJ_SDK_API_ROWS_H_

#include <rocprofiler-sdk/callback_tracing.h>
#include <rocprofiler-sdk/hip/api_args.h>
#include <rocprofiler-sdk/hip/runtime_api_id.h>

#include <cstring>
#include <type_traits>
#include <utility>

#include "../../include/ktj.h"

namespace ktj {
namespace sdk_api {

/* address of member `name` of an argument struct, or null where the struct has no such member */
#define KTJ_SDK_ARG(name)                                                                          \
  template <class T, class = void> struct has_##name : std::false_type {};                         \
  template <class T> struct has_##name<T, std::void_t<decltype(std::declval<const T&>().name)>> : std::true_type {}; \
  template <class T> inline const void* arg_##name(const T& a) {                                   \
    if constexpr (has_##name<T>::value) return &a.name; else { (void)a; return nullptr; }          \
  }
KTJ_SDK_ARG(stream) KTJ_SDK_ARG(numBlocks) KTJ_SDK_ARG(dimBlocks) KTJ_SDK_ARG(sharedMemBytes)
KTJ_SDK_ARG(gridDimX) KTJ_SDK_ARG(gridDimY) KTJ_SDK_ARG(gridDimZ)
KTJ_SDK_ARG(blockDimX) KTJ_SDK_ARG(blockDimY) KTJ_SDK_ARG(blockDimZ)
KTJ_SDK_ARG(globalWorkSizeX) KTJ_SDK_ARG(globalWorkSizeY) KTJ_SDK_ARG(globalWorkSizeZ)
KTJ_SDK_ARG(localWorkSizeX) KTJ_SDK_ARG(localWorkSizeY) KTJ_SDK_ARG(localWorkSizeZ)
KTJ_SDK_ARG(dst) KTJ_SDK_ARG(src) KTJ_SDK_ARG(sizeBytes) KTJ_SDK_ARG(kind)
KTJ_SDK_ARG(ptr) KTJ_SDK_ARG(size)
#undef KTJ_SDK_ARG

template <class V> inline bool read_arg(const void* p, V* out) {
  if (!p) return false;
  std::memcpy(out, p, sizeof(V));
  return true;
}

/* extract_kernel_args (RocprofLogger.cpp:84-143).  The reference's `workgroupSize` (numBlocks,
 * gridDim?, globalWorkSize?) goes to the row's grid and its `gridSize` (dimBlocks, blockDim?,
 * localWorkSize?) to the row's workgroup (rocprofKernelRow's constructor, :583-600). */
template <class T> inline void kernel_args(const T& a, ktj_runtime_rec* r) {
  uint64_t stream = 0;
  if (read_arg(arg_stream(a), &stream)) r->u.kernel.stream = stream;
  uint32_t d3[3];
  if (read_arg(arg_numBlocks(a), &d3)) for (int k = 0; k < 3; ++k) r->u.kernel.grid[k] = d3[k];
  if (read_arg(arg_dimBlocks(a), &d3)) for (int k = 0; k < 3; ++k) r->u.kernel.workgroup[k] = d3[k];
  uint32_t v;
  if (read_arg(arg_sharedMemBytes(a), &v)) r->u.kernel.group_segment_size = v;
  if (read_arg(arg_gridDimX(a), &v)) r->u.kernel.grid[0] = v;
  if (read_arg(arg_gridDimY(a), &v)) r->u.kernel.grid[1] = v;
  if (read_arg(arg_gridDimZ(a), &v)) r->u.kernel.grid[2] = v;
  if (read_arg(arg_blockDimX(a), &v)) r->u.kernel.workgroup[0] = v;
  if (read_arg(arg_blockDimY(a), &v)) r->u.kernel.workgroup[1] = v;
  if (read_arg(arg_blockDimZ(a), &v)) r->u.kernel.workgroup[2] = v;
  if (read_arg(arg_globalWorkSizeX(a), &v)) r->u.kernel.grid[0] = v;
  if (read_arg(arg_globalWorkSizeY(a), &v)) r->u.kernel.grid[1] = v;
  if (read_arg(arg_globalWorkSizeZ(a), &v)) r->u.kernel.grid[2] = v;
  if (read_arg(arg_localWorkSizeX(a), &v)) r->u.kernel.workgroup[0] = v;
  if (read_arg(arg_localWorkSizeY(a), &v)) r->u.kernel.workgroup[1] = v;
  if (read_arg(arg_localWorkSizeZ(a), &v)) r->u.kernel.workgroup[2] = v;
}
/* extract_copy_args (RocprofLogger.cpp:47-82).  The reference keeps, for dst and src, the address
 * of the text the SDK renders the argument to, which is gone when the callback returns; the row
 * here holds the argument's value, which is what that text says. */
template <class T> inline void copy_args(const T& a, ktj_runtime_rec* r) {
  uint64_t v;
  if (read_arg(arg_dst(a), &v)) r->u.copy.dst = v;
  if (read_arg(arg_src(a), &v)) r->u.copy.src = v;
  if (read_arg(arg_sizeBytes(a), &v)) r->u.copy.size = v;
  uint32_t kind;
  if (read_arg(arg_kind(a), &kind)) r->u.copy.copy_kind = kind;
  if (read_arg(arg_stream(a), &v)) r->u.copy.stream = v;
}
/* extract_malloc_args (RocprofLogger.cpp:145-163); `ptr` as for dst and src above */
template <class T> inline void malloc_args(const T& a, ktj_runtime_rec* r) {
  uint64_t v;
  if (read_arg(arg_ptr(a), &v)) r->u.malloc_.ptr = v;
  if (read_arg(arg_size(a), &v)) r->u.malloc_.size = v;
}

/* isKernelApi (RocprofLogger.cpp:212-232), isCopyApi (:167-209), isMallocApi (:235-245) */
#define KTJ_SDK_KERNEL_APIS(X)                                                                     \
  X(hipExtLaunchKernel) X(hipExtLaunchMultiKernelMultiDevice) X(hipLaunchCooperativeKernel)        \
  X(hipLaunchCooperativeKernelMultiDevice) X(hipLaunchKernel) X(hipModuleLaunchCooperativeKernel)  \
  X(hipModuleLaunchCooperativeKernelMultiDevice) X(hipModuleLaunchKernel) X(hipExtModuleLaunchKernel) \
  X(hipHccModuleLaunchKernel) X(hipLaunchCooperativeKernel_spt) X(hipLaunchKernel_spt)
#define KTJ_SDK_COPY_APIS(X)                                                                       \
  X(hipMemcpy) X(hipMemcpy2D) X(hipMemcpy2DAsync) X(hipMemcpy2DFromArray) X(hipMemcpy2DFromArrayAsync) \
  X(hipMemcpy2DToArray) X(hipMemcpy2DToArrayAsync) X(hipMemcpy3D) X(hipMemcpy3DAsync) X(hipMemcpyAsync) \
  X(hipMemcpyAtoH) X(hipMemcpyDtoD) X(hipMemcpyDtoDAsync) X(hipMemcpyDtoH) X(hipMemcpyDtoHAsync)    \
  X(hipMemcpyFromArray) X(hipMemcpyFromSymbol) X(hipMemcpyFromSymbolAsync) X(hipMemcpyHtoA)        \
  X(hipMemcpyHtoD) X(hipMemcpyHtoDAsync) X(hipMemcpyParam2D) X(hipMemcpyParam2DAsync) X(hipMemcpyPeer) \
  X(hipMemcpyPeerAsync) X(hipMemcpyToArray) X(hipMemcpyToSymbol) X(hipMemcpyToSymbolAsync)         \
  X(hipMemcpyWithStream)
#define KTJ_SDK_MALLOC_APIS(X) X(hipMalloc) X(hipFree)
/* RuntimeActivity<T>::flowStart (libkineto/src/RocprofActivity_inl.h:185-200) */
#define KTJ_SDK_FLOW_START_APIS(X)                                                                 \
  X(hipLaunchKernel) X(hipExtLaunchKernel) X(hipLaunchCooperativeKernel) X(hipHccModuleLaunchKernel) \
  X(hipModuleLaunchKernel) X(hipExtModuleLaunchKernel) X(hipMalloc) X(hipFree) X(hipMemcpy)        \
  X(hipMemcpyAsync) X(hipMemcpyWithStream) X(hipGraphLaunch)

/* whether a runtime row of this operation starts a flow to its device rows: what a caller puts into
 * ktj_set_api_table's flow_start_cids for a trace of rocprofiler-sdk HIP runtime API records */
inline bool is_flow_start(uint32_t operation) {
  switch (operation) {
#define X(op) case ROCPROFILER_HIP_RUNTIME_API_ID_##op:
    KTJ_SDK_FLOW_START_APIS(X)
#undef X
      return true;
    default: return false;
  }
}

/* Fills *out (zeroed first) from one HIP runtime API call: operation id, the SDK's internal
 * correlation id, the call's arguments, its begin/end on the caller's clock and the calling
 * process and thread (RocprofLogger.cpp:572-659).  Returns the row kind (KTJ_RT_*). */
inline uint32_t runtime_row(uint32_t operation, uint64_t correlation_id, const rocprofiler_hip_api_args_t& args,
                            uint64_t begin, uint64_t end, uint32_t pid, uint32_t tid, ktj_runtime_rec* out) {
  std::memset(out, 0, sizeof *out);
  out->id = correlation_id;
  out->begin = begin;
  out->end = end;
  out->cid = operation;
  out->pid = pid;
  out->tid = tid;
  out->kind = KTJ_RT_DEFAULT;
  switch (operation) {
#define X(op)                                                                                     \
    case ROCPROFILER_HIP_RUNTIME_API_ID_##op:                                                      \
      out->kind = KTJ_RT_KERNEL;                                                                   \
      out->u.kernel.kernel_name_id = KTJ_NONE; /* no function pointer on this path (:590-591) */     \
      kernel_args(args.op, out);                                                                   \
      break;
    KTJ_SDK_KERNEL_APIS(X)
#undef X
#define X(op)                                                                                     \
    case ROCPROFILER_HIP_RUNTIME_API_ID_##op:                                                      \
      out->kind = KTJ_RT_COPY;                                                                     \
      out->u.copy.copy_kind = static_cast<uint32_t>(hipMemcpyDefault); /* where the call has no `kind` (:53) */ \
      copy_args(args.op, out);                                                                     \
      break;
    KTJ_SDK_COPY_APIS(X)
#undef X
#define X(op)                                                                                     \
    case ROCPROFILER_HIP_RUNTIME_API_ID_##op:                                                      \
      out->kind = KTJ_RT_MALLOC;                                                                   \
      malloc_args(args.op, out);                                                                   \
      break;
    KTJ_SDK_MALLOC_APIS(X)
#undef X
    default: break;
  }
  return out->kind;
}

}  // namespace sdk_api
}  // namespace ktj
#endif
