// Time stamps at the phase boundaries of the long kernels, for the timelines that
// benchmarks/phase_timeline.py prints.  Only a library built with -DATK_TRACE
// (`python build.py --trace`, which writes libapprox_topk_hip_trace.so beside the
// product library) has them; without the macro every stamp is an empty statement
// and the product library holds no trace of this file.
//
// A stamp is the constant 100 MHz clock (s_memrealtime, the same on every CU), written
// to a buffer of kSlots words per workgroup.  The buffer is a device variable
// of the translation unit that includes this header, so every such unit that wants
// to be read names a reader of its own with ATK_TRACE_READER.  Launches of more than
// kGroups workgroups stamp their first kGroups only; a later launch of a traced kernel
// from the same unit overwrites the buffer.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#ifdef ATK_TRACE
namespace atk {
namespace trace {
constexpr int kSlots = 20;
constexpr int kGroups = 16384;
static __device__ uint64_t buf[(size_t)kGroups * kSlots];
// by the workgroup's first thread
__device__ __forceinline__ void stamp_group(int slot) {
  if (threadIdx.x == 0 && blockIdx.x < (unsigned)kGroups) buf[(size_t)blockIdx.x * kSlots + slot] = wall_clock64();
}
// by the first lane of the calling wave (wave-uniform slot)
__device__ __forceinline__ void stamp_wave(int slot) {
  if (threadIdx.x % 64 == 0 && blockIdx.x < (unsigned)kGroups) buf[(size_t)blockIdx.x * kSlots + slot] = wall_clock64();
}
}  // namespace trace
}  // namespace atk
#define ATK_TRACE_GROUP(slot) ::atk::trace::stamp_group(slot)
#define ATK_TRACE_WAVE(slot) ::atk::trace::stamp_wave(slot)
// int name(uint64_t* host, size_t bytes): copies the unit's buffer to the host (hipError_t as int)
#define ATK_TRACE_READER(name)                                                                  \
  extern "C" int name(uint64_t* host, size_t bytes) {                                          \
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(::atk::trace::buf), bytes);               \
  }
#else
#define ATK_TRACE_GROUP(slot) do {} while (0)
#define ATK_TRACE_WAVE(slot) do {} while (0)
#define ATK_TRACE_READER(name)
#endif
