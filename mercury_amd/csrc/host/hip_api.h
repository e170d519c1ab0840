// The few HIP runtime calls the host core makes itself (pinned memory, one copy per step,
// events), looked up at run time in the HIP runtime the process already uses.  PyTorch brings
// a HIP runtime of its own; a process must talk to one runtime only (streams, events and
// pointers are that runtime's), so the host core does not link against one.
#pragma once

#include <hip/hip_runtime_api.h>

namespace mercury {

struct HipApi {
  hipError_t (*host_malloc)(void** ptr, size_t size, unsigned int flags) = nullptr;
  hipError_t (*host_free)(void* ptr) = nullptr;
  hipError_t (*memcpy_async)(void* dst, const void* src, size_t size, hipMemcpyKind kind,
                             hipStream_t stream) = nullptr;
  hipError_t (*event_create)(hipEvent_t* event, unsigned int flags) = nullptr;
  hipError_t (*event_record)(hipEvent_t event, hipStream_t stream) = nullptr;
  hipError_t (*event_synchronize)(hipEvent_t event) = nullptr;
  hipError_t (*event_destroy)(hipEvent_t event) = nullptr;
  const char* (*error_string)(hipError_t error) = nullptr;
};

// Throws KernelError when no HIP runtime is loaded in the process and none can be opened.
const HipApi& hip();

}  // namespace mercury
