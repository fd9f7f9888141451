// A fixed block of device memory that exists from the moment the library's code object is loaded
// on a device until the process ends, for callers that may not allocate (code under HIP graph
// capture, serving loops, harnesses that forbid hipMalloc).  One block per device, shared by
// every call on that device.
#pragma once

#include <cstddef>

namespace eh {

constexpr size_t kStaticScratchBytes = size_t{8} << 20;      // per device
constexpr size_t kStaticScratchAlign = 256;

// Device address of device `index`'s block; that device must be current.  The address is looked
// up once per device and kept.  Throws eh::Error when the runtime cannot resolve the symbol.
void* static_scratch_ptr(int index);

}  // namespace eh
