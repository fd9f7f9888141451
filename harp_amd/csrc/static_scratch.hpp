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

// One call's turn on device `index`'s block.  Several device handles may exist for one GPU, each
// with a stream of its own, and all of them share the block: while a turn lives no other call
// queues launches that use it, `stream` (a hipStream_t) is made to wait for the launches of the
// previous turn when those went to another stream, and the destructor records this turn's end
// behind everything `stream` holds by then.  Nothing is created or allocated.  On a stream that
// is being captured neither the wait nor the record is issued.
class StaticScratchTurn {
 public:
  StaticScratchTurn(int index, void* stream);
  ~StaticScratchTurn();
  StaticScratchTurn(const StaticScratchTurn&) = delete;
  StaticScratchTurn& operator=(const StaticScratchTurn&) = delete;

 private:
  int index_;
  void* stream_;
  bool capturing_ = false;
};

}  // namespace eh
