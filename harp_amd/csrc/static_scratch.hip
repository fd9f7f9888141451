// The library's only statically allocated device memory (see static_scratch.hpp).
#include <hip/hip_runtime.h>

#include <mutex>
#include <string>

#include "ast.hpp"
#include "static_scratch.hpp"

namespace {

// In host code this name is a stand-in for the symbol, not an address a kernel could use: host
// code only ever passes the pointer hipGetSymbolAddress returns for the current device.
static __device__ __align__(256) unsigned char scratch[eh::kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_mu;
struct Slot {
  void* ptr = nullptr;
  std::mutex turn;                // held while one call queues its launches on the block
  hipEvent_t last_use = nullptr;  // recorded behind the launches of the call that used the block last
  hipStream_t last_stream = nullptr;
  bool used = false;
};
Slot g_slot[kMaxDevices];

}  // namespace

namespace eh {

void* static_scratch_ptr(int index) {
  if (index < 0 || index >= kMaxDevices) throw Error("device index " + std::to_string(index) + " has no static scratch block");
  std::lock_guard<std::mutex> lk(g_mu);
  Slot& s = g_slot[index];
  if (!s.ptr) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      throw Error(std::string("hipGetSymbolAddress(static scratch): ") + hipGetErrorString(e) + " (hip error " +
                  std::to_string(static_cast<int>(e)) + ")");
    // the event that orders one call's use of the block behind the previous call's is made here,
    // once, so that the calls themselves create nothing
    hipEvent_t ev = nullptr;
    e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
    if (e != hipSuccess)
      throw Error(std::string("hipEventCreateWithFlags(static scratch): ") + hipGetErrorString(e));
    s.last_use = ev;
    s.ptr = p;
  }
  return s.ptr;
}

StaticScratchTurn::StaticScratchTurn(int index, void* stream) : index_(index), stream_(stream) {
  if (index < 0 || index >= kMaxDevices) throw Error("device index " + std::to_string(index) + " has no static scratch block");
  Slot& s = g_slot[index];
  s.turn.lock();
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  capturing_ = hipStreamIsCapturing(st, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone;
  // launches on one stream run in order anyway; another stream's must wait for the last use.
  // A capturing stream records no such wait: when and beside what a captured sequence is
  // replayed is in the caller's hands.
  if (!capturing_ && s.used && s.last_stream != st && s.last_use) {
    hipError_t e = hipStreamWaitEvent(st, s.last_use, 0);
    if (e != hipSuccess) {
      s.turn.unlock();
      throw Error(std::string("hipStreamWaitEvent(static scratch): ") + hipGetErrorString(e));
    }
  }
}

StaticScratchTurn::~StaticScratchTurn() {
  Slot& s = g_slot[index_];
  hipStream_t st = static_cast<hipStream_t>(stream_);
  if (!capturing_ && s.last_use && hipEventRecord(s.last_use, st) == hipSuccess) {
    s.last_stream = st;
    s.used = true;
  }
  s.turn.unlock();
}

}  // namespace eh
