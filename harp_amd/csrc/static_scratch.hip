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
void* g_ptr[kMaxDevices] = {};

}  // namespace

namespace eh {

void* static_scratch_ptr(int index) {
  if (index < 0 || index >= kMaxDevices) throw Error("device index " + std::to_string(index) + " has no static scratch block");
  std::lock_guard<std::mutex> lk(g_mu);
  if (!g_ptr[index]) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      throw Error(std::string("hipGetSymbolAddress(static scratch): ") + hipGetErrorString(e) + " (hip error " +
                  std::to_string(static_cast<int>(e)) + ")");
    g_ptr[index] = p;
  }
  return g_ptr[index];
}

}  // namespace eh
