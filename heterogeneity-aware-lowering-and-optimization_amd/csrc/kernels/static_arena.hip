// Statically allocated device scratch for the entry point that must not
// allocate (odla_hip_ExecuteComputationStatic): the temporaries of a plan - what
// an ordinary context keeps in the arena it allocates when it is created - live
// in one file-scope device array instead.  Every GPU the library runs on holds
// its own copy of the array, at its own address, from the moment the code
// object is loaded there until the process ends.
//
// In host code the array's name is only a handle for the symbol lookup below,
// never a device address: everything that touches the memory (kernel
// arguments, copies) uses the pointer that hipGetSymbolAddress returned for the
// device at hand.
#include <hip/hip_runtime.h>

#include <mutex>

#include "kernels.h"

namespace ohip {

static __device__ __align__(256) unsigned char scratch[kStaticArenaBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_mu;
void* g_ptr[kMaxDevices] = {nullptr};
}  // namespace

// Address of the calling thread's current device's copy of the array.  The
// first call on a device looks the symbol up (with that device current) and
// keeps the answer; later calls only read the table.
hipError_t static_arena(void** ptr, size_t* bytes) {
  if (ptr == nullptr) return hipErrorInvalidValue;
  *ptr = nullptr;
  if (bytes != nullptr) *bytes = kStaticArenaBytes;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (p == nullptr) return hipErrorInvalidSymbol;
    g_ptr[dev] = p;
  }
  *ptr = g_ptr[dev];
  return hipSuccess;
}

}  // namespace ohip
