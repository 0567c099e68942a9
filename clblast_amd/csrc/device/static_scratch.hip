// =================================================================================================
// Scratch memory that exists without any allocation: one file-scope array in device memory, a copy of
// which every GPU the library runs on holds from the moment the code object is loaded until the process
// ends. It serves the one entry point that must not allocate (CLBlastSgemmNoAlloc: callers under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc). All calls on one GPU share that
// GPU's array, so calls that overlap on one GPU race; the array keeps the last call's contents.
// =================================================================================================
#include <hip/hip_runtime.h>

#include <mutex>

#include "clbh_device.h"

namespace {

constexpr size_t kStaticScratchBytes = size_t{64} << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// In host code `scratch` is a stand-in for the symbol, not an address: the address of each GPU's copy is asked for
// once, with that GPU current, and only these pointers are ever handed to kernels.
constexpr int kMaxDevices = 64;
std::mutex resolve_mutex;
void* device_pointer[kMaxDevices] = {};

}  // namespace

extern "C" {

size_t clbh_static_scratch_bytes(void) { return kStaticScratchBytes; }

int clbh_static_scratch(int device, void** pointer) {
  if (pointer == nullptr || device < 0 || device >= kMaxDevices) { return hipErrorInvalidValue; }
  std::lock_guard<std::mutex> lock(resolve_mutex);
  if (device_pointer[device] == nullptr) {
    int current = 0;
    auto status = hipGetDevice(&current);
    if (status != hipSuccess) { return static_cast<int>(status); }
    if (current != device) {
      status = hipSetDevice(device);
      if (status != hipSuccess) { return static_cast<int>(status); }
    }
    void* resolved = nullptr;
    status = hipGetSymbolAddress(&resolved, HIP_SYMBOL(scratch));
    if (current != device) {
      const auto restored = hipSetDevice(current);
      if (status == hipSuccess) { status = restored; }
    }
    if (status != hipSuccess) { return static_cast<int>(status); }
    if (resolved == nullptr) { return hipErrorInvalidSymbol; }
    device_pointer[device] = resolved;
  }
  *pointer = device_pointer[device];
  return 0;
}

}  // extern "C"
