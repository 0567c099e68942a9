// =================================================================================================
// Counters for kernels whose work-groups meet in memory (kernels/gemm_skinny_cols.hpp: the work-group that draws a
// strip's last ticket adds the partial sums of the others). The counters must be zero when such a kernel starts, and
// every kernel leaves them at zero, so they live in one file-scope array in device memory that is zero from the
// loading of the code object on: no launch has to clear anything. The array is cut into slots, one per (device,
// stream) pair that ever asked: launches on one stream are ordered and may share counters, launches on different
// streams may overlap and may not. A caller that gets no slot (more stream handles than slots, or the per-thread
// stream, whose one handle stands for a stream per host thread) clears counters of its own with a fill kernel instead.
// =================================================================================================
#include <hip/hip_runtime.h>

#include <map>
#include <mutex>
#include <utility>

#include "clbh_device.h"

namespace {

constexpr int kTicketSlots = 64;
static __device__ __align__(256) unsigned int ticket_slots[kTicketSlots * CLBH_TICKETS_PER_STREAM];

constexpr int kMaxDevices = 64;
std::mutex ticket_mutex;
unsigned int* device_base[kMaxDevices] = {};
std::map<std::pair<int, hipStream_t>, int> slot_of;
int slots_taken[kMaxDevices] = {};

}  // namespace

extern "C" int clbh_tickets(hipStream_t stream, unsigned int** pointer) {
  if (pointer == nullptr) { return hipErrorInvalidValue; }
  *pointer = nullptr;
  if (clbh_stream_is_alias(stream) != 0) { return hipErrorNotSupported; }
  int device = 0;
  auto status = clbh_stream_device(stream, &device);
  if (status != 0) { return status; }
  if (device < 0 || device >= kMaxDevices) { return hipErrorInvalidValue; }
  std::lock_guard<std::mutex> lock(ticket_mutex);
  if (device_base[device] == nullptr) {
    // (in host code the array's name stands for the symbol, not for an address: each GPU's copy is asked for once, with
    // that GPU current)
    int current = 0;
    auto hip_status = hipGetDevice(&current);
    if (hip_status != hipSuccess) { return static_cast<int>(hip_status); }
    if (current != device) {
      hip_status = hipSetDevice(device);
      if (hip_status != hipSuccess) { return static_cast<int>(hip_status); }
    }
    void* resolved = nullptr;
    hip_status = hipGetSymbolAddress(&resolved, HIP_SYMBOL(ticket_slots));
    if (current != device) {
      const auto restored = hipSetDevice(current);
      if (hip_status == hipSuccess) { hip_status = restored; }
    }
    if (hip_status != hipSuccess) { return static_cast<int>(hip_status); }
    if (resolved == nullptr) { return hipErrorInvalidSymbol; }
    device_base[device] = static_cast<unsigned int*>(resolved);
  }
  const auto key = std::make_pair(device, stream);
  auto found = slot_of.find(key);
  if (found == slot_of.end()) {
    if (slots_taken[device] >= kTicketSlots) { return hipErrorOutOfMemory; }
    found = slot_of.emplace(key, slots_taken[device]++).first;
  }
  *pointer = device_base[device] + static_cast<size_t>(found->second) * CLBH_TICKETS_PER_STREAM;
  return 0;
}
