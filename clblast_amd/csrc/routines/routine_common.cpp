// =================================================================================================
// Error dispatch and matrix validation shared by the GEMM routines (see routine_common.hpp).
// =================================================================================================
#include "routines/routine_common.hpp"

#include <algorithm>
#include <cstdio>
#include <map>
#include <memory>
#include <mutex>
#include <utility>

namespace clblast {
// =================================================================================================

StatusCode DispatchException(const bool silent) {
  const char* message = nullptr;
  auto status = StatusCode::kUnknownError;
  try {
    throw;
  } catch (const BLASError& e) {
    status = e.status();  // argument errors stay silent
  } catch (const RuntimeErrorCode& e) {
    message = e.what();
    status = e.status();
  } catch (const DeviceError& e) {
    message = e.what();
    status = StatusCode::kUnknownError;
  } catch (const std::runtime_error& e) {
    message = e.what();
    status = StatusCode::kUnknownError;
  }
  // anything else propagates to the caller's catch-all (the C wrappers turn it into kUnexpectedError)
  if (message != nullptr && !silent) {
    fprintf(stderr, "CLBlast: %s\n", message);
  }
  return status;
}

BLASError SwappedOperands(const BLASError& error) {
  switch (error.status()) {
    case StatusCode::kInvalidMatrixA: return BLASError(StatusCode::kInvalidMatrixB, error.details());
    case StatusCode::kInvalidMatrixB: return BLASError(StatusCode::kInvalidMatrixA, error.details());
    case StatusCode::kInvalidLeadDimA: return BLASError(StatusCode::kInvalidLeadDimB, error.details());
    case StatusCode::kInvalidLeadDimB: return BLASError(StatusCode::kInvalidLeadDimA, error.details());
    case StatusCode::kInsufficientMemoryA: return BLASError(StatusCode::kInsufficientMemoryB, error.details());
    case StatusCode::kInsufficientMemoryB: return BLASError(StatusCode::kInsufficientMemoryA, error.details());
    default: return error;
  }
}

namespace {
// The buffer kept for one (device, stream). A call may hold several pieces of it at once (a routine with several
// temporaries, a GEMM called from inside such a routine): pieces are cut off its front in the order they are asked for
// and given back in the opposite order, as the scopes of the StreamScratch objects of one call nest. The mutex is held
// by the calling thread from its first piece to the return of its last one.
struct CachedScratch {
  void* pointer = nullptr;
  size_t bytes = 0;
  size_t used = 0;   // offset of the first free byte
  size_t live = 0;   // pieces handed out and not yet returned
  size_t demand = 0; // what a call would have needed while the buffer could not grow
  bool pinned = false;          // a captured graph holds the buffer's address: it is never freed or replaced again
  unsigned long long last_use = 0;
  std::recursive_mutex taken;
};
constexpr size_t kScratchAlignment = 256;
std::mutex scratch_cache_mutex;
std::map<std::pair<int, hipStream_t>, std::unique_ptr<CachedScratch>> scratch_cache;
unsigned long long scratch_clock = 0;

void FreeScratchBuffer(void* pointer) {
  // (hipFree waits for the device, which covers kernels of earlier calls that still use the buffer)
  const auto status = clbh_free(pointer);
  if (status != 0) { fprintf(stderr, "CLBlast: freeing a scratch buffer failed: %s\n", clbh_error_string(status)); }
}

// With the table full, the idle entry that was used least recently makes room (streams come and go in long-running
// programs). Called with scratch_cache_mutex held.
bool EvictIdleScratch() {
  auto victim = scratch_cache.end();
  for (auto entry = scratch_cache.begin(); entry != scratch_cache.end(); ++entry) {
    auto& cached = *entry->second;
    if (cached.pinned || !cached.taken.try_lock()) { continue; }
    const bool idle = (cached.live == 0);
    cached.taken.unlock();
    if (idle && (victim == scratch_cache.end() || cached.last_use < victim->second->last_use)) { victim = entry; }
  }
  if (victim == scratch_cache.end()) { return false; }
  if (victim->second->pointer != nullptr) { FreeScratchBuffer(victim->second->pointer); }
  scratch_cache.erase(victim);
  return true;
}

// A piece of `bytes` bytes of this stream's buffer (its entry then stays locked by this thread until the piece is
// returned), or nullptr: then the caller allocates on the stream.
CachedScratch* TakeCachedScratch(const size_t bytes, hipStream_t stream, size_t& offset) {
  auto device = 0;
  if (bytes == 0 || bytes > kCachedScratchBytes || clbh_stream_device(stream, &device) != 0) { return nullptr; }
  // hipStreamPerThread is one handle value for a different stream in every host thread: a buffer keyed by it would be
  // shared by streams that nothing orders against each other.
  if (clbh_stream_is_alias(stream) != 0) { return nullptr; }
  // While the stream is being captured into a graph nothing may be allocated or freed with the blocking calls, and the
  // address a captured kernel gets must stay valid for every later replay.
  auto capturing = 0;
  if (clbh_stream_capturing(stream, &capturing) != 0) { return nullptr; }
  CachedScratch* entry = nullptr;
  {
    std::lock_guard<std::mutex> lock(scratch_cache_mutex);
    const auto key = std::make_pair(device, stream);
    auto found = scratch_cache.find(key);
    if (found == scratch_cache.end()) {
      if (capturing != 0) { return nullptr; }  // no buffer in place: the captured call allocates on the stream
      if (scratch_cache.size() >= kCachedScratchStreams && !EvictIdleScratch()) { return nullptr; }
      found = scratch_cache.emplace(key, std::unique_ptr<CachedScratch>(new CachedScratch())).first;
    }
    entry = found->second.get();
    if (!entry->taken.try_lock()) { return nullptr; }  // another host thread is inside a call on this stream
    entry->last_use = ++scratch_clock;
  }
  offset = (entry->used + kScratchAlignment - 1) / kScratchAlignment * kScratchAlignment;
  if (offset + bytes > entry->bytes || (entry->live == 0 && entry->demand > entry->bytes && !entry->pinned && capturing == 0)) {
    // Too small: grow - in powers of two from 1 MiB, so that this happens a few times per stream at most - unless
    // pieces of the buffer are in use (then the size that would have done is remembered, and the next call's first
    // request grows the buffer to it), the stream is being captured, or a captured graph knows the buffer's address.
    auto wanted = size_t{1} << 20;
    while (wanted < std::max(offset + bytes, entry->demand)) { wanted *= 2; }
    if (wanted > kCachedScratchBytes) { wanted = kCachedScratchBytes; }
    if (entry->live > 0 || offset + bytes > wanted || entry->pinned || capturing != 0) {
      if (!entry->pinned) { entry->demand = std::max(entry->demand, std::min(offset + bytes, kCachedScratchBytes)); }
      entry->taken.unlock();
      return nullptr;
    }
    if (entry->pointer != nullptr) { FreeScratchBuffer(entry->pointer); }
    entry->pointer = nullptr;
    entry->bytes = 0;
    if (clbh_alloc(&entry->pointer, wanted) != 0) {
      entry->pointer = nullptr;
      entry->taken.unlock();
      return nullptr;
    }
    entry->bytes = wanted;
  }
  if (capturing != 0) { entry->pinned = true; }
  entry->used = offset + bytes;
  entry->live += 1;
  return entry;
}

void ReturnCachedScratch(CachedScratch* entry, const size_t offset, const size_t bytes) {
  entry->live -= 1;
  if (entry->live == 0) { entry->used = 0; }
  else if (entry->used == offset + bytes) { entry->used = offset; }  // the last piece taken: its space is free again
  entry->taken.unlock();
}
}  // namespace

StreamScratch::StreamScratch(const size_t bytes, hipStream_t stream, const char* what)
    : pointer_(nullptr), bytes_(bytes), stream_(stream), cached_(nullptr), cached_offset_(0) {
  if (auto* entry = TakeCachedScratch(bytes, stream, cached_offset_)) {
    cached_ = entry;
    pointer_ = static_cast<unsigned char*>(entry->pointer) + cached_offset_;
    return;
  }
  if (clbh_alloc_async(&pointer_, bytes, stream) != 0) {
    pointer_ = nullptr;
    throw RuntimeErrorCode(StatusCode::kTempBufferAllocFailure, what);
  }
}

StreamScratch::~StreamScratch() {
  if (cached_ != nullptr) { ReturnCachedScratch(static_cast<CachedScratch*>(cached_), cached_offset_, bytes_); }
  else if (pointer_ != nullptr) { clbh_free_async(pointer_, stream_); }
}

void ReleaseCachedScratch() {
  std::lock_guard<std::mutex> lock(scratch_cache_mutex);
  for (auto entry = scratch_cache.begin(); entry != scratch_cache.end();) {
    if (!entry->second->pinned && entry->second->taken.try_lock()) {
      const bool idle = (entry->second->live == 0);  // not in the hands of a running call (of this thread either)
      if (idle && entry->second->pointer != nullptr) { FreeScratchBuffer(entry->second->pointer); }
      entry->second->taken.unlock();
      if (idle) { entry = scratch_cache.erase(entry); continue; }
    }
    ++entry;
  }
}

StatusCode DispatchExceptionForC() {
  const char* message = nullptr;
  try {
    throw;
  } catch (const std::exception& e) {
    message = e.what();
  } catch (...) {
    message = "unknown exception";
  }
  fprintf(stderr, "CLBlast (unexpected): %s\n", message);
  return StatusCode::kUnexpectedError;
}

// =================================================================================================

template <typename T>
size_t Buffer<T>::GetSize() const {
  if (size_known_) { return known_bytes_; }
  auto bytes = size_t{0};
  if (pointer_ == nullptr || clbh_buffer_extent(pointer_, &bytes) != 0) {
    throw std::runtime_error("not a device allocation");
  }
  return bytes;
}

namespace {
template <typename T>
void TestMatrix(const size_t one, const size_t two, const Buffer<T>& buffer, const size_t offset, const size_t ld,
                const bool test_lead_dim, const StatusCode bad_ld, const StatusCode too_small,
                const StatusCode bad_buffer) {
  if (test_lead_dim && ld < one) {
    throw BLASError(bad_ld);
  }
  auto available = size_t{0};
  try {
    available = buffer.GetSize();
  } catch (const std::runtime_error& e) {
    throw BLASError(bad_buffer, e.what());
  }
  const auto required_size = (ld * (two - 1) + one + offset) * sizeof(T);
  if (available < required_size) {
    throw BLASError(too_small);
  }
}
}  // namespace

template <typename T>
void TestMatrixA(const size_t one, const size_t two, const Buffer<T>& buffer, const size_t offset, const size_t ld,
                 const bool test_lead_dim) {
  TestMatrix(one, two, buffer, offset, ld, test_lead_dim, StatusCode::kInvalidLeadDimA,
             StatusCode::kInsufficientMemoryA, StatusCode::kInvalidMatrixA);
}
template <typename T>
void TestMatrixB(const size_t one, const size_t two, const Buffer<T>& buffer, const size_t offset, const size_t ld,
                 const bool test_lead_dim) {
  TestMatrix(one, two, buffer, offset, ld, test_lead_dim, StatusCode::kInvalidLeadDimB,
             StatusCode::kInsufficientMemoryB, StatusCode::kInvalidMatrixB);
}
template <typename T>
void TestMatrixC(const size_t one, const size_t two, const Buffer<T>& buffer, const size_t offset, const size_t ld) {
  TestMatrix(one, two, buffer, offset, ld, true, StatusCode::kInvalidLeadDimC, StatusCode::kInsufficientMemoryC,
             StatusCode::kInvalidMatrixC);
}

#define CLBLAST_HIP_INSTANTIATE(T)                                                                            \
  template class Buffer<T>;                                                                                   \
  template void TestMatrixA<T>(const size_t, const size_t, const Buffer<T>&, const size_t, const size_t,      \
                               const bool);                                                                   \
  template void TestMatrixB<T>(const size_t, const size_t, const Buffer<T>&, const size_t, const size_t,      \
                               const bool);                                                                   \
  template void TestMatrixC<T>(const size_t, const size_t, const Buffer<T>&, const size_t, const size_t);
CLBLAST_HIP_INSTANTIATE(half)
CLBLAST_HIP_INSTANTIATE(float)
CLBLAST_HIP_INSTANTIATE(double)
CLBLAST_HIP_INSTANTIATE(float2)
CLBLAST_HIP_INSTANTIATE(double2)
#undef CLBLAST_HIP_INSTANTIATE

// =================================================================================================
}  // namespace clblast
