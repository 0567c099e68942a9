// =================================================================================================
// Shared host-side pieces of the GEMM routines: the error convention, integer helpers, the non-owning
// device-buffer view and the argument-validation contract.
//
// Follows the behaviour of the reference's
//   src/utilities/clblast_exceptions.{hpp,cpp}   (BLASError / RuntimeErrorCode / DispatchException)
//   src/utilities/utilities.cpp:480-508          (GetRealArg, Ceil, CeilDiv, IsMultiple)
//   src/utilities/buffer_test.hpp:26-73,169-218  (TestMatrixA/B/C and their batched forms)
//   src/clpp11.hpp:650,763-768                   (non-owning Buffer<T> and GetSize)
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINE_COMMON_HPP_
#define CLBLAST_HIP_ROUTINE_COMMON_HPP_

#include <cstddef>
#include <stdexcept>
#include <string>
#include <vector>

#include "clbh_device.h"
#include "clblast_half.h"
#include "clblast_hip.h"

namespace clblast {
// =================================================================================================

// Invalid user arguments: mapped to their status code without any message (reference:
// clblast_exceptions.cpp:45-52).
class BLASError : public std::invalid_argument {
 public:
  explicit BLASError(const StatusCode status, const std::string& detail = std::string{})
      : std::invalid_argument("BLAS error: " + std::to_string(static_cast<int>(status)) +
                              (detail.empty() ? "" : " (" + detail + ")")),
        status_(status), details_(detail) {}
  StatusCode status() const { return status_; }
  const std::string& details() const { return details_; }

 private:
  StatusCode status_;
  std::string details_;
};

// Failures that are not the caller's fault: reported on stderr as "CLBlast: ..." and mapped to their
// status code (reference: clblast_exceptions.cpp:56-63).
class RuntimeErrorCode : public std::runtime_error {
 public:
  explicit RuntimeErrorCode(const StatusCode status, const std::string& detail = std::string{})
      : std::runtime_error("Run-time error: " + std::to_string(static_cast<int>(status)) +
                           (detail.empty() ? "" : " (" + detail + ")")),
        status_(status) {}
  StatusCode status() const { return status_; }

 private:
  StatusCode status_;
};

// A failing call of the device layer. The reference forwards the raw driver code
// (clblast_exceptions.cpp:54-56); raw HIP codes are positive and would read as success-like values to
// callers testing `status < 0`, so they all map to kUnknownError and the HIP text goes to stderr.
class DeviceError : public std::runtime_error {
 public:
  DeviceError(const int code, const std::string& where)
      : std::runtime_error("HIP error in " + where + ": " + std::to_string(code) + " (" +
                           clbh_error_string(code) + ")"),
        code_(code) {}
  int code() const { return code_; }

 private:
  int code_;
};

inline void CheckDevice(const int code, const char* where) {
  if (code != 0) {
    throw DeviceError(code, where);
  }
}

// To be called from inside a catch(...) block of an API function.
StatusCode DispatchException(const bool silent = false);
// Second line of defence of the C wrappers (reference: clblast_exceptions.cpp:101-114).
StatusCode DispatchExceptionForC();

// =================================================================================================

inline size_t CeilDiv(const size_t x, const size_t y) { return 1 + ((x - 1) / y); }
inline size_t Ceil(const size_t x, const size_t y) { return CeilDiv(x, y) * y; }
inline bool IsMultiple(const size_t a, const size_t b) { return (a % b) == 0; }

template <typename T>
constexpr Precision PrecisionValue();
template <>
constexpr Precision PrecisionValue<half>() { return Precision::kHalf; }
template <>
constexpr Precision PrecisionValue<float>() { return Precision::kSingle; }
template <>
constexpr Precision PrecisionValue<double>() { return Precision::kDouble; }

// The scalar as the kernels consume it: half bit patterns are widened to float on the host
// (reference: utilities.cpp:480-483), everything travels to the device layer as double.
template <typename T>
inline double ScalarToDouble(const T value) { return static_cast<double>(value); }
template <>
inline double ScalarToDouble<half>(const half value) { return static_cast<double>(HalfToFloat(value)); }

// Storage size in bytes of one element of precision T
template <typename T>
constexpr size_t ElementBytes() { return sizeof(T); }

// =================================================================================================

// The constants 0, 1 and -1 in the host type of a precision (fp16: the binary16 bit patterns)
template <typename T> inline T ConstantZero() { return T(0); }
template <typename T> inline T ConstantOne() { return T(1); }
template <typename T> inline T ConstantNegOne() { return T(-1); }
template <> inline half ConstantZero<half>() { return 0x0000; }
template <> inline half ConstantOne<half>() { return 0x3C00; }
template <> inline half ConstantNegOne<half>() { return 0xBC00; }

// Non-owning view of a caller's device allocation (reference: Buffer<T>(cl_mem), clpp11.hpp:650).
template <typename T>
class Buffer {
 public:
  explicit Buffer(const void* pointer) : pointer_(pointer), known_bytes_(0), size_known_(false) {}
  // for memory the library allocated itself (the driver is not asked about it)
  Buffer(const void* pointer, const size_t bytes) : pointer_(pointer), known_bytes_(bytes), size_known_(true) {}
  const void* operator()() const { return pointer_; }
  // Bytes addressable from the pointer to the end of its allocation. Throws std::runtime_error if
  // the pointer is not device memory, which the matrix tests turn into kInvalidMatrix{A,B,C}.
  size_t GetSize() const;

 private:
  const void* pointer_;
  size_t known_bytes_;
  bool size_known_;
};

// The error of a GEMM whose A and B were the caller's B and A, in the caller's terms (reference:
// src/routines/level3/xsymm.cpp:92-109, xtrmm.cpp:110-127).
BLASError SwappedOperands(const BLASError& error);

// Scratch memory of one call, valid for kernels enqueued on `stream` while the object lives. Requests are served from a
// buffer of up to kCachedScratchBytes that the library keeps per (device, stream) - stream order makes its reuse by the
// next call on that stream safe, and nothing is allocated or freed on the way (a stream-ordered free costs about 8 us of
// host time, more than many a small GEMM). The objects of one call share the buffer as a stack: they are expected to be
// destroyed in the opposite order of their construction (anything else only delays the reuse of their space). Requests
// that do not fit, requests while another host thread is inside a call on the same stream, and streams beyond
// kCachedScratchStreams get stream-ordered memory that is freed on the stream when the object goes out of scope, also
// when an error unwinds the call. ReleaseCachedScratch (ClearCache calls it) frees the kept buffers; the caller must
// have synchronised.
constexpr size_t kCachedScratchBytes = size_t{16} << 20;
constexpr size_t kCachedScratchStreams = 16;
class StreamScratch {
 public:
  StreamScratch(const size_t bytes, hipStream_t stream, const char* what);
  ~StreamScratch();
  StreamScratch(const StreamScratch&) = delete;
  StreamScratch& operator=(const StreamScratch&) = delete;
  void* get() const { return pointer_; }
  size_t bytes() const { return bytes_; }

 private:
  void* pointer_;
  size_t bytes_;
  hipStream_t stream_;
  void* cached_;          // the cache entry this object holds a piece of, or nullptr for stream-ordered memory
  size_t cached_offset_;  // where in the entry's buffer the piece starts
};
void ReleaseCachedScratch();

// Argument-validation contract; check order: leading dimension first, then the buffer size.
template <typename T>
void TestMatrixA(const size_t one, const size_t two, const Buffer<T>& buffer, const size_t offset, const size_t ld,
                 const bool test_lead_dim = true);
template <typename T>
void TestMatrixB(const size_t one, const size_t two, const Buffer<T>& buffer, const size_t offset, const size_t ld,
                 const bool test_lead_dim = true);
template <typename T>
void TestMatrixC(const size_t one, const size_t two, const Buffer<T>& buffer, const size_t offset, const size_t ld);

// =================================================================================================
}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINE_COMMON_HPP_
