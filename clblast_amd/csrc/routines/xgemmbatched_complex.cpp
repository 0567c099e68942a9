// =================================================================================================
// XgemmComplexBatched<R> host logic (see xgemmbatched_complex.hpp).
// =================================================================================================
#include "routines/xgemmbatched_complex.hpp"

#include <algorithm>
#include <climits>
#include <cstring>
#include <memory>

namespace clblast {
// =================================================================================================

namespace {
constexpr size_t kMaxRealExtent = static_cast<size_t>(INT_MAX) / 2;
constexpr size_t kSmallExtent = 384;

// One operand of the canonical column-major problems C' = A' * B' (for a row-major call the operands change places)
struct BatchedOperand {
  const void* pointer;
  size_t offset, ld, stride;
  const std::vector<size_t>* offsets;  // per-batch offsets (GemmBatched) or nullptr (strided)
  bool kcontig, conjugate;
};

// The kernel that works on the interleaved data itself reads and writes every matrix once; the real form moves the
// first operand three more times but runs on the large-tile real kernels. The former wins up to about 400 rows and
// columns (256 x 256^3: 321 against 365 us, 64 x 512^3: 589 us both ways).
// A tile forced through OverrideParameters asks for the real kernels.
bool UseSmallKernel(const size_t rows, const size_t columns, const size_t k, const size_t batch_count,
                    const Precision precision) {
  if (rows > kSmallExtent || columns > kSmallExtent || ForcedTileVariant(precision) != 0) { return false; }
  // a few work-groups walking a long k alone are slower than the real kernels, which split such a k
  const auto groups = CeilDiv(rows, size_t{64}) * CeilDiv(columns, size_t{64}) * batch_count;
  return groups >= 512 || k <= 64;
}

clbh_complex_small_operand SmallOperand(const BatchedOperand& operand, const long long* device_offsets) {
  return clbh_complex_small_operand{operand.pointer, static_cast<long long>(operand.offset),
                                    static_cast<long long>(operand.ld), static_cast<long long>(operand.stride),
                                    device_offsets, operand.kcontig ? 1 : 0, operand.conjugate ? 1 : 0};
}
}  // namespace

template <typename R>
XgemmComplexBatched<R>::XgemmComplexBatched(hipStream_t* queue, hipEvent_t* event)
    : GemmRoutineBase(queue, event, PrecisionValue<R>()), queue_(queue), event_(event) {}

// =================================================================================================

template <typename R>
void XgemmComplexBatched<R>::DoGemmStridedBatched(
    const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m, const size_t n,
    const size_t k, const Complex alpha, const Buffer<Complex>& a_buffer, const size_t a_offset, const size_t a_ld,
    const size_t a_stride, const Buffer<Complex>& b_buffer, const size_t b_offset, const size_t b_ld,
    const size_t b_stride, const Complex beta, const Buffer<Complex>& c_buffer, const size_t c_offset, const size_t c_ld,
    const size_t c_stride, const size_t batch_count) {
  // reference: xgemmstridedbatched.cpp:68-75, then the last matrix of the batch decides (buffer_test.hpp:195-218)
  if (batch_count < 1) { throw BLASError(StatusCode::kInvalidBatchCount); }
  if (c_stride == 0) { throw BLASError(StatusCode::kInvalidDimension); }
  if (batch_count > static_cast<size_t>(INT_MAX)) {
    throw BLASError(StatusCode::kInvalidBatchCount, "batch count exceeds 2^31-1");
  }
  const auto shape = Xgemm<R>::ProcessArguments(layout, a_transpose, b_transpose, m, n, k);
  TestMatrixA(shape.a_one, shape.a_two, a_buffer, a_offset + (batch_count - 1) * a_stride, a_ld);
  TestMatrixB(shape.b_one, shape.b_two, b_buffer, b_offset + (batch_count - 1) * b_stride, b_ld);
  TestMatrixC(shape.c_one, shape.c_two, c_buffer, c_offset + (batch_count - 1) * c_stride, c_ld);
  if (m > kMaxRealExtent || n > kMaxRealExtent || k > kMaxRealExtent) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^30");
  }

  const bool col_major = (layout == Layout::kColMajor);
  const auto first = BatchedOperand{a_buffer(), a_offset, a_ld, a_stride, nullptr, shape.a_rotated,
                                    a_transpose == Transpose::kConjugate};
  const auto second = BatchedOperand{b_buffer(), b_offset, b_ld, b_stride, nullptr, !shape.b_rotated,
                                     b_transpose == Transpose::kConjugate};
  const auto left = col_major ? first : second;
  const auto right = col_major ? second : first;
  const auto rows = col_major ? m : n, columns = col_major ? n : m;
  const auto precision = static_cast<int>(8 * sizeof(R));
  const auto batches = static_cast<int>(batch_count);

  if (UseSmallKernel(rows, columns, k, batch_count, PrecisionValue<R>())) {
    auto desc = clbh_complex_small_desc{};
    desc.precision = precision;
    desc.rows = static_cast<int>(rows);
    desc.columns = static_cast<int>(columns);
    desc.k = static_cast<int>(k);
    desc.batch_count = batches;
    desc.left = SmallOperand(left, nullptr);
    desc.right = SmallOperand(right, nullptr);
    desc.c = clbh_complex_small_operand{c_buffer(), static_cast<long long>(c_offset), static_cast<long long>(c_ld),
                                        static_cast<long long>(c_stride), nullptr, 0, 0};
    desc.alpha_re = static_cast<double>(alpha.real());
    desc.alpha_im = static_cast<double>(alpha.imag());
    desc.beta_re = static_cast<double>(beta.real());
    desc.beta_im = static_cast<double>(beta.imag());
    CheckDevice(clbh_complex_gemm_small_batched(&desc, stream()), "clbh_complex_gemm_small_batched");
    Finish();  // records the caller's event
    return;
  }

  // left operands -> real 2 rows x 2k each, densely behind one another
  const auto expanded_elements = 4 * rows * k;
  const auto expanded_bytes = batch_count * expanded_elements * sizeof(R);
  const StreamScratch expanded(expanded_bytes, stream(), "real form of the first operands");
  auto walk = clbh_complex_batches{batches, static_cast<long long>(left.stride), nullptr,
                                   static_cast<long long>(expanded_elements), nullptr};
  CheckDevice(clbh_complex_expand_batched(precision, static_cast<int>(rows), static_cast<int>(k), left.kcontig ? 1 : 0,
                                          left.conjugate ? 1 : 0, right.conjugate ? 1 : 0,
                                          static_cast<double>(alpha.real()), static_cast<double>(alpha.imag()),
                                          left.pointer, static_cast<long long>(left.offset),
                                          static_cast<long long>(left.ld), expanded.get(), &walk, stream()),
              "clbh_complex_expand_batched");
  // right operands: in place when their k index is contiguous, else transposed first
  const void* right_pointer = right.pointer;
  auto right_offset = right.offset, right_ld = right.ld, right_stride = right.stride;
  auto right_bytes = size_t{0};
  std::unique_ptr<StreamScratch> transposed;
  if (!right.kcontig) {
    // a stride of zero shares one matrix between all products: transpose it once
    const auto copies = (right.stride == 0) ? size_t{1} : batch_count;
    right_bytes = copies * 2 * k * columns * sizeof(R);
    transposed.reset(new StreamScratch(right_bytes, stream(), "transposed second operands"));
    walk = clbh_complex_batches{static_cast<int>(copies), static_cast<long long>(right.stride), nullptr,
                                static_cast<long long>(k * columns), nullptr};
    CheckDevice(clbh_complex_transpose_batched(precision, static_cast<int>(k), static_cast<int>(columns), right.pointer,
                                               static_cast<long long>(right.offset), static_cast<long long>(right.ld),
                                               transposed->get(), &walk, stream()),
                "clbh_complex_transpose_batched");
    right_pointer = transposed->get();
    right_offset = 0;
    right_ld = k;
    right_stride = (right.stride == 0) ? 0 : k * columns;
  }
  auto real_beta = beta.real();
  if (beta.imag() != R(0)) {
    walk = clbh_complex_batches{batches, static_cast<long long>(c_stride), nullptr, 0, nullptr};
    CheckDevice(clbh_complex_scale_batched(precision, static_cast<int>(rows), static_cast<int>(columns), 0,
                                           static_cast<double>(beta.real()), static_cast<double>(beta.imag()),
                                           const_cast<void*>(c_buffer()), static_cast<long long>(c_offset),
                                           static_cast<long long>(c_ld), &walk, stream()),
                "clbh_complex_scale_batched");
    real_beta = R(1);
  }
  const auto real_left = Buffer<R>(expanded.get(), expanded_bytes);
  const auto real_right = transposed ? Buffer<R>(right_pointer, right_bytes) : Buffer<R>(right_pointer);
  auto real_routine = XgemmStridedBatched<R>(queue_, event_);  // records the caller's event after its launch
  real_routine.DoGemmStridedBatched(Layout::kColMajor, Transpose::kNo, Transpose::kNo, 2 * rows, columns, 2 * k, R(1),
                                    real_left, 0, 2 * rows, expanded_elements, real_right, 2 * right_offset,
                                    2 * right_ld, 2 * right_stride, real_beta, Buffer<R>(c_buffer()), 2 * c_offset,
                                    2 * c_ld, 2 * c_stride, batch_count);
}

// =================================================================================================

template <typename R>
void XgemmComplexBatched<R>::DoGemmBatched(const Layout layout, const Transpose a_transpose,
                                           const Transpose b_transpose, const size_t m, const size_t n, const size_t k,
                                           const std::vector<Complex>& alphas, const Buffer<Complex>& a_buffer,
                                           const std::vector<size_t>& a_offsets, const size_t a_ld,
                                           const Buffer<Complex>& b_buffer, const std::vector<size_t>& b_offsets,
                                           const size_t b_ld, const std::vector<Complex>& betas,
                                           const Buffer<Complex>& c_buffer, const std::vector<size_t>& c_offsets,
                                           const size_t c_ld, const size_t batch_count) {
  // reference: xgemmbatched.cpp:66-69, then the largest offset decides and the leading dimensions of A and B are not
  // tested (xgemmbatched.cpp:82-84, buffer_test.hpp:169-190)
  if ((batch_count < 1) || (alphas.size() != batch_count) || (betas.size() != batch_count) ||
      (a_offsets.size() != batch_count) || (b_offsets.size() != batch_count) || (c_offsets.size() != batch_count)) {
    throw BLASError(StatusCode::kInvalidBatchCount);
  }
  if (batch_count > static_cast<size_t>(INT_MAX)) {
    throw BLASError(StatusCode::kInvalidBatchCount, "batch count exceeds 2^31-1");
  }
  const auto shape = Xgemm<R>::ProcessArguments(layout, a_transpose, b_transpose, m, n, k);
  TestMatrixA(shape.a_one, shape.a_two, a_buffer, *std::max_element(a_offsets.begin(), a_offsets.end()), a_ld, false);
  TestMatrixB(shape.b_one, shape.b_two, b_buffer, *std::max_element(b_offsets.begin(), b_offsets.end()), b_ld, false);
  TestMatrixC(shape.c_one, shape.c_two, c_buffer, *std::max_element(c_offsets.begin(), c_offsets.end()), c_ld);
  if (m > kMaxRealExtent || n > kMaxRealExtent || k > kMaxRealExtent) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^30");
  }

  const bool col_major = (layout == Layout::kColMajor);
  const auto first = BatchedOperand{a_buffer(), 0, a_ld, 0, &a_offsets, shape.a_rotated,
                                    a_transpose == Transpose::kConjugate};
  const auto second = BatchedOperand{b_buffer(), 0, b_ld, 0, &b_offsets, !shape.b_rotated,
                                     b_transpose == Transpose::kConjugate};
  const auto left = col_major ? first : second;
  const auto right = col_major ? second : first;
  const auto rows = col_major ? m : n, columns = col_major ? n : m;
  const auto precision = static_cast<int>(8 * sizeof(R));
  const auto batches = static_cast<int>(batch_count);

  // What the helper kernels read per matrix, in one upload: [alphas | betas | left | right | c offsets]
  const bool complex_betas = std::any_of(betas.begin(), betas.end(), [](const Complex& b) { return b.imag() != R(0); });
  const auto scalars_block = batch_count * sizeof(Complex);
  const auto offsets_block = batch_count * sizeof(long long);
  auto packed = std::vector<unsigned char>(2 * scalars_block + 3 * offsets_block);
  std::memcpy(&packed[0], alphas.data(), scalars_block);
  std::memcpy(&packed[scalars_block], betas.data(), scalars_block);
  for (auto batch = size_t{0}; batch < batch_count; ++batch) {
    const long long values[3] = {static_cast<long long>((*left.offsets)[batch]),
                                 static_cast<long long>((*right.offsets)[batch]),
                                 static_cast<long long>(c_offsets[batch])};
    for (int which = 0; which < 3; ++which) {
      std::memcpy(&packed[2 * scalars_block + which * offsets_block + batch * sizeof(long long)], &values[which],
                  sizeof(long long));
    }
  }
  const StreamScratch metadata(packed.size(), stream(), "batch metadata");
  CheckDevice(clbh_upload_async(metadata.get(), packed.data(), packed.size(), stream()), "clbh_upload_async");
  const auto base = static_cast<const unsigned char*>(metadata.get());
  const auto device_alphas = static_cast<const void*>(base);
  const auto device_betas = static_cast<const void*>(base + scalars_block);
  const auto device_left = reinterpret_cast<const long long*>(base + 2 * scalars_block);
  const auto device_right = reinterpret_cast<const long long*>(base + 2 * scalars_block + offsets_block);
  const auto device_c = reinterpret_cast<const long long*>(base + 2 * scalars_block + 2 * offsets_block);

  if (UseSmallKernel(rows, columns, k, batch_count, PrecisionValue<R>())) {
    auto desc = clbh_complex_small_desc{};
    desc.precision = precision;
    desc.rows = static_cast<int>(rows);
    desc.columns = static_cast<int>(columns);
    desc.k = static_cast<int>(k);
    desc.batch_count = batches;
    desc.left = SmallOperand(left, device_left);
    desc.right = SmallOperand(right, device_right);
    desc.c = clbh_complex_small_operand{c_buffer(), 0, static_cast<long long>(c_ld), 0, device_c, 0, 0};
    desc.alphas = device_alphas;
    desc.betas = device_betas;
    CheckDevice(clbh_complex_gemm_small_batched(&desc, stream()), "clbh_complex_gemm_small_batched");
    Finish();  // records the caller's event
    return;
  }

  // left operands -> real 2 rows x 2k each (times their alpha), densely behind one another
  const auto expanded_elements = 4 * rows * k;
  const auto expanded_bytes = batch_count * expanded_elements * sizeof(R);
  const StreamScratch expanded(expanded_bytes, stream(), "real form of the first operands");
  auto walk = clbh_complex_batches{batches, 0, device_left, static_cast<long long>(expanded_elements), device_alphas};
  CheckDevice(clbh_complex_expand_batched(precision, static_cast<int>(rows), static_cast<int>(k), left.kcontig ? 1 : 0,
                                          left.conjugate ? 1 : 0, right.conjugate ? 1 : 0, 1.0, 0.0, left.pointer, 0,
                                          static_cast<long long>(left.ld), expanded.get(), &walk, stream()),
              "clbh_complex_expand_batched");
  // right operands: in place (offsets in real numbers) or transposed into a dense temporary
  auto real_right_offsets = std::vector<size_t>(batch_count);
  const void* right_pointer = right.pointer;
  auto right_ld = right.ld;
  auto right_bytes = size_t{0};
  std::unique_ptr<StreamScratch> transposed;
  if (!right.kcontig) {
    right_bytes = batch_count * 2 * k * columns * sizeof(R);
    transposed.reset(new StreamScratch(right_bytes, stream(), "transposed second operands"));
    walk = clbh_complex_batches{batches, 0, device_right, static_cast<long long>(k * columns), nullptr};
    CheckDevice(clbh_complex_transpose_batched(precision, static_cast<int>(k), static_cast<int>(columns), right.pointer, 0,
                                               static_cast<long long>(right.ld), transposed->get(), &walk, stream()),
                "clbh_complex_transpose_batched");
    right_pointer = transposed->get();
    right_ld = k;
    for (auto batch = size_t{0}; batch < batch_count; ++batch) { real_right_offsets[batch] = batch * 2 * k * columns; }
  } else {
    for (auto batch = size_t{0}; batch < batch_count; ++batch) { real_right_offsets[batch] = 2 * (*right.offsets)[batch]; }
  }
  // betas: real ones go to the real GEMM; if any has an imaginary part, all are applied in a pass of their own
  auto real_betas = std::vector<R>(batch_count, R(1));
  if (complex_betas) {
    walk = clbh_complex_batches{batches, 0, device_c, 0, device_betas};
    CheckDevice(clbh_complex_scale_batched(precision, static_cast<int>(rows), static_cast<int>(columns), 0, 1.0, 0.0,
                                           const_cast<void*>(c_buffer()), 0, static_cast<long long>(c_ld), &walk,
                                           stream()),
                "clbh_complex_scale_batched");
  } else {
    for (auto batch = size_t{0}; batch < batch_count; ++batch) { real_betas[batch] = betas[batch].real(); }
  }
  auto real_left_offsets = std::vector<size_t>(batch_count), real_c_offsets = std::vector<size_t>(batch_count);
  for (auto batch = size_t{0}; batch < batch_count; ++batch) {
    real_left_offsets[batch] = batch * expanded_elements;
    real_c_offsets[batch] = 2 * c_offsets[batch];
  }
  const auto real_left = Buffer<R>(expanded.get(), expanded_bytes);
  const auto real_right = transposed ? Buffer<R>(right_pointer, right_bytes) : Buffer<R>(right_pointer);
  auto real_routine = XgemmBatched<R>(queue_, event_);  // records the caller's event after its launch
  real_routine.DoGemmBatched(Layout::kColMajor, Transpose::kNo, Transpose::kNo, 2 * rows, columns, 2 * k,
                             std::vector<R>(batch_count, R(1)), real_left, real_left_offsets, 2 * rows, real_right,
                             real_right_offsets, 2 * right_ld, real_betas, Buffer<R>(c_buffer()), real_c_offsets,
                             2 * c_ld, batch_count);
}

template class XgemmComplexBatched<float>;
template class XgemmComplexBatched<double>;

// =================================================================================================
}  // namespace clblast
