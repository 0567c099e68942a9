// =================================================================================================
// Batched and strided-batched GEMM host logic (see xgemmbatched.hpp).
// =================================================================================================
#include "routines/xgemmbatched.hpp"

#include <algorithm>
#include <memory>
#include <climits>
#include <cstring>

namespace clblast {
// =================================================================================================

template <typename T>
XgemmBatched<T>::XgemmBatched(hipStream_t* queue, hipEvent_t* event)
    : GemmRoutineBase(queue, event, PrecisionValue<T>()) {}

template <typename T>
void XgemmBatched<T>::DoGemmBatched(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                                    const size_t m, const size_t n, const size_t k, const std::vector<T>& alphas,
                                    const Buffer<T>& a_buffer, const std::vector<size_t>& a_offsets,
                                    const size_t a_ld, const Buffer<T>& b_buffer,
                                    const std::vector<size_t>& b_offsets, const size_t b_ld,
                                    const std::vector<T>& betas, const Buffer<T>& c_buffer,
                                    const std::vector<size_t>& c_offsets, const size_t c_ld,
                                    const size_t batch_count) {
  // Batch count and array lengths first (reference: xgemmbatched.cpp:66-69)
  if ((batch_count < 1) || (alphas.size() != batch_count) || (betas.size() != batch_count) ||
      (a_offsets.size() != batch_count) || (b_offsets.size() != batch_count) || (c_offsets.size() != batch_count)) {
    throw BLASError(StatusCode::kInvalidBatchCount);
  }
  if (batch_count > static_cast<size_t>(INT_MAX)) {
    throw BLASError(StatusCode::kInvalidBatchCount, "batch count exceeds 2^31-1");
  }
  const auto shape = Xgemm<T>::ProcessArguments(layout, a_transpose, b_transpose, m, n, k);

  // The largest offset decides; the leading dimensions of A and B are not tested, that of C is
  // (reference: xgemmbatched.cpp:82-84, buffer_test.hpp:169-190)
  const auto a_max = *std::max_element(a_offsets.begin(), a_offsets.end());
  const auto b_max = *std::max_element(b_offsets.begin(), b_offsets.end());
  const auto c_max = *std::max_element(c_offsets.begin(), c_offsets.end());
  TestMatrixA(shape.a_one, shape.a_two, a_buffer, a_max, a_ld, false);
  TestMatrixB(shape.b_one, shape.b_two, b_buffer, b_max, b_ld, false);
  TestMatrixC(shape.c_one, shape.c_two, c_buffer, c_max, c_ld);

  auto desc = Xgemm<T>::Canonicalise(shape, layout, m, n, k, a_buffer(), 0, a_ld, b_buffer(), 0, b_ld,
                                     const_cast<void*>(c_buffer()), 0, c_ld);
  const auto choice = SelectKernel(PrecisionValue<T>(), desc.a_kcontig != 0, desc.b_kcontig != 0,
                                   static_cast<size_t>(desc.m), static_cast<size_t>(desc.n), k, batch_count, true,
                                   min_indirect_size(), false, false, std::max({a_ld, b_ld, c_ld}));
  desc.kernel_class = choice.kernel_class;
  desc.tile_variant = choice.tile_variant;
  desc.split_k = choice.split_k;
  desc.batch_count = static_cast<int>(batch_count);

  // Packs [alphas | betas | a_offsets | b_offsets | c_offsets] into one host block. Scalars are stored
  // in the kernels' compute type: float for fp16/fp32 (half scalars are widened on the host as in
  // utilities.cpp:480-483), double for fp64. After the row-major fold the canonical A is the user's B.
  const auto scalar_bytes = (PrecisionValue<T>() == Precision::kDouble) ? sizeof(double) : sizeof(float);
  const auto scalars_block = Ceil(batch_count * scalar_bytes, 8);
  const auto offsets_block = batch_count * sizeof(long long);
  const auto col_major = (layout == Layout::kColMajor);
  const auto& first_offsets = col_major ? a_offsets : b_offsets;   // of the canonical A
  const auto& second_offsets = col_major ? b_offsets : a_offsets;  // of the canonical B

  // fp16 operands of the tiled kernels are fetched in dwords (see Xgemm::DoGemm): when the matrices of an operand
  // start at odd elements or have an odd leading dimension, all of them are copied into one aligned dense temporary
  // and the kernel gets the offsets in there; the copy kernel reads the caller's offsets from two more blocks
  struct AlignedCopy { bool wanted; size_t one, two, ld; };
  const auto plan_copy = [&](const void* pointer, const long long ld, const std::vector<size_t>& offsets, const bool kcontig,
                             const int extent) {
    auto plan = AlignedCopy{false, static_cast<size_t>(kcontig ? desc.k : extent), static_cast<size_t>(kcontig ? extent : desc.k), 0};
    plan.ld = Ceil(plan.one, 8);
    if (PrecisionValue<T>() != Precision::kHalf || desc.kernel_class != CLBH_KERNEL_MFMA) { return plan; }
    plan.wanted = (reinterpret_cast<unsigned long long>(pointer) % 4 != 0) || (ld % 2 != 0) ||
                  std::any_of(offsets.begin(), offsets.end(), [](const size_t offset) { return offset % 2 != 0; });
    return plan;
  };
  const auto copy_a = plan_copy(desc.a, desc.a_ld, first_offsets, desc.a_kcontig != 0, desc.m);
  const auto copy_b = plan_copy(desc.b, desc.b_ld, second_offsets, desc.b_kcontig != 0, desc.n);
  const auto extra_blocks = (copy_a.wanted ? 1 : 0) + (copy_b.wanted ? 1 : 0);
  const auto total_bytes = 2 * scalars_block + (3 + extra_blocks) * offsets_block;
  auto packed = std::vector<unsigned char>(total_bytes);
  for (auto batch = size_t{0}; batch < batch_count; ++batch) {
    if (PrecisionValue<T>() == Precision::kDouble) {
      const auto alpha = ScalarToDouble(alphas[batch]);
      const auto beta = ScalarToDouble(betas[batch]);
      std::memcpy(&packed[batch * sizeof(double)], &alpha, sizeof(double));
      std::memcpy(&packed[scalars_block + batch * sizeof(double)], &beta, sizeof(double));
    } else {
      const auto alpha = static_cast<float>(ScalarToDouble(alphas[batch]));
      const auto beta = static_cast<float>(ScalarToDouble(betas[batch]));
      std::memcpy(&packed[batch * sizeof(float)], &alpha, sizeof(float));
      std::memcpy(&packed[scalars_block + batch * sizeof(float)], &beta, sizeof(float));
    }
    const auto a_off = static_cast<long long>(copy_a.wanted ? batch * copy_a.ld * copy_a.two : first_offsets[batch]);
    const auto b_off = static_cast<long long>(copy_b.wanted ? batch * copy_b.ld * copy_b.two : second_offsets[batch]);
    const auto c_off = static_cast<long long>(c_offsets[batch]);
    auto extra = 2 * scalars_block + 3 * offsets_block;
    if (copy_a.wanted) {
      const auto original = static_cast<long long>(first_offsets[batch]);
      std::memcpy(&packed[extra + batch * sizeof(long long)], &original, sizeof(long long));
      extra += offsets_block;
    }
    if (copy_b.wanted) {
      const auto original = static_cast<long long>(second_offsets[batch]);
      std::memcpy(&packed[extra + batch * sizeof(long long)], &original, sizeof(long long));
    }
    std::memcpy(&packed[2 * scalars_block + batch * sizeof(long long)], &a_off, sizeof(long long));
    std::memcpy(&packed[2 * scalars_block + offsets_block + batch * sizeof(long long)], &b_off, sizeof(long long));
    std::memcpy(&packed[2 * scalars_block + 2 * offsets_block + batch * sizeof(long long)], &c_off,
                sizeof(long long));
  }

  // what the launcher may assume about the alignment of the per-batch offsets (elements): the largest power
  // of two up to 8 that divides all of them
  auto multiple = size_t{8};
  for (auto batch = size_t{0}; batch < batch_count; ++batch) {
    // (the aligned copies lie at multiples of 8 elements)
    const auto bits = (copy_a.wanted ? 0 : first_offsets[batch]) | (copy_b.wanted ? 0 : second_offsets[batch]) | c_offsets[batch];
    while (multiple > 1 && (bits % multiple) != 0) { multiple /= 2; }
  }
  // an odd offset of C alone does not keep the fp16 kernels from fetching A and B in dwords
  if (PrecisionValue<T>() == Precision::kHalf && multiple < 2 &&
      std::none_of(first_offsets.begin(), first_offsets.end(), [&](const size_t o) { return !copy_a.wanted && o % 2 != 0; }) &&
      std::none_of(second_offsets.begin(), second_offsets.end(), [&](const size_t o) { return !copy_b.wanted && o % 2 != 0; })) {
    multiple = 2;
  }
  desc.batch.offset_multiple = static_cast<int>(multiple);

  const StreamScratch device_block(total_bytes, stream(), "batch metadata");
  std::unique_ptr<StreamScratch> aligned_a, aligned_b;
  auto status = clbh_upload_async(device_block.get(), packed.data(), total_bytes, stream());
  if (status == 0) {
    const auto base = static_cast<unsigned char*>(device_block.get());
    auto extra = 2 * scalars_block + 3 * offsets_block;
    const auto make_copy = [&](const AlignedCopy& plan, const void*& pointer, long long& ld,
                               std::unique_ptr<StreamScratch>& copy) {
      if (!plan.wanted) { return; }
      copy.reset(new StreamScratch(batch_count * plan.ld * plan.two * sizeof(T), stream(), "aligned copies of an operand"));
      CheckDevice(clbh_copy_matrix_batched(16, static_cast<int>(plan.one), static_cast<int>(plan.two),
                                           static_cast<int>(batch_count), pointer, 0, ld, 0,
                                           reinterpret_cast<const long long*>(base + extra), copy->get(),
                                           static_cast<long long>(plan.ld), static_cast<long long>(plan.ld * plan.two), stream()),
                  "clbh_copy_matrix_batched");
      pointer = copy->get();
      ld = static_cast<long long>(plan.ld);
      extra += offsets_block;
    };
    make_copy(copy_a, desc.a, desc.a_ld, aligned_a);
    make_copy(copy_b, desc.b, desc.b_ld, aligned_b);
    desc.batch.alphas = base;
    desc.batch.betas = base + scalars_block;
    desc.batch.a_offsets = reinterpret_cast<const long long*>(base + 2 * scalars_block);
    desc.batch.b_offsets = reinterpret_cast<const long long*>(base + 2 * scalars_block + offsets_block);
    desc.batch.c_offsets = reinterpret_cast<const long long*>(base + 2 * scalars_block + 2 * offsets_block);
    status = clbh_gemm_launch(&desc, stream());
  }
  CheckDevice(status, "batched GEMM launch");
  Finish();
}

// =================================================================================================

template <typename T>
XgemmStridedBatched<T>::XgemmStridedBatched(hipStream_t* queue, hipEvent_t* event)
    : GemmRoutineBase(queue, event, PrecisionValue<T>()) {}

template <typename T>
void XgemmStridedBatched<T>::DoGemmStridedBatched(
    const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m, const size_t n,
    const size_t k, const T alpha, const Buffer<T>& a_buffer, const size_t a_offset, const size_t a_ld,
    const size_t a_stride, const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld, const size_t b_stride,
    const T beta, const Buffer<T>& c_buffer, const size_t c_offset, const size_t c_ld, const size_t c_stride,
    const size_t batch_count) {
  // reference: xgemmstridedbatched.cpp:68-75
  if (batch_count < 1) {
    throw BLASError(StatusCode::kInvalidBatchCount);
  }
  if (c_stride == 0) {
    throw BLASError(StatusCode::kInvalidDimension);
  }
  if (batch_count > static_cast<size_t>(INT_MAX)) {
    throw BLASError(StatusCode::kInvalidBatchCount, "batch count exceeds 2^31-1");
  }
  const auto shape = Xgemm<T>::ProcessArguments(layout, a_transpose, b_transpose, m, n, k);

  // The last matrix of the batch decides (reference: buffer_test.hpp:195-218)
  TestMatrixA(shape.a_one, shape.a_two, a_buffer, a_offset + (batch_count - 1) * a_stride, a_ld);
  TestMatrixB(shape.b_one, shape.b_two, b_buffer, b_offset + (batch_count - 1) * b_stride, b_ld);
  TestMatrixC(shape.c_one, shape.c_two, c_buffer, c_offset + (batch_count - 1) * c_stride, c_ld);

  auto desc = Xgemm<T>::Canonicalise(shape, layout, m, n, k, a_buffer(), a_offset, a_ld, b_buffer(), b_offset, b_ld,
                                     const_cast<void*>(c_buffer()), c_offset, c_ld);
  const auto col_major = (layout == Layout::kColMajor);
  desc.a_stride = static_cast<long long>(col_major ? a_stride : b_stride);
  desc.b_stride = static_cast<long long>(col_major ? b_stride : a_stride);
  desc.c_stride = static_cast<long long>(c_stride);
  desc.batch_count = static_cast<int>(batch_count);
  desc.alpha = ScalarToDouble(alpha);
  desc.beta = ScalarToDouble(beta);
  const auto choice = SelectKernel(PrecisionValue<T>(), desc.a_kcontig != 0, desc.b_kcontig != 0,
                                   static_cast<size_t>(desc.m), static_cast<size_t>(desc.n), k, batch_count, false,
                                   min_indirect_size(), false, desc.beta == 0.0, std::max({a_ld, b_ld, c_ld}));
  desc.kernel_class = choice.kernel_class;
  desc.tile_variant = choice.tile_variant;
  desc.split_k = choice.split_k;

  // fp16 operands of the tiled kernels are fetched in dwords (see Xgemm::DoGemm): matrices at odd elements, with an odd
  // leading dimension or an odd stride are copied into aligned dense temporaries first (4096 x 33 x 65 x 40: 162 us on
  // the element-wise kernel)
  std::unique_ptr<StreamScratch> aligned_a, aligned_b;
  if (PrecisionValue<T>() == Precision::kHalf && desc.kernel_class == CLBH_KERNEL_MFMA) {
    const auto align = [&](const void*& pointer, long long& offset, long long& ld, long long& stride, const bool kcontig,
                           const int extent, std::unique_ptr<StreamScratch>& copy) {
      const auto address = reinterpret_cast<unsigned long long>(pointer) + 2 * static_cast<unsigned long long>(offset);
      if (address % 4 == 0 && ld % 2 == 0 && (stride % 2 == 0 || batch_count == 1)) { return; }
      const auto one = static_cast<size_t>(kcontig ? desc.k : extent), two = static_cast<size_t>(kcontig ? extent : desc.k);
      const auto new_ld = Ceil(one, 8);
      const auto copies = (stride == 0) ? size_t{1} : batch_count;  // a shared matrix is copied once
      copy.reset(new StreamScratch(copies * new_ld * two * sizeof(T), stream(), "aligned copies of an operand"));
      CheckDevice(clbh_copy_matrix_batched(16, static_cast<int>(one), static_cast<int>(two), static_cast<int>(copies), pointer,
                                           offset, ld, stride, nullptr, copy->get(), static_cast<long long>(new_ld),
                                           static_cast<long long>(new_ld * two), stream()),
                  "clbh_copy_matrix_batched");
      pointer = copy->get();
      offset = 0;
      ld = static_cast<long long>(new_ld);
      stride = (stride == 0) ? 0 : static_cast<long long>(new_ld * two);
    };
    align(desc.a, desc.a_offset, desc.a_ld, desc.a_stride, desc.a_kcontig != 0, desc.m, aligned_a);
    align(desc.b, desc.b_offset, desc.b_ld, desc.b_stride, desc.b_kcontig != 0, desc.n, aligned_b);
  }
  // A batch of one matrix gets the tile table's choice for a single product, which may split a long k: the K ranges
  // sum in stream-ordered scratch, as in Xgemm::DoGemm
  const auto temp_bytes = clbh_gemm_workspace_bytes(&desc);
  std::unique_ptr<StreamScratch> scratch;
  if (temp_bytes > 0) {
    scratch.reset(new StreamScratch(temp_bytes, stream(), "temporary buffer"));
    desc.workspace = scratch->get();
  }
  desc.workspace_bytes = temp_bytes;
  CheckDevice(clbh_gemm_launch(&desc, stream()), "strided-batched GEMM launch");
  Finish();
}

template class XgemmBatched<half>;
template class XgemmBatched<float>;
template class XgemmBatched<double>;
template class XgemmStridedBatched<half>;
template class XgemmStridedBatched<float>;
template class XgemmStridedBatched<double>;

// =================================================================================================
}  // namespace clblast
