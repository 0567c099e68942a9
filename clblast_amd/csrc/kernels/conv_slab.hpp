// =================================================================================================
// fp16 and fp32 CONVGEMM with unit strides and no dilation on gfx950, without an im2col matrix and without a padded copy of
// the images (the reference's single-kernel method, src/routines/levelx/xconvgemm.cpp:121-160 with
// src/kernels/levelx/xconvgemm_part1.opencl / xconvgemm_part2.opencl, gathers every patch element from memory; its
// two-kernel method writes the kernel_h * kernel_w times larger im2col matrix first, xconvgemm.cpp:78-119).
//
// (Written out for fp16; fp32 is the same with half as many channels per step: a chunk of 8 channels, 16-byte pieces of
// four pixels of ONE channel, v_mfma_f32_32x32x2_f32 - four of them per 16-byte operand pair, lane group g of the two
// supplying channels 4 g .. 4 g + 3 - and a result that leaves the registers directly, 16 bytes of four pixels per lane.)
//
// A work-group owns `rows` whole output rows of one image (at most 448 output pixels) and 128 kernels. The channels
// are walked in chunks of 16. For a chunk, the part of the image that the tile's patches touch - (rows + kernel_h - 1)
// x (width + 2 pad_w) pixels, zeros outside the image - is staged in LDS with the CHANNEL as the contiguous index
// ([row][column][channel], pitch 24 halves): 16-byte loads along the image rows of two channels at a time, their halves
// interleaved in registers, eight 4-byte LDS writes (the lanes of a wavefront take pieces of eight different slab rows,
// which keeps the 64 dwords of a write on 64 banks). Every tap (kh, kw) of the kernel is then one k-step of
// v_mfma_f32_32x32x16_f16 whose pixel operand is a 16-byte LDS read at the tile pixel's address plus the tap's uniform
// offset: the image is read from memory once per chunk, not once per tap, and no address arithmetic stands between the
// matrix instructions. Two slabs alternate, so that the next chunk is requested before and written after the products
// of the current one (one barrier per chunk). A single wavefront per SIMD hides only what stands between its matrix
// instructions, so the reads of the next tap and the writes of the next chunk's pieces are placed there one by one.
//
// The kernel matrix is read through a copy in k-step order, [chunk][tap][kernel][16 channels] (HconvPermuteKernel; taps
// mirrored there for a true convolution): the tile's 128 kernels of a chunk are taps contiguous pieces of 4 KiB, which
// go straight from memory into LDS next to the slab (two chunks alternate as the slabs do), and a lane's eight k values
// are one 16-byte LDS read. The K walk itself therefore issues no memory instruction that its products wait for: the
// next chunk's image pieces and kernels are requested at the top of a chunk and waited for at its end. Two sets of
// operand registers alternate from tap to tap, so that the reads of the next tap stand under the products of this one.
//
// Wavefront (wm, wn) of the four owns pixels [224 wm, 224 wm + 224) x kernels [64 wn, 64 wn + 64): 7 x 2 blocks of
// 32 x 32, 224 accumulator registers. The pixels are the FIRST operand, so that a lane's four consecutive result
// registers are four consecutive pixels of one kernel: after the walk they go to LDS as [kernel][pixel] with 8-byte
// writes (the slabs are no longer needed) and leave with 16-byte stores along the result's rows.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_CONV_SLAB_HPP_
#define CLBLAST_HIP_KERNELS_CONV_SLAB_HPP_

#include <hip/hip_runtime.h>

#include <type_traits>

#include "device/launch_plans.hpp"
#include "kernels/gemm_mfma.hpp"
#include "kernels/gemm_mfma_f16.hpp"

namespace clbh {

template <typename T>
struct ConvSlabType {
  static constexpr int CHUNK = 32 / sizeof(T);                   // channels per chunk: 32 bytes per pixel (16 halves, 8 floats)
  static constexpr int PITCH = kConvSlabPixelBytes / sizeof(T);  // elements from a pixel to the next
  static constexpr int PIECE = 16 / sizeof(T);                   // pixels of a 16-byte piece of an image row (8, 4)
  static constexpr int PLANES = sizeof(T) == 2 ? 2 : 1;          // channels a staged piece covers (fp16: a pair, one dword per pixel)
  typedef T Vector __attribute__((ext_vector_type(16 / sizeof(T))));  // a 16-byte operand
};

template <typename T>
struct ConvSlabArgs {
  const T* images;   // batch x channels x height x width
  const T* weights;  // [channels / CHUNK][taps][kernels][CHUNK] (ConvPermuteKernel)
  T* result;         // batch x kernels x output_h x output_w
  int channels, height, width;
  int kernel_h, kernel_w, pad_h, pad_w;
  int output_h, output_w;
  int kernels;
  int rows;          // output rows per tile; rows * output_w <= kConvSlabPixels
  int row_tiles;     // ceil(output_h / rows)
  int kernel_tiles;  // ceil(kernels / (64 J))
  int slab_rows, slab_width;  // rows + kernel_h - 1, width + 2 pad_w
  int slab_elements;          // (slab_rows * slab_width + 8) * PITCH
  int spare_at;               // elements from a slab's start to its last 8 pixels, a strip that no product reads
};

// x / d for 0 <= x, d < 2^10, with inverse = 1.0f / d (exact: (x + 0.5) / d is at least 2^-11 away from an integer)
__device__ __forceinline__ int SmallQuotient(const int x, const float inverse) {
  return static_cast<int>((static_cast<float>(x) + 0.5f) * inverse);
}

// out[((chunk * taps + tap) * kernels + n) * CHUNK + i] = weights[n][(CHUNK chunk + i) * taps + (flip ? taps - 1 - tap : tap)],
// one thread per 16 bytes (half of a kernel's chunk)
template <typename T>
__global__ __launch_bounds__(256) void ConvPermuteKernel(const T* __restrict__ weights, T* __restrict__ out, const int kernels,
                                                         const int channels, const int taps, const int flip) {
  using Type = ConvSlabType<T>;
  const int index = blockIdx.x * 256 + threadIdx.x;
  if (index >= kernels * (channels / Type::PIECE) * taps) { return; }
  const int part = index % 2;
  const int n = (index / 2) % kernels;
  const int step = index / (2 * kernels);
  const int chunk = step / taps, tap = step % taps;
  const int stored_tap = flip ? (taps - 1 - tap) : tap;
  const T* from = weights + (static_cast<long long>(n) * channels + chunk * Type::CHUNK + Type::PIECE * part) * taps + stored_tap;
  typename Type::Vector values;
#pragma unroll
  for (int i = 0; i < Type::PIECE; ++i) { values[i] = from[i * taps]; }
  *reinterpret_cast<typename Type::Vector*>(out + static_cast<long long>(index) * Type::PIECE) = values;
}

// grid: batch x row_tiles x kernel_tiles work-groups of 256 threads; dynamic LDS: two slabs and two chunks of the kernel
// matrix, or kConvSlabResultBytes where that is more.
// TASKS: 16-byte pieces of the slab (fp16: of two channels each) a thread stages per chunk, at least
// ceil(8 * slab_rows * (width / PIECE) / 256). TAPS: kernel_h * kernel_w as a constant (the walk over the taps is then
// straight-line code), or 0 for any number of taps. J: blocks of 32 kernels per wavefront - 2: the tile of 128 kernels
// described above; 1: a tile of 64 kernels (wavefronts of 224 pixels x 32 kernels) for calls with at most 64 kernels,
// which would leave half of the large tile's matrix instructions without use.
template <typename T, int TASKS, int TAPS, int J>
__global__ __launch_bounds__(kConvSlabThreads, 1) void ConvSlabKernel(const ConvSlabArgs<T> p) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  typedef unsigned Dwords4 __attribute__((ext_vector_type(4)));
  using Type = ConvSlabType<T>;
  using Vector = typename Type::Vector;
  constexpr bool HALF = sizeof(T) == 2;
  constexpr int CHUNK = Type::CHUNK, PITCH = Type::PITCH, PIECE = Type::PIECE, PLANES = Type::PLANES, BLOCKS = kConvSlabBlocks;
  constexpr int KERNELS = 64 * J;                // of the tile
  constexpr int TAP_ELEMENTS = KERNELS * CHUNK;  // the tile's part of the kernel matrix for one tap (2 or 4 KiB)

  const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wave_m = wave % 2, wave_n = wave / 2;
  int block = blockIdx.x;
  const int kernel_tile = block % p.kernel_tiles;
  block /= p.kernel_tiles;
  const int row_tile = block % p.row_tiles;
  const int batch = block / p.row_tiles;
  const int row0 = row_tile * p.rows;
  const int valid_pixels = min(p.rows, p.output_h - row0) * p.output_w;
  const int n0 = kernel_tile * KERNELS;
  const int plane = p.height * p.width;
  const int taps = TAPS > 0 ? TAPS : p.kernel_h * p.kernel_w;
  const int chunks = p.channels / CHUNK;
  T* const ordered = lds + 2 * p.slab_elements;  // two chunks of the kernel matrix, taps * TAP_ELEMENTS each

  // The pieces this thread stages, the same for every chunk: channel pair (fp32: channel), slab row, 8 (4) columns. Eight
  // neighbouring lanes hold the eight channel pairs (channels) of one piece, the eight groups of a wavefront the pieces of eight consecutive
  // slab rows in the same columns. A pixel is 12 banks from the next and a slab row 8 x (an odd number) banks from
  // the next (the host pads the slab's width to 2 mod 4 pixels), so the 64 dwords of one write instruction fall on 64
  // different banks. A piece that does not exist (a row outside the image, a task beyond the slab) is loaded from the
  // first row of the planes and written to a spare strip behind the slab: no branches, the slab keeps its zeros.
  int piece_source[TASKS], piece_target[TASKS];  // element offsets in the chunk's planes and in LDS
  {
    const int row_vectors = p.width / PIECE;
    const float rows_inverse = 1.0f / static_cast<float>(p.slab_rows);
#pragma unroll
    for (int j = 0; j < TASKS; ++j) {
      const int t = tid + kConvSlabThreads * j;
      const int pair = t % 8, rest = t / 8;
      const int v = SmallQuotient(rest, rows_inverse), h = rest - v * p.slab_rows;
      const int image_row = row0 + h - p.pad_h;
      const bool exists = v < row_vectors && image_row >= 0 && image_row < p.height;
      piece_source[j] = exists ? (PLANES * pair * p.height + image_row) * p.width + PIECE * v : PLANES * pair * plane;
      piece_target[j] = (exists ? (h * p.slab_width + p.pad_w + PIECE * v) * PITCH : p.spare_at) + PLANES * pair;
    }
  }
  Dwords4 even_channel[TASKS], odd_channel[HALF ? TASKS : 1];  // (fp32: the piece's only channel in even_channel)
  const T* image = p.images + static_cast<long long>(batch) * p.channels * plane;
  auto request = [&](const int chunk) {
    const T* planes = image + static_cast<long long>(chunk) * CHUNK * plane;
#pragma unroll
    for (int j = 0; j < TASKS; ++j) {
      even_channel[j] = *reinterpret_cast<const Dwords4*>(planes + piece_source[j]);
      if constexpr (HALF) { odd_channel[j] = *reinterpret_cast<const Dwords4*>(planes + piece_source[j] + plane); }
    }
  };
  auto deposit = [&](T* slab) {
#pragma unroll
    for (int j = 0; j < TASKS; ++j) {
#pragma unroll
      for (int i = 0; i < PIECE; ++i) {  // pixel i of the piece as one dword: fp16 (even channel, odd channel)
        unsigned pixel;
        if constexpr (HALF) {
          pixel = __builtin_amdgcn_perm(odd_channel[j][i / 2], even_channel[j][i / 2], (i % 2) ? 0x07060302u : 0x05040100u);
        } else {
          pixel = even_channel[j][i];
        }
        *reinterpret_cast<unsigned*>(slab + piece_target[j] + i * PITCH) = pixel;
      }
    }
  };
  // The tile's 128 kernels of a chunk, tap by tap, straight from memory into LDS: wavefront w moves kernels
  // [32 w, 32 w + 32) of every tap (1 KiB, contiguous on both sides). Kernels beyond the matrix read what follows them
  // (zeros behind the end of the copy); their results are not stored.
  const int ordered_bytes_left = (p.channels * taps * p.kernels - n0 * CHUNK) * static_cast<int>(sizeof(T));
  const int tap_bytes = p.kernels * CHUNK * static_cast<int>(sizeof(T));
  auto request_kernels = [&](const int chunk) {
    typedef __attribute__((address_space(3))) void* LdsPtr;
    const T* from = p.weights + n0 * CHUNK;
    const auto view = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(from), 0, ordered_bytes_left, kRawBufferFlags);
    T* to = ordered + (chunk & 1) * taps * TAP_ELEMENTS + wave * (1024 / static_cast<int>(sizeof(T)));
    int lane_bytes = chunk * taps * tap_bytes + wave * 1024 + lane * 16;  // (the range check covers this offset only)
    for (int tap = 0; tap < taps; ++tap) {
      // (device pass only: with a pointer of a dependent type here, hipcc's host pass drops the kernel's launch stub
      // without a diagnostic and the library fails to link)
#if defined(__HIP_DEVICE_COMPILE__)
      if (wave < 2 * J) { __builtin_amdgcn_raw_ptr_buffer_load_lds(view, (LdsPtr)(to), 16, lane_bytes, 0, 0, 0); }  // (1 KiB = 32 kernels each)
#endif
      to += TAP_ELEMENTS;
      lane_bytes += tap_bytes;
    }
  };

  request_kernels(0);
  request(0);
  // Zeros in both slabs: what no piece covers (the border columns, rows outside the image) stays zero
  for (int i = tid; i < 2 * p.slab_elements / PIECE; i += kConvSlabThreads) { reinterpret_cast<Dwords4*>(lds)[i] = Dwords4(0u); }

  // Where this lane's pixel of each block sits in a slab (tap (0, 0)), plus its half of the 16 channels
  int pixel_at[BLOCKS];
  const float width_inverse = 1.0f / static_cast<float>(p.output_w);
#pragma unroll
  for (int i = 0; i < BLOCKS; ++i) {
    int pixel = (wave_m * BLOCKS + i) * 32 + lane % 32;
    if (pixel >= valid_pixels) { pixel = 0; }
    const int row = SmallQuotient(pixel, width_inverse);
    pixel_at[i] = (row * p.slab_width + (pixel - row * p.output_w)) * PITCH + PIECE * (lane / 32);
  }
  // This lane's kernels in a tap's part of the ordered kernel matrix
  int kernel_at[J];
#pragma unroll
  for (int j = 0; j < J; ++j) { kernel_at[j] = (wave_n * 32 * J + j * 32 + lane % 32) * CHUNK + PIECE * (lane / 32); }

  // (with TAPS known the first tap of the first chunk takes 0 as its addend instead: 224 register writes less)
  float16_t acc[BLOCKS][J];
  if (TAPS == 0) {
#pragma unroll
    for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
      for (int j = 0; j < J; ++j) { acc[i][j] = float16_t(0.0f); }
    }
  }

  __syncthreads();  // the zeros are in place
  deposit(lds);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's part of the kernels has arrived
  __syncthreads();

  // One set of operands: the pixels' 16 channels at a tap and the kernels' 16 channels at that tap
  struct Operands {
    Vector pixels[BLOCKS], kernels[J];
  };
  auto fetch = [&](const T* slab_at_tap, const T* kernels_at_tap, Operands& set) {
    // (in the order of their first use: the reads are spread over the products of the tap before)
#pragma unroll
    for (int j = 0; j < J; ++j) { set.kernels[j] = *reinterpret_cast<const Vector*>(kernels_at_tap + kernel_at[j]); }
#pragma unroll
    for (int i = 0; i < BLOCKS; ++i) { set.pixels[i] = *reinterpret_cast<const Vector*>(slab_at_tap + pixel_at[i]); }
  };
  auto products = [&](const Operands& set, auto from_zero) {
    if constexpr (HALF) {
#pragma unroll
      for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
        for (int j = 0; j < J; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(set.pixels[i], set.kernels[j],
                                                            decltype(from_zero)::value ? float16_t(0.0f) : acc[i][j], 0, 0, 0);
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {  // channels (e, 4 + e) of the chunk; all blocks between two sums into the same registers
#pragma unroll
        for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
          for (int j = 0; j < J; ++j) {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(set.pixels[i][e], set.kernels[j][e],
                                                            (decltype(from_zero)::value && e == 0) ? float16_t(0.0f) : acc[i][j], 0, 0, 0);
          }
        }
      }
    }
  };

  // The walk over one chunk; `first`: the chunk that starts the sums (a type, so that chunk 0 is code of its own)
  auto walk = [&](const int chunk, auto first) {
    constexpr bool FIRST = decltype(first)::value && TAPS > 0;
    constexpr int PER = HALF ? 1 : 4;  // matrix instructions per pair of 16-byte operands
    const T* slab = lds + (chunk & 1) * p.slab_elements;
    const T* kernels_now = ordered + (chunk & 1) * taps * TAP_ELEMENTS;
    // The next chunk's kernels and pieces are asked for between the products of the first tap (TAPS known) - without a
    // test of the chunk, which would end the scheduling region: the last chunk asks for itself again, into the slab and
    // the kernel buffer that nothing reads any more, and the wait at its end keeps these loads out of the epilogue's LDS.
    const int chunk_ahead = min(chunk + 1, chunks - 1);
    if (TAPS == 0 && chunk + 1 < chunks) {
      request_kernels(chunk_ahead);
      request(chunk_ahead);
    }
    Operands set[2];
    fetch(slab, kernels_now, set[0]);
    __builtin_amdgcn_sched_barrier(0);
    int kh = 0, kw = 0;
    auto next_tap = [&]() {  // the slab's offset of the tap after (kh, kw)
      if (++kw == p.kernel_w) {
        kw = 0;
        ++kh;
      }
      return (kh * p.slab_width + kw) * PITCH;
    };
    // (the scheduler is held to an order: left alone it moves every read down to its first use, and the products then
    // wait for the LDS read by read)
    if (TAPS > 0) {
      if (TAPS == 1) {
        request_kernels(chunk_ahead);
        request(chunk_ahead);
      }
#pragma unroll
      for (int tap = 0; tap + 1 < TAPS; ++tap) {
        if (tap == 0) {
          request_kernels(chunk_ahead);
          request(chunk_ahead);
        }
        fetch(slab + next_tap(), kernels_now + (tap + 1) * TAP_ELEMENTS, set[(tap + 1) % 2]);
        if (tap == 0) { products(set[0], std::integral_constant<bool, FIRST>{}); } else { products(set[tap % 2], std::false_type{}); }
        // one read after every matrix instruction: nine reads in a row wait for room in the LDS queue, and the
        // wavefront issues nothing else meanwhile
#pragma unroll
        for (int i = 0; i < (BLOCKS + J < BLOCKS * J ? BLOCKS + J : BLOCKS * J); ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);  // one matrix instruction (fp32: the four of a block),
          __builtin_amdgcn_sched_group_barrier(0x002, 1, 0);  // the address of
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read,
          if (tap == 0) {
            __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);  // (first tap: the addresses of)
            __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);  // two loads of the next chunk
          }
        }
#pragma unroll
        for (int i = BLOCKS + J; i < BLOCKS * J; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
          if (tap == 0) {
            __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      // The last tap has nothing to fetch: the next chunk's pieces go to their slab between its products (a wavefront
      // alone on its SIMD hides nothing that does not stand between matrix instructions). Without a test of the chunk,
      // which would end the scheduling region: after the last chunk the writes repeat the pieces of that chunk in the
      // slab that nothing reads any more.
      deposit(lds + ((chunk + 1) & 1) * p.slab_elements);
      products(set[(TAPS - 1) % 2], std::integral_constant<bool, FIRST && TAPS == 1>{});
#pragma unroll
      for (int i = 0; i < BLOCKS * J; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);  // one matrix instruction (fp32: four),
        __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);  // two vector ALU instructions,
        __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);  // two LDS writes
      }
      __builtin_amdgcn_sched_barrier(0);
    } else {
      for (int tap = 0; tap < taps; tap += 2) {
        if (tap + 1 < taps) { fetch(slab + next_tap(), kernels_now + (tap + 1) * TAP_ELEMENTS, set[1]); }
        __builtin_amdgcn_sched_barrier(0);
        products(set[0], std::false_type{});
        __builtin_amdgcn_sched_barrier(0);
        if (tap + 1 < taps) {
          if (tap + 2 < taps) { fetch(slab + next_tap(), kernels_now + (tap + 2) * TAP_ELEMENTS, set[0]); }
          __builtin_amdgcn_sched_barrier(0);
          products(set[1], std::false_type{});
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if (TAPS == 0 && chunk + 1 < chunks) { deposit(lds + ((chunk + 1) & 1) * p.slab_elements); }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  walk(0, std::true_type{});
  for (int chunk = 1; chunk < chunks; ++chunk) { walk(chunk, std::false_type{}); }

  const long long pixels = static_cast<long long>(p.output_h) * p.output_w;
  T* result = p.result + static_cast<long long>(batch) * p.kernels * pixels + static_cast<long long>(row0) * p.output_w;
  // Register r of block (i, j): pixel 32 i + 8 (r / 4) + 4 (lane / 32) + r % 4, kernel 32 j + lane % 32.
  if constexpr (HALF) {
    // fp16 epilogue: [kernel][pixel] in LDS (every wavefront its own part), then 16-byte stores along the result's rows
    constexpr int RP = kConvSlabResultPitch;
#pragma unroll
    for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
      for (int j = 0; j < J; ++j) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          half4_t four;
#pragma unroll
          for (int e = 0; e < 4; ++e) { four[e] = static_cast<_Float16>(acc[i][j][4 * g + e]); }
          const int pixel = (wave_m * BLOCKS + i) * 32 + 8 * g + 4 * (lane / 32);
          const int n = wave_n * 32 * J + j * 32 + lane % 32;
          *reinterpret_cast<half4_t*>(lds + n * RP + pixel) = four;
        }
      }
    }
    __syncthreads();
    constexpr int ROW_VECTORS = BLOCKS * 32 / 8;  // 16-byte pieces of a kernel's row in this wavefront's part
#pragma unroll 14
    for (int t = 0; t < ROW_VECTORS * J / 2; ++t) {  // 32 J rows of ROW_VECTORS pieces, 64 at a time
      const int q = lane + 64 * t;
      const int n = wave_n * 32 * J + q / ROW_VECTORS, pixel = wave_m * BLOCKS * 32 + (q % ROW_VECTORS) * 8;
      if (n0 + n < p.kernels && pixel < valid_pixels) {
        const Dwords4 value = *reinterpret_cast<const Dwords4*>(lds + n * RP + pixel);
        *reinterpret_cast<Dwords4*>(result + (n0 + n) * pixels + pixel) = value;
      }
    }
  } else {
    // fp32 epilogue: the same in two halves (the kernels of a wavefront's first block of 32, then of its second: 64 rows
    // of the tile at a time fit LDS). A wavefront writes and reads its own part only.
    constexpr int RP = kConvSlabPixels + 4;       // floats from a kernel to the next
    constexpr int ROW_VECTORS = BLOCKS * 32 / 4;  // 16-byte pieces of a kernel's row in this wavefront's part
#pragma unroll
    for (int j = 0; j < J; ++j) {
#pragma unroll
      for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          Vector four;
#pragma unroll
          for (int e = 0; e < 4; ++e) { four[e] = acc[i][j][4 * g + e]; }
          const int pixel = (wave_m * BLOCKS + i) * 32 + 8 * g + 4 * (lane / 32);
          *reinterpret_cast<Vector*>(lds + (wave_n * 32 + lane % 32) * RP + pixel) = four;
        }
      }
#pragma unroll 14
      for (int t = 0; t < ROW_VECTORS / 2; ++t) {
        const int q = lane + 64 * t;
        const int row = q / ROW_VECTORS, pixel = wave_m * BLOCKS * 32 + (q % ROW_VECTORS) * 4;
        const int n = n0 + wave_n * 32 * J + j * 32 + row;
        if (n < p.kernels && pixel < valid_pixels) {
          const Vector value = *reinterpret_cast<const Vector*>(lds + (wave_n * 32 + row) * RP + pixel);
          *reinterpret_cast<Vector*>(result + n * pixels + pixel) = value;
        }
      }
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_CONV_SLAB_HPP_
