// =================================================================================================
// Large-tile MFMA GEMM kernel for gfx950, fp32 and fp64. It stands where the reference has its
// "indirect" path (src/routines/level3/xgemm.cpp:102-222 with the kernels of
// src/kernels/level3/xgemm_part1-4.opencl, copy_pad/transpose_pad.opencl), but needs none of that
// path's pre- and post-kernels: both operand orientations, arbitrary leading dimensions and offsets
// and ragged edges are handled by the tile loaders and the epilogue of this one kernel.
//
// Structure (one work-group = 256 threads = 4 wavefronts):
//   * the work-group owns a TILE_M x TILE_N block of C; K is walked in slabs of TILE_K;
//   * a ring of three LDS slab buffers: while slab t feeds the matrix cores, slab t+1 has landed or is
//     landing and slab t+2 is being requested into the buffer that the previous barrier released; one
//     barrier per slab;
//   * both operands sit in LDS as [k][x] (x = m for A, n for B; x contiguous) whatever their layout in
//     memory: x-contiguous operands go from global memory straight into LDS (buffer loads with the LDS
//     as destination, 16 bytes per lane), k-contiguous ones are loaded into registers with 16-byte
//     loads along k and scattered into LDS (a transpose on the fly);
//   * each wavefront computes a (MF*FM) x (MF*FN) block with v_mfma_f32_32x32x2_f32 (MF = 32) or
//     v_mfma_f64_16x16x4_f64 (MF = 16). The n-indexed values are fed as the MFMA's A operand and the
//     m-indexed ones as its B operand, so the lanes of a result register run along m: stores to the
//     column-major C are contiguous per lane group. A lane owns FM consecutive m (one LDS read of
//     FM elements, one vector store of FM elements);
//   * the blockIdx -> tile mapping first makes the work-groups that the hardware deals round-robin to
//     one XCD (blockIdx % 8) logically contiguous, then walks C in groups of GROUP_M tile rows, so
//     the tiles in flight on one XCD share A and B panels in that XCD's L2.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_MFMA_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_MFMA_HPP_

#include <tuple>
#include <type_traits>

#include "kernels/gemm_args.hpp"

namespace clbh {

constexpr int kMfmaThreads = 256;
constexpr int kNumXcd = 8;

typedef float float16_t __attribute__((ext_vector_type(16)));
typedef double double4_t __attribute__((ext_vector_type(4)));

// ---- per-precision MFMA traits ---------------------------------------------------------------------
template <typename T> struct MfmaTraits;

template <> struct MfmaTraits<float> {
  static constexpr int MF = 32;       // the instruction computes an MF x MF block
  static constexpr int KP = 2;        // k extent of one instruction
  static constexpr int ACC = 16;      // accumulator elements per lane and block
  using Acc = float16_t;
  static __device__ __forceinline__ Acc Zero() { return Acc(0.0f); }
  static __device__ __forceinline__ Acc Mfma(const float rows, const float cols, const Acc acc) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(rows, cols, acc, 0, 0, 0);
  }
  // row of the MF x MF block held by accumulator element r of a lane in k-group g
  static __device__ __forceinline__ int Row(const int r, const int g) { return 8 * (r / 4) + 4 * g + (r % 4); }
};

template <> struct MfmaTraits<double> {
  static constexpr int MF = 16;
  static constexpr int KP = 4;
  static constexpr int ACC = 4;
  using Acc = double4_t;
  static __device__ __forceinline__ Acc Zero() { return Acc(0.0); }
  static __device__ __forceinline__ Acc Mfma(const double rows, const double cols, const Acc acc) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(rows, cols, acc, 0, 0, 0);
  }
  static __device__ __forceinline__ int Row(const int r, const int g) { return 4 * r + g; }
};

// fp32 with the 16 x 16 x 4 instruction: the same flops per cycle as 32 x 32 x 2 in blocks a quarter of the size, for
// tiles of 32 x 64 and below (more work-groups for mid-sized problems: two wavefronts per SIMD instead of one)
struct MfmaTraitsF32Small {
  static constexpr int MF = 16;
  static constexpr int KP = 4;
  static constexpr int ACC = 4;
  typedef float Acc __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ Acc Zero() { return Acc(0.0f); }
  static __device__ __forceinline__ Acc Mfma(const float rows, const float cols, const Acc acc) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(rows, cols, acc, 0, 0, 0);
  }
  static __device__ __forceinline__ int Row(const int r, const int g) { return 4 * g + r; }
};

// ---- tile configuration ----------------------------------------------------------------------------
// WM x WN wavefronts per work-group (WM * WN == 4), each owning FM x FN MFMA blocks.
template <typename T, int WM_, int WN_, int FM_, int FN_, int TILE_K_, int MIN_WAVES_ = 2, typename Traits_ = MfmaTraits<T>>
struct MfmaConfig {
  static constexpr int MIN_WAVES = MIN_WAVES_;  // wavefronts per SIMD the register budget must allow
  using Traits = Traits_;
  static constexpr int WM = WM_, WN = WN_, FM = FM_, FN = FN_;
  static constexpr int TILE_M = WM * FM * Traits::MF;
  static constexpr int TILE_N = WN * FN * Traits::MF;
  static constexpr int TILE_K = TILE_K_;
  static constexpr int VEC = 16 / sizeof(T);  // elements per 16-byte access
  // Row pitch of the LDS tiles in elements. pitch % (64 / VEC... ) is chosen so that the scattered
  // 4-byte (fp32) or 8-byte (fp64) stores of the k-contiguous loader fall into distinct banks: the 64
  // lanes of a wavefront write (TILE_K / VEC) different k rows, which must be (64 * 4 / sizeof(T)) /
  // (TILE_K / VEC) elements apart modulo the bank window.
  static constexpr int PAD = VEC;
  static constexpr int PITCH_M = TILE_M + PAD;
  static constexpr int PITCH_N = TILE_N + PAD;
  static constexpr int STAGES = 3;                                         // LDS slab buffers (a ring)
  static constexpr int LDS_ELEMS = STAGES * TILE_K * (PITCH_M + PITCH_N);
  static constexpr int CHUNKS_A = TILE_M * TILE_K / VEC / kMfmaThreads;  // 16-byte chunks per thread and slab
  static constexpr int CHUNKS_B = TILE_N * TILE_K / VEC / kMfmaThreads;
  static_assert(WM * WN * 64 == kMfmaThreads, "four wavefronts per work-group");
  static_assert(TILE_M * TILE_K % (VEC * kMfmaThreads) == 0 && TILE_N * TILE_K % (VEC * kMfmaThreads) == 0,
                "slab must divide evenly over the threads");
  static_assert(TILE_K % Traits::KP == 0 && TILE_K % VEC == 0, "slab depth");
};

// Vector types for LDS and global accesses; never assumed to be aligned beyond 16 bytes.
template <typename T, int N> struct VecType { typedef T type __attribute__((ext_vector_type(N), aligned(N * sizeof(T) < 16 ? N * sizeof(T) : 16))); };
template <typename T> struct VecType<T, 1> { typedef T type; };

template <typename V, typename T, int N>
__device__ __forceinline__ T VecGet(const V v, const int i) {
  if constexpr (N == 1) { return v; } else { return v[i]; }
}
template <typename V, typename T, int N>
__device__ __forceinline__ V VecWith(V v, const int i, const T value) {
  if constexpr (N == 1) { v = value; } else { v[i] = value; }
  return v;
}

// ---- slab movement ---------------------------------------------------------------------------------
// One operand slab is TILE_X x TILE_K elements; element (x, k) of the operand lives at
// base[KC ? x*ld + k : k*ld + x]. In LDS a slab is always [k][x]. All global reads are buffer loads: the
// resource of every load is cut off at the end of the operand's valid region, so elements outside the
// matrix are never touched and read as zero (the hardware checks the range per dword), and rows or
// columns of a tile that lie outside the matrix but inside that linear range read finite garbage that
// only reaches results nobody stores. No tile needs a special path.
//
// x-contiguous operand ("direct"): `buffer_load_dword[x4] ... lds` moves LANE_BYTES per lane straight
// into LDS, lane l landing at base + LANE_BYTES * l, so a wavefront fills WAVE_BYTES of contiguous LDS per
// instruction and no vector register or LDS store is spent on staging. A slab is kept as groups of R
// whole rows (R * row bytes == WAVE_BYTES; R == 1 with PARTS loads per row when a row is longer), groups
// GROUP_PITCH elements apart. LANE_BYTES is 16 when every address is 16-byte aligned, else 4.
// k-contiguous operand ("staged"): loaded into registers (16 bytes per piece when aligned, else one
// element) and scattered into LDS transposed; the same description with R == 1, i.e. plain rows.
template <typename T, int TILE_X, int TILE_K, bool DIRECT, int LANE_BYTES>
struct SlabLayout {
  static constexpr int VEC = 16 / sizeof(T);
  static constexpr int ROW_BYTES = TILE_X * sizeof(T), WAVE_BYTES = 64 * LANE_BYTES;
  static constexpr int WAVE_ELEMS = WAVE_BYTES / sizeof(T);
  static constexpr int R = (DIRECT && ROW_BYTES < WAVE_BYTES) ? WAVE_BYTES / ROW_BYTES : 1;      // rows per group
  static constexpr int PARTS = (DIRECT && ROW_BYTES > WAVE_BYTES) ? ROW_BYTES / WAVE_BYTES : 1;  // loads per row
  static constexpr int GROUPS = TILE_K / R;
  static constexpr int GROUP_PITCH = R * TILE_X + VEC;
  static constexpr int ELEMS = GROUPS * GROUP_PITCH;  // one stage
  static constexpr int LOADS = GROUPS * PARTS;        // wavefront-wide loads per slab
  static constexpr int LOADS_PER_WAVE = (LOADS + 3) / 4;
  static_assert(TILE_K % R == 0, "whole groups per slab");
  static_assert(PARTS == 1 || PARTS == 2 || PARTS == 4, "a wavefront always loads the same part of a row");
  // offset of element (k, 0)
  static __device__ __forceinline__ int Row(const int k) { return (k / R) * GROUP_PITCH + (k % R) * TILE_X; }
};

// Bytes from `from` to `end`, clamped to what a buffer resource can hold; both pointers are uniform.
__device__ __forceinline__ int RecordsUpTo(const void* from, const void* end) {
  const long long bytes = static_cast<const char*>(end) - static_cast<const char*>(from);
  // clamp to [0, 2^32 - 1] on the two 32-bit halves: stays on the scalar unit (it has no 64-bit compares)
  int high = static_cast<int>(bytes >> 32);
  const unsigned int low = static_cast<unsigned int>(bytes);
  asm("" : "+s"(high));  // opaque, or the halves are fused back into 64-bit vector compares
  return static_cast<int>(high < 0 ? 0u : (high != 0 ? 0xffffffffu : low));
}

constexpr int kRawBufferFlags = 0x00020000;  // untyped raw buffer (stride 0), range-checked against its byte count
// A buffer view of a tile of C is this many bytes long, so that a piece at this offset lies outside it (loads deliver
// zero, stores move nothing); leading dimensions below kViewMaxLd keep every piece of a tile (up to 128 columns of
// 8-byte elements) at a 32-bit offset inside.
constexpr int kViewOutside = 0x7fffff00;
constexpr long long kViewMaxLd = 1ll << 20;

// Byte offset of this lane inside the chunk a direct load moves.
template <typename T, int TILE_X, int TILE_K, int LANE_BYTES>
__device__ __forceinline__ int DirectLaneBytes(const long long ld, const int lane) {
  using L = SlabLayout<T, TILE_X, TILE_K, true, LANE_BYTES>;
  const int position = lane * LANE_BYTES;
  const int row = (L::R > 1) ? position / L::ROW_BYTES : 0, in_row = (L::R > 1) ? position % L::ROW_BYTES : position;
  return static_cast<int>(row * ld * static_cast<long long>(sizeof(T))) + in_row;
}

// Issues the round-th direct load of this wavefront for one slab. Tag only makes the
// instantiation unique per kernel: the host pass of hipcc 7.2 rejects a second kernel reusing a
// specialization of this function ("no matching function"), while the device pass accepts it. `slab` points at the slab's first
// element (x0, k0), `valid_end` behind the last element of the operand, `stage` at the LDS stage; all
// three are uniform over the work-group.
template <typename T, int TILE_X, int TILE_K, int LANE_BYTES, bool RANGE, typename Tag>
__device__ __forceinline__ void DirectLoad(const T* __restrict__ slab, const T* valid_end, const long long ld, T* stage,
                                           const int wave, const int lane_bytes, const int round) {
  using L = SlabLayout<T, TILE_X, TILE_K, true, LANE_BYTES>;
  static_assert(L::LOADS % 4 == 0, "every wavefront issues the same number of loads (the waits count them)");
  const int index = wave + 4 * round;
  const int group = index / L::PARTS, part = index % L::PARTS;
  const T* chunk = slab + static_cast<long long>(group * L::R) * ld + part * L::WAVE_ELEMS;
  typedef __attribute__((address_space(3))) void* LdsPtr;
  // (the buffer form, unlike the flat-encoded global form, leaves the LDS counter alone, so waits on LDS
  // reads stay counted instead of draining the queue)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(
      __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(chunk), 0, RANGE ? RecordsUpTo(chunk, valid_end) : -1, kRawBufferFlags),
      (LdsPtr)(stage + group * L::GROUP_PITCH + part * L::WAVE_ELEMS), LANE_BYTES, lane_bytes, 0, 0, 0);
}

// Gathered A operand (ConvGather). Once per slab the lanes of a wavefront decompose the TILE_K rows of the slab in
// parallel (lane l: row k0 + l of the patch matrix -> channel and kernel tap -> the offset of that tap in the image
// plane and its distance dh, dw from the top-left corner of a patch); the loads then pick their row's values with
// v_readlane, which keeps the per-load arithmetic to a handful of instructions.
struct GatherRows {
  int plane_offset, dh, dw;
};

template <int TILE_K>
__device__ __forceinline__ GatherRows DecomposeRows(const ConvGather& g, const int k0, const int k_len, const int lane) {
  const unsigned p = static_cast<unsigned>(k0 + lane % TILE_K);
  const unsigned channel = (g.taps == 1) ? p : __umulhi(p, g.taps_magic);
  const unsigned kernel_index = p - channel * g.taps;
  const unsigned tap = g.flip ? (g.taps - 1 - kernel_index) : kernel_index;
  const unsigned kh = (g.kernel_w == 1) ? tap : __umulhi(tap, g.kernel_w_magic);
  const unsigned kw = tap - kh * g.kernel_w;
  GatherRows rows;
  const int dh = static_cast<int>(kh) * g.dilation_h;
  rows.dw = static_cast<int>(kw) * g.dilation_w;
  rows.plane_offset = (static_cast<int>(channel) * g.height + dh) * g.width + rows.dw;
  rows.dh = (static_cast<int>(p) < k_len) ? dh : (1 << 28);  // a row beyond k fails every lane's bounds test
  return rows;
}

// The direct load of a gathered operand: the same instruction as DirectLoad with 4 bytes per lane, but every lane
// brings the offset of its own image element - or one beyond the resource's range, which reads as zero, for the
// padding around the image, for patches beyond m and for rows beyond k. `patch_h`, `patch_w` (top-left corner of the
// lane's patch in the padded image; -2^29 for patches beyond m) and `patch_offset` belong to the lane.
template <typename T, int TILE_X, int TILE_K, typename Tag>
__device__ __forceinline__ void GatherLoad(const T* __restrict__ image, const ConvGather& g, T* stage, const int wave,
                                           const int round, const GatherRows& rows, const int* patch_h,
                                           const int* patch_w, const int* patch_offset) {
  using L = SlabLayout<T, TILE_X, TILE_K, true, 4>;
  static_assert(L::R == 1 && sizeof(T) == 4 && TILE_K <= 64, "one row per load, dword elements, a lane per row");
  static_assert(L::LOADS % 4 == 0, "every wavefront issues the same number of loads (the waits count them)");
  const int index = wave + 4 * round;
  const int row = index / L::PARTS, part = index % L::PARTS;
  const int dh = __builtin_amdgcn_readlane(rows.dh, row), dw = __builtin_amdgcn_readlane(rows.dw, row);
  const int plane_offset = __builtin_amdgcn_readlane(rows.plane_offset, row);
  const int h = patch_h[part] + dh, w = patch_w[part] + dw;
  const bool inside = static_cast<unsigned>(h) < static_cast<unsigned>(g.height) &&
                      static_cast<unsigned>(w) < static_cast<unsigned>(g.width);
  const int offset_bytes = inside ? (plane_offset + patch_offset[part]) * 4 : static_cast<int>(0x80000000u);
  // The resource is uniform, but under register pressure the compiler keeps it in vector registers and then loops over
  // its distinct values around every load: take it from the first lane explicitly.
  const unsigned long long address = reinterpret_cast<unsigned long long>(image);
  const unsigned long long low = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(address)));
  const unsigned long long high = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(address >> 32)));
  T* uniform_image = reinterpret_cast<T*>((high << 32) | low);
  const int bytes = __builtin_amdgcn_readfirstlane(static_cast<int>(g.image_bytes));
  typedef __attribute__((address_space(3))) void* LdsPtr;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(__builtin_amdgcn_make_buffer_rsrc(uniform_image, 0, bytes, kRawBufferFlags),
                                           (LdsPtr)(stage + row * L::GROUP_PITCH + part * L::WAVE_ELEMS), 4, offset_bytes, 0,
                                           0, 0);
}

// Gathered operand, 16 bytes per lane: for images without padding, unit stride along the width and an output width
// that is a multiple of 4, four consecutive patches of an output row are four consecutive image elements for every
// tap, so a lane can fetch them in one piece and a wavefront needs ONE load per slab (64 patches x 16 rows: lanes
// 0..15 bring row 4 * wave of the slab, lanes 16..31 the next one, ...). Each lane decomposes its own row; the row a
// lane serves advances by TILE_K per slab. `patch_offset` is the lane's offset of its first patch in the image plane,
// or negative for patches beyond m.
template <typename T, int TILE_X, int TILE_K, typename Tag>
__device__ __forceinline__ void GatherLoadVector(const T* __restrict__ image, const ConvGather& g, T* stage, const int wave,
                                                 const int round, const int k0, const int k_len, const int lane,
                                                 const int patch_offset) {
  using L = SlabLayout<T, TILE_X, TILE_K, true, 16>;
  static_assert(L::PARTS == 1 && sizeof(T) == 4, "whole rows per load, dword elements");
  static_assert(L::LOADS % 4 == 0, "every wavefront issues the same number of loads (the waits count them)");
  const int group = wave + 4 * round;
  const unsigned p = static_cast<unsigned>(k0 + group * L::R + (lane * 16) / L::ROW_BYTES);
  const unsigned channel = (g.taps == 1) ? p : __umulhi(p, g.taps_magic);
  const unsigned kernel_index = p - channel * g.taps;
  const unsigned tap = g.flip ? (g.taps - 1 - kernel_index) : kernel_index;
  const unsigned kh = (g.kernel_w == 1) ? tap : __umulhi(tap, g.kernel_w_magic);
  const unsigned kw = tap - kh * g.kernel_w;
  const int plane_offset = (static_cast<int>(channel) * g.height + static_cast<int>(kh) * g.dilation_h) * g.width +
                           static_cast<int>(kw) * g.dilation_w;
  const bool inside = static_cast<int>(p) < k_len && patch_offset >= 0;
  const int offset_bytes = inside ? (plane_offset + patch_offset) * 4 : static_cast<int>(0x80000000u);
  const unsigned long long address = reinterpret_cast<unsigned long long>(image);
  const unsigned long long low = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(address)));
  const unsigned long long high = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(address >> 32)));
  T* uniform_image = reinterpret_cast<T*>((high << 32) | low);
  const int bytes = __builtin_amdgcn_readfirstlane(static_cast<int>(g.image_bytes));
  typedef __attribute__((address_space(3))) void* LdsPtr;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(__builtin_amdgcn_make_buffer_rsrc(uniform_image, 0, bytes, kRawBufferFlags),
                                           (LdsPtr)(stage + group * L::GROUP_PITCH), 16, offset_bytes, 0, 0, 0);
}

// Staged operand: thread t moves the pieces t, t + 256, ... of the slab (VL elements each, consecutive
// threads along k); with LINES whole x lines per round, piece c lies c * LINES lines after piece 0.
template <int TILE_X, int TILE_K, int VL>
struct StagedPieces {
  static constexpr int ALONG = TILE_K / VL;  // pieces per x line
  static_assert(kMfmaThreads % ALONG == 0, "whole lines per round of pieces");
  static constexpr int LINES = kMfmaThreads / ALONG;
  static constexpr int PIECES = TILE_X * TILE_K / VL / kMfmaThreads;
  static __device__ __forceinline__ int Line(const int tid) { return tid / ALONG; }
  static __device__ __forceinline__ int K(const int tid) { return (tid % ALONG) * VL; }
};

// `offset`: the lane's byte offset, the one the resource's range check looks at; `uniform_offset`: a byte offset common to
// the wavefront, added behind that check (it travels in a scalar register: no vector arithmetic per access).
template <typename T, int VL, typename Resource>
__device__ __forceinline__ typename VecType<T, VL>::type BufferLoad(const Resource resource, const int offset,
                                                                    const int uniform_offset = 0) {
  using V = typename VecType<T, VL>::type;
  constexpr int BYTES = VL * sizeof(T);
  if constexpr (BYTES == 4) { return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b32(resource, offset, uniform_offset, 0)); }
  else if constexpr (BYTES == 8) { return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b64(resource, offset, uniform_offset, 0)); }
  else if constexpr (BYTES == 16) { return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b128(resource, offset, uniform_offset, 0)); }
  else {
    static_assert(BYTES == 32, "piece size");  // two halves (an offset outside the resource stays outside: it is far from the end of the range)
    struct Halves { decltype(__builtin_amdgcn_raw_buffer_load_b128(resource, 0, 0, 0)) low, high; };
    Halves halves;
    halves.low = __builtin_amdgcn_raw_buffer_load_b128(resource, offset, uniform_offset, 0);
    halves.high = __builtin_amdgcn_raw_buffer_load_b128(resource, offset + 16, uniform_offset, 0);
    return __builtin_bit_cast(V, halves);
  }
}

template <typename T, int VL, typename V, typename Resource>
__device__ __forceinline__ void BufferStore(const V value, const Resource resource, const int offset, const int uniform_offset = 0) {
  typedef unsigned Dwords2 __attribute__((ext_vector_type(2)));
  typedef unsigned Dwords4 __attribute__((ext_vector_type(4)));
  constexpr int BYTES = VL * sizeof(T);
  static_assert(sizeof(V) == BYTES, "value type");
  if constexpr (BYTES == 4) { __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), resource, offset, uniform_offset, 0); }
  else if constexpr (BYTES == 8) { __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(Dwords2, value), resource, offset, uniform_offset, 0); }
  else if constexpr (BYTES == 32) {
    struct Halves { Dwords4 low, high; };
    const Halves halves = __builtin_bit_cast(Halves, value);
    BufferStore<unsigned, 4>(halves.low, resource, offset, uniform_offset);
    BufferStore<unsigned, 4>(halves.high, resource, offset + 16, uniform_offset);
  } else {
    static_assert(BYTES == 16, "piece size");
    const Dwords4 data = __builtin_bit_cast(Dwords4, value);
    __builtin_amdgcn_raw_buffer_store_b128(data, resource, offset, uniform_offset, 0);
    // A store of more than 64 bits reads its data registers over several cycles, and a vector instruction that
    // overwrites them right behind it can get there first: with the uniform offset in a scalar register the compiler
    // places no wait state between the two (it does for the other forms of the instruction), and on gfx950 the lanes
    // 12..15 of every row of 16 then stored the new contents of the upper two registers now and then (fp64 results of
    // the persistent kernel, one piece in fifty tiles). The wait states below read the data registers, so whatever
    // overwrites them comes behind.
    asm volatile("s_nop 1" ::"v"(data) : "memory");
  }
}

// Piece c of this thread for the slab at `slab` (element (x0, k0), uniform).
template <typename T, int TILE_X, int TILE_K, int VL, bool RANGE>
__device__ __forceinline__ typename VecType<T, VL>::type LoadPiece(const T* __restrict__ slab, const T* valid_end,
                                                                   const long long ld, const int lane_bytes, const int c) {
  using P = StagedPieces<TILE_X, TILE_K, VL>;
  const T* round = slab + static_cast<long long>(c * P::LINES) * ld;
  return BufferLoad<T, VL>(__builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(round), 0, RANGE ? RecordsUpTo(round, valid_end) : -1, kRawBufferFlags), lane_bytes);
}

// Registers -> LDS tile [k][x] of row pitch PITCH. CHECK zeroes the elements at k >= k_valid (the K tail:
// such elements lie inside the operand's linear range and hold the next line's data).
template <typename T, int TILE_X, int TILE_K, int PITCH, int VL, bool CHECK>
__device__ __forceinline__ void StorePiece(T* __restrict__ tile, const int tid, const int c,
                                           const typename VecType<T, VL>::type v, const int k_valid) {
  using P = StagedPieces<TILE_X, TILE_K, VL>;
  using V = typename VecType<T, VL>::type;
  const int x = P::Line(tid) + c * P::LINES, k = P::K(tid);
#pragma unroll
  for (int e = 0; e < VL; ++e) {
    T value = VecGet<V, T, VL>(v, e);
    if (CHECK && k + e >= k_valid) { value = T(0); }
    tile[(k + e) * PITCH + x] = value;
  }
}

// ---- blockIdx -> tile ------------------------------------------------------------------------------
// Work-groups are dealt to the XCDs round-robin; this index gives each XCD a contiguous range of 0 .. num_blocks - 1
__device__ __forceinline__ int XcdContiguousIndex(const int block, const int num_blocks) {
  const int per_xcd = (num_blocks + kNumXcd - 1) / kNumXcd;
  const int remainder = num_blocks % kNumXcd;
  const int tall = (remainder == 0) ? kNumXcd : remainder;  // XCDs that own per_xcd blocks
  const int xcd = block % kNumXcd, local = block / kNumXcd;
  return (xcd < tall) ? xcd * per_xcd + local : tall * per_xcd + (xcd - tall) * (per_xcd - 1) + local;
}

template <int GROUP_M = 8>
__device__ __forceinline__ void TileOfBlock(const int block, const int num_blocks, const int tiles_m,
                                            const int tiles_n, int& tile_m, int& tile_n) {
  // (1) a contiguous logical range per XCD
  const int logical = XcdContiguousIndex(block, num_blocks);
  // (2) grouped walk: GROUP_M tile rows at a time, column by column inside a group
  const int in_group = GROUP_M * tiles_n;
  const int group = logical / in_group;
  const int first_m = group * GROUP_M;
  const int group_rows = min(tiles_m - first_m, GROUP_M);
  tile_m = first_m + (logical % in_group) % group_rows;
  tile_n = (logical % in_group) / group_rows;
}

// The walk of launches with uneven work per tile (a triangle of C: tiles outside it leave at once; a triangular
// operand: the K range depends on the tile row or column). Work-groups are dispatched in index order and dealt to the
// XCDs round-robin, so the XCDs stay evenly loaded only if eight consecutive work-groups carry similar work: XCD x
// owns the tile columns x, x + 8, x + 16, ..., eight consecutive work-groups are eight neighbouring columns of one
// tile row, and inside its columns each XCD still walks GROUP_M rows at a time (operand reuse in its L2). The grid
// holds kNumXcd * tiles_m * ceil(tiles_n / kNumXcd) work-groups (see TriangleBlocks in the launchers); the function
// returns false for the ones beyond the last column. `operand_triangle` (kernels that give every tile a work-group of
// its own pass it): the tiles with the longest K range come first (TriangularRange: the last tile rows for 1, the last
// tile columns for 3, the first ones for 2 and 4), so that work-groups which start late fill the time the early ones
// leave instead of ending the launch on the longest tiles.
__device__ __forceinline__ bool TileOfBlockCyclic(const int block, const int tiles_m, const int tiles_n, int& tile_m,
                                                  int& tile_n, const int operand_triangle = 0) {
  const int xcd = block % kNumXcd, local = block / kNumXcd;
  constexpr int GROUP_M = 8;
  const int columns = (tiles_n + kNumXcd - 1) / kNumXcd;  // tile columns per XCD
  const int in_group = GROUP_M * columns;
  const int group = local / in_group;
  const int first_m = group * GROUP_M;
  const int group_rows = min(tiles_m - first_m, GROUP_M);
  tile_m = first_m + (local % in_group) % group_rows;
  const int column = ((local % in_group) / group_rows) * kNumXcd + xcd;
  tile_m = (operand_triangle == 1) ? tiles_m - 1 - tile_m : tile_m;
  tile_n = (operand_triangle == 3) ? tiles_n - 1 - column : column;
  return column < tiles_n;
}

// ---- the kernel ------------------------------------------------------------------------------------
// A_CONV != 0: the A operand is gathered from a batch of images (GemmArgs::conv); needs !A_KC and fp32. 1: one element
// per lane, any convolution; 2: four per lane (GatherLoadVector names the conditions).
template <typename T, typename Config, bool A_KC, bool B_KC, bool ALIGNED, int A_CONV = 0>
__global__ __launch_bounds__(kMfmaThreads, ALIGNED ? Config::MIN_WAVES : 2) void GemmMfmaKernel(const GemmArgs<T> p, const int tiles_m,
                                                               const int tiles_n) {
  using Traits = typename Config::Traits;
  using Acc = typename Traits::Acc;
  constexpr int MF = Traits::MF, KP = Traits::KP, ACC = Traits::ACC;
  constexpr int TILE_M = Config::TILE_M, TILE_N = Config::TILE_N, TILE_K = Config::TILE_K;
  constexpr int FM = Config::FM, FN = Config::FN, VEC = Config::VEC;
  // ALIGNED: 16-byte global accesses. fp32 and fp64 operands always qualify: the memory system wants dword
  // alignment only, whatever the offsets and leading dimensions are.
  constexpr int VL = ALIGNED ? VEC : 1;         // elements per staged global access
  constexpr int LANE_BYTES = ALIGNED ? 16 : 4;  // bytes per lane of a direct load
  constexpr bool A_DIRECT = !A_KC, B_DIRECT = !B_KC;
  static_assert(A_CONV == 0 || !A_KC, "a gathered operand takes the direct path");
  constexpr int LANE_BYTES_A = (A_CONV == 1) ? 4 : LANE_BYTES;  // the general gather moves single elements
  using LA = SlabLayout<T, TILE_M, TILE_K, A_DIRECT, LANE_BYTES_A>;
  using LB = SlabLayout<T, TILE_N, TILE_K, B_DIRECT, LANE_BYTES>;
  using PA = StagedPieces<TILE_M, TILE_K, VL>;
  using PB = StagedPieces<TILE_N, TILE_K, VL>;
  constexpr int STAGES = Config::STAGES;
  static_assert(STAGES == 3, "the tags of the slab walk assume a ring of three");
  static_assert(STAGES * (LA::ELEMS + LB::ELEMS) <= Config::LDS_ELEMS, "LDS allocation covers the layouts");
  constexpr int STAGED_A = A_DIRECT ? 0 : PA::PIECES, STAGED_B = B_DIRECT ? 0 : PB::PIECES;
  constexpr int STAGED = STAGED_A + STAGED_B;
  constexpr int KSTEPS = TILE_K / KP;
  static_assert(KSTEPS % 2 == 0, "fragment register sets alternate per k-step");
  constexpr int SLOTS = KSTEPS - 1;
  constexpr int PER_SLOT = (STAGED + SLOTS - 1) / SLOTS;
  using VM = typename VecType<T, FM>::type;
  using VN = typename VecType<T, FN>::type;
  using VP = typename VecType<T, VL>::type;
  using KernelTag = std::tuple<Config, std::integral_constant<int, A_CONV * 8 + (A_KC ? 4 : 0) | (B_KC ? 2 : 0) | (ALIGNED ? 1 : 0)>>;

  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  T* a_stages = lds;                       // [STAGES][LA::ELEMS]
  T* b_stages = lds + STAGES * LA::ELEMS;  // [STAGES][LB::ELEMS]

  const int tid = threadIdx.x;
  const int lane = tid % 64, wave = tid / 64;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wave_m = wave % Config::WM, wave_n = wave / Config::WM;
  const int lane_x = lane % MF;  // position along the lane dimension of the MFMA block
  const int lane_g = lane / MF;  // k-group of the lane inside one instruction

  // The tile, or the two tiles, of this work-group. With a triangular operand the K range of a tile grows or shrinks
  // with its row (its column, for the second operand): a launch of one work-group per tile leaves the compute units
  // that drew short tiles idle (two work-groups that share a compute unit are placed there by their index, so no order
  // of the walk evens that out). Such launches are folded instead: a work-group takes a tile of the first half of the
  // rows and then its mirror image in the second half, the two K ranges add up to the same length for every work-group.
  int tile_m, tile_n;
  int partner_m = -1, partner_n = -1;
  if ((p.c_triangle | p.operand_triangle) != 0) {
    const bool fold_rows = p.c_triangle == 0 && (p.operand_triangle == 1 || p.operand_triangle == 2);
    const bool fold_columns = p.c_triangle == 0 && p.operand_triangle >= 3;
    const int walk_m = fold_rows ? (tiles_m + 1) / 2 : tiles_m, walk_n = fold_columns ? (tiles_n + 1) / 2 : tiles_n;
    if (!TileOfBlockCyclic(blockIdx.x, walk_m, walk_n, tile_m, tile_n)) { return; }
    if (fold_rows && tiles_m - 1 - tile_m != tile_m) { partner_m = tiles_m - 1 - tile_m; partner_n = tile_n; }
    if (fold_columns && tiles_n - 1 - tile_n != tile_n) { partner_m = tile_m; partner_n = tiles_n - 1 - tile_n; }
  } else {
    // (the 32 tiles that an XCD's CUs hold at a time form GROUP_M rows of 32 / GROUP_M columns: as square a piece of C
    // as the tile's shape allows, so that the fewest operand panels pass through that XCD's L2)
    TileOfBlock<(TILE_M >= 2 * TILE_N) ? 4 : 8>(blockIdx.x, gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
  }
  for (int pass = 0; pass < 2; ++pass) {
    if (pass == 1) {
      if (partner_m < 0) { break; }
      tile_m = partner_m;
      tile_n = partner_n;
      __syncthreads();  // every wavefront has left the LDS buffers of the first tile
    }
    const int m0 = tile_m * TILE_M, n0 = tile_n * TILE_N;
    if (TileOutsideTriangle(p.c_triangle, m0, n0, TILE_M, TILE_N)) { continue; }  // uniform: the whole work-group leaves
    const bool masked = TileCrossesDiagonal(p.c_triangle, m0, n0, TILE_M, TILE_N);

    // LDS read offsets of this lane. Aligned operands: the lane owns FM consecutive m (one vector LDS read,
    // one vector store to C). Otherwise C is stored element-wise, and the lane owns m = lane_x, lane_x + MF,
    // ... so that the lanes of each scalar store cover consecutive addresses.
    constexpr bool M_INTERLEAVED = ALIGNED;
    const int a_read = wave_m * (FM * MF) + (M_INTERLEAVED ? lane_x * FM : lane_x);
    const int b_read = wave_n * (FN * MF) + lane_x * FN;
    static_assert((KP % LA::R == 0 || LA::R % KP == 0) && (KP % LB::R == 0 || LB::R % KP == 0), "row offsets add up");
    const int a_lane_row = LA::Row(lane_g) + a_read, b_lane_row = LB::Row(lane_g) + b_read;

    // Gathered A: the patches this lane loads (one per part of a tile row), as the top-left corner of the patch in the
    // padded image and the offset of that corner in the image plane; patches beyond m never pass the bounds test
    constexpr int GATHER_PARTS = (A_CONV == 1) ? LA::PARTS : 1;
    int patch_h[GATHER_PARTS], patch_w[GATHER_PARTS], patch_offset[GATHER_PARTS];
    if constexpr (A_CONV == 2) {  // the lane's four patches: first one at 4 * (lane % 16) of the tile row
      const int patch = m0 + (lane * 4) % TILE_M;
      const int oh = patch / p.conv.output_w, ow = patch - oh * p.conv.output_w;
      patch_offset[0] = (patch < p.m) ? oh * p.conv.stride_h * p.conv.width + ow : -1;
      patch_h[0] = patch_w[0] = 0;
    }
    if constexpr (A_CONV == 1) {
#pragma unroll
      for (int part = 0; part < GATHER_PARTS; ++part) {
        const int patch = m0 + part * LA::WAVE_ELEMS + lane;
        const int oh = patch / p.conv.output_w, ow = patch - oh * p.conv.output_w;
        const int corner_h = oh * p.conv.stride_h - p.conv.pad_h;
        patch_w[part] = ow * p.conv.stride_w - p.conv.pad_w;
        patch_offset[part] = corner_h * p.conv.width + patch_w[part];
        patch_h[part] = (patch < p.m) ? corner_h : -(1 << 29);
      }
    }

    for (int batch = blockIdx.y; batch < p.batch_count; batch += gridDim.y) {
      const T* a;
      const T* b;
      T* c;
      T alpha, beta;
      ResolveBatch<T, T>(p, batch, a, b, c, alpha, beta);
      int k_len = p.k;
      long long c_ld = p.c_ld;
      if (p.split_chunk > 0) {  // this "batch" is one K range of a single problem
        const int k_begin = batch * p.split_chunk;
        k_len = min(p.split_chunk, p.k - k_begin);
        a = static_cast<const T*>(p.a) + p.a_offset + (A_KC ? k_begin : k_begin * p.a_ld);
        b = static_cast<const T*>(p.b) + p.b_offset + (B_KC ? k_begin : k_begin * p.b_ld);
        c_ld = p.split_ld;
        c = static_cast<T*>(p.split_workspace) + static_cast<long long>(batch) * p.split_ld * p.n;
        alpha = T(1);
        beta = T(0);
      } else if (p.operand_triangle != 0) {  // skip the K range in which a triangular operand is zero
        int k_first;
        TriangularRange(p.operand_triangle, m0, n0, TILE_M, TILE_N, p.k, k_first, k_len);
        a += A_KC ? static_cast<long long>(k_first) : k_first * p.a_ld;
        b += B_KC ? static_cast<long long>(k_first) : k_first * p.b_ld;
      }
      const int slabs = (k_len + TILE_K - 1) / TILE_K;

      Acc acc[FM][FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int j = 0; j < FN; ++j) { acc[i][j] = Traits::Zero(); }
      }

      // Walk over the slabs, explicitly scheduled so that the matrix pipe never waits at a slab boundary even
      // with one wavefront per SIMD. Per k-step: LDS reads of the fragments of the NEXT k-step (other
      // register set), the FM x FN MFMAs of this k-step, then a share of the data movement for the coming
      // slabs: a direct operand's slab t+1 is requested in the first k-step of slab t; a staged operand
      // stores its slab t+1 into the other LDS buffer and refills the staging registers with slab t+2. One
      // barrier per slab, before its last k-step: by then every wavefront has finished its reads of the
      // current buffer and its writes to the other one, so the last k-step already fetches the first
      // fragments of slab t+1.
      const T* a_tile0 = a + (A_KC ? m0 * p.a_ld : static_cast<long long>(m0));  // element (m0, k = 0), uniform
      const T* b_tile0 = b + (B_KC ? n0 * p.b_ld : static_cast<long long>(n0));
      // behind the last element of the operand: (x = extent - 1, k = k_len - 1) + 1
      const T* a_end = a + (A_KC ? (p.m - 1) * p.a_ld + k_len : (k_len - 1) * p.a_ld + p.m);
      const T* b_end = b + (B_KC ? (p.n - 1) * p.b_ld + k_len : (k_len - 1) * p.b_ld + p.n);
      const int a_lane_bytes = A_DIRECT ? DirectLaneBytes<T, TILE_M, TILE_K, LANE_BYTES_A>(p.a_ld, lane)
                                        : static_cast<int>((PA::Line(tid) * p.a_ld + PA::K(tid)) * static_cast<long long>(sizeof(T)));
      const int b_lane_bytes = B_DIRECT ? DirectLaneBytes<T, TILE_N, TILE_K, LANE_BYTES>(p.b_ld, lane)
                                        : static_cast<int>((PB::Line(tid) * p.b_ld + PB::K(tid)) * static_cast<long long>(sizeof(T)));
      auto a_slab = [&](const int k0) { return a_tile0 + (A_KC ? static_cast<long long>(k0) : k0 * p.a_ld); };
      auto b_slab = [&](const int k0) { return b_tile0 + (B_KC ? static_cast<long long>(k0) : k0 * p.b_ld); };
      // The walk exists twice: with range-checked loads (tiles that touch an edge of the matrix, or a K
      // tail), and without (the resources then cover "everything", which saves the scalar arithmetic of one
      // byte count per load).
      auto walk = [&](auto range_tag) {
        constexpr bool RANGE = decltype(range_tag)::value;
        VP a_stage[STAGED_A > 0 ? STAGED_A : 1], b_stage[STAGED_B > 0 ? STAGED_B : 1];
        auto load_piece = [&](const int piece, const int k0) {
          if (piece < STAGED_A) { a_stage[piece] = LoadPiece<T, TILE_M, TILE_K, VL, RANGE>(a_slab(k0), a_end, p.a_ld, a_lane_bytes, piece); }
          else { b_stage[piece - STAGED_A] = LoadPiece<T, TILE_N, TILE_K, VL, RANGE>(b_slab(k0), b_end, p.b_ld, b_lane_bytes, piece - STAGED_A); }
        };
        auto store_piece = [&](const int piece, T* a_dst, T* b_dst, const int k0, auto check_tag) {
          constexpr bool CHECK = RANGE && decltype(check_tag)::value;
          if (piece < STAGED_A) {
            StorePiece<T, TILE_M, TILE_K, LA::GROUP_PITCH, VL, CHECK>(a_dst, tid, piece, a_stage[piece], k_len - k0);
          } else {
            StorePiece<T, TILE_N, TILE_K, LB::GROUP_PITCH, VL, CHECK>(b_dst, tid, piece - STAGED_A, b_stage[piece - STAGED_A], k_len - k0);
          }
        };
        // direct loads of one slab, numbered over both operands: A's rounds first
        constexpr int DIRECT_A = A_DIRECT ? LA::LOADS_PER_WAVE : 0, DIRECT_B = B_DIRECT ? LB::LOADS_PER_WAVE : 0;
        constexpr int DIRECT = DIRECT_A + DIRECT_B;
        constexpr int DIRECT_PER_SLOT = (DIRECT + SLOTS - 1) / SLOTS;
        GatherRows gather_rows{};  // of the slab whose loads are being issued (gathered A only)
        auto direct_load = [&](const int load, const int k0, auto* a_dst, auto* b_dst) {
          if constexpr (DIRECT_A > 0) {
            if (load < DIRECT_A) {
              if constexpr (A_CONV == 1) {
                GatherLoad<T, TILE_M, TILE_K, KernelTag>(a, p.conv, a_dst, wave_u, load, gather_rows, patch_h, patch_w, patch_offset);
              } else if constexpr (A_CONV == 2) {
                GatherLoadVector<T, TILE_M, TILE_K, KernelTag>(a, p.conv, a_dst, wave_u, load, k0, k_len, lane, patch_offset[0]);
              } else {
                DirectLoad<T, TILE_M, TILE_K, LANE_BYTES, RANGE, KernelTag>(a_slab(k0), a_end, p.a_ld, a_dst, wave_u, a_lane_bytes, load);
              }
            }
          }
          if constexpr (DIRECT_B > 0) {
            if (load >= DIRECT_A) { DirectLoad<T, TILE_N, TILE_K, LANE_BYTES, RANGE, KernelTag>(b_slab(k0), b_end, p.b_ld, b_dst, wave_u, b_lane_bytes, load - DIRECT_A); }
          }
        };
        auto read_a = [&](const T* stage, const int ks) {
          const T* src = stage + LA::Row(ks * KP) + a_lane_row;
          VM av;
          if constexpr (M_INTERLEAVED) {
            av = *reinterpret_cast<const VM*>(src);
          } else {
#pragma unroll
            for (int i = 0; i < FM; ++i) { av = VecWith<VM, T, FM>(av, i, src[i * MF]); }
          }
          return av;
        };
        auto read_b = [&](const T* stage, const int ks) {
          return *reinterpret_cast<const VN*>(stage + LB::Row(ks * KP) + b_lane_row);
        };

        // Prologue: slab 0 lands in buffer 0 and slab 1 is requested - its direct loads before the wait for slab 0, so that
        // the two memory latencies overlap (loads complete in order: when at most the direct loads of slab 1 are
        // outstanding, everything of slab 0 has arrived); its staged pieces once slab 0 has left the staging registers.
        if constexpr (A_CONV == 1) { gather_rows = DecomposeRows<TILE_K>(p.conv, 0, k_len, lane); }
#pragma unroll
        for (int load = 0; load < DIRECT; ++load) { direct_load(load, 0, a_stages, b_stages); }
#pragma unroll
        for (int piece = 0; piece < STAGED; ++piece) { load_piece(piece, 0); }
        if (slabs > 1) {
          if constexpr (A_CONV == 1) { gather_rows = DecomposeRows<TILE_K>(p.conv, TILE_K, k_len, lane); }
#pragma unroll
          for (int load = 0; load < DIRECT; ++load) { direct_load(load, TILE_K, a_stages + LA::ELEMS, b_stages + LB::ELEMS); }
          asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DIRECT) : "memory");
        } else {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
#pragma unroll
        for (int piece = 0; piece < STAGED; ++piece) { store_piece(piece, a_stages, b_stages, 0, std::true_type{}); }
        if (slabs > 1) {
#pragma unroll
          for (int piece = 0; piece < STAGED; ++piece) { load_piece(piece, TILE_K); }
        }
        __syncthreads();
        VM av[2];
        VN bv[2];
        av[0] = read_a(a_stages, 0);
        bv[0] = read_b(b_stages, 0);
        int cur = 0;  // ring position of the current slab; slab + 1 is in the next buffer, slab + 2 goes into the one before
        // One slab. STORE: slab + 1 exists (staged operands store it); LOAD: slab + 2 exists (direct operands
        // request it into the buffer that the barrier of the previous slab released, staged operands fetch it
        // into registers). Compile-time, so that the steady state has no branches; the slab stored without a
        // following load is the last one, the only one that can hold a K tail.
        auto slab_body = [&](const int slab, auto store_tag, auto load_tag) {
          constexpr bool STORE = decltype(store_tag)::value, LOAD = decltype(load_tag)::value;
          const int nxt = (cur == STAGES - 1) ? 0 : cur + 1, prv = (cur == 0) ? STAGES - 1 : cur - 1;
          const T* a_cur = a_stages + cur * LA::ELEMS;
          const T* b_cur = b_stages + cur * LB::ELEMS;
          T* a_nxt = a_stages + nxt * LA::ELEMS;
          T* b_nxt = b_stages + nxt * LB::ELEMS;
          T* a_prv = a_stages + prv * LA::ELEMS;
          T* b_prv = b_stages + prv * LB::ELEMS;
          const int k_store = (slab + 1) * TILE_K, k_load = (slab + 2) * TILE_K;
          if constexpr (A_CONV == 1 && LOAD) { gather_rows = DecomposeRows<TILE_K>(p.conv, k_load, k_len, lane); }
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) {
            const int set = ks % 2;
            if (ks + 1 < KSTEPS) {
              av[set ^ 1] = read_a(a_cur, ks + 1);
              bv[set ^ 1] = read_b(b_cur, ks + 1);
            } else {
              av[set ^ 1] = read_a(a_nxt, 0);
              bv[set ^ 1] = read_b(b_nxt, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < FM; ++i) {
#pragma unroll
              for (int j = 0; j < FN; ++j) {
                acc[i][j] = Traits::Mfma(VecGet<VN, T, FN>(bv[set], j), VecGet<VM, T, FM>(av[set], i), acc[i][j]);
              }
            }
            if (ks < KSTEPS - 1) {
#pragma unroll
              for (int u = 0; u < PER_SLOT; ++u) {
                const int piece = ks * PER_SLOT + u;
                if (piece < STAGED) {
                  if (STORE) { store_piece(piece, a_nxt, b_nxt, k_store, std::integral_constant<bool, !LOAD>{}); }
                  if (LOAD) { load_piece(piece, k_load); }
                }
              }
#pragma unroll
              for (int u = 0; u < DIRECT_PER_SLOT; ++u) {
                const int load = ks * DIRECT_PER_SLOT + u;
                if (LOAD && load < DIRECT) { direct_load(load, k_load, a_prv, b_prv); }
              }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (ks == KSTEPS - 2) {
              // slab + 1 must have landed for everybody: everything requested before this slab has to be
              // complete, this slab's own requests (slab + 2) may stay in flight (loads complete in order)
              if (LOAD) { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DIRECT + STAGED) : "memory"); }
              else { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
              asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            }
          }
          cur = nxt;
        };
        int slab = 0;
        for (; slab + 2 < slabs; ++slab) { slab_body(slab, std::true_type{}, std::true_type{}); }
        if (slab + 1 < slabs) { slab_body(slab, std::true_type{}, std::false_type{}); ++slab; }
        slab_body(slab, std::false_type{}, std::false_type{});
        __syncthreads();
      };
      // Lane owns m = m_base + i * M_STEP (i < FM); accumulator element r of block (i, j) is the column
      // n = n_base + FN * Row(r) + j.
      const int m_base = m0 + a_read;
      const int n_base = n0 + wave_n * (FN * MF);
      constexpr int M_STEP = M_INTERLEAVED ? 1 : MF;  // distance in m between the lane's accumulator blocks
      // 16-byte accesses to C need dword alignment only, which every fp32/fp64 address has
      typedef T VMG __attribute__((ext_vector_type(FM > 1 ? FM : 2), aligned(sizeof(T))));
      const bool vector_store = M_INTERLEAVED && (FM > 1) && (m_base + FM <= p.m) && !masked;
      auto writes = [&](const int i, const int n) {  // element i of the lane's piece of column n belongs to the result
        return n < p.n && m_base + i * M_STEP < p.m && (!masked || InTriangle(p.c_triangle, m_base + i * M_STEP, n));
      };
      // Small tiles (at most 16 registers of old C per lane) fetch the old C before the K walk when beta != 0: with a
      // short k the launch is a stream over C, and a work-group that asked for its C only after its last product would
      // wait out a second memory latency with nothing else to do (8191 x 8191 x 127: 0.27 -> 0.14 ms). The loads are the
      // oldest in the queue, so the first wait of the walk covers them.
      constexpr bool PREFETCH_C = FM * FN * ACC * sizeof(T) <= 64;
      T old_c[PREFETCH_C ? FM * FN * ACC : 1];
      if constexpr (PREFETCH_C) {
        if (beta != T(0)) {
#pragma unroll
          for (int j = 0; j < FN; ++j) {
#pragma unroll
            for (int r = 0; r < ACC; ++r) {
              const int n = n_base + FN * Traits::Row(r, lane_g) + j;
#pragma unroll
              for (int i = 0; i < FM; ++i) {
                old_c[(j * ACC + r) * FM + i] = writes(i, n) ? c[n * c_ld + m_base + i * M_STEP] : T(0);
              }
            }
          }
        }
      }

      if (m0 + TILE_M <= p.m && n0 + TILE_N <= p.n && k_len % TILE_K == 0) { walk(std::false_type{}); }
      else { walk(std::true_type{}); }

      // Epilogue.
      if constexpr (PREFETCH_C) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
          for (int r = 0; r < ACC; ++r) {
            const int n = n_base + FN * Traits::Row(r, lane_g) + j;
            T* dst = c + n * c_ld + m_base;
            if (vector_store && n < p.n) {
              VMG out;
#pragma unroll
              for (int i = 0; i < FM; ++i) {
                out[i] = (beta == T(0)) ? alpha * acc[i][j][r] : Combine(alpha, acc[i][j][r], beta, old_c[(j * ACC + r) * FM + i]);
              }
              *reinterpret_cast<VMG*>(dst) = out;
            } else {
#pragma unroll
              for (int i = 0; i < FM; ++i) {
                if (writes(i, n)) {
                  dst[i * M_STEP] = (beta == T(0)) ? alpha * acc[i][j][r] : Combine(alpha, acc[i][j][r], beta, old_c[(j * ACC + r) * FM + i]);
                }
              }
            }
          }
        }
      } else if (M_INTERLEAVED && FM > 1 && c_ld < kViewMaxLd) {
        // Large tiles whose lanes own runs of FM consecutive m: C through a buffer view of the tile, every piece at an
        // offset that lies outside the view where the piece does (columns from n on, lanes at or beyond the last row): such
        // loads deliver zeros and such stores move nothing. No branch stands between the pieces then, and the old C of
        // four columns is in flight together before the first of them is combined and stored (with one branch per piece
        // every load was waited for before the next one left). Lanes whose run straddles the last row, and tiles on the
        // diagonal of a triangle, move their elements one by one afterwards.
        // (64 bytes of old C per lane in flight)
        constexpr int WANTED = 64 / static_cast<int>(sizeof(VMG)) > 0 ? 64 / static_cast<int>(sizeof(VMG)) : 1;
        constexpr int BATCH = (ACC % WANTED == 0) ? WANTED : (ACC % 4 == 0) ? 4 : 1;
        // (the lane's place once more, opaque: what the epilogue derives from it is then computed here and not ahead of
        // the K walk, where it would occupy registers that the large tiles have none to spare of)
        int late_read = a_read, late_g = lane_g;
        asm volatile("" : "+v"(late_read), "+v"(late_g));
        const int late_m = m0 + late_read;
        const bool whole_run = (late_m + FM <= p.m) && !masked;
        const auto view = __builtin_amdgcn_make_buffer_rsrc(c + n0 * c_ld + m0, 0, kViewOutside, kRawBufferFlags);
        const int column_bytes = static_cast<int>(c_ld) * static_cast<int>(sizeof(T));
        const int lane_bytes = (n_base - n0) * column_bytes + late_read * static_cast<int>(sizeof(T));
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
          for (int r0 = 0; r0 < ACC; r0 += BATCH) {
            int offset[BATCH];
            VMG old[BATCH];
#pragma unroll
            for (int rr = 0; rr < BATCH; ++rr) {
              const int column = FN * Traits::Row(r0 + rr, late_g) + j;
              offset[rr] = (whole_run && n_base + column < p.n) ? lane_bytes + column * column_bytes : kViewOutside;
            }
            if (beta != T(0)) {
#pragma unroll
              for (int rr = 0; rr < BATCH; ++rr) { old[rr] = BufferLoad<T, FM>(view, offset[rr]); }
            }
#pragma unroll
            for (int rr = 0; rr < BATCH; ++rr) {
              const int r = r0 + rr;
              VMG out;
              if (beta == T(0)) {
#pragma unroll
                for (int i = 0; i < FM; ++i) { out[i] = alpha * acc[i][j][r]; }
              } else {
#pragma unroll
                for (int i = 0; i < FM; ++i) { out[i] = Combine(alpha, acc[i][j][r], beta, old[rr][i]); }
              }
              BufferStore<T, FM>(out, view, offset[rr]);
            }
            if (!whole_run) {
#pragma unroll
              for (int rr = 0; rr < BATCH; ++rr) {
                const int r = r0 + rr;
                const int n = n_base + FN * Traits::Row(r, late_g) + j;
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                  if (n < p.n && late_m + i < p.m && (!masked || InTriangle(p.c_triangle, late_m + i, n))) {
                    StoreResult<T, T>(c + n * c_ld + late_m, i, acc[i][j][r], alpha, beta);
                  }
                }
              }
            }
          }
        }
      } else {
        // Large tiles: the old C of four columns at a time is fetched before the first of them is combined and stored
        // (a load behind a store to memory that may alias it cannot be hoisted by the compiler).
        constexpr int BATCH = (ACC % 4 == 0) ? 4 : 1;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
          for (int r0 = 0; r0 < ACC; r0 += BATCH) {
            VMG old[BATCH];
            if (vector_store && beta != T(0)) {
#pragma unroll
              for (int rr = 0; rr < BATCH; ++rr) {
                const int n = n_base + FN * Traits::Row(r0 + rr, lane_g) + j;
                if (n < p.n) { old[rr] = *reinterpret_cast<const VMG*>(c + n * c_ld + m_base); }
              }
            }
#pragma unroll
            for (int rr = 0; rr < BATCH; ++rr) {
              const int r = r0 + rr;
              const int n = n_base + FN * Traits::Row(r, lane_g) + j;
              if (n >= p.n) { continue; }
              T* dst = c + n * c_ld + m_base;
              if (vector_store) {
                VMG out;
                if (beta == T(0)) {
#pragma unroll
                  for (int i = 0; i < FM; ++i) { out[i] = alpha * acc[i][j][r]; }
                } else {
#pragma unroll
                  for (int i = 0; i < FM; ++i) { out[i] = Combine(alpha, acc[i][j][r], beta, old[rr][i]); }
                }
                *reinterpret_cast<VMG*>(dst) = out;
              } else {
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                  if (writes(i, n)) { StoreResult<T, T>(dst, i * M_STEP, acc[i][j][r], alpha, beta); }
                }
              }
            }
          }
        }
      }
    }
  }
}

// Second pass of a split-K launch: C = alpha * (sum of the workspace slabs) + beta * C.
template <typename T>
__global__ __launch_bounds__(256) void GemmSplitReduceKernel(const T* __restrict__ workspace, const int splits,
                                                             const int split_ld, T* __restrict__ c, const long long c_ld,
                                                             const int m, const int n, const T alpha, const T beta) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int j = blockIdx.y;
  if (i >= m) { return; }
  const long long slab = static_cast<long long>(split_ld) * n;
  const T* src = workspace + static_cast<long long>(j) * split_ld + i;
  T sum = T(0);
  for (int s = 0; s < splits; ++s) { sum += src[s * slab]; }
  StoreResult<T, T>(c, j * c_ld + i, sum, alpha, beta);
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_MFMA_HPP_
