// =================================================================================================
// MFMA GEMM kernel for gfx950, fp16 storage with fp32 accumulation (HGEMM), for operands whose
// addresses are dword aligned (base and offsets multiples of 4 bytes, even leading dimensions). It
// replaces the reference's whole "indirect" chain (src/routines/level3/xgemm.cpp:102-222,
// src/kernels/level3/xgemm_part1-4.opencl) and its direct kernels (xgemm_direct_part1-3.opencl) with
// one launch that reads the caller's operands in place. Unlike the reference, which accumulates in
// fp16 (src/kernels/common.opencl:44-45), products are accumulated in fp32 by
// v_mfma_f32_16x16x32_f16 and rounded to fp16 once, in the epilogue. (Of the two fp16 shapes of gfx950 this one
// draws less power per flop: on uniform random operands a loop of nothing but MFMAs sustains 1.97 PFLOP/s with
// 16x16x32 and 1.71 PFLOP/s with 32x32x16 under the same power cap, and large HGEMMs run against that cap.)
//
// Structure:
//   * work-group tile (32*WM*FM) x (32*WN*FN), one wavefront per 2FM x 2FN blocks of 16 x 16; K is walked
//     in slabs of 32 - one MFMA deep - that live in a ring of LDS buffers;
//   * every slab goes global -> LDS directly (`buffer_load_dwordx4 ... lds`: lane l's 16 bytes land at
//     base + 16 * l, so LDS is filled in 1 KiB pieces whose inner order is fixed, while which 16 bytes of
//     global memory a lane fetches is free - that freedom carries the bank swizzles). The resources
//     are cut off at the end of the operand: loads beyond it touch no memory and deliver zero, so edge
//     tiles and the K tail of an x-contiguous operand need nothing special; the K tail of a
//     k-contiguous operand (whose out-of-range elements are the next line's data) is zeroed in LDS by
//     the wavefront that requested the piece;
//   * the MFMA wants 8 consecutive k per lane (lane l: row l % 16, k = 8 * (l / 16) ..). A k-contiguous
//     operand is kept as [x][32] (16-byte chunk c of row x at position c ^ ((x >> 2) & 3): the 16-byte reads
//     of 16 consecutive rows cover all 64 banks once) and read with one ds_read_b128 per fragment. An
//     x-contiguous operand is kept as [k][W] (chunk t of row k at t ^ swizzle(k)) and read with the CDNA4
//     transposing LDS read ds_read_b64_tr_b16. LDS serves 32 lanes of such a read per cycle: rows k..k+3 and
//     k+8..k+11, 32 bytes each, which the swizzle spreads over eight different 8-dword bank windows;
//   * explicit schedule, fenced for the compiler. The wavefront's blocks form four quadrants (halves of
//     its A blocks x halves of its B blocks) that are multiplied in the order (A0,B0) (A0,B1) (A1,B0) (A1,B1);
//     under the MFMAs of a quadrant the fragments that the next one lacks are read - B1, A1, then A0 and B0
//     of the next slab - so every fragment register is refilled right after its last use and no second
//     register set is needed. One barrier per slab, after the second quadrant, when all reads of the slab
//     have been issued: the second half of a slab already fetches the first fragments of the next one and
//     the matrix pipe never drains at a slab boundary;
//   * the m-indexed fragment is the MFMA's A operand, so a lane holds runs of four consecutive m; the
//     epilogue stages each block column through LDS and moves C in 16-byte pieces along m.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_DIRECT_F16_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_DIRECT_F16_HPP_

#include <type_traits>

#include "kernels/gemm_args.hpp"
#include "kernels/gemm_mfma.hpp"
#include "kernels/gemm_mfma_f16.hpp"

namespace clbh {

// WM x WN wavefronts per work-group, each owning FM x FN MFMA blocks of 32 x 32 (FM >= FN). MIN_WAVES is the
// number of wavefronts per SIMD the register budget must allow. STAGES slab buffers form the LDS ring: the slab
// STAGES - 1 ahead of the one being multiplied is on its way from memory.
template <int WM_, int WN_, int FM_, int FN_, int MIN_WAVES_, int STAGES_ = 3, bool STAGGER_ = false>
struct HdirectConfig {
  static constexpr bool STAGGER = STAGGER_;
  static constexpr int WM = WM_, WN = WN_, FM = FM_, FN = FN_, MIN_WAVES = MIN_WAVES_;
  static constexpr int WAVES = WM * WN, THREADS = 64 * WAVES;
  static constexpr int TILE_M = WM * FM * 32, TILE_N = WN * FN * 32, TILE_K = 32, STAGES = STAGES_;
  static constexpr int PIECES_A = TILE_M / 16, PIECES_B = TILE_N / 16;  // 1 KiB pieces of a slab
  static constexpr int ROUNDS = (PIECES_A + PIECES_B + WAVES - 1) / WAVES;  // requests per wavefront and slab
  static constexpr bool DUMMY = (PIECES_A + PIECES_B) % WAVES != 0;  // some requests go to a scratch piece
  static constexpr int A_ELEMS = PIECES_A * 512, B_ELEMS = PIECES_B * 512;  // halfs per stage
  static constexpr int RING_BYTES = (STAGES * (A_ELEMS + B_ELEMS) + (DUMMY ? 512 : 0)) * 2;
  static constexpr int EPILOGUE_BYTES = WAVES * 32 * (FM * 32 + 8) * 2;
  static constexpr int LDS_BYTES = RING_BYTES > EPILOGUE_BYTES ? RING_BYTES : EPILOGUE_BYTES;
  static_assert(FM >= FN, "the quarters of a k-step run over the m blocks");
};

// Chunk swizzle of row k of an x-contiguous slab [k][W]: one cycle of a transposing read takes 32 bytes from each
// of the rows k..k+3 and k+8..k+11 (k a multiple of 4), which must fall into eight different 8-dword bank windows.
template <int W>
__device__ __forceinline__ int HSwizzle(const int k) {
  const int by_octet = 2 * ((k >> 3) & 1);
  return by_octet ^ ((W >= 128) ? 4 * (k & 3) : (W == 64) ? 4 * ((k >> 1) & 1) : 0);
}

// Byte offset that lies outside every buffer view of C (views are this long): loads from there deliver zero, stores
// to there move nothing
constexpr int kHOutside = 0x7fffff00;

// Byte count from `from` to `end`, rounded up to whole dwords (the range check works per dword; the last
// one may hold a single valid half) and clamped to what a resource can hold.
__device__ __forceinline__ int HRecordsUpTo(const void* from, const void* end) {
  const long long bytes = (static_cast<const char*>(end) - static_cast<const char*>(from) + 3) & ~3ll;
  int high = static_cast<int>(bytes >> 32);
  const unsigned int low = static_cast<unsigned int>(bytes);
  asm("" : "+s"(high));  // opaque, or the halves are fused back into 64-bit vector compares
  return static_cast<int>(high < 0 ? 0u : (high != 0 ? 0xffffffffu : low));
}

// Requests one 1 KiB piece: `source` points at its first row (uniform), `lane_bytes` is the lane's byte offset
// from there (HPieceLaneBytes), `destination` the piece's place in the LDS stage (uniform).
template <bool RANGE, typename Tag>
__device__ __forceinline__ void HRequestPiece(const _Float16* __restrict__ source, const _Float16* valid_end,
                                              _Float16* destination, const int lane_bytes) {
  typedef __attribute__((address_space(3))) void* LdsPtr;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(
      __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(source), 0, RANGE ? HRecordsUpTo(source, valid_end) : -1,
                                        kRawBufferFlags),
      (LdsPtr)(destination), 16, lane_bytes, 0, 0, 0);
}

// The request of a lane for a piece of a gathered A operand (CONVGEMM without an im2col matrix, see ConvGather): the
// lane's 16 bytes are eight consecutive patches of one output row in row `p` of the patch matrix - eight consecutive
// image elements, for images without padding, unit stride along the width and an output width that is a multiple of
// 8. The loads move dwords, so an odd element offset cannot be fetched from the image itself: the host keeps a second
// copy of the images shifted by one element, copy_stride elements behind the first (copy[j] = image[j + 1]), and odd
// offsets read that one. With an even image width the parity is that of the tap's column offset. `patch_offset` is
// the offset of the lane's first patch in the image plane (even), or negative for patches beyond m; rows beyond k and
// those patches get an offset beyond the resource's range, which reads as zero.
template <typename Tag>
__device__ __forceinline__ void HGatherPiece(const _Float16* __restrict__ image, const ConvGather& g, _Float16* destination,
                                             const int p_row, const int k_len, const int patch_offset) {
  const unsigned p = static_cast<unsigned>(p_row);
  const unsigned channel = (g.taps == 1) ? p : __umulhi(p, g.taps_magic);
  const unsigned kernel_index = p - channel * g.taps;
  const unsigned tap = g.flip ? (g.taps - 1 - kernel_index) : kernel_index;
  const unsigned kh = (g.kernel_w == 1) ? tap : __umulhi(tap, g.kernel_w_magic);
  const unsigned kw = tap - kh * g.kernel_w;
  const int element = (static_cast<int>(channel) * g.height + static_cast<int>(kh) * g.dilation_h) * g.width +
                      static_cast<int>(kw) * g.dilation_w + patch_offset;
  const int aligned = (element & 1) ? element - 1 + g.copy_stride : element;
  const bool inside = p_row < k_len && patch_offset >= 0;
  const int offset_bytes = inside ? aligned * 2 : static_cast<int>(0x80000000u);
  // (the resource is taken from the first lane explicitly: under register pressure the compiler keeps it in vector
  // registers otherwise and loops over its distinct values around every load)
  const unsigned long long address = reinterpret_cast<unsigned long long>(image);
  const unsigned long long low = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(address)));
  const unsigned long long high = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(address >> 32)));
  _Float16* uniform_image = reinterpret_cast<_Float16*>((high << 32) | low);
  const int bytes = __builtin_amdgcn_readfirstlane(static_cast<int>(g.image_bytes));
  typedef __attribute__((address_space(3))) void* LdsPtr;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(__builtin_amdgcn_make_buffer_rsrc(uniform_image, 0, bytes, kRawBufferFlags),
                                           (LdsPtr)(destination), 16, offset_bytes, 0, 0, 0);
}

// Byte offset of a lane's 16 bytes from the first row of piece `piece`. KC: the piece is x rows
// 16*piece..+15 of 32 halfs; XC: k rows (512/W)*piece.. of W halfs. The lane's LDS position is fixed
// (16 * lane), the chunk it fetches carries the swizzle.
template <int W, bool KC>
__device__ __forceinline__ int HPieceLaneBytes(const long long ld, const int piece, const int lane) {
  constexpr int ROWS = KC ? 16 : 512 / W, CHUNKS = KC ? 4 : W / 8;  // rows of the piece, 16-byte chunks per row
  const int row = lane / CHUNKS, position = lane % CHUNKS;
  const int chunk = KC ? position ^ ((row >> 2) & 3) : position ^ HSwizzle<W>(ROWS * piece + row);
  return static_cast<int>((row * ld + 8 * chunk) * 2);
}

// After its own request for a k-contiguous piece has landed, the wavefront zeroes the elements k >= k_valid.
__device__ __forceinline__ void HZeroTail(_Float16* stage, const int piece, const int lane, const int k_valid) {
  const int row = lane / 4, chunk = (lane % 4) ^ ((row >> 2) & 3);
  half8_t* cell = reinterpret_cast<half8_t*>(stage + piece * 512 + lane * 8);
  if (8 * chunk + 7 >= k_valid) {
    half8_t value = *cell;
#pragma unroll
    for (int e = 0; e < 8; ++e) { if (8 * chunk + e >= k_valid) { value[e] = _Float16(0); } }
    *cell = value;
  }
}

// Offset (halfs) of a lane's fragment data for the block starting at x16 (a multiple of 16): the lane feeds row
// x16 + lane % 16 with k = 8 * (lane / 16) .. + 7.
template <int W, bool KC>
__device__ __forceinline__ int HFragmentOffset(const int lane, const int x16) {
  if (KC) {
    const int x = x16 + lane % 16;
    return x * 32 + 8 * ((lane / 16) ^ ((x >> 2) & 3));
  } else {
    // a group of 16 lanes reads a 4 (k) x 16 (x) block, four consecutive x per lane, and gets it back transposed:
    // lane q of the group then holds four consecutive k of column q
    const int group = lane / 16, q = lane % 16;
    const int k = 8 * group + q / 4;
    const int x = x16 + 4 * (q % 4);
    return k * W + 8 * ((x / 8) ^ HSwizzle<W>(k)) + x % 8;
  }
}

// Fragment of a stage.
template <int W, bool KC>
__device__ __forceinline__ half8_t HFragment(const _Float16* __restrict__ stage, const int offset) {
  if (KC) {
    return *reinterpret_cast<const half8_t*>(&stage[offset]);
  } else {
    typedef __attribute__((address_space(3))) short4_t* LdsPtr;
    const _Float16* src = stage + offset;
    const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(src));
    const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(src + 4 * W));  // rows k + 4: the same swizzle
    half8_t out;
    const half4_t lo_h = __builtin_bit_cast(half4_t, lo), hi_h = __builtin_bit_cast(half4_t, hi);
#pragma unroll
    for (int e = 0; e < 4; ++e) { out[e] = lo_h[e]; out[4 + e] = hi_h[e]; }
    return out;
  }
}

// ---- the kernel ------------------------------------------------------------------------------------
// A_CONV: the A operand is gathered from a batch of images (GemmArgs::conv, HGatherPiece); needs !A_KC.
template <typename Config, bool A_KC, bool B_KC, bool A_CONV = false>
__global__ __launch_bounds__(Config::THREADS, Config::MIN_WAVES) void HgemmDirectKernel(const GemmArgs<float> p, const int tiles_m,
                                                                  const int tiles_n) {
  using T = _Float16;
  constexpr int TILE_M = Config::TILE_M, TILE_N = Config::TILE_N, TILE_K = Config::TILE_K;
  constexpr int FM = Config::FM, FN = Config::FN, WAVES = Config::WAVES, STAGES = Config::STAGES, ROUNDS = Config::ROUNDS;
  constexpr int BM = 2 * FM, BN = 2 * FN;  // the wavefront's blocks of 16 x 16
  constexpr int AHEAD = STAGES - 1;        // slabs on their way or landed beyond the current one, in the steady state
  static_assert(TILE_K == 32 && (STAGES == 3 || STAGES == 4), "a slab is one MFMA deep; the waits below count up to three slabs");
  typedef float float4_t __attribute__((ext_vector_type(4)));
  static_assert(!A_CONV || !A_KC, "a gathered operand is x-contiguous in LDS");
  using KernelTag = std::tuple<Config, std::integral_constant<int, (A_CONV ? 4 : 0) | (A_KC ? 2 : 0) | (B_KC ? 1 : 0)>>;

  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  T* a_ring = lds;                               // [STAGES][A_ELEMS]
  T* b_ring = lds + STAGES * Config::A_ELEMS;    // [STAGES][B_ELEMS]
  T* scratch_piece = lds + STAGES * (Config::A_ELEMS + Config::B_ELEMS);

  const int tid = threadIdx.x;
  const int lane = tid % 64, wave = tid / 64;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wave_m = wave % Config::WM, wave_n = wave / Config::WM;

  int tile_m, tile_n;
  if ((p.c_triangle | p.operand_triangle) != 0) {
    if (!TileOfBlockCyclic(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n, p.operand_triangle)) { return; }
  } else {
    TileOfBlock(blockIdx.x, gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
  }
  const int m0 = tile_m * TILE_M, n0 = tile_n * TILE_N;
  if (TileOutsideTriangle(p.c_triangle, m0, n0, TILE_M, TILE_N)) { return; }  // uniform: the whole work-group leaves
  const bool masked = TileCrossesDiagonal(p.c_triangle, m0, n0, TILE_M, TILE_N);

  int a_offset[BM], b_offset[BN];
#pragma unroll
  for (int q = 0; q < BM; ++q) { a_offset[q] = HFragmentOffset<TILE_M, A_KC>(lane, (wave_m * BM + q) * 16); }
#pragma unroll
  for (int q = 0; q < BN; ++q) { b_offset[q] = HFragmentOffset<TILE_N, B_KC>(lane, (wave_n * BN + q) * 16); }

  for (int batch = blockIdx.y; batch < p.batch_count; batch += gridDim.y) {
    const T* a;
    const T* b;
    T* c;
    float alpha, beta;
    ResolveBatch<T, float>(p, batch, a, b, c, alpha, beta);
    int k_len = p.k;
    if (p.split_chunk > 0) {  // this "batch" is one K range of a single problem (ranges are multiples of 64 deep)
      const int k_begin = batch * p.split_chunk;
      k_len = min(p.split_chunk, p.k - k_begin);
      a = static_cast<const T*>(p.a) + p.a_offset + (A_KC ? static_cast<long long>(k_begin) : k_begin * p.a_ld);
      b = static_cast<const T*>(p.b) + p.b_offset + (B_KC ? static_cast<long long>(k_begin) : k_begin * p.b_ld);
    } else if (p.operand_triangle != 0) {  // skip the K range in which a triangular operand is zero
      int k_first;
      TriangularRange(p.operand_triangle, m0, n0, TILE_M, TILE_N, p.k, k_first, k_len);
      a += A_KC ? static_cast<long long>(k_first) : k_first * p.a_ld;
      b += B_KC ? static_cast<long long>(k_first) : k_first * p.b_ld;
    }
    const int slabs = (k_len + TILE_K - 1) / TILE_K;
    const int k_tail = k_len % TILE_K;  // valid depth of the last slab when it is partial

    float4_t acc[BM][BN];
#pragma unroll
    for (int i = 0; i < BM; ++i) {
#pragma unroll
      for (int j = 0; j < BN; ++j) { acc[i][j] = float4_t(0.0f); }
    }

    const T* a_tile0 = a + (A_KC ? m0 * p.a_ld : static_cast<long long>(m0));  // element (m0, k = 0), uniform
    const T* b_tile0 = b + (B_KC ? n0 * p.b_ld : static_cast<long long>(n0));
    // behind the last element of the operand: (x = extent - 1, k = k_len - 1) + 1
    const T* a_end = a + (A_KC ? (p.m - 1) * p.a_ld + k_len : (k_len - 1) * p.a_ld + p.m);
    const T* b_end = b + (B_KC ? (p.n - 1) * p.b_ld + k_len : (k_len - 1) * p.b_ld + p.n);

    // The walk exists twice: with range-checked requests (tiles that touch an edge of the matrix, or a K
    // tail), and without (saves the scalar arithmetic of one byte count per request).
    auto walk = [&](auto range_tag) {
      constexpr bool RANGE = decltype(range_tag)::value;
      // Request `round` of this wavefront: which piece, where its rows start inside a slab (elements), the
      // lane's byte offset and the piece's place inside a stage; all constant over the K walk.
      const T* a_request = a_tile0;  // first row of the slab to be requested next
      const T* b_request = b_tile0;
      const long long a_step = A_KC ? static_cast<long long>(TILE_K) : TILE_K * p.a_ld;
      const long long b_step = B_KC ? static_cast<long long>(TILE_K) : TILE_K * p.b_ld;
      long long piece_start[ROUNDS];
      int piece_lane_bytes[ROUNDS], piece_place[ROUNDS];
      int gather_row[A_CONV ? ROUNDS : 1];  // gathered A: the row of the slab a lane serves in a round
      int request_k = 0;                    // first row of the slab to be requested next
#pragma unroll
      for (int round = 0; round < ROUNDS; ++round) {
        const int piece = wave_u + WAVES * round;
        if ((Config::PIECES_A % WAVES == 0) ? (round < Config::PIECES_A / WAVES) : (piece < Config::PIECES_A)) {
          piece_start[round] = static_cast<long long>((A_KC ? 16 : 512 / TILE_M) * piece) * p.a_ld;
          piece_lane_bytes[round] = HPieceLaneBytes<TILE_M, A_KC>(p.a_ld, piece, lane);
          piece_place[round] = piece * 512;
          if constexpr (A_CONV) {
            // the lane's row of the piece and its (swizzled) chunk of eight patches, as in HPieceLaneBytes; in place of
            // the byte offset the offset of the first of these patches in the image plane, or -1 beyond m
            constexpr int ROWS = 512 / TILE_M, CHUNKS = TILE_M / 8;
            const int row = ROWS * piece + lane / CHUNKS;
            const int chunk = (lane % CHUNKS) ^ HSwizzle<TILE_M>(row);
            const int patch = m0 + 8 * chunk;
            const int oh = patch / p.conv.output_w, ow = patch - oh * p.conv.output_w;
            gather_row[round] = row;
            piece_lane_bytes[round] = (patch < p.m) ? oh * p.conv.stride_h * p.conv.width + ow : -1;
          }
        } else {
          const int b_piece = piece - Config::PIECES_A;
          piece_start[round] = static_cast<long long>((B_KC ? 16 : 512 / TILE_N) * b_piece) * p.b_ld;
          piece_lane_bytes[round] = HPieceLaneBytes<TILE_N, B_KC>(p.b_ld, b_piece, lane);
          piece_place[round] = b_piece * 512;
        }
      }
      // requests piece `round` of the slab at a_request / b_request into ring position `buffer`
      // (when the pieces of A fill whole rounds, the operand of a round is known at compile time: no branch
      // stands between the MFMAs)
      auto is_a = [&](const int round, const int piece) {
        return (Config::PIECES_A % WAVES == 0) ? (round < Config::PIECES_A / WAVES) : (piece < Config::PIECES_A);
      };
      auto request = [&](const int round, const int buffer) {
        const int piece = wave_u + WAVES * round;
        if (is_a(round, piece)) {
          if constexpr (A_CONV) {
            HGatherPiece<KernelTag>(a, p.conv, a_ring + buffer * Config::A_ELEMS + piece_place[round],
                                    request_k + gather_row[round], k_len, piece_lane_bytes[round]);
          } else {
            HRequestPiece<RANGE, KernelTag>(a_request + piece_start[round], a_end,
                                            a_ring + buffer * Config::A_ELEMS + piece_place[round], piece_lane_bytes[round]);
          }
        } else if (!Config::DUMMY || piece < Config::PIECES_A + Config::PIECES_B) {
          HRequestPiece<RANGE, KernelTag>(b_request + piece_start[round], b_end,
                                          b_ring + buffer * Config::B_ELEMS + piece_place[round], piece_lane_bytes[round]);
        } else {
          // keeps the number of outstanding requests equal in all wavefronts (the waits count them): an
          // empty resource moves nothing but zeros, into a piece nobody reads
          typedef __attribute__((address_space(3))) void* LdsPtr;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(__builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(a_tile0), 0, 0, kRawBufferFlags),
                                                   (LdsPtr)(scratch_piece), 16, lane * 16, 0, 0, 0);
        }
      };
      auto next_request_slab = [&]() { a_request += a_step; b_request += b_step; request_k += TILE_K; };
      // zeroes the K tail of the k-contiguous pieces this wavefront requested for the slab in `buffer`
      auto zero_tail = [&](const int buffer) {
        if (!RANGE || k_tail == 0 || !(A_KC || B_KC)) { return; }
#pragma unroll
        for (int round = 0; round < ROUNDS; ++round) {
          const int piece = wave_u + WAVES * round;
          if (piece < Config::PIECES_A) {
            if (A_KC) { HZeroTail(a_ring + buffer * Config::A_ELEMS, piece, lane, k_tail); }
          } else if (piece < Config::PIECES_A + Config::PIECES_B) {
            if (B_KC) { HZeroTail(b_ring + buffer * Config::B_ELEMS, piece - Config::PIECES_A, lane, k_tail); }
          }
        }
      };

      // Prologue: the first AHEAD slabs are requested into ring positions 0, 1, ...; slab 0 must have landed.
      const int first_slabs = min(slabs, AHEAD);
#pragma unroll
      for (int s = 0; s < AHEAD; ++s) {
        if (s < first_slabs) {
#pragma unroll
          for (int round = 0; round < ROUNDS; ++round) { request(round, s); }
          next_request_slab();
        }
      }
      if (first_slabs == 1) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
      else if (first_slabs == 2) { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(ROUNDS) : "memory"); }
      else { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * ROUNDS) : "memory"); }
      if (slabs == 1) { zero_tail(0); }
      __syncthreads();
      // Fragments: the halves A0, A1 of the wavefront's A blocks and B0, B1 of its B blocks, one register set each
      half8_t a_frag[2][FM], b_frag[2][FN];
#pragma unroll
      for (int q = 0; q < FM; ++q) { a_frag[0][q] = HFragment<TILE_M, A_KC>(a_ring, a_offset[q]); }
#pragma unroll
      for (int q = 0; q < FN; ++q) { b_frag[0][q] = HFragment<TILE_N, B_KC>(b_ring, b_offset[q]); }
      int cur = 0;  // ring position of the current slab; slab + s is s positions on, slab + AHEAD goes into the one before
      // One slab. LATER (compile-time, so that the steady state has no branches): how many slabs follow this one, capped
      // at AHEAD. LATER == AHEAD: slab + AHEAD exists and is requested into the buffer that the barrier of the previous
      // slab released.
      // Ring of three: slab + 2 is requested under the first two quadrants, into the buffer whose reads everybody had
      // finished (waited for) at the previous barrier. Ring of four: slab + 3 is requested under the last two quadrants,
      // after this slab's barrier, into the buffer of slab - 1 - every wavefront has consumed its last fragments of that
      // slab before it reached this barrier, so the barrier need not wait for LDS reads and their latency stays hidden.
      constexpr int REQUEST_QUADRANT = (STAGES == 4) ? 2 : 0;
      // STAGGER: the two halves of the work-group issue their requests under different quadrants. (Wavefronts issue in
      // order and a 1 KiB request occupies the memory pipeline's front end for 16 cycles: when all wavefronts reach a
      // request in the same cycles, the last one in the queue cannot issue its next MFMAs for 100 cycles.)
      constexpr int REQUEST_SLOTS = Config::STAGGER ? FM : 2 * FM;  // MFMA groups that carry a share of the requests each
      constexpr int PER_SLOT = (ROUNDS + REQUEST_SLOTS - 1) / REQUEST_SLOTS;
      auto slab_body = [&](auto later_tag, auto phase_tag) {
        constexpr int LATER = decltype(later_tag)::value;
        constexpr int PHASE = decltype(phase_tag)::value;
        constexpr bool LOAD = LATER == AHEAD;
        const int nxt = (cur == STAGES - 1) ? 0 : cur + 1, prv = (cur == 0) ? STAGES - 1 : cur - 1;
        const T* a_cur = a_ring + cur * Config::A_ELEMS;
        const T* b_cur = b_ring + cur * Config::B_ELEMS;
        const T* a_nxt = a_ring + nxt * Config::A_ELEMS;
        const T* b_nxt = b_ring + nxt * Config::B_ELEMS;
        // quadrant (A half ha, B half hb); under its MFMAs the fragments the next quadrant lacks are read: B1, A1 (this
        // slab), then A0, B0 (next slab)
#pragma unroll
        for (int quadrant = 0; quadrant < 4; ++quadrant) {
          const int ha = quadrant / 2, hb = quadrant % 2;
#pragma unroll
          for (int q = 0; q < FM; ++q) {
            // the reads of a quadrant go with its first groups of MFMAs, one fragment each
            if (quadrant == 0 || quadrant == 3) {
              if (q < FN) {
                if (quadrant == 0) { b_frag[1][q] = HFragment<TILE_N, B_KC>(b_cur, b_offset[FN + q]); }
                else { b_frag[0][q] = HFragment<TILE_N, B_KC>(b_nxt, b_offset[q]); }
              }
            } else if (quadrant == 1) {
              a_frag[1][q] = HFragment<TILE_M, A_KC>(a_cur, a_offset[FM + q]);
            } else {
              a_frag[0][q] = HFragment<TILE_M, A_KC>(a_nxt, a_offset[q]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              acc[ha * FM + q][hb * FN + j] =
                  __builtin_amdgcn_mfma_f32_16x16x32_f16(a_frag[ha][q], b_frag[hb][j], acc[ha * FM + q][hb * FN + j], 0, 0, 0);
            }
            // spread over the groups: a burst of identical requests from all work-groups defeats the L2
            if (LOAD && (Config::STAGGER ? quadrant == REQUEST_QUADRANT + PHASE
                                         : (quadrant >= REQUEST_QUADRANT && quadrant < REQUEST_QUADRANT + 2))) {
#pragma unroll
              for (int u = 0; u < PER_SLOT; ++u) {
                const int round = ((Config::STAGGER ? 0 : quadrant - REQUEST_QUADRANT) * FM + q) * PER_SLOT + u;
                if (round < ROUNDS) { request(round, prv); }
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          }
          if (quadrant == 1) {
            // slab + 1 must have landed for everybody; the requests for the slab behind it may stay in flight
            constexpr int IN_FLIGHT = (LATER >= 2) ? ROUNDS : 0;
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IN_FLIGHT) : "memory");
            if (LATER == 1) { zero_tail(nxt); }  // slab + 1 is the last one
            // (the zeroed tail must be in LDS, not on its way, when the others pass the barrier)
            if (STAGES == 4 && LATER != 1) { asm volatile("s_barrier" ::: "memory"); }
            else { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
          }
        }
        cur = nxt;
        if (LOAD) { next_request_slab(); }
      };
      int slab = 0;
      using Phase0 = std::integral_constant<int, 0>;
      if (Config::STAGGER && wave_u >= WAVES / 2) {
        for (; slab + AHEAD < slabs; ++slab) { slab_body(std::integral_constant<int, AHEAD>{}, std::integral_constant<int, 1>{}); }
      } else {
        for (; slab + AHEAD < slabs; ++slab) { slab_body(std::integral_constant<int, AHEAD>{}, Phase0{}); }
      }
      if constexpr (AHEAD >= 3) {
        if (slab + 2 < slabs) { slab_body(std::integral_constant<int, 2>{}, Phase0{}); ++slab; }
      }
      if (slab + 1 < slabs) { slab_body(std::integral_constant<int, 1>{}, Phase0{}); ++slab; }
      slab_body(std::integral_constant<int, 0>{}, Phase0{});
    };
    if (m0 + TILE_M <= p.m && n0 + TILE_N <= p.n && k_tail == 0) { walk(std::false_type{}); }
    else { walk(std::true_type{}); }

    // Epilogue, staged through LDS so that global memory sees whole lines. The four accumulator elements of a
    // lane are the rows m = 4*(lane/16) + 0..3 of column n = lane%16 of a 16 x 16 block. Per pair j of block
    // columns a wavefront owns a [32 n][WAVE_M m] fp16 staging tile of its own: C (when beta != 0) comes in
    // with 16-byte accesses along m, every lane combines its four consecutive m in fp32 and rounds once, and
    // the finished rows leave with 16-byte stores. Only wavefront-local ordering is needed (LDS operations of
    // a wavefront complete in order).
    if (p.split_chunk > 0) {
      // Split-K: the fp32 partial sums go to slab `batch` of the workspace (column-major, leading dimension split_ld,
      // a multiple of 4 >= m), four consecutive m per store; a second kernel adds the slabs and applies alpha and beta.
      float* partial = static_cast<float*>(p.split_workspace) + static_cast<long long>(batch) * p.split_ld * p.n;
      typedef float float4u_t __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int j = 0; j < BN; ++j) {
        const int n_index = n0 + (wave_n * BN + j) * 16 + lane % 16;
#pragma unroll
        for (int i = 0; i < BM; ++i) {
          const int m_index = m0 + (wave_m * BM + i) * 16 + 4 * (lane / 16);
          if (n_index < p.n && m_index < p.split_ld) {
            float4u_t out;
#pragma unroll
            for (int e = 0; e < 4; ++e) { out[e] = acc[i][j][e]; }
            *reinterpret_cast<float4u_t*>(partial + static_cast<long long>(n_index) * p.split_ld + m_index) = out;
          }
        }
      }
      __syncthreads();  // the next K range refills the slab buffers
    } else {
      constexpr int WAVE_M = FM * 32, STAGE_PITCH = WAVE_M + 8;
      constexpr int LANES_PER_ROW = WAVE_M / 8, ROWS_PER_PASS = 64 / LANES_PER_ROW, PASSES = 32 / ROWS_PER_PASS;
      T* stage = lds + wave * (32 * STAGE_PITCH);
      const int wave_m0 = m0 + wave_m * WAVE_M;
      // (the pieces of a block column are addressed by 32-bit byte offsets from its first element)
      const bool vector_rows = (p.c_ld % 2 == 0) && ((reinterpret_cast<unsigned long long>(c) & 3) == 0) && !masked &&
                               p.c_ld < (1 << 24);
      auto wave_fence = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      };
      // (the lane number once more, opaque: what the epilogue derives from it is then computed here and not ahead of the
      // K walk, where it would sit in registers that the walk has none to spare of - the 256 x 256 tile spilled 150)
      int late_lane = lane;
      asm volatile("" : "+v"(late_lane));
      // moves the staging tile's rows from (LOAD) or to (!LOAD) the block column starting at n_blk
      auto rows = [&](const int n_blk, auto load_tag) {
        constexpr bool LOAD = decltype(load_tag)::value;
        if (vector_rows) {
          // C through a buffer view of the block column, every piece at an offset that lies outside the view where the
          // piece does (rows from n on, m from the matrix's last row on): such loads deliver zeros and such stores move
          // nothing, so no branch stands between the passes and all loads of a block column are in flight together
          // (with a branch per pass each load was waited for before the next one left).
          const auto view = __builtin_amdgcn_make_buffer_rsrc(c + n_blk * p.c_ld + wave_m0, 0, kHOutside, kRawBufferFlags);
          const int rows_left = p.n - n_blk;
          const int first_row = late_lane / LANES_PER_ROW, col = 8 * (late_lane % LANES_PER_ROW);
          const int inside = p.m - (wave_m0 + col);  // how many of the lane's eight m lie inside the matrix
          const int lane_offset = (first_row * static_cast<int>(p.c_ld) + col) * 2;
          const int pass_step = ROWS_PER_PASS * static_cast<int>(p.c_ld) * 2;
          T* cells = &stage[first_row * STAGE_PITCH + col];
          // (four passes at a time: more pieces in flight cost the 256 x 256 tile, whose accumulators fill half of the
          // registers, spills)
          constexpr int GROUP = PASSES < 4 ? PASSES : 4;
          const auto offset_of = [&](const int pass) {
            const bool there = pass * ROWS_PER_PASS + first_row < rows_left && inside >= 8;
            return there ? lane_offset + pass * pass_step : kHOutside;
          };
#pragma unroll
          for (int group = 0; group < PASSES; group += GROUP) {
            half8_t pieces[GROUP];
            if (LOAD) {
#pragma unroll
              for (int g = 0; g < GROUP; ++g) { pieces[g] = BufferLoad<T, 8>(view, offset_of(group + g)); }
            }
#pragma unroll
            for (int g = 0; g < GROUP; ++g) {
              half8_t* local = reinterpret_cast<half8_t*>(cells + (group + g) * ROWS_PER_PASS * STAGE_PITCH);
              if (LOAD) { *local = pieces[g]; }
              else { BufferStore<T, 8>(*local, view, offset_of(group + g)); }
            }
          }
          // A wavefront on the m edge of the matrix: the one piece per row that straddles the last row of C moves
          // element by element, in the same way (the pieces before it above, as whole pieces).
          if (wave_m0 + WAVE_M > p.m) {
            const bool straddles = inside > 0 && inside < 8;
#pragma unroll
            for (int pass = 0; pass < PASSES; ++pass) {
              const bool there = pass * ROWS_PER_PASS + first_row < rows_left && straddles;
              T* row_cells = cells + pass * ROWS_PER_PASS * STAGE_PITCH;
              unsigned short values[7];
#pragma unroll
              for (int e = 0; e < 7; ++e) {
                const int element = (there && e < inside) ? lane_offset + pass * pass_step + 2 * e : kHOutside;
                if (LOAD) { values[e] = __builtin_amdgcn_raw_buffer_load_b16(view, element, 0, 0); }
                else { __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, row_cells[e]), view, element, 0, 0); }
              }
              if (LOAD && straddles) {
#pragma unroll
                for (int e = 0; e < 7; ++e) { row_cells[e] = __builtin_bit_cast(T, values[e]); }
              }
            }
          }
        } else {
#pragma unroll 1
          for (int row = 0; row < 32; ++row) {
            if (n_blk + row >= p.n) { break; }
#pragma unroll
            for (int col = lane; col < WAVE_M; col += 64) {
              if (wave_m0 + col < p.m && (!masked || InTriangle(p.c_triangle, wave_m0 + col, n_blk + row))) {
                T* global = c + (n_blk + row) * p.c_ld + wave_m0 + col;
                if (LOAD) { stage[row * STAGE_PITCH + col] = *global; }
                else { *global = stage[row * STAGE_PITCH + col]; }
              }
            }
          }
        }
      };
      __syncthreads();  // every wavefront is done with the slab buffers
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int n_blk = n0 + (wave_n * FN + j) * 32;
        if (n_blk < p.n && wave_m0 < p.m) {
          if (beta != 0.0f) {
            rows(n_blk, std::true_type{});
            wave_fence();
          }
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
            for (int i = 0; i < BM; ++i) {
              half4_t* cell = reinterpret_cast<half4_t*>(&stage[(16 * jj + lane % 16) * STAGE_PITCH + 16 * i + 4 * (lane / 16)]);
              half4_t out;
              if (beta != 0.0f) {
                const half4_t old = *cell;
#pragma unroll
                for (int e = 0; e < 4; ++e) { out[e] = Narrow<T, float>(Combine(alpha, acc[i][2 * j + jj][e], beta, static_cast<float>(old[e]))); }
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) { out[e] = Narrow<T, float>(alpha * acc[i][2 * j + jj][e]); }
              }
              *cell = out;
            }
          }
          wave_fence();
          rows(n_blk, std::false_type{});
          wave_fence();
        }
      }
      __syncthreads();  // the next batch entry refills the slab buffers
    }
  }
}

// Second pass of a split-K launch: C = alpha * (sum of the fp32 workspace slabs) + beta * C, rounded to fp16 once.
// grid: (ceil(m / 256), n).
__global__ __launch_bounds__(256) void HgemmSplitReduceKernel(const float* __restrict__ workspace, const int splits,
                                                              const int split_ld, _Float16* __restrict__ c,
                                                              const long long c_ld, const int m, const int n,
                                                              const float alpha, const float beta) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int j = blockIdx.y;
  if (i >= m || j >= n) { return; }
  const long long slab = static_cast<long long>(split_ld) * n;
  const float* src = workspace + static_cast<long long>(j) * split_ld + i;
  float sum = 0.0f;
  for (int s = 0; s < splits; ++s) { sum += src[s * slab]; }
  StoreResult<_Float16, float>(c, j * c_ld + i, sum, alpha, beta);
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_DIRECT_F16_HPP_
