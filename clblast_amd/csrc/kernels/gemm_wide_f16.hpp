// =================================================================================================
// HGEMM for large products on gfx950: 256 x 256 tiles, ONE wavefront per SIMD, 128 x 128 per wavefront.
// Same role and same operand handling as HgemmDirectKernel (kernels/gemm_direct_f16.hpp), which it
// replaces where the tile table asks for it: the reference's indirect chain for big matrices
// (src/routines/level3/xgemm.cpp:102-222, src/kernels/level3/xgemm_part1-4.opencl) as one launch that
// reads the caller's operands in place, fp32 accumulation in v_mfma_f32_16x16x32_f16, one rounding.
//
// Why another shape. Large HGEMMs run against the board's power limit, not against the matrix pipe: the
// clock settles where the energy per flop allows, and stalls are mostly bought back by a higher clock.
// What counts is the energy spent on moving operands, and of that the LDS -> register traffic depends on
// the wavefront's tile alone: a wavefront of 128 x 128 reads (128 + 128) x 32 halfs per 64 MFMAs, one of
// 128 x 64 reads (128 + 64) x 32 per 32 - a third more. 128 x 128 needs 256 accumulator registers; with
// one wavefront per SIMD they live in the accumulation half of the register file and the other half
// holds two complete sets of fragments, so every fragment is read from LDS a whole slab ahead of its use.
//
// Structure:
//   * 4 wavefronts (2 x 2), slabs of 32 along K in a ring of four LDS buffers, filled by direct
//     global -> LDS loads (layouts, swizzles and transposing reads as in gemm_direct_f16.hpp);
//   * while slab t is multiplied from fragment set t % 2, the wavefront reads the fragments of slab t + 1
//     into the other set and requests slab t + 4 into the buffer of slab t (whose last LDS read finished
//     before this slab began). One barrier per slab, at its start: "my requests for slab t + 1 have landed,
//     my reads of slab t are done". A request has two to three slabs of time to land;
//   * the K walk is unrolled over the ring (buffer and fragment set are compile-time facts: LDS addresses are
//     immediates) and K is padded to a multiple of 128 with slabs beyond the operand, which the range check of
//     the buffer loads turns into zeros without touching memory;
//   * every MFMA is followed by at most one LDS read or one request: with a single wavefront per SIMD nothing
//     else fills the issue slots;
//   * C moves straight between memory and the accumulators' values in 16-byte pieces (v_permlane16_swap gathers eight
//     consecutive rows of a column in one lane): for the length of the epilogue the matrix pipe stands still, and an
//     epilogue staged through LDS - thirteen, later three LDS round trips per 16 columns - took 11 us of a tile's 187.
//   * the GENERAL instances also walk the tiles of a triangle of a square C (tiles on the diagonal store under a mask:
//     the other triangle's elements go back as they were read) and split the tiles of a last round that would fill at
//     most half of the work-groups into K ranges, one item each, whose sums a second kernel adds up
//     (HgemmWideFixupKernel) - 528 tiles on 256 work-groups then cost two rounds and a short one instead of three.
// Requirements (the launcher checks them): dword-aligned operands, no triangular operand, no K ranges as batch
// entries, no gathered operand; a k-contiguous operand needs k % 8 == 0 (its K tail is cut by giving whole 16-byte
// chunks an offset outside the buffer's range); m % 8 == 0 (C moves in pieces of eight rows, each inside the matrix or
// not); a triangle of C needs m == n.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_WIDE_F16_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_WIDE_F16_HPP_

#include <type_traits>

#include "kernels/gemm_direct_f16.hpp"

namespace clbh {

struct HwideConfig {
  static constexpr int WM = 2, WN = 2, WAVES = 4, THREADS = 256;
  static constexpr int TILE_M = 256, TILE_N = 256, TILE_K = 32, STAGES = 4;
  static constexpr int BM = 8, BN = 8;              // blocks of 16 x 16 per wavefront
  static constexpr int PIECES = 16;                 // 1 KiB pieces per operand and slab
  static constexpr int ROUNDS = 2 * PIECES / WAVES;  // requests per wavefront and slab: four for A, then four for B
  static constexpr int OPERAND_ELEMS = 256 * 32;    // halfs of one operand's slab
  static constexpr int RING_BYTES = STAGES * 2 * OPERAND_ELEMS * 2;
  static constexpr int WAVE_M = 128;
  static constexpr int OLD_C_BYTES = WAVES * 8 * 1024;  // one strip of old C per wavefront (eight pieces of 16 bytes per lane)
  static constexpr int LDS_BYTES = RING_BYTES + OLD_C_BYTES;
  static constexpr int STORES = 32;                                   // 16-byte stores per wavefront and tile
};

// One MFMA whose accumulator stays where it is: the instruction is written out with the accumulator as a tied operand
// in the accumulation registers. (Left to the register allocator, several of the 64 accumulator blocks got a
// destination different from their source and were copied back through vector registers at every turn of the K loop.)
// FIRST: the accumulator starts from zero (no register is cleared beforehand). The compiler still sees the operands and
// waits for the LDS reads that fill the fragments, but it does not know the instruction: it would place no wait states
// between an MFMA and a copy of its accumulator. None may exist inside the walk (a test greps the generated code
// between the walk's markers), and whoever reads the accumulators afterwards goes through WideMfmaDrain.
typedef float wide_acc_t __attribute__((ext_vector_type(4)));
template <bool FIRST>
__device__ __forceinline__ void WideMfma(wide_acc_t& acc, const half8_t a, const half8_t b) {
  if (FIRST) { asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b)); }
  else { asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b)); }
}
// Sixteen wait states that every later use of these accumulators depends on: the longest latency from a four-pass MFMA
// to a read of its result by another kind of instruction is shorter.
__device__ __forceinline__ void WideMfmaDrain(wide_acc_t (&acc)[8][8]) {
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    asm volatile("s_nop 15"
                 : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]), "+a"(acc[i][4]), "+a"(acc[i][5]),
                   "+a"(acc[i][6]), "+a"(acc[i][7]), "+a"(acc[i + 1][0]), "+a"(acc[i + 1][1]), "+a"(acc[i + 1][2]),
                   "+a"(acc[i + 1][3]), "+a"(acc[i + 1][4]), "+a"(acc[i + 1][5]), "+a"(acc[i + 1][6]), "+a"(acc[i + 1][7]));
  }
}

// v_permlane16_swap: of two registers, the odd rows of 16 lanes of the first change places with the even rows of the
// second (rows 0..3 of `first` become first.0, second.0, first.2, second.2; of `second`: first.1, second.1, first.3,
// second.3). Four pairs at once, written as instructions (their inputs come from instructions the compiler does not
// know either) between the wait states that the compiler places for the builtin: two between a vector instruction's
// result and this instruction's read of it, two between its results and a vector instruction that reads them.
__device__ __forceinline__ void WidePermlane16Swap(float (&first)[4], float (&second)[4]) {
  asm volatile(
      "s_nop 1\n\tv_permlane16_swap_b32 %0, %4\n\tv_permlane16_swap_b32 %1, %5\n\tv_permlane16_swap_b32 %2, %6\n\t"
      "v_permlane16_swap_b32 %3, %7\n\ts_nop 1"
      : "+v"(first[0]), "+v"(first[1]), "+v"(first[2]), "+v"(first[3]), "+v"(second[0]), "+v"(second[1]), "+v"(second[2]), "+v"(second[3]));
}

// The tiles of a triangle of a square C of `along` x `along` tiles in an order with the locality of TileOfBlock: groups of
// eight tile rows, column by column inside a group (upper triangle, tile row <= tile column: a group holds the
// triangle on its own eight columns, then whole columns of eight), a contiguous range of that order per XCD. The
// lower triangle is the mirror image. `index` counts 0 .. TriangleTiles(along) - 1.
__device__ __host__ __forceinline__ int TriangleTiles(const int along) { return along * (along + 1) / 2; }
__device__ __forceinline__ void TriangleTileOfBlock(const int index, const int along, const bool upper, int& tile_m, int& tile_n) {
  int rest = XcdContiguousIndex(index, TriangleTiles(along));
  int first = 0, rows = min(8, along);
  while (first + rows < along) {  // (at most along / 8 turns, scalar; the last group takes what is left)
    const int in_group = rows * (rows + 1) / 2 + rows * (along - first - rows);
    if (rest < in_group) { break; }
    rest -= in_group;
    first += rows;
    rows = min(8, along - first);
  }
  int row, column;
  const int corner = rows * (rows + 1) / 2;
  if (rest < corner) {  // column first + c of the group's own triangle holds the rows first .. first + c
    int c = 0;
    while (rest >= (c + 1) * (c + 2) / 2) { ++c; }
    column = first + c;
    row = first + rest - c * (c + 1) / 2;
  } else {
    column = first + rows + (rest - corner) / rows;
    row = first + (rest - corner) % rows;
  }
  tile_m = upper ? row : column;
  tile_n = upper ? column : row;
}

// What an item of a launch is: a tile of a matrix of the batch, the turns of the ring (128 k each) it walks, and where
// its sums go - into C (slot < 0) or, for one K range of a split tile, into a slot of partial sums.
struct WideItem {
  int tile_m, tile_n, batch, first_group, groups, slot;
};
// GENERAL: launches over a triangle of C, and launches that split the tiles from p.tail_first on into K ranges.
template <bool GENERAL>
__device__ __forceinline__ WideItem WideItemOf(const GemmArgs<float>& p, const int tiles_m, const int tiles_n, const int item,
                                              const int all_groups) {
  WideItem w;
  const int tiles = tiles_m * tiles_n;
  if constexpr (!GENERAL) {
    w.batch = item / tiles;
    TileOfBlock(item - w.batch * tiles, tiles, tiles_m, tiles_n, w.tile_m, w.tile_n);
    w.first_group = 0;
    w.groups = all_groups;
    w.slot = -1;
  } else {
    int logical = item;
    w.first_group = 0;
    w.groups = all_groups;
    w.slot = -1;
    if (p.tail_parts > 0 && item >= p.tail_first) {
      w.slot = item - p.tail_first;
      logical = p.tail_first + w.slot / p.tail_parts;
      w.first_group = (w.slot % p.tail_parts) * p.tail_groups;
      w.groups = min(p.tail_groups, all_groups - w.first_group);
    }
    const int per_matrix = (p.c_triangle != 0) ? TriangleTiles(tiles_m) : tiles;
    w.batch = logical / per_matrix;
    const int index = logical - w.batch * per_matrix;
    if (p.c_triangle != 0) { TriangleTileOfBlock(index, tiles_m, p.c_triangle == 1, w.tile_m, w.tile_n); }
    else { TileOfBlock(index, tiles, tiles_m, tiles_n, w.tile_m, w.tile_n); }
  }
  return w;
}

// RANGE: range-checked requests (some tile touches an edge of the matrix, or K is not a multiple of 128); without,
// every tile is whole and the byte count per slab and operand is saved.
//
// The work-groups are persistent: grid.x of them (one per compute unit) take the items - tiles of all matrices of the
// batch - g, g + grid.x, ... Under the last turn of the K walk of an item the first turn of the ring of the NEXT item
// is requested, so the epilogue's stores and the next walk's first slabs overlap; the queue of memory operations
// then holds, oldest first: the next item's four slabs, the stores. The waits of a walk's first turn count
// those stores: every epilogue issues exactly HwideConfig::STORES of them per wavefront (pieces outside the matrix go
// to offsets outside the view of C and move nothing), and at the very start as many stores that move nothing are
// issued, so that the first item sees the same queue.
template <bool A_KC, bool B_KC, bool RANGE, bool GENERAL = false>
__global__ __launch_bounds__(HwideConfig::THREADS, 1) void HgemmWideKernel(const GemmArgs<float> p, const int tiles_m,
                                                                           const int tiles_n, const int items) {
  using T = _Float16;
  using Config = HwideConfig;
  constexpr int TILE_M = Config::TILE_M, TILE_N = Config::TILE_N, TILE_K = Config::TILE_K, STAGES = Config::STAGES;
  constexpr int BM = Config::BM, BN = Config::BN, WAVES = Config::WAVES, ROUNDS = Config::ROUNDS;
  constexpr int ELEMS = Config::OPERAND_ELEMS;
  constexpr int PENDING = Config::STORES;  // stores of the previous epilogue behind a first turn's requests
  typedef __attribute__((address_space(3))) void* LdsPtr;

  __shared__ __align__(16) unsigned char lds_raw[Config::LDS_BYTES];
  T* lds = reinterpret_cast<T*>(lds_raw);
  T* a_ring = lds;                         // [STAGES][ELEMS]
  T* b_ring = lds + STAGES * ELEMS;        // [STAGES][ELEMS]

  const int tid = threadIdx.x;
  const int lane = tid % 64, wave = tid / 64;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  T* old_c_lds = lds + 2 * STAGES * ELEMS + wave_u * 4096;  // [8 pieces][64 lanes][8]: the last strip of old C of this wavefront
  const int wave_m = wave_u % Config::WM, wave_n = wave_u / Config::WM;  // (uniform: C is addressed through a buffer view per wavefront)

  // LDS positions of the lane's fragments inside a slab buffer
  const T* a_read[BM];
  const T* b_read[BN];
#pragma unroll
  for (int q = 0; q < BM; ++q) { a_read[q] = a_ring + HFragmentOffset<TILE_M, A_KC>(lane, (wave_m * BM + q) * 16); }
#pragma unroll
  for (int q = 0; q < BN; ++q) { b_read[q] = b_ring + HFragmentOffset<TILE_N, B_KC>(lane, (wave_n * BN + q) * 16); }

  const int k_len = p.k;
  const int slabs = (k_len + TILE_K - 1) / TILE_K;
  const int all_groups = (slabs + STAGES - 1) / STAGES;  // the walk runs whole turns of the ring (of an item's K range: WideItem)

  // A request of this wavefront: round r < 4 fetches piece wave + 4 r of A, round 4 + r that piece of B. The lane's byte
  // offset from the slab's first row is kept per round (the range check of a buffer load looks at the vector offset
  // only, so the piece's rows cannot travel in the scalar offset).
  int a_bytes[ROUNDS / 2], b_bytes[ROUNDS / 2];
  int a_lane_k = 0, b_lane_k = 0;  // k-contiguous operand: first k of the lane's chunk inside a slab
#pragma unroll
  for (int r = 0; r < ROUNDS / 2; ++r) {
    const int piece = wave_u + WAVES * r;
    a_bytes[r] = HPieceLaneBytes<TILE_M, A_KC>(p.a_ld, piece, lane) + static_cast<int>(2 * (A_KC ? 16 : 512 / TILE_M) * piece * p.a_ld);
    b_bytes[r] = HPieceLaneBytes<TILE_N, B_KC>(p.b_ld, piece, lane) + static_cast<int>(2 * (B_KC ? 16 : 512 / TILE_N) * piece * p.b_ld);
  }
  if (A_KC) { a_lane_k = 8 * ((lane % 4) ^ (((lane / 4) >> 2) & 3)); }
  if (B_KC) { b_lane_k = 8 * ((lane % 4) ^ (((lane / 4) >> 2) & 3)); }
  const long long a_step = A_KC ? static_cast<long long>(TILE_K) : TILE_K * p.a_ld;
  const long long b_step = B_KC ? static_cast<long long>(TILE_K) : TILE_K * p.b_ld;

  // State of the requests: the slab to be requested next, of the item whose slabs are on their way
  const T* a_request = nullptr;
  const T* b_request = nullptr;
  const T* a_end = nullptr;
  const T* b_end = nullptr;
  int request_k = 0;
  int request_k_len = k_len;  // extent of the K range whose slabs are being requested
  int request_open = -1;  // 0 behind the last item: the requests of a next item's first turn are issued all the same, and move nothing
  auto a_resource = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(a_request), 0, 0, kRawBufferFlags);
  auto b_resource = a_resource;
  // (every word of a resource is taken from the first lane: the compiler then keeps the resources in scalar registers
  // across the loop over the items, where it would otherwise move them to vector registers and loop over their values)
  const auto uniform_pointer = [](const T* pointer) {
    const auto bits = reinterpret_cast<unsigned long long>(pointer);
    const unsigned int low = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(bits));
    const unsigned int high = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(bits >> 32));
    return reinterpret_cast<T*>((static_cast<unsigned long long>(high) << 32) | low);
  };
  auto refresh_resources = [&]() {
    const int a_records = __builtin_amdgcn_readfirstlane((RANGE ? HRecordsUpTo(a_request, a_end) : -1) & request_open);
    const int b_records = __builtin_amdgcn_readfirstlane((RANGE ? HRecordsUpTo(b_request, b_end) : -1) & request_open);
    a_resource = __builtin_amdgcn_make_buffer_rsrc(uniform_pointer(a_request), 0, a_records, kRawBufferFlags);
    b_resource = __builtin_amdgcn_make_buffer_rsrc(uniform_pointer(b_request), 0, b_records, kRawBufferFlags);
  };
  // request `round` of the slab at a_request / b_request into ring position `buffer`
  auto request = [&](const int round, const int buffer) {
    const int r = round % (ROUNDS / 2);
    const int place = (wave_u + WAVES * r) * 512;
    if (round < ROUNDS / 2) {
      int offset = a_bytes[r];
      if (A_KC && RANGE) { offset = (request_k + a_lane_k < (GENERAL ? request_k_len : k_len)) ? offset : static_cast<int>(0x80000000u); }
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_resource, (LdsPtr)(a_ring + buffer * ELEMS + place), 16, offset, 0, 0, 0);
    } else {
      int offset = b_bytes[r];
      if (B_KC && RANGE) { offset = (request_k + b_lane_k < (GENERAL ? request_k_len : k_len)) ? offset : static_cast<int>(0x80000000u); }
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_resource, (LdsPtr)(b_ring + buffer * ELEMS + place), 16, offset, 0, 0, 0);
    }
  };
  auto next_request_slab = [&]() {
    a_request += a_step;
    b_request += b_step;
    request_k += TILE_K;
    refresh_resources();
  };
  // The slabs of all items of a work-group form ONE stream through the ring: the last turn of an item's walk requests
  // the first four slabs of the next item (without the range check K is a multiple of 128: they all exist) at the usual
  // pace, one request per eight MFMAs - requested in one go between walk and epilogue, those 128 KiB per CU kept the
  // vector memory pipe of the CU busy for 1.8 us with nothing to multiply. Where the next item's operands lie is worked
  // out ahead of the walk (scalar arithmetic with a few divisions and, for batches, loads of pointers).
  const T* planned_a = nullptr;
  const T* planned_b = nullptr;
  const T* planned_a_end = nullptr;
  const T* planned_b_end = nullptr;
  int planned_open = 0;
  int planned_k_len = k_len;
  auto plan_first_turn = [&](const int wanted) {
    planned_open = (wanted < items) ? -1 : 0;
    const WideItem planned = WideItemOf<GENERAL>(p, tiles_m, tiles_n, (wanted < items) ? wanted : 0, all_groups);
    const T* a;
    const T* b;
    T* c;
    float alpha, beta;
    ResolveBatch<T, float>(p, planned.batch, a, b, c, alpha, beta);
    // the item's K range [k_first, k_last): all of K unless the tile is split
    const int k_first = planned.first_group * (STAGES * TILE_K);
    const int k_last = GENERAL ? min(k_len, k_first + planned.groups * (STAGES * TILE_K)) : k_len;
    planned_k_len = k_last - k_first;
    // element (m0, k_first), uniform
    planned_a = a + (A_KC ? planned.tile_m * TILE_M * p.a_ld + k_first : k_first * p.a_ld + planned.tile_m * TILE_M);
    planned_b = b + (B_KC ? planned.tile_n * TILE_N * p.b_ld + k_first : k_first * p.b_ld + planned.tile_n * TILE_N);
    planned_a_end = a + (A_KC ? (p.m - 1) * p.a_ld + k_last : (k_last - 1) * p.a_ld + p.m);
    planned_b_end = b + (B_KC ? (p.n - 1) * p.b_ld + k_last : (k_last - 1) * p.b_ld + p.n);
  };
  auto switch_requests = [&]() {  // from here on the requests fetch the planned item, from its first slab on
    request_open = planned_open;
    a_request = planned_a;
    b_request = planned_b;
    a_end = planned_a_end;
    b_end = planned_b_end;
    request_k = 0;
    request_k_len = planned_k_len;
    refresh_resources();
  };

  // C moves in pieces of 16 bytes, eight consecutive m of one column, straight between memory and the accumulators' values:
  // of two blocks of rows, 2 q and 2 q + 1, a lane holds rows 4 g + r (g = lane / 16, r = 0..3) of each; one
  // v_permlane16_swap per register exchanges the odd rows of 16 lanes of the one with the even rows of the other, and
  // the lane then holds the eight rows 16 (g % 2) + 8 (g / 2) + 0..7 of the pair's 32, all of column lane % 16. A
  // wavefront's 128 x 128 part is four strips of 32 columns; a strip is eight pieces per lane (piece: block of 16
  // columns pass / 4 of the strip, pair of row blocks pass % 4).
  constexpr int WAVE_M = Config::WAVE_M;
  constexpr int PASSES = 8, STRIPS = BN / 2;
  static_assert(STRIPS * PASSES == Config::STORES && BM == 8, "stores per wavefront and tile");
  const int c_lane_m = 16 * ((lane / 16) % 2) + 8 * (lane / 32);
  const int c_lane_offset = ((lane % 16) * static_cast<int>(p.c_ld) + c_lane_m) * 2;
  const int c_block_bytes = 16 * static_cast<int>(p.c_ld) * 2;  // from one block of 16 columns to the next
  // All of old C is asked for under the last turn of the walk, two microseconds (a load's latency under this load)
  // before the epilogue wants it: strip 0 under the first three slabs (3, 3 and 2 loads) into registers the walk leaves
  // free, strips 1 and 2 under the fourth, whose MFMAs need no fragments of a next slab any more (one set of fragment
  // registers is idle there), strip 3 under the second and third slab straight into LDS (four loads each).
  constexpr int kEarlyStrip0[STAGES + 1] = {0, 3, 6, 8, 8};      // loads of strip 0 issued before slab ST of the last turn
  constexpr int kEarlyBefore[STAGES + 1] = {0, 3, 10, 16, 16};   // all loads of old C issued before slab ST of the last turn

  int item = blockIdx.x;
  if (item >= items) { return; }
  plan_first_turn(item);
  switch_requests();
#pragma unroll
  for (int slab = 0; slab < STAGES; ++slab) {
#pragma unroll
    for (int round = 0; round < ROUNDS; ++round) { request(round, slab); }
    next_request_slab();
  }
  {
    // as many stores as an epilogue issues, into a view of no bytes: they move nothing and take their places in the queue
    const auto nothing = __builtin_amdgcn_make_buffer_rsrc(static_cast<T*>(p.c), 0, 0, kRawBufferFlags);
    half8_t zeros;
#pragma unroll
    for (int e = 0; e < 8; ++e) { zeros[e] = T(0); }
#pragma unroll
    for (int i = 0; i < Config::STORES; ++i) { BufferStore<T, 8>(zeros, nothing, 0); }
  }

  for (; item < items; item += gridDim.x) {
    // the tile of C of this item
    const WideItem here = WideItemOf<GENERAL>(p, tiles_m, tiles_n, item, all_groups);
    const int groups = here.groups;
    const int m0 = here.tile_m * TILE_M, n0 = here.tile_n * TILE_N;
    T* c;
    float alpha, beta;
    {
      const T* a;
      const T* b;
      ResolveBatch<T, float>(p, here.batch, a, b, c, alpha, beta);
    }
    // GENERAL: a tile on the diagonal of a triangle of C keeps the old values of the other triangle's elements (they are
    // stored back as they were read); the sums of one K range of a split tile go to their slot as they are
    const bool masked = GENERAL && p.c_triangle != 0 && here.tile_m == here.tile_n;
    const bool to_slot = GENERAL && here.slot >= 0;
    const bool fetch_c = !to_slot && (beta != 0.0f || masked);
    wide_acc_t acc[BM][BN];  // written by the first slab
    plan_first_turn(item + gridDim.x);

    // Old C, fetched under the MFMAs of the last turn of the K walk (see kEarlyStrip0). With beta == 0 the same loads run
    // with an offset outside the view (no memory is touched), so the code and the count of loads in flight do not
    // depend on beta.
    const int wave_m0 = m0 + wave_m * WAVE_M, wave_n0 = n0 + wave_n * (BN * 16);
    const auto c_view = __builtin_amdgcn_make_buffer_rsrc(c + wave_n0 * p.c_ld + wave_m0, 0, kHOutside, kRawBufferFlags);
    const int c_inside = p.m - (wave_m0 + c_lane_m);   // rows of C from the lane's first one (of pair 0) to the matrix's edge
    const int c_cols_left = p.n - wave_n0 - lane % 16; // columns of C from the lane's first one to the matrix's edge
    const auto c_uniform = [&](const int strip, const int pass) { return (2 * strip + pass / 4) * c_block_bytes + 64 * (pass % 4); };
    const auto c_piece_there = [&](const int strip, const int pass) {  // all eight rows of the piece inside the matrix
      return !RANGE || (16 * (2 * strip + pass / 4) < c_cols_left && c_inside - 32 * (pass % 4) >= 8);
    };
    const auto c_load = [&](const int strip, const int pass) {
      if (RANGE) { return BufferLoad<T, 8>(c_view, (fetch_c && c_piece_there(strip, pass)) ? c_lane_offset + c_uniform(strip, pass) : kHOutside); }
      return BufferLoad<T, 8>(c_view, fetch_c ? c_lane_offset : kHOutside, c_uniform(strip, pass));
    };
    const auto c_load_to_lds = [&](const int pass) {  // piece `pass` of strip 3: lane l's 16 bytes land at old_c_lds[pass][l]
      // (every operand of the load worked out beforehand: with a call among the load's own arguments the host pass of
      // the compiler drops this kernel's launch stub without a word)
      const bool wanted = fetch_c && c_piece_there(STRIPS - 1, pass);
      const int piece_offset = c_lane_offset + c_uniform(STRIPS - 1, pass);
      const int offset = wanted ? piece_offset : kHOutside;
      LdsPtr place = (LdsPtr)(old_c_lds + pass * 512);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(c_view, place, 16, offset, 0, 0, 0);
    };
    half8_t old_c[STRIPS - 1][PASSES];

    {
      // the first four slabs of this item have landed: the youngest operations in the queue are the stores of the
      // previous epilogue (or the stores that stand in for them ahead of the first item), all requests are older
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PENDING) : "memory");
      half8_t a_frag[2][BM], b_frag[2][BN];
#pragma unroll
      for (int q = 0; q < BM; ++q) { a_frag[0][q] = HFragment<TILE_M, A_KC>(a_read[q], 0); }
#pragma unroll
      for (int q = 0; q < BN; ++q) { b_frag[0][q] = HFragment<TILE_N, B_KC>(b_read[q], 0); }

      // One slab in ring position ST (compile time): wait and barrier, 64 MFMAs with the fragment reads of the next slab,
      // the requests for the slab four further on (in the last turn: of the next item) and, in the last turn, the first
      // loads of old C between them. TURN1: the first turn of an item - its slabs have landed, but what it requests
      // stands behind the previous epilogue's stores in the queue.
      auto slab_body = [&](auto stage_tag, auto last_tag, auto first_tag, auto turn1_tag) {
        constexpr int ST = decltype(stage_tag)::value;
        constexpr bool LAST = decltype(last_tag)::value;
        constexpr bool FIRST = decltype(first_tag)::value;  // the very first slab: the accumulators start here
        constexpr bool TURN1 = decltype(turn1_tag)::value;
        constexpr int CUR = ST % 2, NXT = 1 - CUR, NEXT_ST = (ST + 1) % STAGES;
        constexpr bool READS_NEXT = !(LAST && ST == STAGES - 1);  // (the next item's first fragments are read at its top)
        // My requests for the next slab have landed - the requests of two later slabs may stay in flight, and so may the
        // loads of old C issued since (last turn) -, my reads of this slab are done. Nothing to wait for where the next
        // slab is one of the item's first four, or is not read here.
        constexpr int IN_FLIGHT = ((TURN1 && ST + 1 < STAGES) || !READS_NEXT) ? 63 : 2 * ROUNDS + (LAST ? kEarlyBefore[ST] : 0);
        static_assert(IN_FLIGHT < 64, "the counter of memory operations holds six bits");
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::"n"(IN_FLIGHT) : "memory");
#pragma unroll
        for (int i = 0; i < BM; ++i) {
#pragma unroll
          for (int j = 0; j < BN; ++j) {
            const int n = i * BN + j;
            WideMfma<FIRST>(acc[i][j], a_frag[CUR][i], b_frag[CUR][j]);
            if (READS_NEXT && n % 4 == 1) {  // one fragment of the next slab per four MFMAs: B first
              const int f = n / 4;
              if (f < BN) { b_frag[NXT][f] = HFragment<TILE_N, B_KC>(b_read[f], NEXT_ST * ELEMS); }
              else { a_frag[NXT][f - BN] = HFragment<TILE_M, A_KC>(a_read[f - BN], NEXT_ST * ELEMS); }
            }
            if (n % 8 == 7) { request(n / 8, ST); }
            if (LAST && ST < STAGES - 1 && n % 16 == 11 && kEarlyStrip0[ST] + n / 16 < kEarlyStrip0[ST + 1]) {
              const int piece = kEarlyStrip0[ST] + n / 16;
              old_c[0][piece] = c_load(0, piece);
            }
            if (LAST && (ST == 1 || ST == 2) && n % 16 == 3) { c_load_to_lds(4 * (ST - 1) + n / 16); }
            if (LAST && ST == STAGES - 1 && n % 8 == 3) { old_c[1][n / 8] = c_load(1, n / 8); }
            if (LAST && ST == STAGES - 1 && n % 8 == 5) { old_c[2][n / 8] = c_load(2, n / 8); }  // (into the idle set of fragment registers)
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        next_request_slab();
      };
      using std::integral_constant;
      using std::false_type;
      using std::true_type;
      asm volatile("; WIDE_WALK_BEGIN" ::: "memory");
      if (groups == 1) {
        switch_requests();
        slab_body(integral_constant<int, 0>{}, true_type{}, true_type{}, true_type{});
        slab_body(integral_constant<int, 1>{}, true_type{}, false_type{}, true_type{});
        slab_body(integral_constant<int, 2>{}, true_type{}, false_type{}, true_type{});
        slab_body(integral_constant<int, 3>{}, true_type{}, false_type{}, true_type{});
      } else {
        slab_body(integral_constant<int, 0>{}, false_type{}, true_type{}, true_type{});
        slab_body(integral_constant<int, 1>{}, false_type{}, false_type{}, true_type{});
        slab_body(integral_constant<int, 2>{}, false_type{}, false_type{}, true_type{});
        slab_body(integral_constant<int, 3>{}, false_type{}, false_type{}, true_type{});
        for (int group = 2; group < groups; ++group) {
          slab_body(integral_constant<int, 0>{}, false_type{}, false_type{}, false_type{});
          slab_body(integral_constant<int, 1>{}, false_type{}, false_type{}, false_type{});
          slab_body(integral_constant<int, 2>{}, false_type{}, false_type{}, false_type{});
          slab_body(integral_constant<int, 3>{}, false_type{}, false_type{}, false_type{});
        }
        switch_requests();
        slab_body(integral_constant<int, 0>{}, true_type{}, false_type{}, false_type{});
        slab_body(integral_constant<int, 1>{}, true_type{}, false_type{}, false_type{});
        slab_body(integral_constant<int, 2>{}, true_type{}, false_type{}, false_type{});
        slab_body(integral_constant<int, 3>{}, true_type{}, false_type{}, false_type{});
      }
      asm volatile("; WIDE_WALK_END" ::: "memory");
      WideMfmaDrain(acc);
    }

    // Epilogue: piece by piece the accumulators' values are exchanged between the rows of lanes (see above), combined
    // with the old values in fp32, rounded once and stored; no LDS, no dependence between pieces.
    {
      auto combine = [&](auto use_c_tag, auto masked_tag) {
        constexpr bool USE_C = decltype(use_c_tag)::value;
        constexpr bool MASKED = decltype(masked_tag)::value;  // a tile on the diagonal of a triangle of C (reads old C)
        static_assert(USE_C || !MASKED, "the elements outside the triangle are stored back as they were read");
#pragma unroll
        for (int strip = 0; strip < STRIPS; ++strip) {
#pragma unroll
          for (int pass = 0; pass < PASSES; ++pass) {
            const int j = 2 * strip + pass / 4, pair = pass % 4;
            if (pass % 2 == 0) { __builtin_amdgcn_sched_barrier(0); }  // (the accumulators leave their registers two pieces at a time, not all at once)
            // (copied to vector registers here, and from nowhere else: with a copy per use the compiler fetches all 256
            // accumulators at the top of the epilogue and spills what else lives there)
            float even[4], odd[4];  // rows 4 g + r of the pair's two blocks, then rows 0..3 and 4..7 of the lane's eight
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(even[r]) : "a"(acc[2 * pair][j][r]));
              asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(odd[r]) : "a"(acc[2 * pair + 1][j][r]));
            }
            WidePermlane16Swap(even, odd);
            float values[8];
#pragma unroll
            for (int r = 0; r < 4; ++r) { values[r] = even[r]; values[4 + r] = odd[r]; }
            half8_t old = half8_t(T(0));
            if (USE_C) {
              if (strip < STRIPS - 1) {
                old = old_c[strip][pass];
              } else {
                // (its loads into LDS are older than every store: all but the stores of the strips before have completed)
                if (pass == 0) { asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STRIPS - 1) * PASSES) : "memory"); }
                old = *reinterpret_cast<const half8_t*>(old_c_lds + pass * 512 + lane * 8);
              }
            }
            half8_t out;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              if constexpr (MASKED) {
                const float fresh = (beta != 0.0f) ? Combine(alpha, values[e], beta, static_cast<float>(old[e])) : alpha * values[e];
                const bool kept = InTriangle(p.c_triangle, wave_m0 + c_lane_m + 32 * pair + e, wave_n0 + 16 * j + lane % 16);
                out[e] = kept ? Narrow<T, float>(fresh) : old[e];
              } else if constexpr (USE_C) {
                out[e] = Narrow<T, float>(Combine(alpha, values[e], beta, static_cast<float>(old[e])));
              } else {
                out[e] = Narrow<T, float>(alpha * values[e]);
              }
            }
            if (RANGE) { BufferStore<T, 8>(out, c_view, c_piece_there(strip, pass) ? c_lane_offset + c_uniform(strip, pass) : kHOutside); }
            else { BufferStore<T, 8>(out, c_view, c_lane_offset, c_uniform(strip, pass)); }
          }
        }
      };
      // The sums of one K range of a split tile: sixteen bytes per lane and block of 16 x 16 (four consecutive rows of a
      // column) into the item's slot, a column-major 256 x 256 matrix of floats. (More stores than the epilogues that the
      // waits of the next walk count on: those waits then wait for more than they need to, never for less.)
      auto store_sums = [&]() {
        float* slot = p.tail_partials + static_cast<long long>(here.slot) * (TILE_M * TILE_N) + wave_n * (BN * 16) * TILE_M + wave_m * WAVE_M;
        const int slot_bytes = (TILE_N - wave_n * (BN * 16)) * TILE_M * 4;
        const auto slot_view = __builtin_amdgcn_make_buffer_rsrc(slot, 0, slot_bytes, kRawBufferFlags);
        const int lane_bytes = ((lane % 16) * TILE_M + 4 * (lane / 16)) * 4;
        typedef float float4_t __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int j = 0; j < BN; ++j) {
#pragma unroll
          for (int i = 0; i < BM; ++i) {
            if (i % 2 == 0) { __builtin_amdgcn_sched_barrier(0); }
            float4_t sums;
            float part[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) { asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(part[r]) : "a"(acc[i][j][r])); }
#pragma unroll
            for (int r = 0; r < 4; ++r) { sums[r] = part[r]; }
            BufferStore<float, 4>(sums, slot_view, lane_bytes, (16 * j * TILE_M + 16 * i) * 4);
          }
        }
      };
      if (GENERAL && to_slot) { store_sums(); }
      else if (GENERAL && masked) { combine(std::true_type{}, std::true_type{}); }
      else if (beta != 0.0f) { combine(std::true_type{}, std::false_type{}); }
      else { combine(std::false_type{}, std::false_type{}); }
    }
  }
}

// Second kernel of a launch with split tiles (GemmArgs::tail_parts > 0): the 32 work-groups t * 32 .. t * 32 + 31 add the
// sums of the K ranges of tile tail_first + t in the order of the ranges, eight columns each, apply alpha and beta and
// store - what lies inside the matrix, and on the diagonal of a triangle of C the triangle's elements. A thread owns
// eight rows of a column (the rows of C are a multiple of 8: such a piece lies inside the matrix or outside).
constexpr int kWideFixupGroupsPerTile = 32;
__global__ __launch_bounds__(256) void HgemmWideFixupKernel(const GemmArgs<float> p, const int tiles_m, const int tiles_n,
                                                            const int all_groups) {
  using T = _Float16;
  constexpr int TILE = 256;
  const int tile = static_cast<int>(blockIdx.x) / kWideFixupGroupsPerTile;
  const WideItem first = WideItemOf<true>(p, tiles_m, tiles_n, p.tail_first + tile * p.tail_parts, all_groups);
  const T* a;
  const T* b;
  T* c;
  float alpha, beta;
  ResolveBatch<T, float>(p, first.batch, a, b, c, alpha, beta);
  const int m0 = first.tile_m * TILE, n0 = first.tile_n * TILE;
  const bool masked = p.c_triangle != 0 && first.tile_m == first.tile_n;
  const float* sums = p.tail_partials + static_cast<long long>(tile) * p.tail_parts * (TILE * TILE);
  const auto c_view = __builtin_amdgcn_make_buffer_rsrc(c + n0 * p.c_ld + m0, 0, kHOutside, kRawBufferFlags);
  typedef float float4_t __attribute__((ext_vector_type(4)));
  const int row = 8 * (threadIdx.x % 32);
  const int column = 8 * (static_cast<int>(blockIdx.x) % kWideFixupGroupsPerTile) + threadIdx.x / 32;
  if (m0 + row >= p.m || n0 + column >= p.n) { return; }
  float total[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) { total[e] = 0.0f; }
  for (int part = 0; part < p.tail_parts; ++part) {
    const float4_t* piece = reinterpret_cast<const float4_t*>(sums + static_cast<long long>(part) * (TILE * TILE) + column * TILE + row);
    const float4_t low = piece[0], high = piece[1];
#pragma unroll
    for (int e = 0; e < 4; ++e) { total[e] += low[e]; total[4 + e] += high[e]; }
  }
  const int offset = (column * static_cast<int>(p.c_ld) + row) * 2;
  half8_t old = half8_t(T(0));
  if (beta != 0.0f || masked) { old = BufferLoad<T, 8>(c_view, offset); }
  half8_t out;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float fresh = (beta != 0.0f) ? Combine(alpha, total[e], beta, static_cast<float>(old[e])) : alpha * total[e];
    const bool kept = !masked || InTriangle(p.c_triangle, m0 + row + e, n0 + column);
    out[e] = kept ? Narrow<T, float>(fresh) : old[e];
  }
  BufferStore<T, 8>(out, c_view, offset);
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_WIDE_F16_HPP_
