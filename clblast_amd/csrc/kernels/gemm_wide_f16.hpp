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
//     else fills the issue slots.
// Requirements (the launcher checks them): dword-aligned operands, no triangles, no split-K, no gathered
// operand; a k-contiguous operand needs k % 8 == 0 (its K tail is cut by giving whole 16-byte chunks an
// offset outside the buffer's range).
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
  static constexpr int WAVE_M = 128, STAGE_PITCH = WAVE_M + 8;
  static constexpr int STAGING_BYTES = WAVES * 16 * STAGE_PITCH * 2;  // the epilogue's tiles of 16 columns, one per wavefront
  static constexpr int LDS_BYTES = RING_BYTES + STAGING_BYTES;        // beside the ring: it is refilled under the epilogue
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

// RANGE: range-checked requests (some tile touches an edge of the matrix, or K is not a multiple of 128); without,
// every tile is whole and the byte count per slab and operand is saved.
//
// The work-groups are persistent: grid.x of them (one per compute unit) take the items - tiles of all matrices of the
// batch - g, g + grid.x, ... Behind the K walk of an item the first turn of the ring of the NEXT item is requested
// before the epilogue starts, so the epilogue's stores and the next walk's first slabs overlap; the queue of memory
// operations then holds, oldest first: the next item's four slabs, the stores. The waits of a walk's first turn count
// those stores: every epilogue issues at least HwideConfig::STORES of them per wavefront (pieces outside the matrix go
// to offsets outside the view of C and move nothing; tiles on the last rows of C add element-wise stores, which only
// makes the waits stricter than needed), and at the very start as many stores that move nothing are issued, so that
// the first item sees the same queue.
template <bool A_KC, bool B_KC, bool RANGE>
__global__ __launch_bounds__(HwideConfig::THREADS, 1) void HgemmWideKernel(const GemmArgs<float> p, const int tiles_m,
                                                                           const int tiles_n) {
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
  T* staging = lds + 2 * STAGES * ELEMS;   // [WAVES][16][STAGE_PITCH]

  const int tid = threadIdx.x;
  const int lane = tid % 64, wave = tid / 64;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wave_m = wave_u % Config::WM, wave_n = wave_u / Config::WM;  // (uniform: C is addressed through a buffer view per wavefront)
  const int tiles = tiles_m * tiles_n, items = tiles * p.batch_count;

  // LDS positions of the lane's fragments inside a slab buffer
  const T* a_read[BM];
  const T* b_read[BN];
#pragma unroll
  for (int q = 0; q < BM; ++q) { a_read[q] = a_ring + HFragmentOffset<TILE_M, A_KC>(lane, (wave_m * BM + q) * 16); }
#pragma unroll
  for (int q = 0; q < BN; ++q) { b_read[q] = b_ring + HFragmentOffset<TILE_N, B_KC>(lane, (wave_n * BN + q) * 16); }

  const int k_len = p.k;
  const int slabs = (k_len + TILE_K - 1) / TILE_K;
  const int groups = (slabs + STAGES - 1) / STAGES;  // the walk runs whole turns of the ring

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
      if (A_KC && RANGE) { offset = (request_k + a_lane_k < k_len) ? offset : static_cast<int>(0x80000000u); }
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_resource, (LdsPtr)(a_ring + buffer * ELEMS + place), 16, offset, 0, 0, 0);
    } else {
      int offset = b_bytes[r];
      if (B_KC && RANGE) { offset = (request_k + b_lane_k < k_len) ? offset : static_cast<int>(0x80000000u); }
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_resource, (LdsPtr)(b_ring + buffer * ELEMS + place), 16, offset, 0, 0, 0);
    }
  };
  auto next_request_slab = [&]() {
    a_request += a_step;
    b_request += b_step;
    request_k += TILE_K;
    refresh_resources();
  };
  // The first turn of the ring of `item` (without the range check K is a multiple of 128: all four slabs exist)
  auto request_first_turn = [&](const int wanted) {
    request_open = (wanted < items) ? -1 : 0;
    const int item = (wanted < items) ? wanted : 0;
    const int batch = item / tiles;
    int tile_m, tile_n;
    TileOfBlock(item - batch * tiles, tiles, tiles_m, tiles_n, tile_m, tile_n);
    const T* a;
    const T* b;
    T* c;
    float alpha, beta;
    ResolveBatch<T, float>(p, batch, a, b, c, alpha, beta);
    a_request = a + (A_KC ? tile_m * TILE_M * p.a_ld : static_cast<long long>(tile_m * TILE_M));  // element (m0, k = 0), uniform
    b_request = b + (B_KC ? tile_n * TILE_N * p.b_ld : static_cast<long long>(tile_n * TILE_N));
    a_end = a + (A_KC ? (p.m - 1) * p.a_ld + k_len : (k_len - 1) * p.a_ld + p.m);
    b_end = b + (B_KC ? (p.n - 1) * p.b_ld + k_len : (k_len - 1) * p.b_ld + p.n);
    request_k = 0;
    refresh_resources();
#pragma unroll
    for (int s = 0; s < STAGES; ++s) {
#pragma unroll
      for (int round = 0; round < ROUNDS; ++round) { request(round, s); }
      next_request_slab();
    }
  };

  constexpr int WAVE_M = Config::WAVE_M, STAGE_PITCH = Config::STAGE_PITCH;
  constexpr int LANES_PER_ROW = WAVE_M / 8, ROWS_PER_PASS = 64 / LANES_PER_ROW, PASSES = 32 / ROWS_PER_PASS, STRIPS = BN / 2;
  static_assert(STRIPS * PASSES == Config::STORES, "stores per wavefront and tile");
  const int c_first_row = lane / LANES_PER_ROW, c_col = 8 * (lane % LANES_PER_ROW);
  const int c_lane_offset = (c_first_row * static_cast<int>(p.c_ld) + c_col) * 2;
  const int c_pass_bytes = ROWS_PER_PASS * static_cast<int>(p.c_ld) * 2;
  // strip 0 of old C comes in under the first three slabs of the last turn (3, 3 and 2 loads), strip 1 under the fourth,
  // whose MFMAs need no fragments of a next slab any more
  constexpr int EARLY_STRIPS = 2;
  constexpr int kEarlyBefore[STAGES + 1] = {0, 3, 6, 8, 8};  // loads of old C issued before slab ST of the last turn

  int item = blockIdx.x;
  if (item >= items) { return; }
  request_first_turn(item);
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
    const int batch = item / tiles;
    int tile_m, tile_n;
    TileOfBlock(item - batch * tiles, tiles, tiles_m, tiles_n, tile_m, tile_n);
    const int m0 = tile_m * TILE_M, n0 = tile_n * TILE_N;
    T* c;
    float alpha, beta;
    {
      const T* a;
      const T* b;
      ResolveBatch<T, float>(p, batch, a, b, c, alpha, beta);
    }
    wide_acc_t acc[BM][BN];  // written by the first slab

    // Old C. The wavefront's 128 x 128 part of the tile is handled as four strips of 32 columns; a strip moves in eight
    // passes of 16 bytes per lane (lane: 8 consecutive m, pass g: columns 4 g + lane / 16 of the strip). The first two
    // strips are fetched under the MFMAs of the last turn of the K walk, into registers the walk leaves free, the other
    // two right behind the walk into the registers of the fragments. With beta == 0 the same loads run with an offset
    // outside the view (no memory is touched), so the code and the count of loads in flight do not depend on beta.
    const int wave_m0 = m0 + wave_m * WAVE_M, wave_n0 = n0 + wave_n * (BN * 16);
    const auto c_view = __builtin_amdgcn_make_buffer_rsrc(c + wave_n0 * p.c_ld + wave_m0, 0, kHOutside, kRawBufferFlags);
    const int c_inside = p.m - (wave_m0 + c_col);   // how many of the lane's eight m lie inside the matrix
    const int c_rows_left = p.n - wave_n0;          // columns of C from the wavefront's first one to the matrix's edge
    const auto c_piece_there = [&](const int strip, const int pass) {
      return !RANGE || ((32 * strip + pass * ROWS_PER_PASS + c_first_row < c_rows_left) && c_inside >= 8);
    };
    const auto c_load = [&](const int strip, const int pass) {
      const int uniform = (strip * PASSES + pass) * c_pass_bytes;
      if (RANGE) { return BufferLoad<T, 8>(c_view, (beta != 0.0f && c_piece_there(strip, pass)) ? c_lane_offset + uniform : kHOutside); }
      return BufferLoad<T, 8>(c_view, (beta != 0.0f) ? c_lane_offset : kHOutside, uniform);
    };
    half8_t old_c[STRIPS][PASSES];

    {
      // slab 0 of this item has landed (behind it in the queue: three slabs and the stores of the previous epilogue)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 1) * ROUNDS + PENDING) : "memory");
      __syncthreads();
      half8_t a_frag[2][BM], b_frag[2][BN];
#pragma unroll
      for (int q = 0; q < BM; ++q) { a_frag[0][q] = HFragment<TILE_M, A_KC>(a_read[q], 0); }
#pragma unroll
      for (int q = 0; q < BN; ++q) { b_frag[0][q] = HFragment<TILE_N, B_KC>(b_read[q], 0); }

      // One slab in ring position ST (compile time). LAST: the final turn of the ring - nothing is requested any more
      // and the waits count what is still in flight. TURN1: the first turn - the stores of the previous epilogue stand
      // in the queue behind the requests of this turn's slabs.
      auto slab_body = [&](auto stage_tag, auto last_tag, auto first_tag, auto turn1_tag) {
        constexpr int ST = decltype(stage_tag)::value;
        constexpr bool LAST = decltype(last_tag)::value;
        constexpr bool FIRST = decltype(first_tag)::value;  // the very first slab: the accumulators start here
        constexpr bool TURN1 = decltype(turn1_tag)::value;
        constexpr int CUR = ST % 2, NXT = 1 - CUR, NEXT_ST = (ST + 1) % STAGES;
        // my requests for the next slab have landed (two later slabs may stay in flight), my reads of this slab are done
        // (in the last turn the loads of old C issued under its earlier slabs stand behind the requests in the queue)
        constexpr int IN_FLIGHT = (LAST ? (ST + 2 < STAGES ? (STAGES - 2 - ST) * ROUNDS : 0) + kEarlyBefore[ST] : 2 * ROUNDS) +
                                  ((TURN1 && ST + 1 < STAGES) ? PENDING : 0);
        static_assert(IN_FLIGHT < 64, "the counter of memory operations holds six bits");
        if (!(LAST && ST == STAGES - 1)) {
          asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::"n"(IN_FLIGHT) : "memory");
        }
#pragma unroll
        for (int i = 0; i < BM; ++i) {
#pragma unroll
          for (int j = 0; j < BN; ++j) {
            const int n = i * BN + j;
            WideMfma<FIRST>(acc[i][j], a_frag[CUR][i], b_frag[CUR][j]);
            if (!(LAST && ST == STAGES - 1) && n % 4 == 1) {  // one fragment of the next slab per four MFMAs: B first
              const int f = n / 4;
              if (f < BN) { b_frag[NXT][f] = HFragment<TILE_N, B_KC>(b_read[f], NEXT_ST * ELEMS); }
              else { a_frag[NXT][f - BN] = HFragment<TILE_M, A_KC>(a_read[f - BN], NEXT_ST * ELEMS); }
            }
            if (!LAST && n % 8 == 7) { request(n / 8, ST); }
            if (LAST && ST < STAGES - 1 && n % 16 == 11 && kEarlyBefore[ST] + n / 16 < kEarlyBefore[ST + 1]) {
              const int piece = kEarlyBefore[ST] + n / 16;
              old_c[0][piece] = c_load(0, piece);
            }
            if (LAST && ST == STAGES - 1 && n % 8 == 3) { old_c[1][n / 8] = c_load(1, n / 8); }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if (!LAST) { next_request_slab(); }
      };
      using std::integral_constant;
      using std::false_type;
      using std::true_type;
      asm volatile("; WIDE_WALK_BEGIN" ::: "memory");
      if (groups == 1) {
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
        slab_body(integral_constant<int, 0>{}, true_type{}, false_type{}, false_type{});
        slab_body(integral_constant<int, 1>{}, true_type{}, false_type{}, false_type{});
        slab_body(integral_constant<int, 2>{}, true_type{}, false_type{}, false_type{});
        slab_body(integral_constant<int, 3>{}, true_type{}, false_type{}, false_type{});
      }
      asm volatile("; WIDE_WALK_END" ::: "memory");
      WideMfmaDrain(acc);
    }

    // Epilogue, staged through LDS so that global memory sees whole lines: per half strip (16 columns) a wavefront fills
    // its [16 n][128 m] fp16 staging tile; old C goes in with 16 bytes per lane, every lane combines its four consecutive
    // m per block in fp32 and rounds once, the finished rows leave with 16-byte stores. Only wavefront-local ordering is
    // needed (the LDS operations of a wavefront complete in order).
    {
      auto wave_fence = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      };
#pragma unroll
      for (int strip = EARLY_STRIPS; strip < STRIPS; ++strip) {
#pragma unroll
        for (int g = 0; g < PASSES; ++g) { old_c[strip][g] = c_load(strip, g); }
      }
      __syncthreads();  // every wavefront is done with the slab buffers
      // the next item's first slabs are requested now, ahead of this item's stores
      request_first_turn(item + gridDim.x);
      const bool wave_has_rows = wave_m0 < p.m;
      // (the lane number once more, opaque: the LDS addresses the epilogue derives from it are then computed here and
      // not ahead of the K walk, where they would sit in registers all through it)
      int late_lane = lane;
      asm volatile("" : "+v"(late_lane));
      const int late_first_row = late_lane / LANES_PER_ROW, late_col = 8 * (late_lane % LANES_PER_ROW);
      // RANGE: the piece per row that straddles the last row of C moves element by element
      const bool straddles = RANGE && c_inside > 0 && c_inside < 8;
      T* stage = staging + wave_u * (16 * STAGE_PITCH);
      T* cells = &stage[late_first_row * STAGE_PITCH + late_col];
      constexpr int HALF_PASSES = PASSES / 2;
#pragma unroll
      for (int half_strip = 0; half_strip < 2 * STRIPS; ++half_strip) {
        const int strip = half_strip / 2, half = half_strip % 2;
        if (RANGE && !(16 * half_strip < c_rows_left && wave_has_rows)) {  // (uniform) nothing of C here: the stores alone
          half8_t nothing;
#pragma unroll
          for (int e = 0; e < 8; ++e) { nothing[e] = T(0); }
#pragma unroll
          for (int g = 0; g < HALF_PASSES; ++g) { BufferStore<T, 8>(nothing, c_view, kHOutside); }
          continue;
        }
        __builtin_amdgcn_sched_barrier(0);  // (the accumulators leave their registers half strip by half strip, not all at once)
        if (beta != 0.0f) {
#pragma unroll
          for (int g = 0; g < HALF_PASSES; ++g) {
            *reinterpret_cast<half8_t*>(cells + g * ROWS_PER_PASS * STAGE_PITCH) = old_c[strip][half * HALF_PASSES + g];
          }
          if (RANGE && wave_m0 + WAVE_M > p.m) {
#pragma unroll 1
            for (int g = 0; g < HALF_PASSES; ++g) {
              const int pass = half * HALF_PASSES + g;
              const bool there = 32 * strip + pass * ROWS_PER_PASS + c_first_row < c_rows_left && straddles;
              unsigned short values[7];
#pragma unroll
              for (int e = 0; e < 7; ++e) {
                const int element = (there && e < c_inside) ? c_lane_offset + (strip * PASSES + pass) * c_pass_bytes + 2 * e : kHOutside;
                values[e] = __builtin_amdgcn_raw_buffer_load_b16(c_view, element, 0, 0);
              }
              if (straddles) {
#pragma unroll
                for (int e = 0; e < 7; ++e) { cells[g * ROWS_PER_PASS * STAGE_PITCH + e] = __builtin_bit_cast(T, values[e]); }
              }
            }
          }
          wave_fence();
        }
        // (the half strip's accumulators are copied to vector registers here, and from nowhere else: with a copy per
        // use the compiler fetches all 256 of them at the top of the epilogue and spills what else lives there)
        float values[BM][4];
#pragma unroll
        for (int i = 0; i < BM; ++i) {
#pragma unroll
          for (int e = 0; e < 4; ++e) { asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(values[i][e]) : "a"(acc[i][half_strip][e])); }
        }
#pragma unroll
        for (int i = 0; i < BM; ++i) {
          half4_t* cell = reinterpret_cast<half4_t*>(&stage[(late_lane % 16) * STAGE_PITCH + 16 * i + 4 * (late_lane / 16)]);
          half4_t out;
          if (beta != 0.0f) {
            const half4_t old = *cell;
#pragma unroll
            for (int e = 0; e < 4; ++e) { out[e] = static_cast<T>(Combine(alpha, values[i][e], beta, static_cast<float>(old[e]))); }
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) { out[e] = static_cast<T>(alpha * values[i][e]); }
          }
          *cell = out;
        }
        wave_fence();
#pragma unroll
        for (int g = 0; g < HALF_PASSES; ++g) {
          const int pass = half * HALF_PASSES + g;
          const half8_t row = *reinterpret_cast<const half8_t*>(cells + g * ROWS_PER_PASS * STAGE_PITCH);
          const int uniform = (strip * PASSES + pass) * c_pass_bytes;
          if (RANGE) { BufferStore<T, 8>(row, c_view, c_piece_there(strip, pass) ? c_lane_offset + uniform : kHOutside); }
          else { BufferStore<T, 8>(row, c_view, c_lane_offset, uniform); }
        }
        if (RANGE && wave_m0 + WAVE_M > p.m) {
#pragma unroll 1
          for (int g = 0; g < HALF_PASSES; ++g) {
            const int pass = half * HALF_PASSES + g;
            const bool there = 32 * strip + pass * ROWS_PER_PASS + c_first_row < c_rows_left && straddles;
#pragma unroll
            for (int e = 0; e < 7; ++e) {
              const int element = (there && e < c_inside) ? c_lane_offset + (strip * PASSES + pass) * c_pass_bytes + 2 * e : kHOutside;
              __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, cells[g * ROWS_PER_PASS * STAGE_PITCH + e]), c_view, element, 0, 0);
            }
          }
        }
        wave_fence();
      }
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_WIDE_F16_HPP_
