// =================================================================================================
// fp32 GEMM kernel for skinny problems on gfx950 whose large operand is x-contiguous: one extent of C is at most 32
// (n <= 32 with a long m and a plain column-major A, or m <= 32 with a long n and a B of contiguous rows) and k is
// long, e.g. 4099 x 17 x 4096 N/N. Such a product is one pass over the large operand X, bound by HBM. The counterpart
// for a k-contiguous X is kernels/gemm_skinny.hpp; the reference sends all of these shapes to its direct kernel with
// 16 x 16 tiles (src/routines/level3/xgemm.cpp:228-268, src/kernels/level3/xgemm_direct_part3.opencl:17-212).
//
// The lanes of a wavefront run along the rows of X, four consecutive rows per lane and 64 per wavefront load, so every
// load covers whole 256-byte runs of four rows of k; with so few rows per work-group K has to be split, and that is
// done twice: over the eight wavefronts of a work-group, whose sums meet in LDS, and over `ranges` work-groups per
// strip of 64 rows, whose sums meet in memory WITHOUT a second launch - every work-group stores its partial sums,
// takes a ticket of the strip's counter, and the one that draws the last ticket adds all partial sums of the strip in
// the order of the ranges (not of arrival: the result does not depend on timing), applies alpha and beta and writes C.
// It also puts the counter back to zero: the counters are zero before and after every launch.
//
// Products: v_mfma_f32_16x16x4_f32. Of a run of 16 k, lane group g = lane / 16 takes the four k from 4 g on. In step
// s = 0..3 the lane loads its four rows at k = 4 g + s (16 bytes) and feeds them to four instructions, component j to
// instruction j: that instruction's row lane % 16 stands for row 4 (lane % 16) + j of the strip, its four k are
// s, 4 + s, 8 + s, 12 + s of the run. The other operand is the small matrix S, 16 columns per block of instructions and
// one or two blocks: with k contiguous in S a lane's four values for the four steps are one 16-byte load. A lane's
// sixteen results per block are rows 16 g + 4 r + j (r = 0..3: result register, j: instruction) of column lane % 16, so
// the four instructions' registers r form runs of four consecutive rows and everything moves in 16-byte pieces.
// Loads are requested DEPTH runs ahead through range-checked buffer resources: beyond the end of an operand they
// deliver zeros, rows of X beyond its extent deliver a neighbour's data that only reaches sums nobody stores, and the
// K tail is cut by offsets outside the resource (X) and by zeroing (S, whose columns could hold anything there).
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_SKINNY_COLS_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_SKINNY_COLS_HPP_

#include <type_traits>

#include "kernels/gemm_mfma.hpp"

namespace clbh {

constexpr int kSkinnyColsWaves = 8;     // wavefronts per work-group
constexpr int kSkinnyColsRows = 64;     // rows of X per work-group
constexpr int kSkinnyColsRun = 16;      // k per step of a wavefront
constexpr int kSkinnyColsPitch = 68;    // floats per column of a wavefront's sums in LDS (64 rows and a shift of the banks)

struct SkinnyColsArgs {
  const float* x;          // the large operand: element (row, k) at x[k * x_ld + row]
  const float* s;          // the small operand: element (k, col) at s[k * s_k_stride + col * s_col_stride]
  float* c;                // result: element (row, col) at c[row * c_row_stride + col * c_col_stride]
  float* partials;         // ranges > 1: [range][col][partial_ld] sums of the ranges
  unsigned int* tickets;   // ranges > 1: one counter per strip, zero before and after the launch
  long long x_ld, s_k_stride, s_col_stride, c_row_stride, c_col_stride;
  int extent;              // rows of X
  int small;               // columns of S (<= 16 * BLOCKS)
  int k;
  int ranges;              // work-groups per strip
  int k_per_group;         // K range of a work-group: a multiple of kSkinnyColsWaves * kSkinnyColsRun
  int partial_ld;          // a multiple of kSkinnyColsRows, >= extent
  float alpha, beta;
};

// Columns of S beyond the last whole block of 16: up to kSkinnyColsMaxExtra of them are multiplied on the vector ALUs
// (17 columns as two blocks of matrix instructions would double the matrix pipe's work, which with two blocks is about
// as long as the stream itself: 4099 x 17 x 4096 ran at 2.2 to 3 TB/s that way)
constexpr int kSkinnyColsMaxExtra = 4;
constexpr size_t SkinnyColsLdsBytes(const int blocks, const int extra) {
  return sizeof(float) * kSkinnyColsWaves * (16 * blocks + 4 * extra) * kSkinnyColsPitch;
}

// grid: strips * ranges work-groups of 512 threads (which strip and range a work-group serves: see below).
template <int BLOCKS, int EXTRA, int DEPTH, bool S_KC>
__global__ __launch_bounds__(64 * kSkinnyColsWaves, 2) void GemmSkinnyColsKernel(const SkinnyColsArgs p) {
  constexpr int WAVES = kSkinnyColsWaves, RUN = kSkinnyColsRun, PITCH = kSkinnyColsPitch;
  constexpr int BLOCK_COLS = 16 * BLOCKS, COLS = BLOCK_COLS + EXTRA;  // columns on the matrix pipe, all columns
  typedef float float4_t __attribute__((ext_vector_type(4)));
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* sums = reinterpret_cast<float*>(lds_raw);  // [WAVES][BLOCK_COLS][PITCH]
  float* extra_sums = sums + WAVES * BLOCK_COLS * PITCH;  // [WAVES * 4 lane groups][EXTRA][PITCH]
  __shared__ unsigned int ticket_drawn;

  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  // Neighbouring strips go to the same XCD (work-groups are dealt to the XCDs in turn, each XCD has its own L2): a
  // strip's 256-byte runs start wherever the leading dimension puts them, so a run shares its first and last 128-byte
  // line with the neighbours' runs, and the work-groups of an XCD walk K at the same pace - one of them fetches such a
  // line, the other finds it in the L2. (Strip after strip dealt across the XCDs, 4099 x 17 x 4096 with a leading
  // dimension of 4102 read 1.56 times the bytes of X from memory.)
  const int strips = gridDim.x / p.ranges;
  const int logical = XcdContiguousIndex(blockIdx.x, gridDim.x);
  const int strip = logical / p.ranges, range = logical % p.ranges;
  const int row0 = strip * kSkinnyColsRows;
  const int lane_row = 4 * (lane % 16), lane_g = lane / 16;

  // this wavefront's share of the work-group's K range: runs wave, wave + WAVES, ... of it
  const int k_begin = range * p.k_per_group;
  const int k_end = min(p.k, k_begin + p.k_per_group);
  const int runs = (k_end - k_begin + RUN - 1) / RUN;           // of the work-group
  const int my_runs = (runs - wave + WAVES - 1) / WAVES;        // of this wavefront (may be zero or negative)

  const float* x_strip = p.x + row0;
  const float* x_end = p.x + static_cast<long long>(p.k - 1) * p.x_ld + p.extent;
  const float* s_end = p.s + static_cast<long long>(p.k - 1) * p.s_k_stride + static_cast<long long>(p.small - 1) * p.s_col_stride + 1;
  const int x_step_bytes = static_cast<int>(p.x_ld * 4);        // from one k to the next
  const int x_lane_bytes = static_cast<int>((4 * lane_g * p.x_ld + lane_row) * 4);
  constexpr int kOutside = static_cast<int>(0x80000000u);
  int s_lane_bytes[BLOCKS];
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) {
    const int col = 16 * b + lane % 16;
    s_lane_bytes[b] = (col < p.small) ? static_cast<int>((col * p.s_col_stride + 4 * lane_g * p.s_k_stride) * 4) : kOutside;
  }

  int extra_lane_bytes[EXTRA > 0 ? EXTRA : 1];  // (the sixteen lanes of a group read the same values: one column each)
#pragma unroll
  for (int c = 0; c < EXTRA; ++c) {
    extra_lane_bytes[c] = (BLOCK_COLS + c < p.small) ? static_cast<int>(((BLOCK_COLS + c) * p.s_col_stride + 4 * lane_g * p.s_k_stride) * 4) : kOutside;
  }
  float4_t extra_acc[EXTRA > 0 ? EXTRA : 1];  // rows 4 (lane % 16) + j of column BLOCK_COLS + c, over the lane group's k only
#pragma unroll
  for (int c = 0; c < EXTRA; ++c) { extra_acc[c] = float4_t(0.0f); }
  float4_t acc[BLOCKS][4];
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) {
#pragma unroll
    for (int j = 0; j < 4; ++j) { acc[b][j] = float4_t(0.0f); }
  }

  // At the end thread t holds the piece (col, rows 4 q .. 4 q + 3) of the strip's sums, t = 16 col + q; with two blocks
  // of columns every thread has a piece, with one block the first half of the threads. The old values of C that such
  // a piece is combined with are fetched here, ahead of the walk over K, by every work-group of the strip (only the
  // one that finishes the strip uses them, and only that one writes C, after all others have come by): the fetch
  // would otherwise stand at the end of a chain of memory round trips - partial sums, ticket, partial sums, C.
  const int col = tid / 16, q = tid % 16;
  const bool has_piece = col < COLS;
  const int row = row0 + 4 * q;
  const bool stores = has_piece && col < p.small && row < p.extent;
  const bool whole_piece = p.c_row_stride == 1 && row + 3 < p.extent;
  typedef float float4u_t __attribute__((ext_vector_type(4), aligned(4)));
  float* const c_piece = p.c + row * p.c_row_stride + col * p.c_col_stride;
  float4_t old_c = float4_t(0.0f);
  if (stores && p.beta != 0.0f) {
    if (whole_piece) {
      old_c = *reinterpret_cast<const float4u_t*>(c_piece);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (row + e < p.extent) { old_c[e] = c_piece[e * p.c_row_stride]; }
      }
    }
  }

  // One run of 16 k: the lane's four pieces of X (steps s = 0..3) and its values of S per block
  struct Run {
    float4_t x[4];
    float4_t s[BLOCKS];
    float4_t e[EXTRA > 0 ? EXTRA : 1];
    int k_left;  // how many of the lane's four k lie inside the K range (the rest of S is zeroed when the run is multiplied:
                 // touching the values here would wait for the loads at once)
  };
  auto request = [&](const int index) {  // run `index` of this wavefront
    Run run;
    const int k0 = k_begin + (wave + index * WAVES) * RUN;
    const float* x_run = x_strip + static_cast<long long>(k0) * p.x_ld;
    const float* s_run = p.s + static_cast<long long>(k0) * p.s_k_stride;
    const auto x_view = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x_run), 0, RecordsUpTo(x_run, x_end), kRawBufferFlags);
    const auto s_view = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(s_run), 0, RecordsUpTo(s_run, s_end), kRawBufferFlags);
    const int k_lane = k0 + 4 * lane_g;  // the lane's first k of the run
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      run.x[s] = BufferLoad<float, 4>(x_view, (k_lane + s < k_end) ? x_lane_bytes + s * x_step_bytes : kOutside);
    }
#pragma unroll
    for (int b = 0; b < BLOCKS; ++b) {
      if (S_KC) {
        run.s[b] = BufferLoad<float, 4>(s_view, (k_lane < k_end) ? s_lane_bytes[b] : kOutside);
      } else {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          run.s[b][s] = BufferLoad<float, 1>(s_view, (k_lane + s < k_end && s_lane_bytes[b] != kOutside)
                                                        ? s_lane_bytes[b] + s * static_cast<int>(p.s_k_stride * 4) : kOutside);
        }
      }
    }
#pragma unroll
    for (int c = 0; c < EXTRA; ++c) {
      if (S_KC) {
        run.e[c] = BufferLoad<float, 4>(s_view, (k_lane < k_end) ? extra_lane_bytes[c] : kOutside);
      } else {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          run.e[c][s] = BufferLoad<float, 1>(s_view, (k_lane + s < k_end && extra_lane_bytes[c] != kOutside)
                                                        ? extra_lane_bytes[c] + s * static_cast<int>(p.s_k_stride * 4) : kOutside);
        }
      }
    }
    run.k_left = k_end - k_lane;
    return run;
  };
  auto multiply = [&](const Run& run) {
    float4_t small[BLOCKS];
#pragma unroll
    for (int b = 0; b < BLOCKS; ++b) {
#pragma unroll
      for (int s = 0; s < 4; ++s) { small[b][s] = (s < run.k_left) ? run.s[b][s] : 0.0f; }  // (S may hold anything beyond K)
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int b = 0; b < BLOCKS; ++b) {
          acc[b][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(run.x[s][j], small[b][s], acc[b][j], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int c = 0; c < EXTRA; ++c) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const float value = (s < run.k_left) ? run.e[c][s] : 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) { extra_acc[c][j] = __builtin_fmaf(run.x[s][j], value, extra_acc[c][j]); }
      }
    }
  };
  // (no branch stands between the requests: one beyond the wavefront's last run has all its offsets outside the
  // resources and moves nothing - with a branch per request the compiler waits for every load at the join)
  Run ahead[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    // (in the order of the turns below: the wait at the top of the loop is one count for both ways into it)
    __builtin_amdgcn_sched_barrier(0);
    ahead[d] = request(d);
    __builtin_amdgcn_sched_barrier(0);
  }
  // (the order is pinned: left alone, the compiler moves all requests of a turn behind all its products and waits for
  // them at the top of the next turn - nothing would be in flight under the products)
  for (int index = 0; index < my_runs; index += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      multiply(ahead[d]);
      __builtin_amdgcn_sched_barrier(0);
      ahead[d] = request(index + d + DEPTH);  // into the registers whose values the products above have taken
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // The wavefronts' sums meet in LDS: [wave][col][row], 16-byte pieces of four consecutive rows
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float4_t piece;
#pragma unroll
      for (int j = 0; j < 4; ++j) { piece[j] = acc[b][j][r]; }
      *reinterpret_cast<float4_t*>(&sums[(wave * BLOCK_COLS + 16 * b + lane % 16) * PITCH + 16 * lane_g + 4 * r]) = piece;
    }
  }
#pragma unroll
  for (int c = 0; c < EXTRA; ++c) {
    *reinterpret_cast<float4_t*>(&extra_sums[((wave * 4 + lane_g) * EXTRA + c) * PITCH + lane_row]) = extra_acc[c];
  }
  __syncthreads();
  // thread t adds its piece of all wavefronts in their order
  float4_t total = float4_t(0.0f);
  if (has_piece && col < BLOCK_COLS) {
#pragma unroll
    for (int w = 0; w < WAVES; ++w) { total += *reinterpret_cast<const float4_t*>(&sums[(w * BLOCK_COLS + col) * PITCH + 4 * q]); }
  } else if (has_piece) {
#pragma unroll
    for (int w = 0; w < WAVES * 4; ++w) { total += *reinterpret_cast<const float4_t*>(&extra_sums[(w * EXTRA + col - BLOCK_COLS) * PITCH + 4 * q]); }
  }
  auto finish = [&](const float4_t sum) {  // C = alpha * sum + beta * C for the thread's piece
    float4_t out;
#pragma unroll
    for (int e = 0; e < 4; ++e) { out[e] = (p.beta != 0.0f) ? Combine(p.alpha, sum[e], p.beta, old_c[e]) : p.alpha * sum[e]; }
    if (whole_piece) {
      *reinterpret_cast<float4u_t*>(c_piece) = out;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (row + e < p.extent) { c_piece[e * p.c_row_stride] = out[e]; }
      }
    }
  };
  if (p.ranges == 1) {
    if (stores) { finish(total); }
    return;
  }
  // Several work-groups per strip: the sums of this range go to memory, then a ticket; whoever draws the last one adds
  // the ranges in their order. The work-groups of a strip run on different XCDs, whose L2 caches do not see each other's
  // lines. A fence of device scope would write back and invalidate the whole L2 of the XCD, twice per work-group, under
  // the other work-groups' streams (measured: the launch took 88 us instead of 16). Instead the few accesses that cross
  // work-groups say so themselves: the partial sums are stored and loaded with the cache bits of device-coherent
  // accesses (written through to memory, read past the L2), the ticket is a relaxed device-scope atomic, and the order
  // between them is the order of completion - the stores have been acknowledged (vmcnt) before the ticket is taken, the
  // ticket has come back before the loads are issued.
  const long long slab = static_cast<long long>(p.partial_ld) * COLS;
  if (has_piece) {
    float* place = &p.partials[range * slab + static_cast<long long>(col) * p.partial_ld + row];
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(place), "v"(total) : "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) { ticket_drawn = __hip_atomic_fetch_add(&p.tickets[strip], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
  __syncthreads();
  if (ticket_drawn != static_cast<unsigned int>(p.ranges - 1)) { return; }
  // (nobody else touches this strip's counter any more: back to zero for the next launch)
  if (tid == 0) { __hip_atomic_store(&p.tickets[strip], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
  if (stores) {
    float4_t sum = float4_t(0.0f);
    for (int first = 0; first < p.ranges; first += 8) {  // eight loads in flight, added in the order of the ranges
      float4_t piece[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float* place = &p.partials[min(first + i, p.ranges - 1) * slab + static_cast<long long>(col) * p.partial_ld + row];
        asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=v"(piece[i]) : "v"(place) : "memory");
      }
      asm volatile("s_waitcnt vmcnt(0)"
                   : "+v"(piece[0]), "+v"(piece[1]), "+v"(piece[2]), "+v"(piece[3]), "+v"(piece[4]), "+v"(piece[5]), "+v"(piece[6]), "+v"(piece[7])
                   :: "memory");
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (first + i < p.ranges) { sum += piece[i]; }
      }
    }
    finish(sum);
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_SKINNY_COLS_HPP_
