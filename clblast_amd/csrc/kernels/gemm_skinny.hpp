// =================================================================================================
// fp32 GEMM kernel for skinny problems on gfx950: one extent of C is at most 32 (n <= 32 with a long m, or
// m <= 32 with a long n) and k is long, e.g. 4099 x 17 x 4096. Such a product is a stream over the large operand
// (8.4 flop per byte: HBM-bound), which the tiled kernel of gemm_mfma.hpp cannot keep up: its ring of LDS slabs holds
// two slabs in flight per work-group, a few KB per CU against the roughly 60 KB per CU that 8 TB/s times the memory
// latency asks for, and its tiles pad the short extent to 32 (fp32 matrix cores deliver 157 TFLOP/s: at 32 columns
// the products take as long as the stream). (The reference sends these shapes to its direct kernel with 16 x 16 tiles,
// src/routines/level3/xgemm.cpp:228-268, xgemm_direct_part3.opencl.)
//
// Here the large operand X (extent x K) never touches LDS: every wavefront streams its share - 256 rows of X times its
// own K range - straight into registers in the layout the matrix instruction wants, sixteen 1 KiB loads in flight per
// wavefront. The small operand S (K x at most 32) goes through a wavefront-private LDS tile, 16 rows of k at a time, so
// the K walk needs no work-group barrier. The wavefronts of a work-group split the work-group's K range; their partial
// sums meet through LDS at the end in a fixed tree. Work-groups split K further (blockIdx.y); their partial sums go to
// the workspace and GemmSkinnyReduceKernel adds them in slab order.
//
// Matrix instruction v_mfma_f32_4x4x1_16b_f32: sixteen independent 4 x 4 outer products. Block b = lane / 4 multiplies
// four values of S (one per lane % 4, the same in every block: columns 4g .. 4g + 3 of S at one k) with the block's
// four values of X (one per lane: the lane's own row x at that k). A lane's four result registers are the four columns
// of ITS x: lanes own rows of X, registers run along the short extent, which is padded to a multiple of 4 only.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_SKINNY_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_SKINNY_HPP_

#include <type_traits>

#include "kernels/gemm_mfma.hpp"

namespace clbh {

constexpr int kSkinnyTileX = 256;    // rows of X per work-group: four per lane
constexpr int kSkinnyChunk = 16;     // k per chunk: 16 loads of 1 KiB per wavefront, one LDS tile of S
constexpr int kSkinnyLoads = 16;     // loads of X per chunk and wavefront
constexpr int kSkinnySTile = kSkinnyChunk * 4 * 8;  // floats of an S tile: [16 k][4 columns of a group][8 groups]

// LDS floats of a work-group: two S tiles per wavefront during the walk, WAVES / 2 buffers of partial sums after it
constexpr int SkinnyLdsFloats(const int waves, const int groups) {
  const int tiles = waves * 2 * kSkinnySTile, sums = (waves / 2) * groups * 16 * 64;
  return tiles > sums ? tiles : sums;
}

struct SkinnyArgs {
  const float* x;        // the streamed operand: element (row, k) at x[X_KC ? row * x_ld + k : k * x_ld + row]
  const float* s;        // the small operand: element (k, col) at s[S_KC ? col * s_ld + k : k * s_ld + col]
  float* c;              // result: element (row, col) at c[X_IS_A ? col * c_ld + row : row * c_ld + col]
  long long x_ld, s_ld, c_ld;
  int extent;            // rows of X
  int small;             // columns of S (<= 4 * GROUPS)
  int k;
  int k_per_group;       // K range of a work-group: a multiple of kSkinnyChunk * WAVES
  float alpha, beta;
  float* partial;        // not null: K is split over blockIdx.y; range y writes slab y here (laid out like a C with
  long long partial_ld;  // this leading dimension, slab_elements apart), alpha and beta are left to the reduction
  long long slab_elements;
};

// WAVES wavefronts per work-group (a power of two). GROUPS: column groups of four (the short extent is at most
// 4 * GROUPS). X_KC / S_KC: the k index of the operand is the contiguous one. X_IS_A: X is the canonical A (its rows
// are m), else the canonical B (its rows are n).
template <int WAVES, int GROUPS, bool X_KC, bool S_KC, bool X_IS_A>
__global__ __launch_bounds__(64 * WAVES) void GemmSkinnyKernel(const SkinnyArgs p) {
  typedef float float4_t __attribute__((ext_vector_type(4)));
  typedef float float4u_t __attribute__((ext_vector_type(4), aligned(4)));
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* lds = reinterpret_cast<float*>(lds_raw);
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int x0 = blockIdx.x * kSkinnyTileX;
  // this wavefront's K range
  const int group_begin = blockIdx.y * p.k_per_group;
  const int per_wave = p.k_per_group / WAVES;
  const int k_begin = group_begin + wave * per_wave;
  const int k_end = min(k_begin + per_wave, p.k);
  const int chunks = (k_end > k_begin) ? (k_end - k_begin + kSkinnyChunk - 1) / kSkinnyChunk : 0;

  // acc[q][g][i]: row x = x0 + (X_KC ? 64 * q + lane : 4 * lane + q), column 4 * g + i
  float4_t acc[4][GROUPS];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) { acc[q][g] = float4_t(0.0f); }
  }

  // ---- X: sixteen loads of 16 bytes per lane and chunk. x-contiguous: load d brings row k = d of the chunk, the lane's
  // four consecutive x. k-contiguous: load d brings k = 4 * (d / 4) .. + 3 of the row 64 * (d % 4) + lane.
  // Every load goes through a range-checked buffer resource that ends with the tile's last valid element, so that no
  // lane ever touches memory outside the operand and rows of X beyond its extent read as zeros or as other rows (their
  // results are never stored). x-contiguous X: the range also ends with row k_end - 1, so k beyond the range reads as
  // zero. k-contiguous X: k beyond the range only occurs behind the last k of the operand (ranges are multiples of a
  // chunk), where a lane reads the next row or padding; the last chunk of a wavefront replaces such elements by zeros.
  const int x_rows = min(p.extent - x0, kSkinnyTileX);  // > 0
  const float* x_tile = p.x + static_cast<long long>(x0) * (X_KC ? p.x_ld : 1);
  const int lane_offset = X_KC ? static_cast<int>(lane * p.x_ld * 4) : 16 * lane;
  const int block_bytes = static_cast<int>(64 * p.x_ld * 4);  // (k-contiguous X: from one block of 64 rows to the next)
  float4_t ring[kSkinnyLoads];
  auto load_x = [&](const int d, const int chunk_k) {  // chunk_k: first k of the chunk
    long long first, valid;  // the load's uniform first element and the elements from there to the end of the range
    if constexpr (!X_KC) {
      first = static_cast<long long>(chunk_k + d) * p.x_ld;
      valid = (static_cast<long long>(k_end) - 1) * p.x_ld + x_rows - first;
    } else {
      first = chunk_k + 4 * (d / 4);
      valid = static_cast<long long>(x_rows - 1) * p.x_ld + p.k - first;
    }
    const int records = static_cast<int>(min(max(valid, 0ll) * 4, 0x7fffffffll));
    const int offset = lane_offset + (X_KC ? (d % 4) * block_bytes : 0);
    return __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x_tile + first), 0, records, kRawBufferFlags), offset, 0, 0));
  };

  // ---- S: a tile of 16 k x 32 columns per chunk, private to the wavefront, in two LDS buffers, laid out
  // [k][column % 4][column / 4]: the eight floats a lane needs at one k (its lane % 4, every group) are contiguous.
  // k >= k_end and columns >= p.small become zeros (their loads read the last valid k or column instead, so that every
  // load is issued and the counter of outstanding loads is the same for every lane).
  // k-contiguous S: load g brings column group g, lanes along k (16) then the group's four columns.
  // column-contiguous S: load h brings k = 2h, 2h + 1, lanes along the 32 columns.
  constexpr int S_LOADS = S_KC ? GROUPS : 8;
  float* s_tile = lds + wave * (2 * kSkinnySTile);
  float s_regs[S_LOADS];
  auto s_element = [&](const int h, int& kk, int& col) {
    kk = S_KC ? lane % 16 : 2 * h + lane / 32;
    col = S_KC ? 4 * h + lane / 16 : lane % 32;
  };
  auto load_s = [&](const int chunk_k) {
#pragma unroll
    for (int h = 0; h < S_LOADS; ++h) {
      int kk, col;
      s_element(h, kk, col);
      const int k = min(chunk_k + kk, p.k - 1), column = min(col, p.small - 1);
      s_regs[h] = p.s[S_KC ? column * p.s_ld + k : k * p.s_ld + column];
    }
  };
  auto store_s = [&](float* tile, const int chunk_k) {
#pragma unroll
    for (int h = 0; h < S_LOADS; ++h) {
      int kk, col;
      s_element(h, kk, col);
      tile[(kk * 4 + col % 4) * 8 + col / 4] = (chunk_k + kk < k_end && col < p.small) ? s_regs[h] : 0.0f;
    }
  };
  // the products of the X values of one k (a lane's four rows) with the row k of S
  auto multiply_k = [&](const int kk, const float* tile, const float4_t x_values) {
    float s_values[8];
    const float4_t* source = reinterpret_cast<const float4_t*>(tile + (kk * 4 + lane % 4) * 8);
    const float4_t low = source[0];
    float4_t high = float4_t(0.0f);
    if constexpr (GROUPS > 4) { high = source[1]; }
#pragma unroll
    for (int g = 0; g < 4; ++g) { s_values[g] = low[g]; s_values[4 + g] = high[g]; }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int g = 0; g < GROUPS; ++g) {
        acc[q][g] = __builtin_amdgcn_mfma_f32_4x4x1f32(s_values[g], x_values[q], acc[q][g], 0, 0, 0);
      }
    }
  };

  if (chunks > 0) {
    load_s(k_begin);
#pragma unroll
    for (int d = 0; d < kSkinnyLoads; ++d) { ring[d] = load_x(d, k_begin); }
    store_s(s_tile, k_begin);
    int chunk_k = k_begin;
    for (int chunk = 0; chunk + 1 < chunks; ++chunk, chunk_k += kSkinnyChunk) {
      const float* tile = s_tile + (chunk % 2) * kSkinnySTile;
      load_s(chunk_k + kSkinnyChunk);
      __builtin_amdgcn_wave_barrier();  // (LDS operations of a wavefront complete in order: the tile is written)
      if constexpr (!X_KC) {
#pragma unroll
        for (int d = 0; d < kSkinnyLoads; ++d) {
          const float4_t piece = ring[d];
          ring[d] = load_x(d, chunk_k + kSkinnyChunk);
          multiply_k(d, tile, piece);
        }
      } else {
#pragma unroll
        for (int d4 = 0; d4 < kSkinnyLoads; d4 += 4) {
          float4_t pieces[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            pieces[q] = ring[d4 + q];
            ring[d4 + q] = load_x(d4 + q, chunk_k + kSkinnyChunk);
          }
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const float4_t x_values = {pieces[0][t], pieces[1][t], pieces[2][t], pieces[3][t]};
            multiply_k(d4 + t, tile, x_values);
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
      store_s(s_tile + ((chunk + 1) % 2) * kSkinnySTile, chunk_k + kSkinnyChunk);
    }
    // the last chunk: nothing follows it, and it may hold the K tail
    const float* tile = s_tile + ((chunks - 1) % 2) * kSkinnySTile;
    __builtin_amdgcn_wave_barrier();
    if constexpr (!X_KC) {
#pragma unroll
      for (int d = 0; d < kSkinnyLoads; ++d) { multiply_k(d, tile, ring[d]); }
    } else {
#pragma unroll
      for (int d4 = 0; d4 < kSkinnyLoads; d4 += 4) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const bool inside = chunk_k + d4 + t < k_end;
          const float4_t x_values = {inside ? ring[d4][t] : 0.0f, inside ? ring[d4 + 1][t] : 0.0f,
                                     inside ? ring[d4 + 2][t] : 0.0f, inside ? ring[d4 + 3][t] : 0.0f};
          multiply_k(d4 + t, tile, x_values);
        }
      }
    }
  }

  // ---- the wavefronts' partial sums meet in a tree: in every round the upper half of the remaining wavefronts hands
  // its sums to the lower half through LDS (register by register, lane to the same lane), until wavefront 0 holds the
  // sum ((w0 + w4) + (w2 + w6)) + ((w1 + w5) + (w3 + w7)) for eight wavefronts: the same order in every launch.
  __syncthreads();  // every wavefront is done with its S tiles
  float4_t* sums = reinterpret_cast<float4_t*>(lds);
#pragma unroll
  for (int half = WAVES / 2; half >= 1; half /= 2) {
    if (wave >= half && wave < 2 * half) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) { sums[((wave - half) * 4 * GROUPS + q * GROUPS + g) * 64 + lane] = acc[q][g]; }
      }
    }
    __syncthreads();
    if (wave < half) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) { acc[q][g] += sums[(wave * 4 * GROUPS + q * GROUPS + g) * 64 + lane]; }
      }
    }
    if (half > 1) { __syncthreads(); }
  }
  if (wave != 0) { return; }

  // ---- wavefront 0 writes the tile: to C, or to this K range's slab
  const bool to_slab = (p.partial != nullptr);
  float* target = to_slab ? p.partial + blockIdx.y * p.slab_elements : p.c;
  const long long ld = to_slab ? p.partial_ld : p.c_ld;
  const float alpha = to_slab ? 1.0f : p.alpha, beta = to_slab ? 0.0f : p.beta;
  if constexpr (X_IS_A && !X_KC) {
    // the lane's four consecutive rows are contiguous in a column of C
    const int row = 4 * lane;
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int col = 4 * g + i;
        if (col < p.small && row < x_rows) {
          float* destination = target + col * ld + x0 + row;
          if (row + 3 < x_rows) {
            float4_t result;
            if (beta != 0.0f) {
              const float4_t old = *reinterpret_cast<const float4u_t*>(destination);
#pragma unroll
              for (int q = 0; q < 4; ++q) { result[q] = Combine(alpha, acc[q][g][i], beta, old[q]); }
            } else {
#pragma unroll
              for (int q = 0; q < 4; ++q) { result[q] = alpha * acc[q][g][i]; }
            }
            *reinterpret_cast<float4u_t*>(destination) = result;
          } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              if (row + q < x_rows) { StoreResult<float, float>(destination, q, acc[q][g][i], alpha, beta); }
            }
          }
        }
      }
    }
  } else {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int row = X_KC ? 64 * q + lane : 4 * lane + q;
      if (row < x_rows) {
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int col = 4 * g + i;
            if (col < p.small) {
              const long long index = X_IS_A ? col * ld + x0 + row : (x0 + row) * ld + col;
              StoreResult<float, float>(target, index, acc[q][g][i], alpha, beta);
            }
          }
        }
      }
    }
  }
}

// =================================================================================================
// The same problem when the k index of X is the contiguous one (a transposed A, a plain B): rows of X are long
// contiguous runs, and a wavefront that put its lanes along the rows of X would touch 64 rows with every load (measured:
// twice the time of the tiled kernel). Here the lanes of a wavefront run along k: block b = lane / 4 of the matrix
// instruction takes the four k from 4b on of every 64 (a 16-byte load per lane, 256 contiguous bytes per row and load),
// the four lanes of a block take four rows of X. A work-group owns 4 * RG rows of X and ALL of K, split over its
// wavefronts: no second pass, no workspace. A lane's sums cover its share of k only; they meet at the end - first the
// four lanes of a 16-lane row that hold the same row of X (two rotations), then rows and wavefronts through LDS, added
// in a fixed order.
// S must be k-contiguous as well (element (k, col) at s[col * s_ld + k]): a lane loads the four k of its block for
// column 4g + lane % 4 in one piece, which is the A operand of its block as it stands. Both operands are requested
// DEPTH steps (of 64 k) ahead: the counter of outstanding loads completes in order, a wait for a late request of S
// would wait for every earlier request of X too.
// =================================================================================================
constexpr int kSkinnyRowsStep = 64;  // k per step and wavefront

constexpr int SkinnyRowsLdsFloats(const int waves, const int groups, const int rg) { return waves * 4 * (4 * rg) * (4 * groups); }

template <int WAVES, int GROUPS, int RG, int DEPTH, bool X_IS_A, int WAVES_PER_SIMD = 2>
__global__ __launch_bounds__(64 * WAVES, WAVES_PER_SIMD) void GemmSkinnyRowsKernel(const SkinnyArgs p) {
  typedef float float4_t __attribute__((ext_vector_type(4)));
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* lds = reinterpret_cast<float*>(lds_raw);
  constexpr int ROWS = 4 * RG, COLS = 4 * GROUPS;
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int slot = lane / 4, quad_lane = lane % 4;  // the block's k slot; row of X (as B operand) and column of S (as A)
  const int row0 = blockIdx.x * ROWS;
  const int rows = min(p.extent - row0, ROWS);  // > 0
  // this wavefront's K range (p.k_per_group: the range of a wavefront here, a multiple of a step) and, per lane, the
  // number of k from the lane's first one to the end of the range
  const int k_begin = wave * p.k_per_group;
  const int k_end = min(k_begin + p.k_per_group, p.k);
  const int steps = (k_end > k_begin) ? (k_end - k_begin + kSkinnyRowsStep - 1) / kSkinnyRowsStep : 0;
  const int lane_length = k_end - k_begin - 4 * slot;
  // Work-groups walk the steps of a range in different rotations: every work-group reads all of S, and with a common
  // order all of them would ask the same few L2 channels for the same lines at the same time.
  const int rotation = (steps > 0) ? static_cast<int>(blockIdx.x % static_cast<unsigned>(steps)) : 0;
  auto rotated = [&](const int step) {  // the step of the range that comes at position `step` of the walk
    const int shifted = step + rotation;
    return (step >= steps) ? step : (shifted >= steps ? shifted - steps : shifted);
  };

  float4_t acc[RG][GROUPS];
#pragma unroll
  for (int r = 0; r < RG; ++r) {
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) { acc[r][g] = float4_t(0.0f); }
  }

  // The elements of the work-group's tile of C, ordered so that consecutive ones are neighbours in memory; thread t
  // finishes the elements t, t + threads, ... at the end and fetches their old values now, when beta asks for them
  constexpr int ELEMENTS = ROWS * COLS, THREADS = 64 * WAVES, PER_THREAD = (ELEMENTS + THREADS - 1) / THREADS;
  auto c_index = [&](const int e, bool& inside) {
    const int row = X_IS_A ? e % ROWS : e / COLS, col = X_IS_A ? e / ROWS : e % COLS;
    inside = e < ELEMENTS && row < rows && col < p.small;
    return X_IS_A ? col * p.c_ld + row0 + row : (row0 + row) * p.c_ld + col;
  };
  float old_c[PER_THREAD];
#pragma unroll
  for (int q = 0; q < PER_THREAD; ++q) {
    bool inside;
    const long long index = c_index(tid + q * THREADS, inside);
    old_c[q] = (inside && p.beta != 0.0f) ? p.c[index] : 0.0f;
  }

  // Range-checked resources over the work-group's rows of X and over S: a piece that starts at or behind the end of
  // the lane's range is requested at an offset outside the resource and reads as zeros without touching memory; one that
  // straddles the end reads what lies there (the next row, padding; zeros behind the operand) and is cleaned below.
  // Rows of X beyond its extent and columns of S beyond p.small read the last valid one (their results are not stored).
  const float* x_base = p.x + static_cast<long long>(row0) * p.x_ld + k_begin;
  const float* s_base = p.s + k_begin;
  const long long x_valid = static_cast<long long>(rows - 1) * p.x_ld + p.k - k_begin;
  const long long s_valid = static_cast<long long>(p.small - 1) * p.s_ld + p.k - k_begin;
  constexpr int kOutside = 0x7fffff00;  // (an offset no resource reaches)
  const int x_records = static_cast<int>(min(max(x_valid, 0ll) * 4, static_cast<long long>(kOutside)));
  const int s_records = static_cast<int>(min(max(s_valid, 0ll) * 4, static_cast<long long>(kOutside)));
  int x_offset[RG], s_offset[GROUPS];
#pragma unroll
  for (int r = 0; r < RG; ++r) { x_offset[r] = static_cast<int>((min(4 * r + quad_lane, rows - 1) * p.x_ld + 4 * slot) * 4); }
#pragma unroll
  for (int g = 0; g < GROUPS; ++g) { s_offset[g] = static_cast<int>((min(4 * g + quad_lane, p.small - 1) * p.s_ld + 4 * slot) * 4); }

  float4_t x_ring[DEPTH][RG], s_ring[DEPTH][GROUPS];
  auto request = [&](const int d, const int position) {
    const int step = rotated(position);
    // (the offsets go through an empty asm statement: the compiler would otherwise turn each select into a branch
    // around two loads, and could no longer count the loads in flight)
    const int step_bytes = (step * kSkinnyRowsStep < lane_length) ? step * kSkinnyRowsStep * 4 : kOutside;
    const auto x_resource = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x_base), 0, x_records, kRawBufferFlags);
    const auto s_resource = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(s_base), 0, s_records, kRawBufferFlags);
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      int offset = s_offset[g] + step_bytes;
      asm volatile("" : "+v"(offset));
      s_ring[d][g] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(s_resource, offset, 0, 0));
    }
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      int offset = x_offset[r] + step_bytes;
      asm volatile("" : "+v"(offset));
      x_ring[d][r] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(x_resource, offset, 0, 0));
    }
  };

#pragma unroll
  for (int d = 0; d < DEPTH; ++d) { request(d, d); }
  for (int first = 0; first < steps; first += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int step = first + d;
      // the piece that straddles the end of the range (only where the operand's K ends, and K is no multiple of 4)
      const int left = lane_length - rotated(step) * kSkinnyRowsStep;  // k of this piece inside the range
      if (__builtin_amdgcn_readfirstlane(rotated(step) == steps - 1 && (k_end - k_begin) % 4 != 0)) {
#pragma unroll
        for (int t = 1; t < 4; ++t) {
#pragma unroll
          for (int r = 0; r < RG; ++r) { x_ring[d][r][t] = (t < left) ? x_ring[d][r][t] : 0.0f; }
#pragma unroll
          for (int g = 0; g < GROUPS; ++g) { s_ring[d][g][t] = (t < left) ? s_ring[d][g][t] : 0.0f; }
        }
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int r = 0; r < RG; ++r) {
#pragma unroll
          for (int g = 0; g < GROUPS; ++g) {
            acc[r][g] = __builtin_amdgcn_mfma_f32_4x4x1f32(s_ring[d][g][t], x_ring[d][r][t], acc[r][g], 0, 0, 0);
          }
        }
      }
      // (behind the products, which have read their operands by then: the ring slot needs no second set of registers)
      request(d, step + DEPTH);
    }
  }

  // ---- the sums of the four lanes of a 16-lane row that hold the same row of X (lanes l, l + 4, l + 8, l + 12): two
  // rotations within the row leave the sum in every one of them
  auto rotate = [](const float value, auto control) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, value), decltype(control)::value, 0xf, 0xf, false));
  };
#pragma unroll
  for (int r = 0; r < RG; ++r) {
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float value = acc[r][g][i];
        value += rotate(value, std::integral_constant<int, 0x124>{});  // row_ror:4
        value += rotate(value, std::integral_constant<int, 0x128>{});  // row_ror:8
        acc[r][g][i] = value;
      }
    }
  }
  // ---- the four 16-lane rows of every wavefront hand their sums over: partial sum (wave, lane / 16) of every element
  auto element = [](const int row, const int col) { return X_IS_A ? col * ROWS + row : row * COLS + col; };
  if (lane % 16 < 4) {
    float* mine = lds + (wave * 4 + lane / 16) * ELEMENTS;
#pragma unroll
    for (int r = 0; r < RG; ++r) {
#pragma unroll
      for (int g = 0; g < GROUPS; ++g) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { mine[element(4 * r + quad_lane, 4 * g + i)] = acc[r][g][i]; }
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < PER_THREAD; ++q) {
    const int e = tid + q * THREADS;
    bool inside;
    const long long index = c_index(e, inside);
    if (inside) {
      float sum = 0.0f;
#pragma unroll
      for (int part = 0; part < 4 * WAVES; ++part) { sum += lds[part * ELEMENTS + e]; }
      p.c[index] = (p.beta != 0.0f) ? Combine(p.alpha, sum, p.beta, old_c[q]) : p.alpha * sum;
    }
  }
}

// Copies S (element (k, col) at s[k * s_ld + col]) into a k-contiguous one (at target[col * target_ld + k]) for
// GemmSkinnyRowsKernel: 32 x 32 tiles through LDS.
__global__ __launch_bounds__(256) void SkinnyTransposeKernel(const float* __restrict__ s, const long long s_ld, const int k,
                                                             const int columns, float* __restrict__ target,
                                                             const long long target_ld) {
  __shared__ float tile[32][33];
  const int k0 = blockIdx.x * 32, lane_x = threadIdx.x % 32, lane_y = threadIdx.x / 32;
  for (int kk = lane_y; kk < 32; kk += 8) {
    tile[kk][lane_x] = (k0 + kk < k && lane_x < columns) ? s[(k0 + kk) * s_ld + lane_x] : 0.0f;
  }
  __syncthreads();
  for (int col = lane_y; col < columns; col += 8) {
    if (k0 + lane_x < k) { target[col * target_ld + k0 + lane_x] = tile[lane_x][col]; }
  }
}

// Second pass of a launch whose K is split over work-groups: C = alpha * (sum of the slabs, in slab order) + beta * C.
// One thread per element of a slab (partial_ld x n, the padding rows idle), so that a C of 17 x 4099 fills its
// work-groups as well as one of 4099 x 17.
__global__ __launch_bounds__(256) void GemmSkinnyReduceKernel(const float* __restrict__ partial, const int splits,
                                                              const int partial_ld, float* __restrict__ c,
                                                              const long long c_ld, const int m, const int n,
                                                              const float alpha, const float beta) {
  const long long slab = static_cast<long long>(partial_ld) * n;
  const long long e = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= slab) { return; }
  const int i = static_cast<int>(e % partial_ld), j = static_cast<int>(e / partial_ld);
  if (i >= m) { return; }
  float sum = 0.0f;
  for (int s = 0; s < splits; ++s) { sum += partial[s * slab + e]; }
  StoreResult<float, float>(c, j * c_ld + i, sum, alpha, beta);
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_SKINNY_HPP_
