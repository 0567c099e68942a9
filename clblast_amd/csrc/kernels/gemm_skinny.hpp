// =================================================================================================
// fp32 GEMM kernel for skinny problems on gfx950 whose large operand is k-contiguous: one extent of C is at most 32
// (n <= 32 with a long m and a transposed A, or m <= 32 with a long n and a plain B) and k is long, e.g.
// 4099 x 17 x 4096. Such a product is one pass over the large operand X (8.4 flop per byte: HBM-bound). The tiled kernel
// of gemm_mfma.hpp does not keep up with it: its tiles pad the short extent to 32 (fp32 matrix cores deliver
// 157 TFLOP/s: at 32 columns the products take as long as the stream), and the few tiles of such a problem make it split
// K over work-groups, with a second launch that adds the partial sums. (The reference sends these shapes to its direct
// kernel with 16 x 16 tiles, src/routines/level3/xgemm.cpp:228-268, xgemm_direct_part3.opencl.)
//
// Matrix instruction v_mfma_f32_4x4x1_16b_f32: sixteen independent 4 x 4 outer products, so the short extent is padded
// to a multiple of 4 only. Block b = lane / 4 multiplies four values of S (A operand, one per lane % 4: columns
// 4g .. 4g + 3 at one k) with four values of X (B operand, one per lane % 4: four rows of X at the same k); a lane's
// four result registers are the four columns of ITS row of X.
//
// Measured on the MI355X, 4099 x 17 x 4096 with a transposed A: 16.4 us against 27.5 us of the tiled kernel with K split
// (a plain read of the operand with the same access pattern takes 10.5 us). Parts, from switching them off: launch and
// drain 3 us, the stream of X 10.5 us, the re-read of S by every work-group 2 us, the products 7.5 us (overlapped but
// for about 1 us), the epilogue 2.6 us. An x-contiguous X (a plain A) stays with the tiled kernel: there the lanes must
// run along the rows of X, K has to be split over work-groups again, and the variant of this kernel built that way
// (register streaming, wavefront-private LDS tiles of S, tree of partial sums) was no faster than the tiled one (25.9
// against 25.6 us; its epilogue and the reduction launch took 10 us of that). Nor does it help to give a work-group
// a few such rows and all of K, which needs no second launch: with sixteen rows per work-group (runs of 64 bytes, half
// a cache line) X streams at 3 TB/s (4099 x 17 x 4096: 46 us, 16384 x 4 x 16384: 345 against 176 us), with 32 rows
// per work-group, the two halves of the lines fetched by two wavefronts side by side, at 3.5 TB/s (34 and 307 us) -
// every load of a wavefront touches sixteen lines, one per k. Only below about 8 MB of X is that ahead (4099 x 17 x 512:
// 9.8 against 11.0 us).
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_SKINNY_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_SKINNY_HPP_

#include <type_traits>

#include "kernels/gemm_mfma.hpp"

namespace clbh {

struct SkinnyArgs {
  const float* x;        // the large operand: element (row, k) at x[row * x_ld + k]
  const float* s;        // the small operand: element (k, col) at s[col * s_ld + k]
  float* c;              // result: element (row, col) at c[X_IS_A ? col * c_ld + row : row * c_ld + col]
  long long x_ld, s_ld, c_ld;
  int extent;            // rows of X
  int small;             // columns of S (<= 4 * GROUPS)
  int k;
  int k_per_wave;        // K range of a wavefront: a multiple of kSkinnyRowsStep
  float alpha, beta;
};

// =================================================================================================
// Rows of X are long contiguous runs, and a wavefront that put its lanes along the rows of X would touch 64 rows with
// every load (measured: twice the time of the tiled kernel). Here the lanes of a wavefront run along k: block b = lane / 4 of the matrix
// instruction takes the four k from 4b on of every 64 (a 16-byte load per lane, 256 contiguous bytes per row and load),
// the four lanes of a block take four rows of X. A work-group owns 4 * RG rows of X and ALL of K, split over its
// wavefronts: no second pass, no workspace. A lane's sums cover its share of k only; they meet at the end - first the
// four lanes of a 16-lane row that hold the same row of X (two rotations), then rows and wavefronts through LDS, added
// in a fixed order.
// S comes straight from memory (L2 holds all of it) in the layout of the A operand. S_KC, element (k, col) at
// s[col * s_ld + k]: a lane loads the four k of its block for column 4g + lane % 4 in one piece. Otherwise, element at
// s[k * s_ld + col]: lane % 4 = i takes the GROUPS consecutive columns from i * GROUPS on, one piece per k (which
// column a result register stands for is a matter of the epilogue only). Both operands are requested DEPTH steps (of
// 64 k) ahead: the counter of outstanding loads completes in order, a wait for a late request of S would wait for every
// earlier request of X too.
// =================================================================================================
constexpr int kSkinnyRowsStep = 64;  // k per step and wavefront

constexpr int SkinnyRowsLdsFloats(const int waves, const int groups, const int rg) { return waves * 4 * (4 * rg) * (4 * groups); }

template <int WAVES, int GROUPS, int RG, int DEPTH, bool X_IS_A, bool S_KC, int WAVES_PER_SIMD = 2>
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
  // this wavefront's K range and, per lane, the
  // number of k from the lane's first one to the end of the range
  const int k_begin = wave * p.k_per_wave;
  const int k_end = min(k_begin + p.k_per_wave, p.k);
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
  const float* s_base = p.s + (S_KC ? k_begin : k_begin * p.s_ld);
  const long long x_valid = static_cast<long long>(rows - 1) * p.x_ld + p.k - k_begin;
  const long long s_valid = S_KC ? static_cast<long long>(p.small - 1) * p.s_ld + p.k - k_begin
                                 : static_cast<long long>(p.k - k_begin - 1) * p.s_ld + p.small;
  constexpr int kOutside = 0x7fffff00;  // (an offset no resource reaches)
  const int x_records = static_cast<int>(min(max(x_valid, 0ll) * 4, static_cast<long long>(kOutside)));
  const int s_records = static_cast<int>(min(max(s_valid, 0ll) * 4, static_cast<long long>(kOutside)));
  int x_offset[RG], s_offset[GROUPS];
#pragma unroll
  for (int r = 0; r < RG; ++r) { x_offset[r] = static_cast<int>((min(4 * r + quad_lane, rows - 1) * p.x_ld + 4 * slot) * 4); }
#pragma unroll
  for (int g = 0; g < GROUPS; ++g) { s_offset[g] = static_cast<int>((min(4 * g + quad_lane, p.small - 1) * p.s_ld + 4 * slot) * 4); }
  const int s_row_bytes = static_cast<int>(p.s_ld * 4);                                     // (column-contiguous S)
  const int s_lane_bytes = static_cast<int>((4 * slot * p.s_ld + quad_lane * GROUPS) * 4);  // (k = 4 * slot, column i * GROUPS)

  float4_t x_ring[DEPTH][RG], s_ring[DEPTH][S_KC ? GROUPS : 1];
  float s_pieces[DEPTH][4][S_KC ? 1 : GROUPS];  // (column-contiguous S: [t][g])
  auto request = [&](const int d, const int position) {
    const int step = rotated(position);
    // (the offsets go through an empty asm statement: the compiler would otherwise turn each select into a branch
    // around two loads, and could no longer count the loads in flight)
    const int step_bytes = (step * kSkinnyRowsStep < lane_length) ? step * kSkinnyRowsStep * 4 : kOutside;
    const auto x_resource = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x_base), 0, x_records, kRawBufferFlags);
    // (a column-contiguous S advances by whole rows of it per step: the resource moves along, the lane's offset stays small)
    const long long s_step = S_KC ? 0 : static_cast<long long>(step) * kSkinnyRowsStep * p.s_ld;
    const int s_step_records = static_cast<int>(min(max(s_valid - s_step, 0ll) * 4, static_cast<long long>(kOutside)));
    const auto s_resource = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(s_base + s_step), 0,
                                                              S_KC ? s_records : s_step_records, kRawBufferFlags);
    if constexpr (S_KC) {
#pragma unroll
      for (int g = 0; g < GROUPS; ++g) {
        int offset = s_offset[g] + step_bytes;
        asm volatile("" : "+v"(offset));
        s_ring[d][g] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(s_resource, offset, 0, 0));
      }
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t) {  // k = 64 * step + 4 * slot + t: valid while inside the lane's range. (The column
        // offsets of the pieces are part of the lane's offset, which is what the resource's range is checked against.)
        int offset = (step * kSkinnyRowsStep + t < lane_length) ? s_lane_bytes + t * s_row_bytes : kOutside;
        asm volatile("" : "+v"(offset));
        int g = 0;
#pragma unroll
        for (; g + 4 <= GROUPS; g += 4) {
          const float4_t piece = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(s_resource, offset + 4 * g, 0, 0));
          s_pieces[d][t][g] = piece[0]; s_pieces[d][t][g + 1] = piece[1]; s_pieces[d][t][g + 2] = piece[2]; s_pieces[d][t][g + 3] = piece[3];
        }
        if (g + 2 <= GROUPS) {
          typedef float float2_t __attribute__((ext_vector_type(2)));
          const float2_t piece = __builtin_bit_cast(float2_t, __builtin_amdgcn_raw_buffer_load_b64(s_resource, offset + 4 * g, 0, 0));
          s_pieces[d][t][g] = piece[0]; s_pieces[d][t][g + 1] = piece[1];
          g += 2;
        }
        if (g < GROUPS) { s_pieces[d][t][g] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(s_resource, offset + 4 * g, 0, 0)); }
      }
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
          if constexpr (S_KC) {
#pragma unroll
            for (int g = 0; g < GROUPS; ++g) { s_ring[d][g][t] = (t < left) ? s_ring[d][g][t] : 0.0f; }
          }
        }
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int r = 0; r < RG; ++r) {
#pragma unroll
          for (int g = 0; g < GROUPS; ++g) {
            const float s_value = S_KC ? s_ring[d][g][t] : s_pieces[d][t][g];
            acc[r][g] = __builtin_amdgcn_mfma_f32_4x4x1f32(s_value, x_ring[d][r][t], acc[r][g], 0, 0, 0);
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
        for (int i = 0; i < 4; ++i) { mine[element(4 * r + quad_lane, S_KC ? 4 * g + i : i * GROUPS + g)] = acc[r][g][i]; }
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

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_SKINNY_HPP_
