// =================================================================================================
// Batched GEMMs of matrices of a few tiles on gfx950: GemmComplexSmallKernel (complex64 / complex128, below) and
// GemmSmallTiledKernel (fp32 / fp64, at the end of the file). Both keep ONE slab of k = 16 per operand in LDS, so that
// many work-groups share a CU and hide each other's latencies, load the next slab into registers under the products of
// the current one, and use the 16 x 16 x 4 matrix instructions.
//
// Batched complex GEMM of small matrices, on interleaved (re, im) data as it lies in memory. It serves the
// shapes for which the reference launches XgemmDirectBatched / XgemmDirectStridedBatched on float2 / double2
// (src/kernels/level3/xgemm_direct_batched.opencl:24-212 with the complex MultiplyAdd of
// src/kernels/common.opencl:244-251). Such a batch is bound by HBM bandwidth, so every operand is read once and C is
// written once: a work-group owns a 64 x 64 (or 32 x 32) tile of one matrix of the batch, walks k in slabs of 16, splits
// each slab into planes of real and imaginary parts in LDS ([k][x]) and feeds the 16 x 16 x 4 matrix instruction four
// times per block and k-step:
//     Cre += Lre * Rre - Lim * Rim        Cim += Lre * Rim + Lim * Rre
// (the minus sign and the conjugations are applied to the imaginary plane when it is read or stored).
// The canonical problem is column-major: C'(rows x columns) = alpha * L(rows x k) * R(k x columns) + beta * C'.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_SMALL_TILED_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_SMALL_TILED_HPP_

#include "kernels/gemm_mfma.hpp"

namespace clbh {

constexpr int kComplexSmallSlab = 16;  // complex k per slab
constexpr int kComplexSmallThreads = 256;

// One operand or the result: matrix b of the batch starts at pointer + offset + (offsets ? offsets[b] : b * stride),
// all in complex elements.
struct ComplexSmallOperand {
  const void* pointer;
  long long offset, ld, stride;
  const long long* offsets;
  int conjugate;
};

template <typename R>
struct ComplexSmallArgs {
  int rows, columns, k, tiles_r, tiles_c;
  ComplexSmallOperand left, right, c;
  R alpha_re, alpha_im, beta_re, beta_im;
  const R* alphas;  // per matrix (re, im) pairs replacing alpha / beta, or nullptr
  const R* betas;
};

template <typename R> struct ComplexSmallTraits;
template <> struct ComplexSmallTraits<float> { using Mfma = MfmaTraitsF32Small; };
template <> struct ComplexSmallTraits<double> { using Mfma = MfmaTraits<double>; };

// A work-group of four wavefronts owns a TILE x TILE piece of C', each wavefront BLOCKS x BLOCKS blocks of 16 x 16.
template <int BLOCKS>
struct ComplexSmallTile {
  static constexpr int TILE = 32 * BLOCKS;
  static constexpr int PITCH = TILE + 4;  // plane row pitch in real numbers: k rows four banks apart
  static constexpr int PIECES = TILE * kComplexSmallSlab / kComplexSmallThreads;  // complex numbers per thread and slab
  // position (x, p) of a thread's piece q in a slab; consecutive threads run along the contiguous index
  template <bool KC> static __device__ __forceinline__ int X(const int thread, const int q) {
    return KC ? thread / kComplexSmallSlab + (kComplexSmallThreads / kComplexSmallSlab) * q : thread % TILE;
  }
  template <bool KC> static __device__ __forceinline__ int P(const int thread, const int q) {
    return KC ? thread % kComplexSmallSlab : thread / TILE + (kComplexSmallThreads / TILE) * q;
  }
};

// This thread's share of a TILE x 16 slab of an operand: element (x, p) lies at src[KC ? x * ld + p : p * ld + x].
// The loads carry no branch (a branch would make the wavefront wait for the data at once instead of after the
// products of the slab before): a piece outside the matrix reads the matrix' first element, and `valid` says which
// pieces count. Callers make sure the matrix has an element (k > 0).
template <typename R, int BLOCKS, bool KC>
struct ComplexSlabLoader {
  using Tile = ComplexSmallTile<BLOCKS>;
  typedef R Pair __attribute__((ext_vector_type(2)));
  const R* src;
  long long first;       // index of piece 0 in slab 0
  long long piece_step;  // from one piece to the next (uniform)
  long long slab_step;   // from one slab to the next (uniform)
  int x_valid;           // bit q: piece q lies in a row / column of the matrix
  int p_first, p_end;    // k index of piece 0 in slab 0; k

  __device__ __forceinline__ ComplexSlabLoader(const R* src_, const long long ld, const int x0, const int x_end,
                                               const int p_end_, const int thread)
      : src(src_), p_end(p_end_) {
    const int x = x0 + Tile::template X<KC>(thread, 0), p = Tile::template P<KC>(thread, 0);
    first = KC ? x * ld + p : p * ld + x;
    piece_step = KC ? (kComplexSmallThreads / kComplexSmallSlab) * ld : (kComplexSmallThreads / Tile::TILE) * ld;
    slab_step = KC ? kComplexSmallSlab : kComplexSmallSlab * ld;
    p_first = p;
    x_valid = 0;
#pragma unroll
    for (int q = 0; q < Tile::PIECES; ++q) {
      if (x0 + Tile::template X<KC>(thread, q) < x_end) { x_valid |= 1 << q; }
    }
  }

  __device__ __forceinline__ int Load(Pair (&values)[Tile::PIECES], const int slab) const {
    int valid = 0;
#pragma unroll
    for (int q = 0; q < Tile::PIECES; ++q) {
      const int p = slab * kComplexSmallSlab + p_first + (KC ? 0 : (kComplexSmallThreads / Tile::TILE) * q);
      const bool inside = ((x_valid >> q) & 1) != 0 && p < p_end;
      const long long index = inside ? first + q * piece_step + slab * slab_step : 0;
      values[q] = *reinterpret_cast<const Pair*>(src + 2 * index);
      valid |= inside ? 1 << q : 0;
    }
    return valid;
  }
};

template <typename R, int BLOCKS, bool KC>
__device__ __forceinline__ void StoreComplexSlab(R* __restrict__ plane_re, R* __restrict__ plane_im,
                                                 const R __attribute__((ext_vector_type(2))) (&values)[ComplexSmallTile<BLOCKS>::PIECES],
                                                 const int valid, const R sign, const int thread) {
  using Tile = ComplexSmallTile<BLOCKS>;
#pragma unroll
  for (int q = 0; q < Tile::PIECES; ++q) {
    const int at = Tile::template P<KC>(thread, q) * Tile::PITCH + Tile::template X<KC>(thread, q);
    const bool inside = ((valid >> q) & 1) != 0;
    plane_re[at] = inside ? values[q][0] : R(0);
    plane_im[at] = inside ? sign * values[q][1] : R(0);
  }
}

template <typename R, int BLOCKS, bool LEFT_KC, bool RIGHT_KC>
__global__ __launch_bounds__(kComplexSmallThreads, (sizeof(R) == 8 && BLOCKS == 2) ? 3 : 1) void GemmComplexSmallKernel(const ComplexSmallArgs<R> args) {
  using Traits = typename ComplexSmallTraits<R>::Mfma;
  using Acc = typename Traits::Acc;
  using Tile = ComplexSmallTile<BLOCKS>;
  static_assert(Traits::MF == 16 && Traits::KP == 4 && Traits::ACC == 4, "written for the 16 x 16 x 4 instructions");
  constexpr int PLANE = kComplexSmallSlab * Tile::PITCH;
  __shared__ R planes[4 * PLANE];  // left re, left im, right re, right im
  R* const left_re = planes;
  R* const left_im = planes + PLANE;
  R* const right_re = planes + 2 * PLANE;
  R* const right_im = planes + 3 * PLANE;

  const int thread = threadIdx.x, wave = thread / 64, lane = thread % 64;
  const int tiles = args.tiles_r * args.tiles_c;
  const int batch = blockIdx.x / tiles, tile = blockIdx.x % tiles;
  const int r0 = (tile % args.tiles_r) * Tile::TILE, c0 = (tile / args.tiles_r) * Tile::TILE;

  const auto start = [batch](const ComplexSmallOperand& operand) {
    return operand.offset + (operand.offsets != nullptr ? operand.offsets[batch] : batch * operand.stride);
  };
  const R* const left = static_cast<const R*>(args.left.pointer) + 2 * start(args.left);
  const R* const right = static_cast<const R*>(args.right.pointer) + 2 * start(args.right);
  R* const c = static_cast<R*>(const_cast<void*>(args.c.pointer)) + 2 * start(args.c);
  const R left_sign = args.left.conjugate ? R(-1) : R(1), right_sign = args.right.conjugate ? R(-1) : R(1);

  // wavefront w owns the rows from 16 * BLOCKS * (w % 2) and the columns from 16 * BLOCKS * (w / 2) of the tile
  const int wave_r = 16 * BLOCKS * (wave % 2), wave_c = 16 * BLOCKS * (wave / 2);
  const int in_block = lane % 16, k_group = lane / 16;
  Acc acc_re[BLOCKS][BLOCKS], acc_im[BLOCKS][BLOCKS];
#pragma unroll
  for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
    for (int j = 0; j < BLOCKS; ++j) {
      acc_re[i][j] = Traits::Zero();
      acc_im[i][j] = Traits::Zero();
    }
  }

  typedef R Pair __attribute__((ext_vector_type(2)));
  const ComplexSlabLoader<R, BLOCKS, LEFT_KC> left_loader(left, args.left.ld, r0, args.rows, args.k, thread);
  const ComplexSlabLoader<R, BLOCKS, RIGHT_KC> right_loader(right, args.right.ld, c0, args.columns, args.k, thread);
  Pair left_values[Tile::PIECES], right_values[Tile::PIECES];
  int left_valid = 0, right_valid = 0;
  const int slabs = (args.k + kComplexSmallSlab - 1) / kComplexSmallSlab;
  if (slabs > 0) {
    left_valid = left_loader.Load(left_values, 0);
    right_valid = right_loader.Load(right_values, 0);
  }
  for (int slab = 0; slab < slabs; ++slab) {
    __syncthreads();  // the previous slab has been consumed
    StoreComplexSlab<R, BLOCKS, LEFT_KC>(left_re, left_im, left_values, left_valid, left_sign, thread);
    StoreComplexSlab<R, BLOCKS, RIGHT_KC>(right_re, right_im, right_values, right_valid, right_sign, thread);
    __syncthreads();
    if (slab + 1 < slabs) {  // the next slab travels while this one is multiplied
      left_valid = left_loader.Load(left_values, slab + 1);
      right_valid = right_loader.Load(right_values, slab + 1);
    }
#pragma unroll
    for (int step = 0; step < kComplexSmallSlab / 4; ++step) {
      const int line = (4 * step + k_group) * Tile::PITCH + in_block;
      R a_re[BLOCKS], a_im[BLOCKS], a_minus[BLOCKS], b_re[BLOCKS], b_im[BLOCKS];
#pragma unroll
      for (int i = 0; i < BLOCKS; ++i) {
        a_re[i] = left_re[line + wave_r + 16 * i];
        a_im[i] = left_im[line + wave_r + 16 * i];
        a_minus[i] = -a_im[i];
        b_re[i] = right_re[line + wave_c + 16 * i];
        b_im[i] = right_im[line + wave_c + 16 * i];
      }
      // The right operand goes first: a lane then holds one row of C' in four columns, and the lanes of a result
      // register run along the rows, the contiguous index of C'. One product after the other over all blocks, so that
      // no instruction waits for the accumulator of the one before it.
#pragma unroll
      for (int product = 0; product < 4; ++product) {
#pragma unroll
        for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
          for (int j = 0; j < BLOCKS; ++j) {
            if (product == 0) { acc_re[i][j] = Traits::Mfma(b_re[j], a_re[i], acc_re[i][j]); }
            if (product == 1) { acc_im[i][j] = Traits::Mfma(b_im[j], a_re[i], acc_im[i][j]); }
            if (product == 2) { acc_re[i][j] = Traits::Mfma(b_im[j], a_minus[i], acc_re[i][j]); }
            if (product == 3) { acc_im[i][j] = Traits::Mfma(b_re[j], a_im[i], acc_im[i][j]); }
          }
        }
      }
    }
  }

  // C' = alpha * product + beta * C'; C' is read only when beta is not zero
  R alpha_re = args.alpha_re, alpha_im = args.alpha_im, beta_re = args.beta_re, beta_im = args.beta_im;
  if (args.alphas != nullptr) {
    alpha_re = args.alphas[2 * batch];
    alpha_im = args.alphas[2 * batch + 1];
  }
  if (args.betas != nullptr) {
    beta_re = args.betas[2 * batch];
    beta_im = args.betas[2 * batch + 1];
  }
  const bool with_c = (beta_re != R(0)) || (beta_im != R(0));
#pragma unroll
  for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
    for (int j = 0; j < BLOCKS; ++j) {
      const int row = r0 + wave_r + 16 * i + in_block;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int column = c0 + wave_c + 16 * j + Traits::Row(r, k_group);
        if (row < args.rows && column < args.columns) {
          Pair* const target = reinterpret_cast<Pair*>(c + 2 * (column * args.c.ld + row));
          const R re = acc_re[i][j][r], im = acc_im[i][j][r];
          Pair result = {alpha_re * re - alpha_im * im, alpha_re * im + alpha_im * re};
          if (with_c) {
            const Pair old = *target;
            result[0] += beta_re * old[0] - beta_im * old[1];
            result[1] += beta_re * old[1] + beta_im * old[0];
          }
          *target = result;
        }
      }
    }
  }
}

// ---- the same scheme for batches of small REAL matrices (fp32, fp64) -------------------------------------------
// Batches of matrices of a few tiles with a short k are bound by HBM and by latency: the ring of three slabs of the
// large-tile kernel costs LDS (three work-groups per CU) and a long prologue. Here a work-group keeps one slab per
// operand in LDS (two planes of 16 x (TILE + 4)), loads the next one into registers while it multiplies, and eight
// or more work-groups share a CU. Arguments as for the other GEMM kernels (column-major canonical problem).
template <typename T, int BLOCKS, bool KC>
struct RealSlabLoader {
  using Tile = ComplexSmallTile<BLOCKS>;
  const T* src;
  long long first, piece_step, slab_step;
  int x_valid, p_first, p_end;

  __device__ __forceinline__ RealSlabLoader(const T* src_, const long long ld, const int x0, const int x_end,
                                            const int p_end_, const int thread)
      : src(src_), p_end(p_end_) {
    const int x = x0 + Tile::template X<KC>(thread, 0), p = Tile::template P<KC>(thread, 0);
    first = KC ? x * ld + p : p * ld + x;
    piece_step = KC ? (kComplexSmallThreads / kComplexSmallSlab) * ld : (kComplexSmallThreads / Tile::TILE) * ld;
    slab_step = KC ? kComplexSmallSlab : kComplexSmallSlab * ld;
    p_first = p;
    x_valid = 0;
#pragma unroll
    for (int q = 0; q < Tile::PIECES; ++q) {
      if (x0 + Tile::template X<KC>(thread, q) < x_end) { x_valid |= 1 << q; }
    }
  }

  // branch-free like ComplexSlabLoader::Load: a piece outside the matrix reads its first element
  __device__ __forceinline__ int Load(T (&values)[Tile::PIECES], const int slab) const {
    int valid = 0;
#pragma unroll
    for (int q = 0; q < Tile::PIECES; ++q) {
      const int p = slab * kComplexSmallSlab + p_first + (KC ? 0 : (kComplexSmallThreads / Tile::TILE) * q);
      const bool inside = ((x_valid >> q) & 1) != 0 && p < p_end;
      const long long index = inside ? first + q * piece_step + slab * slab_step : 0;
      values[q] = src[index];
      valid |= inside ? 1 << q : 0;
    }
    return valid;
  }
};

// (the register budget is set for many wavefronts per SIMD: what hides the latencies here is other work-groups)
template <typename T, int BLOCKS, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kComplexSmallThreads, sizeof(T) == 8 ? (BLOCKS == 2 ? 3 : 6) : (BLOCKS == 2 ? 4 : 8))
void GemmSmallTiledKernel(const GemmArgs<T> p, const int tiles_m,
                                                                             const int tiles_n) {
  using Traits = typename ComplexSmallTraits<T>::Mfma;
  using Acc = typename Traits::Acc;
  using Tile = ComplexSmallTile<BLOCKS>;
  constexpr int PLANE = kComplexSmallSlab * Tile::PITCH;
  __shared__ T planes[2 * PLANE];
  T* const a_plane = planes;
  T* const b_plane = planes + PLANE;

  const int thread = threadIdx.x, wave = thread / 64, lane = thread % 64;
  const int m0 = (blockIdx.x % tiles_m) * Tile::TILE, n0 = (blockIdx.x / tiles_m) * Tile::TILE;
  const int wave_m = 16 * BLOCKS * (wave % 2), wave_n = 16 * BLOCKS * (wave / 2);
  const int in_block = lane % 16, k_group = lane / 16;
  const int slabs = (p.k + kComplexSmallSlab - 1) / kComplexSmallSlab;

  for (int batch = blockIdx.y; batch < p.batch_count; batch += gridDim.y) {
    const T* a;
    const T* b;
    T* c;
    T alpha, beta;
    ResolveBatch<T, T>(p, batch, a, b, c, alpha, beta);
    Acc acc[BLOCKS][BLOCKS];
#pragma unroll
    for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
      for (int j = 0; j < BLOCKS; ++j) { acc[i][j] = Traits::Zero(); }
    }
    const RealSlabLoader<T, BLOCKS, A_KC> a_loader(a, p.a_ld, m0, p.m, p.k, thread);
    const RealSlabLoader<T, BLOCKS, B_KC> b_loader(b, p.b_ld, n0, p.n, p.k, thread);
    T a_values[Tile::PIECES], b_values[Tile::PIECES];
    int a_valid = a_loader.Load(a_values, 0), b_valid = b_loader.Load(b_values, 0);  // the host guarantees k > 0
    for (int slab = 0; slab < slabs; ++slab) {
      __syncthreads();  // the previous slab (or matrix) has been consumed
#pragma unroll
      for (int q = 0; q < Tile::PIECES; ++q) {
        a_plane[Tile::template P<A_KC>(thread, q) * Tile::PITCH + Tile::template X<A_KC>(thread, q)] =
            ((a_valid >> q) & 1) != 0 ? a_values[q] : T(0);
        b_plane[Tile::template P<B_KC>(thread, q) * Tile::PITCH + Tile::template X<B_KC>(thread, q)] =
            ((b_valid >> q) & 1) != 0 ? b_values[q] : T(0);
      }
      __syncthreads();
      if (slab + 1 < slabs) {
        a_valid = a_loader.Load(a_values, slab + 1);
        b_valid = b_loader.Load(b_values, slab + 1);
      }
#pragma unroll
      for (int step = 0; step < kComplexSmallSlab / 4; ++step) {
        const int line = (4 * step + k_group) * Tile::PITCH + in_block;
        T a_fragment[BLOCKS], b_fragment[BLOCKS];
#pragma unroll
        for (int i = 0; i < BLOCKS; ++i) {
          a_fragment[i] = a_plane[line + wave_m + 16 * i];
          b_fragment[i] = b_plane[line + wave_n + 16 * i];
        }
        // B's fragment goes first: the lanes of a result register then run along m, the contiguous index of C
#pragma unroll
        for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
          for (int j = 0; j < BLOCKS; ++j) { acc[i][j] = Traits::Mfma(b_fragment[j], a_fragment[i], acc[i][j]); }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < BLOCKS; ++i) {
#pragma unroll
      for (int j = 0; j < BLOCKS; ++j) {
        const int row = m0 + wave_m + 16 * i + in_block;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int column = n0 + wave_n + 16 * j + Traits::Row(r, k_group);
          if (row < p.m && column < p.n) { StoreResult<T, T>(c, column * p.c_ld + row, acc[i][j][r], alpha, beta); }
        }
      }
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_SMALL_TILED_HPP_
