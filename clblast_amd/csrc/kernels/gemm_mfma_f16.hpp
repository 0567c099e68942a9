// =================================================================================================
// Register-staged MFMA GEMM kernel for gfx950, fp16 storage with fp32 accumulation: the fallback of the
// direct-load kernel (gemm_direct_f16.hpp) for operands that are not dword aligned (odd element offsets
// or odd leading dimensions), which it reads element by element. Same arithmetic: products are
// accumulated in fp32 by v_mfma_f32_32x32x16_f16 and rounded to fp16 once, in the epilogue (the reference
// accumulates in fp16, src/kernels/common.opencl:44-45).
//
// Structure (one work-group = 256 threads = 4 wavefronts in a 2 x 2 arrangement):
//   * work-group tile (64*FM) x (64*FN), K walked in slabs of TILE_K, two LDS buffers, global loads
//     of slab t+1 in flight while slab t is multiplied, one barrier per slab; edge tiles and the K tail
//     are filled element-wise with bounds checks;
//   * the MFMA wants 8 consecutive k per lane. A k-contiguous operand is kept in LDS as [x][k]
//     (pitch TILE_K + 8 halfs: conflict-free 16-byte reads) and read with one ds_read_b128 per
//     operand block. An x-contiguous operand (x = m for A, n for B) is kept as [k][x] (pitch
//     tile + 32 halfs) and read with the CDNA4 transposing LDS read ds_read_b64_tr_b16, which hands
//     each lane four consecutive k of its own x: the transpose costs no VALU work and no extra pass;
//   * the m-indexed fragment is the MFMA's A operand, so a lane holds runs of four consecutive m; the
//     epilogue stages each block column through LDS and moves C in whole 16-byte pieces along m.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_MFMA_F16_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_MFMA_F16_HPP_

#include <type_traits>

#include "kernels/gemm_args.hpp"
#include "kernels/gemm_mfma.hpp"

namespace clbh {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));

// WM x WN wavefronts per work-group, each owning FM x FN MFMA blocks of 32 x 32. MIN_WAVES is the number
// of wavefronts per SIMD the register budget must allow.
template <int WM_, int WN_, int FM_, int FN_, int TILE_K_, int MIN_WAVES_>
struct HgemmConfig {
  static constexpr int WM = WM_, WN = WN_, FM = FM_, FN = FN_, MIN_WAVES = MIN_WAVES_;
  static constexpr int THREADS = 64 * WM * WN;
  static constexpr int TILE_M = WM * FM * 32;
  static constexpr int TILE_N = WN * FN * 32;
  static constexpr int TILE_K = TILE_K_;
  static constexpr int PITCH_KC = TILE_K + 8;    // halfs per x row of a [x][k] tile
  static constexpr int PITCH_XM = TILE_M + 32;   // halfs per k row of a [k][m] tile
  static constexpr int PITCH_XN = TILE_N + 32;
  static constexpr int A_ELEMS_KC = TILE_M * PITCH_KC, A_ELEMS_XC = TILE_K * PITCH_XM;
  static constexpr int B_ELEMS_KC = TILE_N * PITCH_KC, B_ELEMS_XC = TILE_K * PITCH_XN;
  static constexpr int A_ELEMS = A_ELEMS_KC > A_ELEMS_XC ? A_ELEMS_KC : A_ELEMS_XC;
  static constexpr int B_ELEMS = B_ELEMS_KC > B_ELEMS_XC ? B_ELEMS_KC : B_ELEMS_XC;
  static constexpr int LDS_BYTES = 2 * (A_ELEMS + B_ELEMS) * 2;
  static_assert(TILE_K % 16 == 0, "slab depth is a multiple of the MFMA k extent");
  static_assert((TILE_M * TILE_K) % (8 * THREADS) == 0 && (TILE_N * TILE_K) % (8 * THREADS) == 0, "slab split");
};

// ---- slab movement ---------------------------------------------------------------------------------
// piece -> (x, k) of a slab moved in pieces of VL elements: consecutive threads run along the contiguous
// index of the operand in memory, so a wavefront's accesses coalesce for either orientation.
template <int TILE_X, int TILE_K, int VL, bool KC>
struct PieceMap {
  static constexpr int ALONG = (KC ? TILE_K : TILE_X) / VL;  // pieces per contiguous line of the slab
  static __device__ __forceinline__ void Get(const int piece, int& x, int& k) {
    const int line = piece / ALONG, pos = (piece % ALONG) * VL;
    x = KC ? line : pos;
    k = KC ? pos : line;
  }
};

// Slab of TILE_X x TILE_K halfs; element (x, k) at base[KC ? x*ld + k : k*ld + x]. Threads move pieces
// of VL halfs (8 when every address is 16-byte aligned, else 1), consecutive threads along the
// contiguous index.
template <int THREADS, int TILE_X, int TILE_K, int PIECES, int VL, bool KC>
__device__ __forceinline__ void HLoadSlab(const _Float16* __restrict__ base, const long long ld, const int x0,
                                          const int k0, const int tid,
                                          typename VecType<_Float16, VL>::type (&regs)[PIECES]) {
  using Map = PieceMap<TILE_X, TILE_K, VL, KC>;
  using V = typename VecType<_Float16, VL>::type;
#pragma unroll
  for (int c = 0; c < PIECES; ++c) {
    int x, k;
    Map::Get(tid + c * THREADS, x, k);
    const _Float16* src = KC ? base + (x0 + x) * ld + (k0 + k) : base + (k0 + k) * ld + (x0 + x);
    regs[c] = *reinterpret_cast<const V*>(src);
  }
}

// Edge tiles and the K tail: element-wise, bounds-checked copy straight into LDS (no register staging, no
// overlap with the multiplication). Elements outside the matrix become zero.
template <int THREADS, int TILE_X, int TILE_K, int PITCH, bool KC>
__device__ __forceinline__ void HFillSlabChecked(_Float16* __restrict__ tile, const _Float16* __restrict__ base,
                                                 const long long ld, const int x0, const int k0, const int x_end,
                                                 const int k_end, const int tid) {
  using Map = PieceMap<TILE_X, TILE_K, 1, KC>;
#pragma unroll 4
  for (int piece = tid; piece < TILE_X * TILE_K; piece += THREADS) {
    int x, k;
    Map::Get(piece, x, k);
    const int gx = x0 + x, gk = k0 + k;
    _Float16 value = _Float16(0);
    if (gx < x_end && gk < k_end) { value = KC ? base[gx * ld + gk] : base[gk * ld + gx]; }
    tile[KC ? x * PITCH + k : k * PITCH + x] = value;
  }
}

// Registers -> LDS in the same orientation as memory: [x][k] for KC, [k][x] otherwise.
template <int THREADS, int TILE_X, int TILE_K, int PITCH, int PIECES, int VL, bool KC>
__device__ __forceinline__ void HStoreSlab(_Float16* __restrict__ tile, const int tid,
                                           const typename VecType<_Float16, VL>::type (&regs)[PIECES]) {
  using Map = PieceMap<TILE_X, TILE_K, VL, KC>;
  using V = typename VecType<_Float16, VL>::type;
#pragma unroll
  for (int c = 0; c < PIECES; ++c) {
    int x, k;
    Map::Get(tid + c * THREADS, x, k);
    _Float16* dst = KC ? &tile[x * PITCH + k] : &tile[k * PITCH + x];
    *reinterpret_cast<V*>(dst) = regs[c];
  }
}

// One MFMA operand fragment: the 8 halfs of k = k16 + 8*(lane/32) .. +8 for x = x32 + lane%32.
template <int PITCH, bool KC>
__device__ __forceinline__ half8_t HReadFragment(const _Float16* __restrict__ tile, const int x32, const int k16,
                                                 const int lane) {
  if (KC) {
    return *reinterpret_cast<const half8_t*>(&tile[(x32 + lane % 32) * PITCH + k16 + 8 * (lane / 32)]);
  } else {
    // Transposing read: within each group of 16 lanes, lane q addresses 4 halfs at row k + q/4, columns
    // 4*(q%4)..+3, and receives the 4 halfs of rows k..k+3 at column q. Groups 0/1 take x 0-15/16-31
    // of k 0-7, groups 2/3 the same x of k 8-15; two reads give the 8 consecutive k of a lane.
    const int group = lane / 16, q = lane % 16;
    const int x = x32 + 16 * (group % 2) + 4 * (q % 4);
    const int k = k16 + 8 * (group / 2) + q / 4;
    typedef __attribute__((address_space(3))) short4_t* LdsPtr;
    const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(&tile[k * PITCH + x]));
    const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(&tile[(k + 4) * PITCH + x]));
    half8_t out;
    const half4_t lo_h = __builtin_bit_cast(half4_t, lo), hi_h = __builtin_bit_cast(half4_t, hi);
#pragma unroll
    for (int e = 0; e < 4; ++e) { out[e] = lo_h[e]; out[4 + e] = hi_h[e]; }
    return out;
  }
}

// ---- the kernel ------------------------------------------------------------------------------------
template <typename Config, bool A_KC, bool B_KC, bool ALIGNED>
__global__ __launch_bounds__(Config::THREADS, Config::MIN_WAVES) void HgemmMfmaKernel(const GemmArgs<float> p, const int tiles_m,
                                                                const int tiles_n) {
  using T = _Float16;
  constexpr int TILE_M = Config::TILE_M, TILE_N = Config::TILE_N, TILE_K = Config::TILE_K;
  constexpr int FM = Config::FM, FN = Config::FN;
  constexpr int PITCH_A = A_KC ? Config::PITCH_KC : Config::PITCH_XM;
  constexpr int PITCH_B = B_KC ? Config::PITCH_KC : Config::PITCH_XN;
  constexpr int VL = ALIGNED ? 8 : 1;
  constexpr int THREADS = Config::THREADS;
  constexpr int PIECES_A = TILE_M * TILE_K / VL / THREADS, PIECES_B = TILE_N * TILE_K / VL / THREADS;

  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  T* a_tiles = lds;                          // two buffers of A_ELEMS
  T* b_tiles = lds + 2 * Config::A_ELEMS;    // two buffers of B_ELEMS

  const int tid = threadIdx.x;
  const int lane = tid % 64, wave = tid / 64;
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
  const bool interior = (m0 + TILE_M <= p.m) && (n0 + TILE_N <= p.n);
  const int full_slabs = p.k / TILE_K;
  const int slabs = (p.k + TILE_K - 1) / TILE_K;

  for (int batch = blockIdx.y; batch < p.batch_count; batch += gridDim.y) {
    const T* a;
    const T* b;
    T* c;
    float alpha, beta;
    ResolveBatch<T, float>(p, batch, a, b, c, alpha, beta);

    float16_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
      for (int j = 0; j < FN; ++j) { acc[i][j] = float16_t(0.0f); }
    }

    typename VecType<T, VL>::type a_regs[PIECES_A];
    typename VecType<T, VL>::type b_regs[PIECES_B];

    auto load = [&](const int slab) {
      HLoadSlab<THREADS, TILE_M, TILE_K, PIECES_A, VL, A_KC>(a, p.a_ld, m0, slab * TILE_K, tid, a_regs);
      HLoadSlab<THREADS, TILE_N, TILE_K, PIECES_B, VL, B_KC>(b, p.b_ld, n0, slab * TILE_K, tid, b_regs);
    };
    auto store = [&](const int buffer) {
      HStoreSlab<THREADS, TILE_M, TILE_K, PITCH_A, PIECES_A, VL, A_KC>(a_tiles + buffer * Config::A_ELEMS, tid, a_regs);
      HStoreSlab<THREADS, TILE_N, TILE_K, PITCH_B, PIECES_B, VL, B_KC>(b_tiles + buffer * Config::B_ELEMS, tid, b_regs);
    };
    auto read_fragments = [&](const T* a_tile, const T* b_tile, const int ks, half8_t (&a_frag)[FM],
                              half8_t (&b_frag)[FN]) {
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        a_frag[i] = HReadFragment<PITCH_A, A_KC>(a_tile, (wave_m * FM + i) * 32, ks * 16, lane);
      }
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        b_frag[j] = HReadFragment<PITCH_B, B_KC>(b_tile, (wave_n * FN + j) * 32, ks * 16, lane);
      }
    };
    auto multiply_fragments = [&](const half8_t (&a_frag)[FM], const half8_t (&b_frag)[FN]) {
#pragma unroll
      for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_frag[i], b_frag[j], acc[i][j], 0, 0, 0);
        }
      }
    };
    auto multiply = [&](const int buffer) {
      const T* a_tile = a_tiles + buffer * Config::A_ELEMS;
      const T* b_tile = b_tiles + buffer * Config::B_ELEMS;
#pragma unroll
      for (int ks = 0; ks < TILE_K / 16; ++ks) {
        half8_t a_frag[FM], b_frag[FN];
        read_fragments(a_tile, b_tile, ks, a_frag, b_frag);
        multiply_fragments(a_frag, b_frag);
      }
    };

    // Interior tiles: software-pipelined walk over the full slabs.
    const int fast_slabs = interior ? full_slabs : 0;
    if (fast_slabs > 0) {
      load(0);
      store(0);
      __syncthreads();
      for (int slab = 0; slab < fast_slabs; ++slab) {
        const int buffer = slab & 1;
        if (slab + 1 < fast_slabs) { load(slab + 1); }
        multiply(buffer);
        if (slab + 1 < fast_slabs) { store(buffer ^ 1); }
        __syncthreads();
      }
    }
    // Edge tiles (all slabs) and the K tail of interior tiles: checked, unpipelined.
    for (int slab = fast_slabs; slab < slabs; ++slab) {
      HFillSlabChecked<THREADS, TILE_M, TILE_K, PITCH_A, A_KC>(a_tiles, a, p.a_ld, m0, slab * TILE_K, p.m, p.k, tid);
      HFillSlabChecked<THREADS, TILE_N, TILE_K, PITCH_B, B_KC>(b_tiles, b, p.b_ld, n0, slab * TILE_K, p.n, p.k, tid);
      __syncthreads();
      multiply(0);
      __syncthreads();
    }

    // Epilogue, staged through LDS so that global memory sees whole lines. The m-indexed fragment is the
    // MFMA's A operand: accumulator elements 4g..4g+3 of a lane are the rows m = 8g + 4*(lane/32) + 0..3 of
    // column n = lane%32 of the 32 x 32 block. Per block column j a wavefront owns a [32 n][WAVE_M m] fp16
    // staging tile of its own: C (when beta != 0) comes in with 16-byte accesses along m, every lane
    // combines its four consecutive m in fp32 and rounds once, and the finished rows leave with 16-byte
    // stores. Only wavefront-local ordering is needed (LDS operations of a wavefront complete in order).
    {
      constexpr int WAVE_M = FM * 32, STAGE_PITCH = WAVE_M + 8;
      constexpr int LANES_PER_ROW = WAVE_M / 8, ROWS_PER_PASS = 64 / LANES_PER_ROW, PASSES = 32 / ROWS_PER_PASS;
      static_assert((THREADS / 64) * 32 * STAGE_PITCH * 2 <= Config::LDS_BYTES, "staging tiles fit the slab buffers");
      T* stage = lds + wave * (32 * STAGE_PITCH);
      const int wave_m0 = m0 + wave_m * WAVE_M;
      const bool vector_rows = ALIGNED && (wave_m0 + WAVE_M <= p.m) && (p.c_ld % 8 == 0) &&
                               ((reinterpret_cast<unsigned long long>(c) & 15) == 0) && !masked;
      auto wave_fence = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      };
      // moves the staging tile's rows from (LOAD) or to (!LOAD) the block column starting at n_blk
      auto rows = [&](const int n_blk, auto load_tag) {
        constexpr bool LOAD = decltype(load_tag)::value;
        if (vector_rows) {
#pragma unroll
          for (int pass = 0; pass < PASSES; ++pass) {
            const int row = pass * ROWS_PER_PASS + lane / LANES_PER_ROW, col = 8 * (lane % LANES_PER_ROW);
            if (n_blk + row < p.n) {
              T* global = c + (n_blk + row) * p.c_ld + wave_m0 + col;
              half8_t* local = reinterpret_cast<half8_t*>(&stage[row * STAGE_PITCH + col]);
              if (LOAD) { *local = *reinterpret_cast<const half8_t*>(global); }
              else { *reinterpret_cast<half8_t*>(global) = *local; }
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
          for (int i = 0; i < FM; ++i) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              half4_t* cell = reinterpret_cast<half4_t*>(&stage[(lane % 32) * STAGE_PITCH + 32 * i + 8 * g + 4 * (lane / 32)]);
              half4_t out;
              if (beta != 0.0f) {
                const half4_t old = *cell;
#pragma unroll
                for (int e = 0; e < 4; ++e) { out[e] = Narrow<T, float>(Combine(alpha, acc[i][j][4 * g + e], beta, static_cast<float>(old[e]))); }
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) { out[e] = Narrow<T, float>(alpha * acc[i][j][4 * g + e]); }
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

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_MFMA_F16_HPP_
