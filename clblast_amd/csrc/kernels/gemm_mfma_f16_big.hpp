// =================================================================================================
// HGEMM kernel for large problems on gfx950: 256 x 256 x 64 work-group tile, fp16 storage, fp32
// accumulation with v_mfma_f32_32x32x16_f16. Same role as gemm_mfma_f16.hpp (the reference's indirect
// chain src/routines/level3/xgemm.cpp:102-222 + src/kernels/level3/xgemm_part1-4.opencl in one launch)
// for 16-byte aligned operands; the differences are what measurements on the chip asked for:
//
//   * LDS always holds both operands as [x][k] (x = m or n, 64 k per row = 8 chunks of 16 bytes, no
//     padding) with the chunk index XOR-swizzled by the row, so that every MFMA fragment is ONE
//     ds_read_b128 and those reads are bank-conflict free. Plain 16-byte LDS reads overlap completely
//     with MFMA issue on this chip, whereas the transposing ds_read_b64_tr_b16 reads measurably steal
//     MFMA issue slots.
//   * An operand that is x-contiguous in memory is therefore transposed on its way into LDS: a thread
//     loads R rows (k) of 8 consecutive x, transposes the R x 8 block of halfs in registers with
//     v_perm_b32 (VALU work that hides behind the MFMAs) and writes 8 rows (x) of R halfs.
//   * The main loop is software-pipelined by hand and pinned with scheduling fences: fragments of
//     k-step s+1 are read while k-step s multiplies; the staged slab t+1 is written to the other LDS
//     buffer and the staging registers are refilled with slab t+2 in between; one barrier per slab sits
//     before the last k-step, so the first fragments of slab t+1 are fetched behind it at no cost.
//   * 4 wavefronts (one per SIMD, 128 x 128 each) or 8 wavefronts (two per SIMD, 128 x 64 each).
// Edge tiles and the K tail take an unpipelined, bounds-checked path through the same LDS layout.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_MFMA_F16_BIG_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_MFMA_F16_BIG_HPP_

#include <type_traits>

#include "kernels/gemm_args.hpp"
#include "kernels/gemm_mfma.hpp"
#include "kernels/gemm_mfma_f16.hpp"

namespace clbh {

typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));

template <int WM_, int WN_, int FM_, int FN_, int MIN_WAVES_>
struct HgemmBigConfig {
  static constexpr int WM = WM_, WN = WN_, FM = FM_, FN = FN_, MIN_WAVES = MIN_WAVES_;
  static constexpr int THREADS = 64 * WM * WN;
  static constexpr int TILE_M = WM * FM * 32;
  static constexpr int TILE_N = WN * FN * 32;
  static constexpr int TILE_K = 64;
  static constexpr int A_ELEMS = TILE_M * TILE_K, B_ELEMS = TILE_N * TILE_K;
  static constexpr int LDS_BYTES = 2 * (A_ELEMS + B_ELEMS) * 2;
  static constexpr int PIECES_A = A_ELEMS / 8 / THREADS, PIECES_B = B_ELEMS / 8 / THREADS;  // 16-byte pieces
  static_assert(FM >= FN, "block rows drive the schedule");
  static_assert(TILE_M % 256 == 0 && TILE_N % 256 == 0, "the transposing loader covers 256 x per pass");
  static_assert((PIECES_A == 4 || PIECES_A == 8) && (PIECES_B == 4 || PIECES_B == 8), "pieces per thread");
};

// Offset in halfs of (row x, 16-byte chunk c of the row's 64 k) inside a swizzled [x][64] tile. Rows x,
// x+1 sit in different halves of the 256-byte bank window; the XOR term walks the 8 chunks over 16
// consecutive rows (fragment reads) and over rows 8 apart (transposed stores).
__device__ __forceinline__ int SwizzledOffset(const int x, const int chunk) {
  return x * 64 + ((chunk ^ (((x >> 1) & 7) ^ ((x >> 4) & 7))) << 3);
}

// Staging of one operand slab (TILE_X x 64 halfs) in registers and its way into LDS.
template <int THREADS, int TILE_X, int PIECES, bool KC>
struct SlabStage {
  uint4_t regs[PIECES];
  static constexpr int STORES = KC ? PIECES : 8;

  // KC: piece c covers row x = (tid + c*THREADS) / 8, chunk (tid + c*THREADS) % 8.
  // XC: thread owns columns x8*8..+7 (x8 = tid % 32) of rows k = kg*PIECES + c (kg = tid / 32).
  __device__ __forceinline__ void Load(const int c, const _Float16* __restrict__ base, const long long ld, const int x0,
                                       const int k0, const int tid) {
    const _Float16* src;
    if (KC) {
      const int piece = tid + c * THREADS;
      src = base + (x0 + piece / 8) * ld + (k0 + (piece % 8) * 8);
    } else {
      static_assert(KC || TILE_X == 256, "one pass of 32 threads spans 256 x");
      src = base + (k0 + (tid / 32) * PIECES + c) * ld + (x0 + (tid % 32) * 8);
    }
    regs[c] = *reinterpret_cast<const uint4_t*>(src);
  }

  __device__ __forceinline__ void Store(const int s, _Float16* __restrict__ tile, const int tid) const {
    if (KC) {
      const int piece = tid + s * THREADS;
      *reinterpret_cast<uint4_t*>(&tile[SwizzledOffset(piece / 8, piece % 8)]) = regs[s];
    } else {
      // Row x = x8*8 + s of the transposed block: PIECES consecutive k starting at kg*PIECES. Dword s/2 of
      // every staged row holds x = 2*(s/2), 2*(s/2)+1; pick the low or high half of each.
      const int x = (tid % 32) * 8 + s;
      const int k_first = (tid / 32) * PIECES;
      const unsigned selector = (s % 2 == 0) ? 0x05040100u : 0x07060302u;
      unsigned out[PIECES / 2];
#pragma unroll
      for (int b = 0; b < PIECES / 2; ++b) {
        out[b] = __builtin_amdgcn_perm(regs[2 * b + 1][s / 2], regs[2 * b][s / 2], selector);
      }
      _Float16* dst = &tile[SwizzledOffset(x, k_first / 8) + (k_first % 8)];
      if (PIECES == 8) {
        uint4_t v = {out[0], out[1], out[2 % (PIECES / 2)], out[3 % (PIECES / 2)]};
        *reinterpret_cast<uint4_t*>(dst) = v;
      } else {
        uint2_t v = {out[0], out[1]};
        *reinterpret_cast<uint2_t*>(dst) = v;
      }
    }
  }
};

// Bounds-checked element-wise fill of a swizzled tile (edge tiles, K tail).
template <int THREADS, int TILE_X, bool KC>
__device__ __forceinline__ void FillSwizzledChecked(_Float16* __restrict__ tile, const _Float16* __restrict__ base,
                                                    const long long ld, const int x0, const int k0, const int x_end,
                                                    const int k_end, const int tid) {
  using Map = PieceMap<TILE_X, 64, 1, KC>;
#pragma unroll 4
  for (int piece = tid; piece < TILE_X * 64; piece += THREADS) {
    int x, k;
    Map::Get(piece, x, k);
    const int gx = x0 + x, gk = k0 + k;
    _Float16 value = _Float16(0);
    if (gx < x_end && gk < k_end) { value = KC ? base[gx * ld + gk] : base[gk * ld + gx]; }
    tile[SwizzledOffset(x, k / 8) + (k % 8)] = value;
  }
}

__device__ __forceinline__ half8_t ReadSwizzledFragment(const _Float16* __restrict__ tile, const int x32, const int ks,
                                                        const int lane) {
  return *reinterpret_cast<const half8_t*>(&tile[SwizzledOffset(x32 + lane % 32, ks * 2 + lane / 32)]);
}

template <typename Config, bool A_KC, bool B_KC>
__global__ __launch_bounds__(Config::THREADS, Config::MIN_WAVES) void HgemmBigKernel(const GemmArgs<float> p,
                                                                                   const int tiles_m,
                                                                                   const int tiles_n) {
  using T = _Float16;
  constexpr int THREADS = Config::THREADS, TILE_M = Config::TILE_M, TILE_N = Config::TILE_N, TILE_K = Config::TILE_K;
  constexpr int FM = Config::FM, FN = Config::FN, KSTEPS = TILE_K / 16;
  using StageA = SlabStage<THREADS, TILE_M, Config::PIECES_A, A_KC>;
  using StageB = SlabStage<THREADS, TILE_N, Config::PIECES_B, B_KC>;

  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* a_tiles = reinterpret_cast<T*>(lds_raw);   // two buffers of A_ELEMS
  T* b_tiles = a_tiles + 2 * Config::A_ELEMS;   // two buffers of B_ELEMS

  const int tid = threadIdx.x;
  const int lane = tid % 64, wave = tid / 64;
  const int wave_m = wave % Config::WM, wave_n = wave / Config::WM;

  int tile_m, tile_n;
  TileOfBlock(blockIdx.x, gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
  const int m0 = tile_m * TILE_M, n0 = tile_n * TILE_N;
  const bool interior = (m0 + TILE_M <= p.m) && (n0 + TILE_N <= p.n);
  const int slabs = (p.k + TILE_K - 1) / TILE_K;
  const int fast_slabs = interior ? p.k / TILE_K : 0;

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

    if (fast_slabs > 0) {
      StageA stage_a;
      StageB stage_b;
      auto load_all = [&](const int slab) {
#pragma unroll
        for (int s = 0; s < Config::PIECES_A; ++s) { stage_a.Load(s, a, p.a_ld, m0, slab * TILE_K, tid); }
#pragma unroll
        for (int s = 0; s < Config::PIECES_B; ++s) { stage_b.Load(s, b, p.b_ld, n0, slab * TILE_K, tid); }
      };
      load_all(0);
#pragma unroll
      for (int s = 0; s < StageA::STORES; ++s) { stage_a.Store(s, a_tiles, tid); }
#pragma unroll
      for (int s = 0; s < StageB::STORES; ++s) { stage_b.Store(s, b_tiles, tid); }
      if (fast_slabs > 1) { load_all(1); }
      __syncthreads();

      half8_t a_frag[2][FM], b_frag[2][FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) { a_frag[0][i] = ReadSwizzledFragment(a_tiles, (wave_m * FM + i) * 32, 0, lane); }
#pragma unroll
      for (int j = 0; j < FN; ++j) { b_frag[0][j] = ReadSwizzledFragment(b_tiles, (wave_n * FN + j) * 32, 0, lane); }

      // Work items between the MFMA groups of one slab, in order: store A, load A, store B, load B.
      constexpr int ITEMS_A0 = 0, ITEMS_A1 = ITEMS_A0 + StageA::STORES, ITEMS_B0 = ITEMS_A1 + Config::PIECES_A;
      constexpr int ITEMS_B1 = ITEMS_B0 + StageB::STORES, ITEMS = ITEMS_B1 + Config::PIECES_B;
      constexpr int SLOTS = (KSTEPS - 1) * FM;
      constexpr int PER_SLOT = (ITEMS + SLOTS - 1) / SLOTS;

      auto slab_body = [&](const int slab, auto store_tag, auto load_tag) {
        constexpr bool STORE = decltype(store_tag)::value, LOAD = decltype(load_tag)::value;
        const int cur = slab & 1;
        const T* a_cur = a_tiles + cur * Config::A_ELEMS;
        const T* b_cur = b_tiles + cur * Config::B_ELEMS;
        T* a_nxt = a_tiles + (cur ^ 1) * Config::A_ELEMS;
        T* b_nxt = b_tiles + (cur ^ 1) * Config::B_ELEMS;
        const int k_load = (slab + 2) * TILE_K;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const int set = ks % 2;
          const T* a_src = (ks + 1 < KSTEPS) ? a_cur : a_nxt;
          const T* b_src = (ks + 1 < KSTEPS) ? b_cur : b_nxt;
          const int ks_src = (ks + 1 < KSTEPS) ? ks + 1 : 0;
#pragma unroll
          for (int q = 0; q < FM; ++q) {
            if (!CLBH_EXPERIMENT_NO_READS) {
              a_frag[set ^ 1][q] = ReadSwizzledFragment(a_src, (wave_m * FM + q) * 32, ks_src, lane);
              if (q < FN) { b_frag[set ^ 1][q] = ReadSwizzledFragment(b_src, (wave_n * FN + q) * 32, ks_src, lane); }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              acc[q][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b_frag[set][j], a_frag[set][q], acc[q][j], 0, 0, 0);
            }
            if (ks < KSTEPS - 1) {
#pragma unroll
              for (int u = 0; u < PER_SLOT; ++u) {
                const int item = (ks * FM + q) * PER_SLOT + u;
                if (item < ITEMS_A1) {
                  if (STORE && !CLBH_EXPERIMENT_NO_STORES) { stage_a.Store(item - ITEMS_A0, a_nxt, tid); }
                } else if (item < ITEMS_B0) {
                  if (LOAD && !CLBH_EXPERIMENT_NO_LOADS) { stage_a.Load(item - ITEMS_A1, a, p.a_ld, m0, k_load, tid); }
                } else if (item < ITEMS_B1) {
                  if (STORE && !CLBH_EXPERIMENT_NO_STORES) { stage_b.Store(item - ITEMS_B0, b_nxt, tid); }
                } else if (item < ITEMS) {
                  if (LOAD && !CLBH_EXPERIMENT_NO_LOADS) { stage_b.Load(item - ITEMS_B1, b, p.b_ld, n0, k_load, tid); }
                }
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          }
          if (ks == KSTEPS - 2) {
            if (CLBH_EXPERIMENT_NO_BARRIER) { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
            else { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
          }
        }
      };
      int slab = 0;
      for (; slab + 2 < fast_slabs; ++slab) { slab_body(slab, std::true_type{}, std::true_type{}); }
      if (slab + 1 < fast_slabs) { slab_body(slab, std::true_type{}, std::false_type{}); ++slab; }
      slab_body(slab, std::false_type{}, std::false_type{});
      __syncthreads();
    }

    // Edge tiles (all slabs) and the K tail of interior tiles: checked, unpipelined.
    for (int slab = fast_slabs; slab < slabs; ++slab) {
      FillSwizzledChecked<THREADS, TILE_M, A_KC>(a_tiles, a, p.a_ld, m0, slab * TILE_K, p.m, p.k, tid);
      FillSwizzledChecked<THREADS, TILE_N, B_KC>(b_tiles, b, p.b_ld, n0, slab * TILE_K, p.n, p.k, tid);
      __syncthreads();
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        half8_t a_frag[FM], b_frag[FN];
#pragma unroll
        for (int i = 0; i < FM; ++i) { a_frag[i] = ReadSwizzledFragment(a_tiles, (wave_m * FM + i) * 32, ks, lane); }
#pragma unroll
        for (int j = 0; j < FN; ++j) { b_frag[j] = ReadSwizzledFragment(b_tiles, (wave_n * FN + j) * 32, ks, lane); }
#pragma unroll
        for (int i = 0; i < FM; ++i) {
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b_frag[j], a_frag[i], acc[i][j], 0, 0, 0);
          }
        }
      }
      __syncthreads();
    }

    // Epilogue: lane owns m = m_blk + lane%32; accumulator element r is the column n_blk + Row(r).
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int m = m0 + (wave_m * FM + i) * 32 + lane % 32;
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int n_blk = n0 + (wave_n * FN + j) * 32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int n = n_blk + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
          if (m < p.m && n < p.n) { StoreResult<T, float>(c, n * p.c_ld + m, acc[i][j][r], alpha, beta); }
        }
      }
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_MFMA_F16_BIG_HPP_
