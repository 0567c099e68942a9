// =================================================================================================
// Large-tile MFMA GEMM kernel for gfx950, fp16 storage with fp32 accumulation (HGEMM). Like the
// fp32/fp64 kernel (gemm_mfma.hpp) it replaces the reference's whole "indirect" chain
// (src/routines/level3/xgemm.cpp:102-222, src/kernels/level3/xgemm_part1-4.opencl) with one launch
// that reads the caller's operands in place. Unlike the reference, which accumulates in fp16
// (src/kernels/common.opencl:44-45), products are accumulated in fp32 by v_mfma_f32_32x32x16_f16 and
// rounded to fp16 once, in the epilogue.
//
// Structure (one work-group = 256 threads = 4 wavefronts in a 2 x 2 arrangement):
//   * work-group tile (64*FM) x (64*FN), K walked in slabs of TILE_K, two LDS buffers, global loads
//     of slab t+1 in flight while slab t is multiplied, one barrier per slab;
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
// of wavefronts per SIMD the register budget must allow. PIPELINED selects the explicitly scheduled main
// loop (see HgemmMfmaKernel); it needs FM >= FN and an even number of k-steps per slab.
template <int WM_, int WN_, int FM_, int FN_, int TILE_K_, int MIN_WAVES_, bool PIPELINED_, int STAGES_ = 2>
struct HgemmConfig {
  static constexpr int STAGES = STAGES_;  // LDS slab buffers of the pipelined loop
  static constexpr int WM = WM_, WN = WN_, FM = FM_, FN = FN_, MIN_WAVES = MIN_WAVES_;
  static constexpr bool PIPELINED = PIPELINED_;
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
  // the pipelined loop keeps STAGES slabs per operand in the direct-load layouts (HDirectLayout, <= 576 halfs
  // per KiB of slab)
  static constexpr int DIRECT_ELEMS = (TILE_M + TILE_N) * TILE_K / 512 * 576;
  static constexpr int PLAIN_BYTES = 2 * (A_ELEMS + B_ELEMS) * 2;
  static constexpr int DIRECT_BYTES = PIPELINED_ ? STAGES_ * DIRECT_ELEMS * 2 : 0;
  static constexpr int LDS_BYTES = PLAIN_BYTES > DIRECT_BYTES ? PLAIN_BYTES : DIRECT_BYTES;
  static_assert(TILE_K % 16 == 0, "slab depth is a multiple of the MFMA k extent");
  static_assert((TILE_M * TILE_K) % (8 * THREADS) == 0 && (TILE_N * TILE_K) % (8 * THREADS) == 0, "slab split");
  static_assert(!PIPELINED || (FM >= FN && TILE_K == 32 && TILE_M == 256 && TILE_N == 256 && THREADS == 512 && STAGES >= 2),
                "pipelined loop shape");
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

// Single pieces of a slab (16 bytes), for the explicitly scheduled loop.
template <int THREADS, int TILE_X, int TILE_K, bool KC>
__device__ __forceinline__ half8_t HLoadPiece(const _Float16* __restrict__ base, const long long ld, const int x0,
                                              const int k0, const int tid, const int c) {
  int x, k;
  PieceMap<TILE_X, TILE_K, 8, KC>::Get(tid + c * THREADS, x, k);
  const _Float16* src = KC ? base + (x0 + x) * ld + (k0 + k) : base + (k0 + k) * ld + (x0 + x);
  return *reinterpret_cast<const half8_t*>(src);
}

template <int THREADS, int TILE_X, int TILE_K, int PITCH, bool KC>
__device__ __forceinline__ void HStorePiece(_Float16* __restrict__ tile, const int tid, const int c,
                                            const half8_t value) {
  int x, k;
  PieceMap<TILE_X, TILE_K, 8, KC>::Get(tid + c * THREADS, x, k);
  *reinterpret_cast<half8_t*>(KC ? &tile[x * PITCH + k] : &tile[k * PITCH + x]) = value;
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

// ---- direct global -> LDS slabs for the pipelined loop (256 x 32 halfs per operand and slab) ---------
// `buffer_load_dwordx4 ... lds` puts lane l's 16 bytes at base + 16 * l, so LDS is filled in 1 KiB pieces
// whose inner layout is fixed; which 16 bytes of global memory a lane fetches is free, and that freedom
// carries the bank swizzle.
//   x-contiguous operand: a piece is two k rows of 256 halfs; in the odd row the 16-byte chunk t of the
//     row sits at position t ^ 4. Pieces are 576 halfs apart. LDS serves 32 lanes of a transposing read per
//     cycle: rows k..k+3, 64 bytes each, which this layout spreads over eight different 32-byte bank windows.
//   k-contiguous operand: a piece is 16 x rows of 32 halfs (4 chunks); chunk c of row r sits at position
//     c ^ ((r >> 2) & 3), so the 16-byte reads of 16 consecutive rows cover all 64 banks once.
template <bool KC>
struct HDirectLayout {
  static constexpr int PIECE_PITCH = KC ? 512 : 576;  // halfs
  static constexpr int PIECES = 16;                   // per operand and slab
  static constexpr int ELEMS = PIECES * PIECE_PITCH;
};

// Issues the round-th (0 or 1) piece load of this wavefront; `slab` points at element (x0, k0), uniform.
template <bool KC>
__device__ __forceinline__ void HDirectLoad(const _Float16* __restrict__ slab, const long long ld, _Float16* stage,
                                            const int wave, const int lane, const int round) {
  const int piece = wave + 8 * round;
  const _Float16* source;
  int lane_elems;
  if (KC) {
    const int row = lane / 4, chunk = (lane % 4) ^ ((row >> 2) & 3);
    source = slab + static_cast<long long>(16 * piece) * ld;
    lane_elems = static_cast<int>(row * ld) + 8 * chunk;
  } else {
    const int row = lane / 32, chunk = (lane % 32) ^ (4 * row);
    source = slab + static_cast<long long>(2 * piece) * ld;
    lane_elems = static_cast<int>(row * ld) + 8 * chunk;
  }
  const __amdgpu_buffer_rsrc_t resource = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(source), 0, -1, 0x00020000);
  typedef __attribute__((address_space(3))) void* LdsPtr;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(resource, (LdsPtr)(stage + piece * HDirectLayout<KC>::PIECE_PITCH), 16,
                                           lane_elems * 2, 0, 0, 0);
}

// Offset of a lane's fragment data for the block starting at x32 (a multiple of 32), k-step 0, in a
// direct-layout stage; constant over the whole K walk.
template <bool KC>
__device__ __forceinline__ int HDirectLaneOffset(const int lane, const int x32) {
  if (KC) {
    const int row = lane % 16;
    return (x32 / 16 + (lane % 32) / 16) * 512 + row * 32 + 8 * ((lane / 32) ^ ((row >> 2) & 3));
  } else {
    const int group = lane / 16, q = lane % 16, parity = (q / 4) % 2;
    const int x = (x32 + 16 * (group % 2) + 4 * (q % 4)) ^ (32 * parity);  // odd rows hold chunk t at t ^ 4
    return (4 * (group / 2) + (q / 4) / 2) * 576 + parity * 256 + x;
  }
}

// Fragment of k-step ks (0 or 1) of a direct-layout stage, for the lane offset of its block.
template <bool KC>
__device__ __forceinline__ half8_t HDirectFragment(const _Float16* __restrict__ stage, const int lane_offset, const int ks) {
  if (KC) {
    // chunk index of the k-step is 2*ks + lane/32; the swizzle is an XOR, so k-step 1 flips bit 1 of it
    return *reinterpret_cast<const half8_t*>(&stage[lane_offset ^ (ks * 16)]);
  } else {
    typedef __attribute__((address_space(3))) short4_t* LdsPtr;
    const _Float16* src = stage + ks * 8 * 576 + lane_offset;
    const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(src));
    const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(src + 2 * 576));
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
  TileOfBlock(blockIdx.x, gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
  const int m0 = tile_m * TILE_M, n0 = tile_n * TILE_N;
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
    if constexpr (Config::PIPELINED && ALIGNED) {
      // Explicit schedule for few wavefronts per SIMD, where little but the instruction order inside the
      // wavefront hides latency. Slabs go global -> LDS directly into a ring of STAGES buffers: the loads
      // of slab t+STAGES-1 are issued at the start of slab t (its buffer was released by the barrier of
      // slab t-1) and have STAGES-2 slabs plus one k-step to land. Per slab (2 k-steps of FM quarters):
      //   quarter q of k-step s:  LDS reads of the a/b fragments q of k-step s+1 (other register set),
      //                           then the FN MFMAs of block row q of k-step s.
      //   One barrier per slab, before the last k-step: by then every wavefront has issued all its reads
      //   of the current buffer, and slab t+1 has landed for everybody, so the last k-step can already
      //   fetch the first fragments of slab t+1. Scheduling fences pin this order for the compiler.
      constexpr int KSTEPS = TILE_K / 16, STAGES = Config::STAGES;
      constexpr int LOADS_PER_SLAB = 4;  // per wavefront: two pieces of A, two of B
      using LA = HDirectLayout<A_KC>;
      using LB = HDirectLayout<B_KC>;
      static_assert(STAGES * (LA::ELEMS + LB::ELEMS) * 2 <= Config::LDS_BYTES, "LDS allocation covers the ring");
      static_assert(LOADS_PER_SLAB <= FM, "one request per quarter of the first k-step");
      if (fast_slabs > 0) {
        T* a_ring = lds;
        T* b_ring = lds + STAGES * LA::ELEMS;
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        const T* a_tile0 = a + (A_KC ? m0 * p.a_ld : static_cast<long long>(m0));  // element (m0, k = 0), uniform
        const T* b_tile0 = b + (B_KC ? n0 * p.b_ld : static_cast<long long>(n0));
        // load 0..3 of a slab: piece rounds A0, B0, A1, B1 of this wavefront
        auto issue = [&](const int load, const int slab, const int buffer) {
          const int k0 = slab * TILE_K;
          if (load % 2 == 0) {
            HDirectLoad<A_KC>(a_tile0 + (A_KC ? static_cast<long long>(k0) : k0 * p.a_ld), p.a_ld, a_ring + buffer * LA::ELEMS,
                              wave_u, lane, load / 2);
          } else {
            HDirectLoad<B_KC>(b_tile0 + (B_KC ? static_cast<long long>(k0) : k0 * p.b_ld), p.b_ld, b_ring + buffer * LB::ELEMS,
                              wave_u, lane, load / 2);
          }
        };
        int a_lane[FM], b_lane[FN];
#pragma unroll
        for (int q = 0; q < FM; ++q) { a_lane[q] = HDirectLaneOffset<A_KC>(lane, (wave_m * FM + q) * 32); }
#pragma unroll
        for (int q = 0; q < FN; ++q) { b_lane[q] = HDirectLaneOffset<B_KC>(lane, (wave_n * FN + q) * 32); }
#pragma unroll
        for (int s = 0; s < STAGES - 1; ++s) {
          if (s < fast_slabs) {
#pragma unroll
            for (int load = 0; load < LOADS_PER_SLAB; ++load) { issue(load, s, s); }
          }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        half8_t a_frag[2][FM], b_frag[2][FN];
#pragma unroll
        for (int q = 0; q < FM; ++q) { a_frag[0][q] = HDirectFragment<A_KC>(a_ring, a_lane[q], 0); }
#pragma unroll
        for (int q = 0; q < FN; ++q) { b_frag[0][q] = HDirectFragment<B_KC>(b_ring, b_lane[q], 0); }
        int cur = 0;  // buffer of the current slab; the next slab is in cur + 1, the free one is cur - 1 (mod STAGES)
        // One slab. ISSUE: slab + STAGES - 1 exists and is requested; compile-time, so that the steady state has
        // no branches.
        auto slab_body = [&](const int slab, auto issue_tag) {
          constexpr bool ISSUE = decltype(issue_tag)::value;
          const int nxt = (cur + 1 == STAGES) ? 0 : cur + 1;
          const int free_buffer = (cur == 0) ? STAGES - 1 : cur - 1;
          const T* a_cur = a_ring + cur * LA::ELEMS;
          const T* b_cur = b_ring + cur * LB::ELEMS;
          const T* a_nxt = a_ring + nxt * LA::ELEMS;
          const T* b_nxt = b_ring + nxt * LB::ELEMS;
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) {
            const int set = ks % 2;
            const T* a_src = (ks + 1 < KSTEPS) ? a_cur : a_nxt;
            const T* b_src = (ks + 1 < KSTEPS) ? b_cur : b_nxt;
            const int ks_src = (ks + 1 < KSTEPS) ? ks + 1 : 0;
#pragma unroll
            for (int q = 0; q < FM; ++q) {
              a_frag[set ^ 1][q] = HDirectFragment<A_KC>(a_src, a_lane[q], ks_src);
              if (q < FN) { b_frag[set ^ 1][q] = HDirectFragment<B_KC>(b_src, b_lane[q], ks_src); }
              __builtin_amdgcn_sched_barrier(0);
#pragma unroll
              for (int j = 0; j < FN; ++j) {
                acc[q][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_frag[set][q], b_frag[set][j], acc[q][j], 0, 0, 0);
              }
              // one request per quarter: a burst of identical requests from all work-groups defeats the L2
              if (ISSUE && ks == 0 && q < LOADS_PER_SLAB) { issue(q, slab + STAGES - 1, free_buffer); }
              __builtin_amdgcn_sched_barrier(0);
            }
            if (ks == KSTEPS - 2) {
              // slab + 1 must have landed; in the steady state the loads of the STAGES - 2 slabs after it may
              // still be in flight (loads complete in order)
              if (ISSUE) { asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * LOADS_PER_SLAB) : "memory"); }
              else { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
              asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            }
          }
          cur = nxt;
        };
        int slab = 0;
        for (; slab + STAGES - 1 < fast_slabs; ++slab) { slab_body(slab, std::true_type{}); }
        for (; slab < fast_slabs; ++slab) { slab_body(slab, std::false_type{}); }
        __syncthreads();
      }
    } else if (fast_slabs > 0) {
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
                               ((reinterpret_cast<unsigned long long>(c) & 15) == 0);
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
              if (wave_m0 + col < p.m) {
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
                for (int e = 0; e < 4; ++e) { out[e] = static_cast<T>(alpha * acc[i][j][4 * g + e] + beta * static_cast<float>(old[e])); }
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) { out[e] = static_cast<T>(alpha * acc[i][j][4 * g + e]); }
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
