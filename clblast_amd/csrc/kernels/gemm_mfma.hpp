// =================================================================================================
// Large-tile MFMA GEMM kernel for gfx950, fp32 and fp64. It stands where the reference has its
// "indirect" path (src/routines/level3/xgemm.cpp:102-222 with the kernels of
// src/kernels/level3/xgemm_part1-4.opencl, copy_pad/transpose_pad.opencl), but needs none of that
// path's pre- and post-kernels: both operand orientations, arbitrary leading dimensions and offsets
// and ragged edges are handled by the tile loaders and the epilogue of this one kernel.
//
// Structure (one work-group = 256 threads = 4 wavefronts):
//   * the work-group owns a TILE_M x TILE_N block of C; K is walked in slabs of TILE_K;
//   * global -> registers -> LDS staging with two LDS buffers, so that the loads of slab t+1 are in
//     flight while slab t feeds the matrix cores, with one barrier per slab;
//   * both operands sit in LDS as [k][x] (x = m for A, n for B; x contiguous) whatever their layout in
//     memory: x-contiguous operands are copied with 16-byte loads and stores, k-contiguous ones are
//     loaded with 16-byte loads along k and scattered into LDS (a transpose on the fly);
//   * each wavefront computes a (MF*FM) x (MF*FN) block with v_mfma_f32_32x32x2_f32 (MF = 32) or
//     v_mfma_f64_16x16x4_f64 (MF = 16). The n-indexed values are fed as the MFMA's A operand and the
//     m-indexed ones as its B operand, so the lanes of a result register run along m: stores to the
//     column-major C are contiguous per lane group. A lane owns FM consecutive m (one LDS read of
//     FM elements, one vector store of FM elements);
//   * the blockIdx -> tile mapping first makes the work-groups that the hardware deals round-robin to
//     one XCD (blockIdx % 8) logically contiguous, then walks C in groups of GROUP_M tile rows, so
//     the tiles in flight on one XCD share A and B panels in that XCD's L2.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_MFMA_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_MFMA_HPP_

#include <type_traits>

#ifndef CLBH_EXP_NO_DIRECT
#define CLBH_EXP_NO_DIRECT 0
#endif

#include "kernels/gemm_args.hpp"

namespace clbh {

constexpr int kMfmaThreads = 256;
constexpr int kNumXcd = 8;

typedef float float16_t __attribute__((ext_vector_type(16)));
typedef double double4_t __attribute__((ext_vector_type(4)));

// ---- per-precision MFMA traits ---------------------------------------------------------------------
template <typename T> struct MfmaTraits;

template <> struct MfmaTraits<float> {
  static constexpr int MF = 32;       // the instruction computes an MF x MF block
  static constexpr int KP = 2;        // k extent of one instruction
  static constexpr int ACC = 16;      // accumulator elements per lane and block
  using Acc = float16_t;
  static __device__ __forceinline__ Acc Zero() { return Acc(0.0f); }
  static __device__ __forceinline__ Acc Mfma(const float rows, const float cols, const Acc acc) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(rows, cols, acc, 0, 0, 0);
  }
  // row of the MF x MF block held by accumulator element r of a lane in k-group g
  static __device__ __forceinline__ int Row(const int r, const int g) { return 8 * (r / 4) + 4 * g + (r % 4); }
};

template <> struct MfmaTraits<double> {
  static constexpr int MF = 16;
  static constexpr int KP = 4;
  static constexpr int ACC = 4;
  using Acc = double4_t;
  static __device__ __forceinline__ Acc Zero() { return Acc(0.0); }
  static __device__ __forceinline__ Acc Mfma(const double rows, const double cols, const Acc acc) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(rows, cols, acc, 0, 0, 0);
  }
  static __device__ __forceinline__ int Row(const int r, const int g) { return 4 * r + g; }
};

// ---- tile configuration ----------------------------------------------------------------------------
// WM x WN wavefronts per work-group (WM * WN == 4), each owning FM x FN MFMA blocks.
template <typename T, int WM_, int WN_, int FM_, int FN_, int TILE_K_, int MIN_WAVES_ = 2>
struct MfmaConfig {
  static constexpr int MIN_WAVES = MIN_WAVES_;  // wavefronts per SIMD the register budget must allow
  using Traits = MfmaTraits<T>;
  static constexpr int WM = WM_, WN = WN_, FM = FM_, FN = FN_;
  static constexpr int TILE_M = WM * FM * Traits::MF;
  static constexpr int TILE_N = WN * FN * Traits::MF;
  static constexpr int TILE_K = TILE_K_;
  static constexpr int VEC = 16 / sizeof(T);  // elements per 16-byte access
  // Row pitch of the LDS tiles in elements. pitch % (64 / VEC... ) is chosen so that the scattered
  // 4-byte (fp32) or 8-byte (fp64) stores of the k-contiguous loader fall into distinct banks: the 64
  // lanes of a wavefront write (TILE_K / VEC) different k rows, which must be (64 * 4 / sizeof(T)) /
  // (TILE_K / VEC) elements apart modulo the bank window.
  static constexpr int PAD = VEC;
  static constexpr int PITCH_M = TILE_M + PAD;
  static constexpr int PITCH_N = TILE_N + PAD;
  static constexpr int LDS_ELEMS = 2 * TILE_K * (PITCH_M + PITCH_N);  // two buffers
  static constexpr int CHUNKS_A = TILE_M * TILE_K / VEC / kMfmaThreads;  // 16-byte chunks per thread and slab
  static constexpr int CHUNKS_B = TILE_N * TILE_K / VEC / kMfmaThreads;
  static_assert(WM * WN * 64 == kMfmaThreads, "four wavefronts per work-group");
  static_assert(TILE_M * TILE_K % (VEC * kMfmaThreads) == 0 && TILE_N * TILE_K % (VEC * kMfmaThreads) == 0,
                "slab must divide evenly over the threads");
  static_assert(TILE_K % Traits::KP == 0 && TILE_K % VEC == 0, "slab depth");
};

// Vector types for LDS and global accesses; never assumed to be aligned beyond 16 bytes.
template <typename T, int N> struct VecType { typedef T type __attribute__((ext_vector_type(N), aligned(N * sizeof(T) < 16 ? N * sizeof(T) : 16))); };
template <typename T> struct VecType<T, 1> { typedef T type; };

template <typename V, typename T, int N>
__device__ __forceinline__ T VecGet(const V v, const int i) {
  if constexpr (N == 1) { return v; } else { return v[i]; }
}
template <typename V, typename T, int N>
__device__ __forceinline__ V VecWith(V v, const int i, const T value) {
  if constexpr (N == 1) { v = value; } else { v[i] = value; }
  return v;
}

// ---- slab loaders ----------------------------------------------------------------------------------
// One operand slab is TILE_X x TILE_K elements. `base` points at element (x = 0, k = 0) of the matrix of
// this batch; the element (x, k) lives at base[KC ? x*ld + k : k*ld + x]. Every thread moves PIECES
// pieces of VL elements (VL = 16 bytes' worth when every address is 16-byte aligned, else 1). The
// piece -> (x, k) mapping puts consecutive threads along the contiguous index of the operand in
// memory, so a wavefront's accesses coalesce for either orientation.
template <int TILE_X, int TILE_K, int VL, bool KC>
struct PieceMap {
  static constexpr int ALONG = (KC ? TILE_K : TILE_X) / VL;  // pieces per contiguous line of the slab
  static __device__ __forceinline__ void Get(const int piece, int& x, int& k) {
    const int line = piece / ALONG, pos = (piece % ALONG) * VL;
    x = KC ? line : pos;
    k = KC ? pos : line;
  }
};

// Fast path: the whole slab is inside the matrix.
template <typename T, int TILE_X, int TILE_K, int PIECES, int VL, bool KC>
__device__ __forceinline__ void LoadSlab(const T* __restrict__ base, const long long ld, const int x0, const int k0,
                                         const int tid, T (&regs)[PIECES][VL]) {
  using Map = PieceMap<TILE_X, TILE_K, VL, KC>;
  using V = typename VecType<T, VL>::type;
#pragma unroll
  for (int c = 0; c < PIECES; ++c) {
    int x, k;
    Map::Get(tid + c * kMfmaThreads, x, k);
    const T* src = KC ? base + (x0 + x) * ld + (k0 + k) : base + (k0 + k) * ld + (x0 + x);
    const V v = *reinterpret_cast<const V*>(src);
#pragma unroll
    for (int e = 0; e < VL; ++e) { regs[c][e] = VecGet<V, T, VL>(v, e); }
  }
}

// Register-staged load of a slab whose x range sticks out of the matrix (the k range is complete):
// elements beyond x_end read as zero. Keeps edge tiles on the pipelined path.
template <typename T, int TILE_X, int TILE_K, int PIECES, int VL, bool KC>
__device__ __forceinline__ void LoadSlabEdge(const T* __restrict__ base, const long long ld, const int x0, const int k0,
                                             const int x_end, const int tid, T (&regs)[PIECES][VL]) {
  using Map = PieceMap<TILE_X, TILE_K, VL, KC>;
#pragma unroll
  for (int c = 0; c < PIECES; ++c) {
    int x, k;
    Map::Get(tid + c * kMfmaThreads, x, k);
#pragma unroll
    for (int e = 0; e < VL; ++e) {
      const int gx = x0 + x + (KC ? 0 : e), gk = k0 + k + (KC ? e : 0);
      regs[c][e] = (gx < x_end) ? (KC ? base[gx * ld + gk] : base[gk * ld + gx]) : T(0);
    }
  }
}

// Edge tiles and the K tail: element-wise, bounds-checked copy straight into the LDS tile [k][x] (no
// register staging, no overlap with the multiplication). Elements outside the matrix become zero.
template <typename T, int TILE_X, int TILE_K, int PITCH, bool KC>
__device__ __forceinline__ void FillSlabChecked(T* __restrict__ tile, const T* __restrict__ base, const long long ld,
                                                const int x0, const int k0, const int x_end, const int k_end,
                                                const int tid) {
  using Map = PieceMap<TILE_X, TILE_K, 1, KC>;
#pragma unroll 4
  for (int piece = tid; piece < TILE_X * TILE_K; piece += kMfmaThreads) {
    int x, k;
    Map::Get(piece, x, k);
    const int gx = x0 + x, gk = k0 + k;
    T value = T(0);
    if (gx < x_end && gk < k_end) { value = KC ? base[gx * ld + gk] : base[gk * ld + gx]; }
    tile[k * PITCH + x] = value;
  }
}

// Registers -> LDS tile [k][x] with row pitch PITCH.
template <typename T, int TILE_X, int TILE_K, int PITCH, int PIECES, int VL, bool KC>
__device__ __forceinline__ void StoreSlab(T* __restrict__ tile, const int tid, const T (&regs)[PIECES][VL]) {
  using Map = PieceMap<TILE_X, TILE_K, VL, KC>;
  using V = typename VecType<T, VL>::type;
#pragma unroll
  for (int c = 0; c < PIECES; ++c) {
    int x, k;
    Map::Get(tid + c * kMfmaThreads, x, k);
    if (KC) {
#pragma unroll
      for (int e = 0; e < VL; ++e) { tile[(k + e) * PITCH + x] = regs[c][e]; }
    } else {
      V v;
#pragma unroll
      for (int e = 0; e < VL; ++e) { v = VecWith<V, T, VL>(v, e, regs[c][e]); }
      *reinterpret_cast<V*>(&tile[k * PITCH + x]) = v;
    }
  }
}

// One piece of a full slab: global memory -> register vector, and register vector -> LDS tile [k][x].
// Thread t moves the pieces t, t + THREADS, ... of the slab; with LINES = THREADS / ALONG whole lines per
// round, piece c of a thread lies c * LINES lines after its piece 0. The address is split into a part that
// is uniform over the work-group (64-bit, scalar registers) and the thread's byte offset inside the slab
// (32-bit, one vector register for all pieces of an operand): a global load takes exactly this pair.
template <int TILE_X, int TILE_K, int VL, bool KC>
struct PieceRounds {
  static constexpr int ALONG = PieceMap<TILE_X, TILE_K, VL, KC>::ALONG;
  static_assert(kMfmaThreads % ALONG == 0, "whole lines per round of pieces");
  static constexpr int LINES = kMfmaThreads / ALONG;
};

template <typename T, int TILE_X, int TILE_K, int VL, bool KC>
__device__ __forceinline__ unsigned int PieceLaneBytes(const long long ld, const int tid) {
  using Rounds = PieceRounds<TILE_X, TILE_K, VL, KC>;
  const int line = tid / Rounds::ALONG, pos = (tid % Rounds::ALONG) * VL;
  return static_cast<unsigned int>((line * ld + pos) * static_cast<long long>(sizeof(T)));
}

// `slab` points at the slab's first element (x0, k0) and must be uniform over the work-group.
template <typename T, int TILE_X, int TILE_K, int VL, bool KC>
__device__ __forceinline__ typename VecType<T, VL>::type LoadPiece(const T* __restrict__ slab, const long long ld,
                                                                   const unsigned int lane_bytes, const int c) {
  using Rounds = PieceRounds<TILE_X, TILE_K, VL, KC>;
  const char* round = reinterpret_cast<const char*>(slab + static_cast<long long>(c * Rounds::LINES) * ld);
  return *reinterpret_cast<const typename VecType<T, VL>::type*>(round + lane_bytes);
}

template <typename T, int TILE_X, int TILE_K, int PITCH, int VL, bool KC>
__device__ __forceinline__ void StorePiece(T* __restrict__ tile, const int tid, const int c,
                                           const typename VecType<T, VL>::type v) {
  using V = typename VecType<T, VL>::type;
  int x, k;
  PieceMap<TILE_X, TILE_K, VL, KC>::Get(tid + c * kMfmaThreads, x, k);
  if (KC) {
#pragma unroll
    for (int e = 0; e < VL; ++e) { tile[(k + e) * PITCH + x] = VecGet<V, T, VL>(v, e); }
  } else {
    *reinterpret_cast<V*>(&tile[k * PITCH + x]) = v;
  }
}

// ---- direct global -> LDS loads (x-contiguous, 16-byte aligned operands on interior tiles) ----------
// One `buffer_load_dwordx4 ... lds` moves 16 bytes per lane straight into LDS, lane l landing at
// base + 16 * l: a wavefront fills 1 KiB of contiguous LDS per instruction and no vector register or
// LDS store instruction is spent on staging. A slab [k][x] is therefore kept as groups of R whole rows
// (R * TILE_X * sizeof(T) == 1 KiB, or one row in several instructions when a row is longer), groups
// GROUP_PITCH elements apart. An operand that is staged through registers uses the same description
// with R == 1, i.e. plain rows of pitch TILE_X + PAD.
template <typename T, int TILE_X, int TILE_K, bool DIRECT>
struct SlabLayout {
  static constexpr int VEC = 16 / sizeof(T);
  static constexpr int WAVE_ELEMS = 1024 / sizeof(T);                       // elements per wavefront-wide load
  static constexpr int R = (DIRECT && TILE_X < WAVE_ELEMS) ? WAVE_ELEMS / TILE_X : 1;  // rows per group
  static constexpr int PARTS = (DIRECT && TILE_X > WAVE_ELEMS) ? TILE_X / WAVE_ELEMS : 1;  // loads per row
  static constexpr int GROUPS = TILE_K / R;
  static constexpr int GROUP_PITCH = R * TILE_X + VEC;
  static constexpr int ELEMS = GROUPS * GROUP_PITCH;                         // one stage
  static constexpr int LOADS = GROUPS * PARTS;                               // wavefront-wide loads per slab
  static constexpr int LOADS_PER_WAVE = (LOADS + 3) / 4;
  static_assert(TILE_K % R == 0, "whole groups per slab");
  // offset of element (k, 0)
  static __device__ __forceinline__ int Row(const int k) { return (k / R) * GROUP_PITCH + (k % R) * TILE_X; }
};

// Issues the `round`-th direct load of this wavefront for one slab. `slab` points at the slab's first
// element (x0, k0), `stage` at the LDS stage; both are uniform over the work-group.
template <typename T, int TILE_X, int TILE_K>
__device__ __forceinline__ void DirectLoad(const T* __restrict__ slab, const long long ld, T* stage, const int wave,
                                           const int lane, const int round) {
  using L = SlabLayout<T, TILE_X, TILE_K, true>;
  const int index = wave + 4 * round;
  if (L::LOADS % 4 != 0 && index >= L::LOADS) { return; }
  const int group = index / L::PARTS, part = index % L::PARTS;
  const int in_group = lane * L::VEC;                                      // element of the 1 KiB chunk
  const int row = (L::R > 1) ? in_group / TILE_X : 0, x = (L::R > 1) ? in_group % TILE_X : in_group;
  const int lane_bytes = static_cast<int>((row * ld + x) * static_cast<long long>(sizeof(T)));
  const T* chunk = slab + static_cast<long long>(group * L::R) * ld + part * L::WAVE_ELEMS;
  // Buffer form of the load (untyped raw buffer over the rest of the address space, no range check
  // needed on interior tiles): unlike the flat-encoded global form it leaves the LDS counter alone, so
  // waits on LDS reads stay counted instead of draining the queue.
  const __amdgpu_buffer_rsrc_t resource = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(chunk), 0, -1, 0x00020000);
  typedef __attribute__((address_space(3))) void* LdsPtr;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(resource, (LdsPtr)(stage + group * L::GROUP_PITCH + part * L::WAVE_ELEMS), 16,
                                           lane_bytes, 0, 0, 0);
}

// ---- blockIdx -> tile ------------------------------------------------------------------------------
__device__ __forceinline__ void TileOfBlock(const int block, const int num_blocks, const int tiles_m,
                                            const int tiles_n, int& tile_m, int& tile_n) {
  // (1) work-groups are dealt to the XCDs round-robin: give each XCD a contiguous logical range
  const int per_xcd = (num_blocks + kNumXcd - 1) / kNumXcd;
  const int remainder = num_blocks % kNumXcd;
  const int tall = (remainder == 0) ? kNumXcd : remainder;  // XCDs that own per_xcd blocks
  const int xcd = block % kNumXcd, local = block / kNumXcd;
  const int logical = (xcd < tall) ? xcd * per_xcd + local
                                   : tall * per_xcd + (xcd - tall) * (per_xcd - 1) + local;
  // (2) grouped walk: GROUP_M tile rows at a time, column by column inside a group
  constexpr int GROUP_M = 8;
  const int in_group = GROUP_M * tiles_n;
  const int group = logical / in_group;
  const int first_m = group * GROUP_M;
  const int group_rows = min(tiles_m - first_m, GROUP_M);
  tile_m = first_m + (logical % in_group) % group_rows;
  tile_n = (logical % in_group) / group_rows;
}

// ---- the kernel ------------------------------------------------------------------------------------
template <typename T, typename Config, bool A_KC, bool B_KC, bool ALIGNED>
__global__ __launch_bounds__(kMfmaThreads, ALIGNED ? Config::MIN_WAVES : 2) void GemmMfmaKernel(const GemmArgs<T> p, const int tiles_m,
                                                               const int tiles_n) {
  using Traits = typename Config::Traits;
  using Acc = typename Traits::Acc;
  constexpr int MF = Traits::MF, KP = Traits::KP, ACC = Traits::ACC;
  constexpr int TILE_M = Config::TILE_M, TILE_N = Config::TILE_N, TILE_K = Config::TILE_K;
  constexpr int FM = Config::FM, FN = Config::FN, VEC = Config::VEC;
  constexpr int PITCH_M = Config::PITCH_M, PITCH_N = Config::PITCH_N;
  constexpr int VL = ALIGNED ? VEC : 1;  // elements per global access
  constexpr int PIECES_A = Config::CHUNKS_A * VEC / VL, PIECES_B = Config::CHUNKS_B * VEC / VL;
  using VM = typename VecType<T, FM>::type;
  using VN = typename VecType<T, FN>::type;

  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  T* a_tiles = lds;                             // [2][TILE_K][PITCH_M]
  T* b_tiles = lds + 2 * TILE_K * PITCH_M;      // [2][TILE_K][PITCH_N]

  const int tid = threadIdx.x;
  const int lane = tid % 64, wave = tid / 64;
  const int wave_m = wave % Config::WM, wave_n = wave / Config::WM;
  const int lane_x = lane % MF;  // position along the lane dimension of the MFMA block
  const int lane_g = lane / MF;  // k-group of the lane inside one instruction

  int tile_m, tile_n;
  TileOfBlock(blockIdx.x, gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
  const int m0 = tile_m * TILE_M, n0 = tile_n * TILE_N;
  const bool a_full = (m0 + TILE_M <= p.m), b_full = (n0 + TILE_N <= p.n);

  // LDS read offsets of this lane. Aligned operands: the lane owns FM consecutive m (one vector LDS read,
  // one vector store to C). Otherwise C is stored element-wise, and the lane owns m = lane_x, lane_x + MF,
  // ... so that the lanes of each scalar store cover consecutive addresses.
  constexpr bool M_INTERLEAVED = ALIGNED;
  const int a_read = wave_m * (FM * MF) + (M_INTERLEAVED ? lane_x * FM : lane_x);
  const int b_read = wave_n * (FN * MF) + lane_x * FN;

  for (int batch = blockIdx.y; batch < p.batch_count; batch += gridDim.y) {
    const T* a;
    const T* b;
    T* c;
    T alpha, beta;
    ResolveBatch<T, T>(p, batch, a, b, c, alpha, beta);
    int k_len = p.k;
    long long c_ld = p.c_ld;
    bool c_aligned = ALIGNED;
    if (p.split_chunk > 0) {  // this "batch" is one K range of a single problem
      const int k_begin = batch * p.split_chunk;
      k_len = min(p.split_chunk, p.k - k_begin);
      a = static_cast<const T*>(p.a) + p.a_offset + (A_KC ? k_begin : k_begin * p.a_ld);
      b = static_cast<const T*>(p.b) + p.b_offset + (B_KC ? k_begin : k_begin * p.b_ld);
      c_ld = p.split_ld;
      c = static_cast<T*>(p.split_workspace) + static_cast<long long>(batch) * p.split_ld * p.n;
      alpha = T(1);
      beta = T(0);
      c_aligned = true;  // the workspace is 256-byte aligned and split_ld a multiple of 4
    }
    const int full_slabs = k_len / TILE_K;
    const int slabs = (k_len + TILE_K - 1) / TILE_K;

    Acc acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
      for (int j = 0; j < FN; ++j) { acc[i][j] = Traits::Zero(); }
    }

    T a_regs[PIECES_A][VL];
    T b_regs[PIECES_B][VL];

    auto load = [&](const int slab) {
      if (a_full) { LoadSlab<T, TILE_M, TILE_K, PIECES_A, VL, A_KC>(a, p.a_ld, m0, slab * TILE_K, tid, a_regs); }
      else { LoadSlabEdge<T, TILE_M, TILE_K, PIECES_A, VL, A_KC>(a, p.a_ld, m0, slab * TILE_K, p.m, tid, a_regs); }
      if (b_full) { LoadSlab<T, TILE_N, TILE_K, PIECES_B, VL, B_KC>(b, p.b_ld, n0, slab * TILE_K, tid, b_regs); }
      else { LoadSlabEdge<T, TILE_N, TILE_K, PIECES_B, VL, B_KC>(b, p.b_ld, n0, slab * TILE_K, p.n, tid, b_regs); }
    };
    auto store = [&](const int buffer) {
      StoreSlab<T, TILE_M, TILE_K, PITCH_M, PIECES_A, VL, A_KC>(a_tiles + buffer * TILE_K * PITCH_M, tid, a_regs);
      StoreSlab<T, TILE_N, TILE_K, PITCH_N, PIECES_B, VL, B_KC>(b_tiles + buffer * TILE_K * PITCH_N, tid, b_regs);
    };
    auto multiply = [&](const int buffer) {
      const T* a_tile = a_tiles + buffer * TILE_K * PITCH_M + a_read;
      const T* b_tile = b_tiles + buffer * TILE_K * PITCH_N + b_read;
#pragma unroll
      for (int ks = 0; ks < TILE_K / KP; ++ks) {
        const int k = ks * KP + lane_g;
        VM av;
        if constexpr (M_INTERLEAVED) {
          av = *reinterpret_cast<const VM*>(&a_tile[k * PITCH_M]);
        } else {
#pragma unroll
          for (int i = 0; i < FM; ++i) { av = VecWith<VM, T, FM>(av, i, a_tile[k * PITCH_M + i * MF]); }
        }
        const VN bv = *reinterpret_cast<const VN*>(&b_tile[k * PITCH_N]);
#pragma unroll
        for (int i = 0; i < FM; ++i) {
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            acc[i][j] = Traits::Mfma(VecGet<VN, T, FN>(bv, j), VecGet<VM, T, FM>(av, i), acc[i][j]);
          }
        }
      }
    };

    // Software-pipelined walk over the full slabs.
    const int fast_slabs = full_slabs;
    if (a_full && b_full && fast_slabs > 0) {
      // Interior tiles: explicit schedule, so that the matrix pipe never waits at a slab boundary even
      // with one wavefront per SIMD. Per k-step: LDS reads of the fragments of the NEXT k-step (other
      // register set), the FM x FN MFMAs of this k-step, then a share of the data movement for the
      // coming slabs. An x-contiguous aligned operand goes global -> LDS directly (slab t+1, issued in
      // the first k-step of slab t); any other operand is staged through registers ("store staged slab
      // t+1 into the other LDS buffer, refill the staging registers with slab t+2"). One barrier per
      // slab, before its last k-step: by then every wavefront has finished its reads of the current
      // buffer and its writes to the other one, so the last k-step already fetches the first fragments
      // of slab t+1.
      constexpr int KSTEPS = TILE_K / KP;
      static_assert(KSTEPS % 2 == 0, "fragment register sets alternate per k-step");
      constexpr bool A_DIRECT = !A_KC && ALIGNED && !CLBH_EXP_NO_DIRECT, B_DIRECT = !B_KC && ALIGNED && !CLBH_EXP_NO_DIRECT;
      using LA = SlabLayout<T, TILE_M, TILE_K, A_DIRECT>;
      using LB = SlabLayout<T, TILE_N, TILE_K, B_DIRECT>;
      static_assert(2 * (LA::ELEMS + LB::ELEMS) <= Config::LDS_ELEMS, "LDS allocation covers both layouts");
      constexpr int STAGED_A = A_DIRECT ? 0 : PIECES_A, STAGED_B = B_DIRECT ? 0 : PIECES_B;
      constexpr int STAGED = STAGED_A + STAGED_B;
      constexpr int SLOTS = KSTEPS - 1;
      constexpr int PER_SLOT = (STAGED + SLOTS - 1) / SLOTS;
      T* a_stages = lds;                        // [2][LA::ELEMS]
      T* b_stages = lds + 2 * LA::ELEMS;        // [2][LB::ELEMS]
      const int wave_u = __builtin_amdgcn_readfirstlane(wave);
      using VP = typename VecType<T, VL>::type;
      VP a_stage[STAGED_A > 0 ? STAGED_A : 1], b_stage[STAGED_B > 0 ? STAGED_B : 1];
      const unsigned int a_lane_bytes = PieceLaneBytes<T, TILE_M, TILE_K, VL, A_KC>(p.a_ld, tid);
      const unsigned int b_lane_bytes = PieceLaneBytes<T, TILE_N, TILE_K, VL, B_KC>(p.b_ld, tid);
      const T* a_tile0 = a + (A_KC ? m0 * p.a_ld : static_cast<long long>(m0));  // element (m0, k = 0), uniform
      const T* b_tile0 = b + (B_KC ? n0 * p.b_ld : static_cast<long long>(n0));
      auto a_slab = [&](const int k0) { return a_tile0 + (A_KC ? static_cast<long long>(k0) : k0 * p.a_ld); };
      auto b_slab = [&](const int k0) { return b_tile0 + (B_KC ? static_cast<long long>(k0) : k0 * p.b_ld); };
      auto load_piece = [&](const int piece, const int k0) {
        if (piece < STAGED_A) { a_stage[piece] = LoadPiece<T, TILE_M, TILE_K, VL, A_KC>(a_slab(k0), p.a_ld, a_lane_bytes, piece); }
        else { b_stage[piece - STAGED_A] = LoadPiece<T, TILE_N, TILE_K, VL, B_KC>(b_slab(k0), p.b_ld, b_lane_bytes, piece - STAGED_A); }
      };
      auto store_piece = [&](const int piece, T* a_dst, T* b_dst) {
        if (piece < STAGED_A) { StorePiece<T, TILE_M, TILE_K, LA::GROUP_PITCH, VL, A_KC>(a_dst, tid, piece, a_stage[piece]); }
        else { StorePiece<T, TILE_N, TILE_K, LB::GROUP_PITCH, VL, B_KC>(b_dst, tid, piece - STAGED_A, b_stage[piece - STAGED_A]); }
      };
      auto direct_loads = [&](const int k0, T* a_dst, T* b_dst) {
        if constexpr (A_DIRECT) {
#pragma unroll
          for (int round = 0; round < LA::LOADS_PER_WAVE; ++round) { DirectLoad<T, TILE_M, TILE_K>(a_slab(k0), p.a_ld, a_dst, wave_u, lane, round); }
        }
        if constexpr (B_DIRECT) {
#pragma unroll
          for (int round = 0; round < LB::LOADS_PER_WAVE; ++round) { DirectLoad<T, TILE_N, TILE_K>(b_slab(k0), p.b_ld, b_dst, wave_u, lane, round); }
        }
      };
      const int a_lane_row = LA::Row(lane_g) + a_read, b_lane_row = LB::Row(lane_g) + b_read;
      auto read_a = [&](const T* stage, const int ks) {
        const T* src = stage + LA::Row(ks * KP) + a_lane_row;
        VM av;
        if constexpr (M_INTERLEAVED) {
          av = *reinterpret_cast<const VM*>(src);
        } else {
#pragma unroll
          for (int i = 0; i < FM; ++i) { av = VecWith<VM, T, FM>(av, i, src[i * MF]); }
        }
        return av;
      };
      auto read_b = [&](const T* stage, const int ks) {
        return *reinterpret_cast<const VN*>(stage + LB::Row(ks * KP) + b_lane_row);
      };
      static_assert((KP % LA::R == 0 || LA::R % KP == 0) && (KP % LB::R == 0 || LB::R % KP == 0), "row offsets add up");
      direct_loads(0, a_stages, b_stages);
#pragma unroll
      for (int piece = 0; piece < STAGED; ++piece) { load_piece(piece, 0); }
#pragma unroll
      for (int piece = 0; piece < STAGED; ++piece) { store_piece(piece, a_stages, b_stages); }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (fast_slabs > 1) {
#pragma unroll
        for (int piece = 0; piece < STAGED; ++piece) { load_piece(piece, TILE_K); }
      }
      __syncthreads();
      VM av[2];
      VN bv[2];
      av[0] = read_a(a_stages, 0);
      bv[0] = read_b(b_stages, 0);
      auto slab_body = [&](const int slab, auto store_tag, auto load_tag) {
        constexpr bool STORE = decltype(store_tag)::value, LOAD = decltype(load_tag)::value;
        const int cur = slab & 1;
        const T* a_cur = a_stages + cur * LA::ELEMS;
        const T* b_cur = b_stages + cur * LB::ELEMS;
        T* a_nxt = a_stages + (cur ^ 1) * LA::ELEMS;
        T* b_nxt = b_stages + (cur ^ 1) * LB::ELEMS;
        const int k_load = (slab + 2) * TILE_K;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const int set = ks % 2;
          if (ks + 1 < KSTEPS) {
            av[set ^ 1] = read_a(a_cur, ks + 1);
            bv[set ^ 1] = read_b(b_cur, ks + 1);
          } else {
            av[set ^ 1] = read_a(a_nxt, 0);
            bv[set ^ 1] = read_b(b_nxt, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int i = 0; i < FM; ++i) {
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              acc[i][j] = Traits::Mfma(VecGet<VN, T, FN>(bv[set], j), VecGet<VM, T, FM>(av[set], i), acc[i][j]);
            }
          }
          // the other buffer is free since the barrier of the previous slab
          if (ks == 0 && STORE) { direct_loads((slab + 1) * TILE_K, a_nxt, b_nxt); }
          if (ks < KSTEPS - 1) {
#pragma unroll
            for (int u = 0; u < PER_SLOT; ++u) {
              const int piece = ks * PER_SLOT + u;
              if (piece < STAGED) {
                if (STORE) { store_piece(piece, a_nxt, b_nxt); }
                if (LOAD) { load_piece(piece, k_load); }
              }
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          if (ks == KSTEPS - 2) {
            // direct loads of this slab are older than its register loads: all but those must have landed
            if ((A_DIRECT || B_DIRECT) && STORE) {
              if (LOAD && STAGED > 0) { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(STAGED) : "memory"); }
              else { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
            }
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
          }
        }
      };
      int slab = 0;
      for (; slab + 2 < fast_slabs; ++slab) { slab_body(slab, std::true_type{}, std::true_type{}); }
      if (slab + 1 < fast_slabs) { slab_body(slab, std::true_type{}, std::false_type{}); ++slab; }
      slab_body(slab, std::false_type{}, std::false_type{});
      __syncthreads();
    } else if (fast_slabs > 0) {
      // Edge tiles: same double buffering, loads predicated along x, order left to the compiler.
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
    // The K tail: checked, unpipelined.
    for (int slab = fast_slabs; slab < slabs; ++slab) {
      FillSlabChecked<T, TILE_M, TILE_K, PITCH_M, A_KC>(a_tiles, a, p.a_ld, m0, slab * TILE_K, p.m, k_len, tid);
      FillSlabChecked<T, TILE_N, TILE_K, PITCH_N, B_KC>(b_tiles, b, p.b_ld, n0, slab * TILE_K, p.n, k_len, tid);
      __syncthreads();
      multiply(0);
      __syncthreads();
    }

    // Epilogue. Lane owns m = m_base + i (i < FM); accumulator element r of block (i, j) is the
    // column n = n_base + FN * Row(r) + j.
    const int m_base = m0 + a_read;
    const int n_base = n0 + wave_n * (FN * MF);
    constexpr int M_STEP = M_INTERLEAVED ? 1 : MF;  // distance in m between the lane's accumulator blocks
    const bool vector_store = M_INTERLEAVED && c_aligned && (FM > 1) && (m_base + FM <= p.m);
#pragma unroll
    for (int j = 0; j < FN; ++j) {
#pragma unroll
      for (int r = 0; r < ACC; ++r) {
        const int n = n_base + FN * Traits::Row(r, lane_g) + j;
        if (n >= p.n) { continue; }
        T* dst = c + n * c_ld + m_base;
        if (vector_store) {
          VM out;
          if (beta == T(0)) {
#pragma unroll
            for (int i = 0; i < FM; ++i) { out = VecWith<VM, T, FM>(out, i, alpha * acc[i][j][r]); }
          } else {
            const VM old = *reinterpret_cast<const VM*>(dst);
#pragma unroll
            for (int i = 0; i < FM; ++i) {
              out = VecWith<VM, T, FM>(out, i, alpha * acc[i][j][r] + beta * VecGet<VM, T, FM>(old, i));
            }
          }
          *reinterpret_cast<VM*>(dst) = out;
        } else {
#pragma unroll
          for (int i = 0; i < FM; ++i) {
            if (m_base + i * M_STEP < p.m) { StoreResult<T, T>(dst, i * M_STEP, acc[i][j][r], alpha, beta); }
          }
        }
      }
    }
  }
}

// Second pass of a split-K launch: C = alpha * (sum of the workspace slabs) + beta * C.
template <typename T>
__global__ __launch_bounds__(256) void GemmSplitReduceKernel(const T* __restrict__ workspace, const int splits,
                                                             const int split_ld, T* __restrict__ c, const long long c_ld,
                                                             const int m, const int n, const T alpha, const T beta) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int j = blockIdx.y;
  if (i >= m) { return; }
  const long long slab = static_cast<long long>(split_ld) * n;
  const T* src = workspace + static_cast<long long>(j) * split_ld + i;
  T sum = T(0);
  for (int s = 0; s < splits; ++s) { sum += src[s * slab]; }
  StoreResult<T, T>(c, j * c_ld + i, sum, alpha, beta);
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_MFMA_HPP_
