// =================================================================================================
// Persistent fp32 / fp64 MFMA GEMM kernel for launches of MANY tiles with a SHORT K walk (8191 x 8191 x 127, batches
// of mid-sized matrices). Such a launch streams C: every tile reads and writes its piece of C once and multiplies only
// a few slabs in between, so with one work-group per tile (kernels/gemm_mfma.hpp) the per-tile costs that nothing
// overlaps - dispatch of the work-group, the first slab's way from memory, the read of the old C, the stores - take as
// long as the products (measured at 8191 x 8191 x k: 1.0 us per unit of k plus 130 us).
//
// Here a work-group stays on its CU and walks a sequence of tiles (items); the slabs of all its items form ONE stream
// through the ring of LDS buffers of gemm_mfma.hpp: the first slabs of the next item are requested under the last
// products of the current one, the old C of an item is fetched two slabs before its epilogue, and the stores of an
// item drain under the products of the next. Operand handling (direct global -> LDS loads of x-contiguous operands,
// register-staged k-contiguous ones, range-checked resources for edges and the K tail), fragment layout and MFMA
// schedule are those of GemmMfmaKernel (reference counterpart: the same Xgemm / XgemmDirect kernels,
// src/kernels/level3/xgemm_part1-4.opencl, xgemm_direct_part1-3.opencl).
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_STREAM_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_STREAM_HPP_

#include "kernels/gemm_mfma.hpp"

namespace clbh {

constexpr int kStreamOutside = 0x7fffff00;  // byte count of the view of a tile's C, and the offset of a store that is to move nothing

// USE_C: the old C is read (some beta is not zero). Needs at least four slabs per item (k > 3 * TILE_K) and tiles whose
// accumulators are few enough for a second register set of the same size (the old C).
template <typename T, typename Config, bool A_KC, bool B_KC, bool USE_C>
__global__ __launch_bounds__(kMfmaThreads, Config::MIN_WAVES) void GemmStreamKernel(const GemmArgs<T> p, const int tiles_m,
                                                                                  const int tiles_n, const int items) {
  using Traits = typename Config::Traits;
  using Acc = typename Traits::Acc;
  constexpr int MF = Traits::MF, KP = Traits::KP, ACC = Traits::ACC;
  constexpr int TILE_M = Config::TILE_M, TILE_N = Config::TILE_N, TILE_K = Config::TILE_K;
  constexpr int FM = Config::FM, FN = Config::FN, VEC = Config::VEC;
  constexpr bool A_DIRECT = !A_KC, B_DIRECT = !B_KC;
  using LA = SlabLayout<T, TILE_M, TILE_K, A_DIRECT, 16>;
  using LB = SlabLayout<T, TILE_N, TILE_K, B_DIRECT, 16>;
  using PA = StagedPieces<TILE_M, TILE_K, VEC>;
  using PB = StagedPieces<TILE_N, TILE_K, VEC>;
  constexpr int STAGES = Config::STAGES;
  static_assert(STAGES == 3, "ring of three: the slab two ahead is requested under the current one");
  static_assert(STAGES * (LA::ELEMS + LB::ELEMS) <= Config::LDS_ELEMS, "LDS allocation covers the layouts");
  constexpr int STAGED_A = A_DIRECT ? 0 : PA::PIECES, STAGED_B = B_DIRECT ? 0 : PB::PIECES;
  constexpr int STAGED = STAGED_A + STAGED_B;
  constexpr int KSTEPS = TILE_K / KP;
  static_assert(KSTEPS % 2 == 0, "fragment register sets alternate per k-step");
  constexpr int SLOTS = KSTEPS - 1;
  constexpr int PER_SLOT = (STAGED + SLOTS - 1) / SLOTS;
  constexpr int DIRECT_A = A_DIRECT ? LA::LOADS_PER_WAVE : 0, DIRECT_B = B_DIRECT ? LB::LOADS_PER_WAVE : 0;
  constexpr int DIRECT = DIRECT_A + DIRECT_B;
  constexpr int DIRECT_PER_SLOT = (DIRECT + SLOTS - 1) / SLOTS;
  constexpr int REQUESTS = DIRECT + STAGED;   // vector memory loads per thread and slab
  constexpr int OLD_C = FN * ACC;             // loads of old C per thread and item (FM consecutive elements each)
  static_assert(OLD_C * FM * sizeof(T) <= 256 && REQUESTS + OLD_C < 64, "the old C of an item waits in registers");
  using VM = typename VecType<T, FM>::type;
  using VN = typename VecType<T, FN>::type;
  using VP = typename VecType<T, VEC>::type;
  using KernelTag = std::tuple<Config, std::integral_constant<int, 64 + (A_KC ? 4 : 0) | (B_KC ? 2 : 0) | (USE_C ? 1 : 0)>>;

  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  T* a_stages = lds;                       // [STAGES][LA::ELEMS]
  T* b_stages = lds + STAGES * LA::ELEMS;  // [STAGES][LB::ELEMS]

  const int tid = threadIdx.x;
  const int lane = tid % 64, wave = tid / 64;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wave_m = wave % Config::WM, wave_n = wave / Config::WM;
  const int lane_x = lane % MF, lane_g = lane / MF;
  const int a_read = wave_m * (FM * MF) + lane_x * FM;  // the lane owns FM consecutive m
  const int b_read = wave_n * (FN * MF) + lane_x * FN;
  const int a_lane_row = LA::Row(lane_g) + a_read, b_lane_row = LB::Row(lane_g) + b_read;
  const int a_lane_bytes = A_DIRECT ? DirectLaneBytes<T, TILE_M, TILE_K, 16>(p.a_ld, lane)
                                    : static_cast<int>((PA::Line(tid) * p.a_ld + PA::K(tid)) * static_cast<long long>(sizeof(T)));
  const int b_lane_bytes = B_DIRECT ? DirectLaneBytes<T, TILE_N, TILE_K, 16>(p.b_ld, lane)
                                    : static_cast<int>((PB::Line(tid) * p.b_ld + PB::K(tid)) * static_cast<long long>(sizeof(T)));

  const int k_len = p.k;
  const int slabs = (k_len + TILE_K - 1) / TILE_K;  // >= 4 (the host's condition for this kernel)
  const int tiles = tiles_m * tiles_n;

  // One item: a tile of one matrix of the batch. Everything here is uniform over the work-group. An index beyond the
  // last item gives an item whose operands are empty (its requests move nothing and deliver zeros).
  struct Item {
    const T* a_tile0;  // element (m0, k = 0)
    const T* b_tile0;
    const T* a_end;    // behind the last element of the operand
    const T* b_end;
    T* c;
    T alpha, beta;
    int m0, n0;
  };
  auto make_item = [&](const int index) {
    Item item;
    if (index >= items) {
      item.a_tile0 = item.a_end = static_cast<const T*>(p.a);
      item.b_tile0 = item.b_end = static_cast<const T*>(p.b);
      item.c = static_cast<T*>(p.c);
      item.alpha = item.beta = T(0);
      item.m0 = p.m;
      item.n0 = p.n;
      return item;
    }
    const int batch = index / tiles;
    int tile_m, tile_n;
    TileOfBlock(index - batch * tiles, tiles, tiles_m, tiles_n, tile_m, tile_n);
    const T* a;
    const T* b;
    ResolveBatch<T, T>(p, batch, a, b, item.c, item.alpha, item.beta);
    item.m0 = tile_m * TILE_M;
    item.n0 = tile_n * TILE_N;
    item.a_tile0 = a + (A_KC ? item.m0 * p.a_ld : static_cast<long long>(item.m0));
    item.b_tile0 = b + (B_KC ? item.n0 * p.b_ld : static_cast<long long>(item.n0));
    item.a_end = a + (A_KC ? (p.m - 1) * p.a_ld + k_len : (k_len - 1) * p.a_ld + p.m);
    item.b_end = b + (B_KC ? (p.n - 1) * p.b_ld + k_len : (k_len - 1) * p.b_ld + p.n);
    return item;
  };
  auto a_slab = [&](const Item& item, const int k0) { return item.a_tile0 + (A_KC ? static_cast<long long>(k0) : k0 * p.a_ld); };
  auto b_slab = [&](const Item& item, const int k0) { return item.b_tile0 + (B_KC ? static_cast<long long>(k0) : k0 * p.b_ld); };

  VP a_stage[STAGED_A > 0 ? STAGED_A : 1], b_stage[STAGED_B > 0 ? STAGED_B : 1];
  auto load_piece = [&](const int piece, const Item& item, const int k0) {
    if (piece < STAGED_A) { a_stage[piece] = LoadPiece<T, TILE_M, TILE_K, VEC, true>(a_slab(item, k0), item.a_end, p.a_ld, a_lane_bytes, piece); }
    else { b_stage[piece - STAGED_A] = LoadPiece<T, TILE_N, TILE_K, VEC, true>(b_slab(item, k0), item.b_end, p.b_ld, b_lane_bytes, piece - STAGED_A); }
  };
  auto store_piece = [&](const int piece, T* a_dst, T* b_dst, const int k0) {
    if (piece < STAGED_A) { StorePiece<T, TILE_M, TILE_K, LA::GROUP_PITCH, VEC, true>(a_dst, tid, piece, a_stage[piece], k_len - k0); }
    else { StorePiece<T, TILE_N, TILE_K, LB::GROUP_PITCH, VEC, true>(b_dst, tid, piece - STAGED_A, b_stage[piece - STAGED_A], k_len - k0); }
  };
  auto direct_load = [&](const int load, const Item& item, const int k0, T* a_dst, T* b_dst) {
    if constexpr (DIRECT_A > 0) {
      if (load < DIRECT_A) { DirectLoad<T, TILE_M, TILE_K, 16, true, KernelTag>(a_slab(item, k0), item.a_end, p.a_ld, a_dst, wave_u, a_lane_bytes, load); }
    }
    if constexpr (DIRECT_B > 0) {
      if (load >= DIRECT_A) { DirectLoad<T, TILE_N, TILE_K, 16, true, KernelTag>(b_slab(item, k0), item.b_end, p.b_ld, b_dst, wave_u, b_lane_bytes, load - DIRECT_A); }
    }
  };
  auto read_a = [&](const T* stage, const int ks) { return *reinterpret_cast<const VM*>(stage + LA::Row(ks * KP) + a_lane_row); };
  auto read_b = [&](const T* stage, const int ks) { return *reinterpret_cast<const VN*>(stage + LB::Row(ks * KP) + b_lane_row); };

  int index = blockIdx.x;
  if (index >= items) { return; }
  Item current = make_item(index);
  Item next = make_item(index + gridDim.x);

  // Prologue of the stream: slab 0 of the first item lands in buffer 0, slab 1 is requested.
#pragma unroll
  for (int load = 0; load < DIRECT; ++load) { direct_load(load, current, 0, a_stages, b_stages); }
#pragma unroll
  for (int piece = 0; piece < STAGED; ++piece) { load_piece(piece, current, 0); }
#pragma unroll
  for (int piece = 0; piece < STAGED; ++piece) { store_piece(piece, a_stages, b_stages, 0); }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int load = 0; load < DIRECT; ++load) { direct_load(load, current, TILE_K, a_stages + LA::ELEMS, b_stages + LB::ELEMS); }
#pragma unroll
  for (int piece = 0; piece < STAGED; ++piece) { load_piece(piece, current, TILE_K); }
  __syncthreads();
  VM av[2];
  VN bv[2];
  av[0] = read_a(a_stages, 0);
  bv[0] = read_b(b_stages, 0);
  int cur = 0;  // ring position of the current slab; the next one is in the next buffer, the one after goes into the one before

  Acc acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
#pragma unroll
    for (int j = 0; j < FN; ++j) { acc[i][j] = Traits::Zero(); }
  }
  typedef T VMG __attribute__((ext_vector_type(FM > 1 ? FM : 2), aligned(sizeof(T))));  // FM consecutive m of one column of C
  using OldC = typename std::conditional<(FM > 1), VMG, T>::type;
  OldC old_c[USE_C ? OLD_C : 1];

  // Position of the lane's accumulators in C: m = m_base + i (i < FM); column n0 + lane_n + u of block j and accumulator
  // element r, with u = FN * Row(r, 0) + j known at compile time. The C of an item is addressed through a range-checked
  // view that starts at the item's first column: the lane's byte offset holds its own column and row - or lies outside
  // the view for a piece that is not to move, which then touches no memory (a load delivers zero) - and the u columns
  // travel as the access's uniform offset, so a piece costs a comparison and a select, not a 64-bit address.
  auto m_base = [&](const Item& item) { return item.m0 + a_read; };
  const int c_ld = static_cast<int>(p.c_ld);  // (the host admits leading dimensions whose tile offsets fit 31 bits)
  const int lane_n = wave_n * (FN * MF) + FN * Traits::Row(0, lane_g);
  const int lane_columns = lane_n * c_ld;
  auto c_view = [&](const Item& item) {
    return __builtin_amdgcn_make_buffer_rsrc(item.c + static_cast<long long>(item.n0) * p.c_ld, 0, kStreamOutside, kRawBufferFlags);
  };
  auto columns_of = [](const int j, const int r) { return FN * Traits::Row(r, 0) + j; };
  // the lane's offset for piece (j, r): `lane_offset` while the piece's column is one of the `columns_left` of the matrix
  auto piece_offset = [&](const int lane_offset, const int columns, const int columns_left) {
    int offset = (lane_n + columns < columns_left) ? lane_offset : kStreamOutside;
    asm volatile("" : "+v"(offset));  // (a plain value: no branch around the access)
    return offset;
  };
  // The old C of an item: one load per column piece, none of them under a branch (the waits below count them). A lane
  // whose piece would reach beyond the last row reads the piece FM rows up from the last row instead (the epilogue
  // picks its elements out of it).
  auto fetch_old_c = [&](const Item& item) {
    if constexpr (USE_C) {
      const auto view = c_view(item);
      const int lane_offset = static_cast<int>((lane_columns + max(min(m_base(item), p.m - FM), 0)) * sizeof(T));
      const int columns_left = p.n - item.n0;
#pragma unroll
      for (int j = 0; j < FN; ++j) {
#pragma unroll
        for (int r = 0; r < ACC; ++r) {
          old_c[j * ACC + r] = __builtin_bit_cast(OldC, BufferLoad<T, FM>(view, piece_offset(lane_offset, columns_of(j, r), columns_left),
                                                                        static_cast<int>(columns_of(j, r) * c_ld * sizeof(T))));
        }
      }
    }
  };

  // One slab of the stream: the products of the current slab of `current`; the slab after it (store_k0, of this item or
  // the next) moves from the staging registers into the next buffer, the slab two ahead (`load_item`, load_k0) is
  // requested. FETCH: the old C of `current` is asked for, behind this slab's wait. EXTRA: vector memory operations,
  // beyond this slab's own requests, that were issued behind the requests this slab's wait is about and may stay in
  // flight - the loads of old C in the slab after a FETCH slab, the stores of the previous item in an item's first slab.
  auto slab_body = [&](const int store_k0, const Item& load_item, const int load_k0, auto fetch_tag, auto extra_tag) {
    constexpr bool FETCH = decltype(fetch_tag)::value;
    constexpr int EXTRA = decltype(extra_tag)::value;
    const int nxt = (cur == STAGES - 1) ? 0 : cur + 1, prv = (cur == 0) ? STAGES - 1 : cur - 1;
    const T* a_cur = a_stages + cur * LA::ELEMS;
    const T* b_cur = b_stages + cur * LB::ELEMS;
    T* a_nxt = a_stages + nxt * LA::ELEMS;
    T* b_nxt = b_stages + nxt * LB::ELEMS;
    T* a_prv = a_stages + prv * LA::ELEMS;
    T* b_prv = b_stages + prv * LB::ELEMS;
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
      if (ks < KSTEPS - 1) {
#pragma unroll
        for (int u = 0; u < PER_SLOT; ++u) {
          const int piece = ks * PER_SLOT + u;
          if (piece < STAGED) {
            store_piece(piece, a_nxt, b_nxt, store_k0);
            load_piece(piece, load_item, load_k0);
          }
        }
#pragma unroll
        for (int u = 0; u < DIRECT_PER_SLOT; ++u) {
          const int load = ks * DIRECT_PER_SLOT + u;
          if (load < DIRECT) { direct_load(load, load_item, load_k0, a_prv, b_prv); }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (ks == KSTEPS - 2) {
        // The next slab must have landed for everybody: what was requested before this slab has to be complete; this
        // slab's own requests may stay in flight (loads complete in order), and so may EXTRA younger operations.
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(REQUESTS + EXTRA) : "memory");
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        // The old C is asked for behind this wait: the next slab's wait still lets these loads fly (they are younger
        // than the requests it needs), the one after it covers them - two slabs for the way from memory.
        if constexpr (FETCH) { fetch_old_c(current); }
      }
    }
    cur = nxt;
  };
  using Fetch = std::true_type;
  using NoFetch = std::false_type;
  using NoExtra = std::integral_constant<int, 0>;
  using OldCInFlight = std::integral_constant<int, USE_C ? OLD_C : 0>;
  constexpr int INTERIOR_STORES = OLD_C;  // store instructions of every epilogue (a tile cut by the last row issues more)
  using StoresInFlight = std::integral_constant<int, INTERIOR_STORES>;

  // What the prologue requested has landed (a wait the compiler knows of, unlike the waits written as text: it counts
  // the operations in flight to place its own waits for the staging registers, and where the start of the stream joins
  // the loop it would otherwise have to assume the smallest count on either path).
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), the other counters at their maximum
  while (true) {
    // The slabs of the item (at least four). Every slab requests the slab two ahead: of the same item, then the first two
    // of the next item. The old C is fetched under the third slab from the end. The first slab's wait lets the stores of
    // the previous item's epilogue fly on (the first item has none, and nothing its wait is about is outstanding either).
    slab_body(TILE_K, current, 2 * TILE_K, NoFetch{}, StoresInFlight{});
    for (int s = 1; s + 3 < slabs; ++s) { slab_body((s + 1) * TILE_K, current, (s + 2) * TILE_K, NoFetch{}, NoExtra{}); }
    slab_body((slabs - 2) * TILE_K, current, (slabs - 1) * TILE_K, Fetch{}, NoExtra{});
    slab_body((slabs - 1) * TILE_K, next, 0, NoFetch{}, OldCInFlight{});
    slab_body(0, next, TILE_K, NoFetch{}, NoExtra{});

    // Epilogue of the item; its stores drain under the products of the next item. Every tile issues the same store
    // instructions, none of them under a branch, through a range-checked view of the tile's part of C: a lane whose piece
    // is not wholly inside the matrix stores at an offset outside that view, which moves nothing. So the number of stores
    // in flight behind an epilogue is fixed (INTERIOR_STORES, more for the rare tile below), and the waits of the next
    // item's first slab - the one written here and the ones the compiler places for the staging registers - can let
    // them fly on. (Stores under bounds tests would come in a number nobody knows: where such a path joins the loop, the
    // compiler's waits have to assume that no store was issued and drain the memory pipe at every item.)
    {
      const int mb = m_base(current);
      const auto view = c_view(current);
      const int columns_left = p.n - current.n0;
      const int row_offset = static_cast<int>((lane_columns + mb) * sizeof(T));
      const int whole_offset = (mb + FM <= p.m) ? row_offset : kStreamOutside;
#pragma unroll
      for (int j = 0; j < FN; ++j) {
#pragma unroll
        for (int r = 0; r < ACC; ++r) {
          OldC out;
#pragma unroll
          for (int i = 0; i < FM; ++i) {
            T value = current.alpha * acc[i][j][r];
            if constexpr (USE_C) {
              if (current.beta != T(0)) {
                value = Combine(current.alpha, acc[i][j][r], current.beta, VecGet<OldC, T, FM>(old_c[j * ACC + r], i));
              }
            }
            out = VecWith<OldC, T, FM>(out, i, value);
          }
          BufferStore<T, FM>(out, view, piece_offset(whole_offset, columns_of(j, r), columns_left),
                             static_cast<int>(columns_of(j, r) * c_ld * sizeof(T)));
        }
      }
      if (FM > 1 && current.m0 + TILE_M > p.m) {
        // A tile that the last row of the matrix cuts: a piece that straddles the edge stores its elements one by one.
        // Its old C has come with the others - fetch_old_c moved the lane's piece back into the matrix, so the lane's
        // element i is element i + shift of the piece it holds, whenever that element exists.
        const int shift = mb - max(min(mb, p.m - FM), 0);
        const int straddling_offset = (mb < p.m && mb + FM > p.m) ? row_offset : kStreamOutside;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
          for (int r = 0; r < ACC; ++r) {
            const int offset = piece_offset(straddling_offset, columns_of(j, r), columns_left);
#pragma unroll
            for (int i = 0; i < FM - 1; ++i) {  // (the last element of a straddling piece is never inside)
              T value = current.alpha * acc[i][j][r];
              if constexpr (USE_C) {
                if (current.beta != T(0)) {
                  T old = VecGet<OldC, T, FM>(old_c[j * ACC + r], FM - 1);
#pragma unroll
                  for (int e = 0; e < FM - 1; ++e) { if (i + shift == e) { old = VecGet<OldC, T, FM>(old_c[j * ACC + r], e); } }
                  value = Combine(current.alpha, acc[i][j][r], current.beta, old);
                }
              }
              int element = (mb + i < p.m) ? offset + i * static_cast<int>(sizeof(T)) : kStreamOutside;
              asm volatile("" : "+v"(element));
              BufferStore<T, 1>(value, view, element, static_cast<int>(columns_of(j, r) * c_ld * sizeof(T)));
            }
          }
        }
      }
#pragma unroll
      for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int j = 0; j < FN; ++j) { acc[i][j] = Traits::Zero(); }
      }
    }
    index += gridDim.x;
    if (index >= items) { break; }
    current = next;
    next = make_item(index + gridDim.x);
  }
  // the requests made for items beyond the last one moved nothing; they must have retired before the LDS is given back
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_STREAM_HPP_
