// bf16 GEMM on the gfx950 matrix cores: C[M,N] = A . B with fp32 accumulation, bf16 store.
//
// Roofline: MFMA (v_mfma_f32_32x32x16_bf16, 32768 FLOP per wave instruction).  Algorithmic
// work per launch is 2*M*N*K FLOP.
//
// Structure ("8-wave ping-pong")
//   * A workgroup of 8 waves owns a 256 x 256 tile of C and walks K in steps of 64.  Each wave
//     owns 128 x 64 of the tile as 4 x 2 MFMA tiles of 32x32 held in registers for the whole
//     K loop.
//   * The waves form two groups of four, one wave of each group per SIMD.  Time is cut into
//     half-periods by workgroup barriers.  In every half-period one group only issues MFMAs
//     (all 32 of a K-step, operands already in registers) while the other group only moves
//     data: it issues the global loads of one operand tile of K-step k+2 and reads its operand
//     fragments of the next K-step out of LDS.  Then the roles swap.  The matrix pipe of every
//     SIMD always has exactly one wave feeding it, and no wave ever waits on memory in the
//     middle of its MFMA burst.
//   * Global memory goes straight into LDS (global_load_lds_dwordx4): no staging registers, no
//     LDS store instructions.  The hardware places the 64 lanes of such a load contiguously in
//     LDS, so bank conflicts are avoided by an XOR swizzle applied on the *global* side — each
//     lane fetches the 16-byte chunk that belongs at its LDS slot.
//   * All 160 KB of LDS form a ring of five 32 KB slots, one operand tile (A or B of one
//     K-step) per slot: two slots are being consumed, three are being filled.  Group 1 requests
//     the A tiles (a flight window of three half-periods), group 0 the B tiles (two
//     half-periods), so the texture-address path sees an even 32 KB per half-period — half of
//     what it can carry — and every load has at least a full half-period to land after the
//     last request of its tile went out.  With only two 64 KB stages the loads of a whole
//     K-step had to be pushed out back to back and their tail had no time left.
//   * Loads are 16-byte vectors along whichever dimension is contiguous in memory.  An operand
//     whose contraction dimension is contiguous ("K-major") is fetched from LDS with
//     ds_read_b128; an operand whose contraction dimension is the row index ("transposed": the
//     weight in dgrad, both operands in wgrad) with the transposing LDS read
//     ds_read_b64_tr_b16.  No transposed copy of any operand is ever made.
//   * The MFMA is issued with the operands swapped (the B tile feeds the instruction's A
//     port), so a lane ends up with four consecutive N-columns of one C row and the epilogue
//     stores 8-byte bf16 quads contiguous along the row.
//   * Rows beyond the matrix edge are clamped to the last valid row instead of predicated: an
//     output element depends only on its own A row and B row, and out-of-range outputs are
//     never stored.  A contraction tail (K not a multiple of 64) is zeroed in LDS after its
//     tile has landed.
//   * Workgroup ids are remapped so that the tiles resident on one XCD (ids congruent mod 8)
//     form a compact band of C and share A/B panels in that XCD's L2.
//   * Split-K: when C has too few tiles to fill 256 CUs (weight gradients: a small N x K
//     output contracted over all tokens), the contraction is cut into up to 16 ranges, each
//     workgroup writes an fp32 partial tile into a caller-provided workspace, and a small
//     HBM-bound kernel sums the partials and rounds to bf16.
#include "kr_common.h"

namespace {

constexpr int BK = 64;
constexpr int BM = 256, BN = 256;
constexpr int TM = 4, TN = 2;  // 32x32 MFMA tiles per wave: 128 rows x 64 columns
constexpr int NTHREADS = 512;
constexpr int TILE = 256 * BK;  // elements of one operand tile (either layout)
constexpr int NSLOTS = 5;          // 5 x 32 KB = the whole 160 KB of LDS
constexpr int kXcds = 8;
constexpr int kGroupM = 4;

// ---- LDS layouts (element offsets inside one operand tile) ----------------------------------
// K-major tile [256 rows][64]: 128-byte rows, 16-byte chunk index XORed with (row>>1)&7.
__device__ __forceinline__ int kmajor_off(int row, int chunk) {
  return row * BK + ((chunk ^ ((row >> 1) & 7)) << 3);
}
// transposed tile [64 k-rows][256]: 512-byte rows, chunk index XORed with 4*(krow&3).
__device__ __forceinline__ int transp_off(int krow, int col) {
  return krow * 256 + ((((col >> 3) ^ ((krow & 3) << 2))) << 3) + (col & 7);
}

// ---- direct global -> LDS loads ---------------------------------------------------------------
// Issued through inline assembly on purpose.  A workgroup barrier is a release fence for LDS,
// and the compiler drains every LDS-direct load it knows of (vmcnt(0)) in front of one — which
// would empty the prefetch pipeline twice per K-step.  Written this way the loads are invisible
// to its wait-count bookkeeping; their completion is tracked by hand with explicit vmcnt waits
// placed before the barrier that publishes the data.  The loads have no register destination,
// so nothing can be clobbered behind the register allocator's back.
// base: wave-uniform global address; byte_off: this lane's unsigned 32-bit byte offset from it;
// lds_byte: wave-uniform LDS byte address of a 1-KiB block (lane p lands at +16p).
__device__ __forceinline__ void dma_b128(const void* base, uint32_t byte_off, uint32_t lds_byte) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_byte), "v"(byte_off), "s"(base)
               : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_addr(const bf16* p) {
  return (uint32_t)(uintptr_t)(KR_LDS const bf16*)p;
}

// ---- direct global -> LDS tile loads, issued by the 4 waves of the loading group -----------
// One wave-level load moves 1 KiB into LDS at [base + lane*16].  Block b of a K-major tile
// holds rows 8b..8b+7; block b of a transposed tile holds contraction rows 2b, 2b+1.
template <bool TRANSPOSED>
struct TileLoader {
  // K-major:    load i covers tile row r0 + 32*i (clamped to rmax), 16-byte chunk `chunk`
  // transposed: load i covers contraction row k0 + 8*i, column offset `chunk` (clamped)
  int r0, rmax, chunk;
  int64_t ld;
  __device__ __forceinline__ void init(int64_t ld_, int row0, int rows_total, int wave4, int lane) {
    ld = ld_;
    if (!TRANSPOSED) {
      const int row = 8 * wave4 + (lane >> 3);  // + 32*i; (row >> 1) & 7 does not depend on i
      chunk = ((lane & 7) ^ ((row >> 1) & 7)) * 8;
      r0 = row0 + row;
      rmax = rows_total - 1;
    } else {
      const int krow = 2 * wave4 + (lane >> 5);  // + 8*i; krow & 3 does not depend on i
      int c = row0 + ((lane & 31) ^ ((krow & 3) << 2)) * 8;
      chunk = c + 8 <= rows_total ? c : rows_total - 8;
      r0 = krow;
      rmax = 0;
    }
  }
  // k_left: contraction elements from this K-step's base to the end of the operand (>= 8).
  // A chunk that would start beyond it is redirected to a valid address; it is zeroed in LDS
  // afterwards, so what it fetches does not matter — only that the address is inside the matrix.
  __device__ __forceinline__ uint32_t goff(int i, int k_left) const {
    if (!TRANSPOSED) {
      int r = r0 + 32 * i;
      r = r < rmax ? r : rmax;
      const int kc = chunk + 8 <= k_left ? chunk : k_left - 8;
      return (uint32_t)(r * (int)ld + kc);
    }
    int kr = r0 + 8 * i;
    kr = kr < k_left ? kr : k_left - 1;
    return (uint32_t)(kr * (int)ld + chunk);
  }
  // contraction index (relative to the K-step) covered by load i of this lane
  __device__ __forceinline__ int k_of(int i, int wave4, int lane) const {
    if (!TRANSPOSED) {
      const int row = 8 * wave4 + (lane >> 3);
      return ((lane & 7) ^ ((row >> 1) & 7)) * 8;
    }
    return 2 * (wave4 + 4 * i) + (lane >> 5);
  }
  __device__ __forceinline__ void issue_one(const bf16* __restrict__ kbase, bf16* tile, int wave4,
                                            int k_left, int i) const {
    dma_b128(kbase, goff(i, k_left) * 2u, lds_addr(tile + (wave4 + 4 * i) * 512));
  }
  __device__ __forceinline__ void issue(const bf16* __restrict__ kbase, bf16* tile, int wave4,
                                        int k_left) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int b = wave4 + 4 * i;
      dma_b128(kbase, goff(i, k_left) * 2u, lds_addr(tile + b * 512));
    }
  }
  // zero this lane's chunks whose contraction index is >= k_valid (tile already landed)
  __device__ __forceinline__ void zero_tail(bf16* tile, int k_valid, int wave4, int lane) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int b = wave4 + 4 * i;
      if (k_of(i, wave4, lane) >= k_valid)
        *reinterpret_cast<bf16x8*>(tile + b * 512 + lane * 8) = zero8();
    }
  }
};

// ---- LDS -> MFMA operand fragments ----------------------------------------------------------
// Fragment (t, kk): lane gets tile row (row0 + 32*t + lane%32), k = 16*kk + 8*(lane/32) + 0..7.
// Per-lane base offsets are computed once; everything that varies inside the K loop is an
// instruction immediate.
template <bool TRANSPOSED, int NTILES>
struct FragReader {
  // K-major: one base per kk (the swizzle XOR depends on kk), tile index t is an immediate
  // transposed: one base per t (the XOR depends on the column), kk / half are immediates
  int base[TRANSPOSED ? NTILES : BK / 16];
  __device__ __forceinline__ void init(int row0, int lane) {
    if (!TRANSPOSED) {
      const int row = row0 + (lane & 31);
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) base[kk] = kmajor_off(row, 2 * kk + (lane >> 5));
    } else {
      const int p = lane & 15;
      const int krow = (lane >> 5) * 8 + (p >> 2);
#pragma unroll
      for (int t = 0; t < NTILES; ++t)
        base[t] = transp_off(krow, row0 + 32 * t + ((lane >> 4) & 1) * 16 + (p & 3) * 4);
    }
  }
  // LDS byte address of this lane's base n inside `tile`, made opaque so that the compiler adds
  // nothing but instruction immediates (all below 64 KiB) to it and keeps no per-slot copies.
  __device__ __forceinline__ uint32_t addr(const bf16* tile, int n) const {
    uint32_t v = (uint32_t)(uintptr_t)(KR_LDS const bf16*)tile + 2u * (uint32_t)base[n];
    asm volatile("" : "+v"(v));
    return v;
  }
  static constexpr int NBASE = TRANSPOSED ? NTILES : BK / 16;
  // a[]: addr(tile, n) for every base n
  __device__ __forceinline__ bf16x8 read(const uint32_t (&a)[NBASE], int t, int kk) const {
    if (!TRANSPOSED) {
      return *(KR_LDS const bf16x8*)(a[kk] + 2u * (uint32_t)(t * 32 * BK));
    } else {
      // Transposing read: within each group of 16 lanes, lane p supplies the address of 4
      // consecutive row-of-C elements in contraction row (p/4); it receives, for its own
      // row-of-C, the elements of the group's 4 contraction rows.
      const uint32_t a0 = a[t] + 2u * (uint32_t)(kk * 16 * 256);
      union {
        struct { s16x4 lo, hi; } s;
        bf16x8 v;
      } u;
      u.s.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a0));
      u.s.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a0 + 2u * 4 * 256));
      return u.v;
    }
  }
};

__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ void remap_block(int pid, int nblocks, int tiles_m, int tiles_n,
                                            int& tm, int& tn) {
  // ids congruent mod 8 run on the same XCD: give each XCD a contiguous range of tile ids
  const int q = nblocks / kXcds, r = nblocks % kXcds;
  const int xcd = pid % kXcds, local = pid / kXcds;
  const int lid = xcd * q + (xcd < r ? xcd : r) + local;
  // walk C in bands of kGroupM tile rows, column by column inside a band
  const int per_band = kGroupM * tiles_n;
  const int band = lid / per_band;
  const int first_m = band * kGroupM;
  const int band_rows = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
  const int in_band = lid % per_band;
  tm = first_m + in_band % band_rows;
  tn = in_band / band_rows;
}

template <bool A_T, bool B_T>
__global__ __launch_bounds__(NTHREADS) void gemm_kernel(const bf16* __restrict__ A, int lda,
                                                        const bf16* __restrict__ B, int ldb,
                                                        bf16* __restrict__ C, int ldc, int M,
                                                        int N, int K, int accumulate, int k_per,
                                                        int splits, float* __restrict__ partial) {
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int group = wave >> 2;  // 0: computes first and requests the B tiles, 1: the A tiles
  const int wave4 = wave & 3;
  const int wm = group, wn = wave4;  // wave tile: rows wm*128.., columns wn*64..
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int ntiles = tiles_m * tiles_n;
  const bool split_k = partial != nullptr;

  // Persistent workgroups: work item v = (output tile, split-K range); this workgroup takes
  // items blockIdx.x, blockIdx.x + gridDim.x, ...  The state below describes the current item.
  // (element offsets fit 32 bits: the host checks rows * ld < 2^31 and the workspace size)
  int m0, n0, nk, k_tail, kc = K, a_off = 0, b_off = 0, p_off = 0;
  auto select_item = [&](int v) {
    const int split = v / ntiles;
    int tile_m, tile_n;
    remap_block(v - split * ntiles, ntiles, tiles_m, tiles_n, tile_m, tile_n);
    m0 = tile_m * BM;
    n0 = tile_n * BN;
    if (split_k) {
      // split-K: contraction range [split*k_per, split*k_per + kc), fp32 partial tile out
      // (k_per is a multiple of 64)
      const int k0 = split * k_per;
      a_off = A_T ? k0 * lda : k0;
      b_off = B_T ? k0 * ldb : k0;
      kc = (K - k0) < k_per ? (K - k0) : k_per;
      p_off = split * M * N;
    }
    nk = (kc + BK - 1) / BK;
    k_tail = kc - (nk - 1) * BK;  // valid contraction rows of the last K-step (1..64)
  };

  f32x16 acc[TN][TM];
  bf16x8 af[BK / 16][TM], bfr[BK / 16][TN];

  // Per-lane fragment offsets are recomputed from an opaque copy of the lane id whenever
  // fragments are read (a handful of VALU instructions in the data-movement half-period)
  // instead of occupying eight registers through the MFMA phases.
  auto read_frags = [&](int t) {
    int lf = lane;
    asm volatile("" : "+v"(lf));
    FragReader<A_T, TM> fa;
    FragReader<B_T, TN> fb;
    fa.init(wm * TM * 32, lf);
    fb.init(wn * TN * 32, lf);
    const bf16* at = smem + ((2 * t) % NSLOTS) * TILE;
    const bf16* bt = smem + ((2 * t + 1) % NSLOTS) * TILE;
    uint32_t aa[fa.NBASE], ba[fb.NBASE];
#pragma unroll
    for (int n = 0; n < fa.NBASE; ++n) aa[n] = fa.addr(at, n);
#pragma unroll
    for (int n = 0; n < fb.NBASE; ++n) ba[n] = fb.addr(bt, n);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
#pragma unroll
      for (int i = 0; i < TM; ++i) af[kk][i] = fa.read(aa, i, kk);
#pragma unroll
      for (int j = 0; j < TN; ++j) bfr[kk][j] = fb.read(ba, j, kk);
    }
  };
  auto compute = [&]() {
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i)
          acc[j][i] =
              __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[kk][j], af[kk][i], acc[j][i], 0, 0, 0);
    __builtin_amdgcn_s_setprio(0);
  };

  // LDS is a ring of five 32 KB slots; operand tile x (0 = A, 1 = B) of K-step t lives in slot
  // (2t + x) mod 5.  Two slots hold the K-step being consumed, three are being filled.
  auto slot_of = [&](int t, int x) { return smem + ((2 * t + x) % NSLOTS) * TILE; };
  // Each group loads one operand: group 1 the A tiles, group 0 the B tiles, 8 loads per wave.
  // The per-lane load coordinates are recomputed from an opaque copy of the lane id every time:
  // keeping them alive across the MFMA phases would push the wave over its register budget.
  auto issue_mine = [&](int t) {
    int l2 = lane;
    asm volatile("" : "+v"(l2));
    if (group) {
      TileLoader<A_T> la;
      la.init(lda, m0, M, wave4, l2);
      la.issue(A + a_off + (int64_t)t * (A_T ? BK * lda : BK), slot_of(t, 0), wave4, kc - t * BK);
    } else {
      TileLoader<B_T> lb;
      lb.init(ldb, n0, N, wave4, l2);
      lb.issue(B + b_off + (int64_t)t * (B_T ? BK * ldb : BK), slot_of(t, 1), wave4, kc - t * BK);
    }
  };
  // The data-movement half-period: read this wave's fragments of K-step t_read and request
  // this wave's 8 blocks of K-step t_load, one request after every third fragment read.  The
  // texture-address path takes about as long to accept a group's 32 KB as LDS takes to deliver
  // its fragments; back to back the two would outlast the other group's MFMA burst, woven
  // together they fit inside it.
  auto move_data = [&](int t_read, int t_load) {
    int lf = lane;
    asm volatile("" : "+v"(lf));
    FragReader<A_T, TM> fa;
    FragReader<B_T, TN> fb;
    fa.init(wm * TM * 32, lf);
    fb.init(wn * TN * 32, lf);
    const bf16* at = smem + ((2 * t_read) % NSLOTS) * TILE;
    const bf16* bt = smem + ((2 * t_read + 1) % NSLOTS) * TILE;
    uint32_t aa[fa.NBASE], ba[fb.NBASE];
#pragma unroll
    for (int n = 0; n < fa.NBASE; ++n) aa[n] = fa.addr(at, n);
#pragma unroll
    for (int n = 0; n < fb.NBASE; ++n) ba[n] = fb.addr(bt, n);
    auto body = [&](const auto& loader, const bf16* kbase, bf16* dst) {
      const int k_left = kc - t_load * BK;
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          af[kk][i] = fa.read(aa, i, kk);
          const int n = kk * (TM + TN) + i;
          if (n % 3 == 2) loader.issue_one(kbase, dst, wave4, k_left, n / 3);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          bfr[kk][j] = fb.read(ba, j, kk);
          const int n = kk * (TM + TN) + TM + j;
          if (n % 3 == 2) loader.issue_one(kbase, dst, wave4, k_left, n / 3);
        }
      }
    };
    int l2 = lane;
    asm volatile("" : "+v"(l2));
    if (group) {
      TileLoader<A_T> la;
      la.init(lda, m0, M, wave4, l2);
      body(la, A + a_off + (int64_t)t_load * (A_T ? BK * lda : BK), slot_of(t_load, 0));
    } else {
      TileLoader<B_T> lb;
      lb.init(ldb, n0, N, wave4, l2);
      body(lb, B + b_off + (int64_t)t_load * (B_T ? BK * ldb : BK), slot_of(t_load, 1));
    }
  };
  // After this wave's loads of tile t have landed: zero a contraction tail of the last K-step.
  auto fix_tail_mine = [&](int t) {
    if (t != nk - 1 || k_tail == BK) return;
    int l2 = lane;
    asm volatile("" : "+v"(l2));
    if (group) {
      TileLoader<A_T> la;
      la.init(lda, m0, M, wave4, l2);
      la.zero_tail(slot_of(t, 0), k_tail, wave4, l2);
    } else {
      TileLoader<B_T> lb;
      lb.init(ldb, n0, N, wave4, l2);
      lb.zero_tail(slot_of(t, 1), k_tail, wave4, l2);
    }
  };

  // Two barriers per K-step delimit the half-periods.  The one in the middle of a K-step (after
  // it, group 1 computes and group 0 moves) orders every LDS hazard: data of the next K-step
  // visible, slots of the current one free.  The one at the start of a K-step only keeps the two
  // groups' MFMA bursts apart; every slot a group overwrites after it was last read before the
  // previous middle barrier.  With a transposed B operand the kernel is a little faster when the
  // hand-over at the start is left to the hardware (the next burst may begin while the last one
  // drains); with both operands K-major it is clearly slower, so there the barrier stays.
  constexpr bool kFreeHandoff = B_T;
  const int total_items = ntiles * (split_k ? splits : 1);
  int item = blockIdx.x;
  select_item(item);
  // K-steps 0 and 1 of the first item
  issue_mine(0);
  if (nk > 1) issue_mine(1);

  for (;;) {
  // K-steps 0 and 1 complete in LDS (requested above, or before the previous item's epilogue)
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0); lgkmcnt and expcnt untouched
  if (nk == 1) fix_tail_mine(0);
  __syncthreads();
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[j][i][e] = 0.f;

  if (group == 0) {
    read_frags(0);
    for (int ks = 0; ks < nk; ++ks) {
      // half-period 2ks: this group computes, the other moves data
      if (!kFreeHandoff) lds_barrier();
      compute();
      if (ks + 1 < nk) {
        // B of step ks+1 was requested one K-step ago
        __builtin_amdgcn_s_waitcnt(0x0f70);
        fix_tail_mine(ks + 1);
      }
      lds_barrier();  // half-period 2ks+1: this group moves data, the other computes
      // B(ks+2) replaces A(ks), which group 1 finished reading before the barrier above
      if (ks + 2 < nk)
        move_data(ks + 1, ks + 2);
      else if (ks + 1 < nk)
        read_frags(ks + 1);
    }
  } else {
    for (int ks = 0; ks < nk; ++ks) {
      if (!kFreeHandoff) lds_barrier();
      // A(ks+2) replaces B(ks-1), dead since the previous K-step
      if (ks + 2 < nk)
        move_data(ks, ks + 2);
      else
        read_frags(ks);
      if (ks + 1 < nk) {
        // A of step ks+1 (requested one K-step ago) must be in LDS before group 0 reads it
        // after the next barrier; the 8 loads just issued may stay in flight (loads retire in
        // order)
        if (ks + 2 < nk)
          __builtin_amdgcn_s_waitcnt(0x0f78);  // vmcnt(8)
        else
          __builtin_amdgcn_s_waitcnt(0x0f70);
        fix_tail_mine(ks + 1);
      }
      lds_barrier();
      compute();
    }
  }


  // Every LDS read of this item finished before the last barrier, so the ring is free: request
  // the first two K-steps of the next item now and let them fly during the epilogue.
  const int out_m0 = m0, out_n0 = n0;
  float* const out_partial = split_k ? partial + p_off : nullptr;
  const int next = item + (int)gridDim.x;
  const bool more = next < total_items;
  if (more) {
    select_item(next);
    issue_mine(0);
    if (nk > 1) issue_mine(1);
  }

  // Epilogue.  A lane holds C[m][n..n+3] for m = tile row (lane%32), n = 8g + 4*(lane/32):
  // stored from there, every instruction would scatter 64 eight-byte pieces over 32 rows and
  // the texture-address path, which takes such pieces one at a time, would need ~10 us per
  // tile.  Instead each wave transposes through its own 4 KB of ring slot 4 (idle until K-step
  // 2 of the next item is requested, after the next workgroup barrier): 32 rows of 128 bytes
  // go in from the MFMA layout and come out as whole rows, 8 lanes per row, so an instruction
  // writes 8 full 128-byte (bf16 output) or 8 contiguous row segments (fp32 partial tiles and
  // accumulation into C, staged as fp32 so that the sum is rounded once).  Only lanes of the
  // same wave exchange data: program order of its LDS instructions is all the ordering needed.
  {
    char* const stage = reinterpret_cast<char*>(smem + (NSLOTS - 1) * TILE) + wave * 4096;
    int le = lane;  // opaque copy: nothing derived from it is kept alive through the K loop
    asm volatile("" : "+v"(le));
    const int r = le & 31, h = le >> 5;
    const int wr = r * 128, wsw = (r >> 1) & 7;       // write side: row of the MFMA layout
    const int rrow = le >> 3, rch = le & 7;           // read side: row 8q + rrow, 16-byte chunk rch
    const int m_wave = out_m0 + wm * TM * 32, n_wave = out_n0 + wn * TN * 32;
    auto wave_sync = [&]() {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
    };
    // Global addresses are a wave-uniform block base plus a 32-bit lane offset (row 8q + rrow
    // of the block, this lane's chunk): four offset registers serve every access of the tile.
    const bool rows_in = m_wave + TM * 32 <= M;  // wave-uniform: no row of the wave tile is cut off
    if (out_partial == nullptr && !accumulate) {
      uint32_t lo[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) lo[q] = (uint32_t)((8 * q + rrow) * ldc + 8 * rch);
      const bool cols_in = n_wave + 8 * rch < N;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            bf16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (bf16)acc[j][i][g * 4 + e];
            *reinterpret_cast<bf16x4*>(stage + wr + (((4 * j + g) ^ wsw) << 4) + 8 * h) = o;
          }
        wave_sync();
        bf16* const cb = C + ((int64_t)(m_wave + i * 32) * ldc + n_wave);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int rr = 8 * q + rrow;
          const bf16x8 v =
              *reinterpret_cast<const bf16x8*>(stage + rr * 128 + ((rch ^ ((rr >> 1) & 7)) << 4));
          if (cols_in && (rows_in || m_wave + i * 32 + rr < M)) stg8(cb + lo[q], v);
        }
        wave_sync();
      }
    } else {
      // fp32 staging, one 32 x 32 block per pass; `emit(i, j, q, v)` gets four consecutive
      // columns of row 8q + rrow of block (i, j)
      auto fp32_passes = [&](auto&& before_block_row, auto&& emit) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          before_block_row(i);
#pragma unroll
          for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              f32x4 pv;
#pragma unroll
              for (int e = 0; e < 4; ++e) pv[e] = acc[j][i][g * 4 + e];
              *reinterpret_cast<f32x4*>(stage + wr + (((2 * g + h) ^ wsw) << 4)) = pv;
            }
            wave_sync();
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int rr = 8 * q + rrow;
              const f32x4 v = *reinterpret_cast<const f32x4*>(stage + rr * 128 +
                                                              ((rch ^ ((rr >> 1) & 7)) << 4));
              emit(i, j, q, v);
            }
            wave_sync();
          }
        }
      };
      if (out_partial != nullptr) {
        uint32_t lo[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) lo[q] = (uint32_t)((8 * q + rrow) * N + 4 * rch);
        fp32_passes([](int) {},
                    [&](int i, int j, int q, const f32x4& v) {
                      float* const pb = out_partial + ((int64_t)(m_wave + i * 32) * N + n_wave + j * 32);
                      if (n_wave + j * 32 + 4 * rch < N && (rows_in || m_wave + i * 32 + 8 * q + rrow < M))
                        *reinterpret_cast<f32x4*>(pb + lo[q]) = v;
                    });
      } else {
        // accumulation into C: the old values of a 32-row block (the same row segments the
        // results go to) are requested one block ahead of the passes that use them, so their
        // memory latency is paid once per tile, not once per pass.  Positions beyond the matrix
        // read a valid neighbour instead and are never stored back.
        uint32_t lo[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) lo[q] = (uint32_t)((8 * q + rrow) * ldc + 4 * rch);
        bf16x4 oldc[2][TN][4];
        auto fetch_old = [&](int i) {
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const bf16* const cb = C + ((int64_t)(m_wave + i * 32) * ldc + n_wave + j * 32);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const bool in = n_wave + j * 32 + 4 * rch < N && (rows_in || m_wave + i * 32 + 8 * q + rrow < M);
              oldc[i & 1][j][q] = *reinterpret_cast<const bf16x4*>(in ? cb + lo[q] : C);
            }
          }
        };
        fetch_old(0);
        fp32_passes([&](int i) { if (i + 1 < TM) fetch_old(i + 1); },
                    [&](int i, int j, int q, const f32x4& v) {
                      bf16* const cb = C + ((int64_t)(m_wave + i * 32) * ldc + n_wave + j * 32);
                      if (n_wave + j * 32 + 4 * rch < N && (rows_in || m_wave + i * 32 + 8 * q + rrow < M)) {
                        bf16x4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = (bf16)(v[e] + (float)oldc[i & 1][j][q][e]);
                        *reinterpret_cast<bf16x4*>(cb + lo[q]) = o;
                      }
                    });
      }
    }
  }
  if (!more) break;
  item = next;
  }
}

// the three layouts the library serves
template __global__ void gemm_kernel<false, false>(const bf16*, int, const bf16*, int, bf16*,
                                                   int, int, int, int, int, int, int, float*);
template __global__ void gemm_kernel<false, true>(const bf16*, int, const bf16*, int, bf16*,
                                                  int, int, int, int, int, int, int, float*);
template __global__ void gemm_kernel<true, true>(const bf16*, int, const bf16*, int, bf16*,
                                                 int, int, int, int, int, int, int, float*);

// C = bf16(sum over splits of the fp32 partial tiles [+ C]); one thread per 8 columns.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial,
                                                            bf16* __restrict__ C, int64_t ldc, int M,
                                                            int N, int splits, int accumulate) {
  const int nv = N / 8;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * nv) return;
  const int m = (int)(idx / nv), n = (int)(idx % nv) * 8;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  for (int sp = 0; sp < splits; ++sp) {
    const float* src = partial + ((int64_t)sp * M + m) * N + n;
    const f32x4 a = *reinterpret_cast<const f32x4*>(src);
    const f32x4 b = *reinterpret_cast<const f32x4*>(src + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc[e] += a[e];
      acc[4 + e] += b[e];
    }
  }
  bf16* dst = C + (int64_t)m * ldc + n;
  if (accumulate) {
    const bf16x8 old = ldg8(dst);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += (float)old[e];
  }
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (bf16)acc[e];
  stg8(dst, o);
}

// How many ways to cut the contraction when the output has too few tiles to occupy the GPU.
// 1 = no split.  Two estimates, in units of one K-step of one workgroup (~1.5 us):
//   latency  rounds of work items over the CUs, each item paying its K-steps plus a fixed
//            prologue/epilogue, plus the traffic of the fp32 partial tiles (written once, read
//            once by the reduce kernel at ~5 TB/s);
//   CU-time  the same work summed over the CUs it occupies, per CU of the device.
// A GEMM that has the GPU to itself wants the smallest latency (latency_weight 1); one that
// runs beside kernels of other streams, which can use the CUs it leaves idle, should mostly
// keep its CU-time small (latency_weight ~0.3).
inline int choose_splits(int M, int N, int K, float latency_weight) {
  constexpr int kCus = 256, kItemOverhead = 4;
  const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  if (tiles >= 192) return 1;
  const double w = latency_weight < 0.f ? 0.0 : (latency_weight > 1.f ? 1.0 : (double)latency_weight);
  const int nk = (K + BK - 1) / BK;
  const double reduce_per_split = (double)M * N * 8.0 / 5.0e12 / 1.5e-6;
  auto cost = [&](int sp) {
    const int items = tiles * sp, rounds = (items + kCus - 1) / kCus;
    const int per_item = (nk + sp - 1) / sp + kItemOverhead;
    const double reduce = sp > 1 ? sp * reduce_per_split : 0.0;
    const double latency = (double)rounds * per_item + reduce;
    const double cu_time = (double)items * per_item / kCus + reduce;
    return w * latency + (1.0 - w) * cu_time;
  };
  int best = 1;
  double best_cost = cost(1);
  for (int sp = 2; sp <= 16 && nk / sp >= 8; ++sp) {
    const double c = cost(sp);
    if (c < best_cost * 0.95) {  // a split must pay for itself clearly
      best_cost = c;
      best = sp;
    }
  }
  return best;
}

template <bool A_T, bool B_T>
int launch(const bf16* A, int64_t lda, const bf16* B, int64_t ldb, bf16* C, int64_t ldc, int M,
           int N, int K, int accumulate, float* workspace, size_t workspace_bytes,
           hipStream_t stream) {
  constexpr size_t lds_bytes = NSLOTS * TILE * sizeof(bf16);
  // raise the dynamic-LDS limit once per instantiation (thread-safe static initialisation)
  static const hipError_t attr_status =
      hipFuncSetAttribute((const void*)gemm_kernel<A_T, B_T>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (attr_status != hipSuccess) return KR_ELAUNCH;
  const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  // the latency-optimal count, capped by what the caller's workspace holds (a caller that wants
  // fewer splits says so by passing the smaller workspace kr_gemm_workspace_bytes_shared sizes)
  int splits = choose_splits(M, N, K, 1.f);
  const size_t one = (size_t)M * N * sizeof(float);
  if (workspace == nullptr) {
    splits = 1;
  } else if ((size_t)splits * one > workspace_bytes) {
    splits = (int)(workspace_bytes / one);
  }
  if (splits < 2 || (int64_t)splits * M * N >= ((int64_t)1 << 31)) splits = 1;
  // one persistent workgroup per compute unit (a workgroup owns a whole CU's LDS)
  static const int num_cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  if (splits == 1) {
    const int grid = tiles < num_cus ? tiles : num_cus;
    hipLaunchKernelGGL((gemm_kernel<A_T, B_T>), dim3(grid), dim3(NTHREADS), lds_bytes, stream, A,
                       (int)lda, B, (int)ldb, C, (int)ldc, M, N, K, accumulate, 0, 1, (float*)nullptr);
    return kr_launch_status();
  }
  int k_per = (K + splits - 1) / splits;
  k_per = (k_per + BK - 1) / BK * BK;
  splits = (K + k_per - 1) / k_per;
  const int items = tiles * splits;
  hipLaunchKernelGGL((gemm_kernel<A_T, B_T>), dim3(items < num_cus ? items : num_cus), dim3(NTHREADS),
                     lds_bytes, stream, A, (int)lda, B, (int)ldb, C, (int)ldc, M, N, K, 0, k_per, splits, workspace);
  if (hipGetLastError() != hipSuccess) return KR_ELAUNCH;
  const int64_t work = (int64_t)M * (N / 8);
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, stream,
                     (const float*)workspace, C, ldc, M, N, splits, accumulate);
  return kr_launch_status();
}

}  // namespace

extern "C" size_t kr_gemm_workspace_bytes(int layout, int M, int N, int K) {
  (void)layout;
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int splits = choose_splits(M, N, K, 1.f);
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

extern "C" size_t kr_gemm_workspace_bytes_shared(int layout, int M, int N, int K, float latency_weight) {
  (void)layout;
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int splits = choose_splits(M, N, K, latency_weight);
  const int cap = choose_splits(M, N, K, 1.f);
  if (splits > cap) splits = cap;
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

extern "C" int kr_gemm_bf16(int layout, int M, int N, int K, const void* A, int64_t lda,
                            const void* B, int64_t ldb, void* C, int64_t ldc, int accumulate,
                            void* workspace, size_t workspace_bytes, void* stream) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return KR_EINVAL;
  if (!kr_aligned16(A) || !kr_aligned16(B) || !kr_aligned16(C)) return KR_EINVAL;
  if (workspace && !kr_aligned16(workspace)) return KR_EINVAL;
  if ((M | N | K) % 8 || (lda | ldb | ldc) % 8) return KR_EUNSUPPORTED;
  // chunk offsets inside an operand are kept in 32 bits
  const int64_t a_rows = layout == KR_GEMM_NT ? 64 : M, b_rows = layout == KR_GEMM_TN ? N : 64;
  // ... and so are the offsets of the 32 rows of an output block from the block's first element
  if (a_rows * lda >= (int64_t)1 << 31 || b_rows * ldb >= (int64_t)1 << 31 || ldc >= (int64_t)1 << 26 ||
      N >= 1 << 26)
    return KR_EUNSUPPORTED;
  const bf16* a = (const bf16*)A;
  const bf16* b = (const bf16*)B;
  bf16* c = (bf16*)C;
  float* ws = (float*)workspace;
  hipStream_t st = (hipStream_t)stream;
  switch (layout) {
    case KR_GEMM_TN:  // A [M,K], B [N,K]
      if (lda < K || ldb < K || ldc < N) return KR_EINVAL;
      return launch<false, false>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, ws, workspace_bytes, st);
    case KR_GEMM_NN:  // A [M,K], B [K,N]
      if (lda < K || ldb < N || ldc < N) return KR_EINVAL;
      return launch<false, true>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, ws, workspace_bytes, st);
    case KR_GEMM_NT:  // A [K,M], B [K,N]
      if (lda < M || ldb < N || ldc < N) return KR_EINVAL;
      return launch<true, true>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, ws, workspace_bytes, st);
    default:
      return KR_EINVAL;
  }
}
