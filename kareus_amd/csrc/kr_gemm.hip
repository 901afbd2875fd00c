// bf16 GEMM on the gfx950 matrix cores: C[M,N] = A . B with fp32 accumulation, bf16 store.
//
// Roofline: MFMA (v_mfma_f32_16x16x32_bf16, 16384 FLOP per wave instruction).  Algorithmic
// work per launch is 2*M*N*K FLOP.
//
// Structure ("one instruction stream per SIMD")
//   * A workgroup of 4 waves, one per SIMD, owns a 256 x 256 tile of C and walks K in steps of
//     64.  Each wave owns 128 x 128 of the tile as 8 x 8 MFMA tiles of 16x16: 256 accumulator
//     registers, which are the wave's accumulation registers (the MFMAs are written as inline
//     assembly to pin them there); its 256 ordinary registers hold two sets of operand
//     fragments and the addressing.
//   * The K loop is a fixed, hand-ordered sequence.  A half-step is the 64 MFMAs of one
//     32-element half of a K-step; woven between them, one behind each MFMA, are the 16
//     fragment reads of the next half-step and the 8 global loads of one operand tile two
//     K-steps ahead.  An MFMA holds the matrix pipe for 16 cycles and the wave can issue
//     another instruction every 4-5, so these ride along without opening a gap in the pipe.
//     One workgroup barrier per K-step publishes the next tiles and retires the current ones.
//   * Global memory goes straight into LDS (global_load_lds_dwordx4): no staging registers, no
//     LDS store instructions.  The hardware places the 64 lanes of such a load contiguously in
//     LDS, so bank conflicts are avoided by an XOR swizzle applied on the *global* side — each
//     lane fetches the 16-byte chunk that belongs at its LDS slot.
//   * All 160 KB of LDS form a ring of five 32 KB slots, one operand tile (A or B of one
//     K-step) per slot.  In K-step t the first half-step requests A(t+2) into the slot B(t-1)
//     left at the previous barrier, the second half-step B(t+2) into the slot A(t) leaves at
//     this one: an even 32 KB per half-step, and every tile has one to two K-steps to land.
//   * Loads are 16-byte vectors along whichever dimension is contiguous in memory.  An operand
//     whose contraction dimension is contiguous ("K-major") is fetched from LDS with
//     ds_read_b128; an operand whose contraction dimension is the row index ("transposed": the
//     weight in dgrad, both operands in wgrad) with the transposing LDS read
//     ds_read_b64_tr_b16.  No transposed copy of any operand is ever made.
//   * The MFMA is issued with the operands swapped (the B tile feeds the instruction's A
//     port), so a lane ends up with four consecutive N-columns of one C row; the epilogue
//     transposes 16-row blocks through LDS and stores whole rows.
//   * Rows beyond the matrix edge are clamped to the last valid row instead of predicated: an
//     output element depends only on its own A row and B row, and out-of-range outputs are
//     never stored.  A contraction tail (K not a multiple of 64) is zeroed in LDS after its
//     tile has landed.
//   * Workgroups are persistent (one per compute unit); ids are remapped so that the tiles
//     resident on one XCD (ids congruent mod 8) form a compact band of C and share A/B panels
//     in that XCD's L2.
//   * Split-K: when C has too few tiles to fill 256 CUs (weight gradients: a small N x K
//     output contracted over all tokens), the contraction is cut into up to 16 ranges, each
//     workgroup writes an fp32 partial tile into a caller-provided workspace, and a small
//     HBM-bound kernel sums the partials and rounds to bf16.
#include "kr_common.h"

namespace {

constexpr int BK = 64;
constexpr int BM = 256, BN = 256;  // BN: the widest tile; a kernel instance covers 32 * WN columns
constexpr int WT = 8;  // 16x16 MFMA tiles per wave along M: a wave owns 128 rows x 16 * WN columns of C
constexpr int NTHREADS = 256;
constexpr int TILE = 256 * BK;  // elements of one operand tile (either layout)
constexpr uint32_t SLOT_BYTES = TILE * sizeof(bf16);
constexpr int NSLOTS = 5;          // 5 x 32 KB = the whole 160 KB of LDS
constexpr int kXcds = 8;
constexpr int KR_GEMM_EPI_TRANSPOSED_OUT = 100;  // internal: not part of the C ABI's epilogue values
constexpr int kGroupM = 4;

// ---- LDS layouts (element offsets inside one operand tile) ----------------------------------
// K-major tile [256 rows][64]: 128-byte rows, 16-byte chunk index XORed with (row>>1)&7.
// Output stores carry the non-temporal hint: nothing in the launch reads an output tile again.  Measured on
// the 8B shard's layer at 16384 tokens: the out-projection forward 7 % shorter, the fc1 forward with its
// SwiGLU epilogue 3-6 %, fc2's forward 2 %, the one-nanobatch step 1 %.  The bytes a launch fetches from
// memory are the same with and without the hint (FETCH_SIZE), so the time is won on the store path, not on
// operand re-reads; the same hint on other kernels' stores or on the epilogues' residual loads changed nothing.
__device__ __forceinline__ void stg8_out(bf16* p, bf16x8 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<bf16x8*>(p));
}

__device__ __forceinline__ int kmajor_off(int row, int chunk) {
  return row * BK + ((chunk ^ ((row >> 1) & 7)) << 3);
}
// transposed tile [64 k-rows][256]: 512-byte rows, 16-byte chunk index XORed with a value made of
// k-row bits 0, 1 (the four k-rows one 16-lane group reads together) and bit 3 (the two groups
// of a 32-lane half read k-rows 8 apart).
__device__ __forceinline__ int transp_swz(int krow) { return ((krow & 3) << 2) | (((krow >> 3) & 1) << 1); }
__device__ __forceinline__ int transp_off(int krow, int col) {
  return krow * 256 + (((col >> 3) ^ transp_swz(krow)) << 3) + (col & 7);
}

// ---- direct global -> LDS loads ---------------------------------------------------------------
// Issued through inline assembly on purpose.  A workgroup barrier is a release fence for LDS,
// and the compiler drains every LDS-direct load it knows of (vmcnt(0)) in front of one — which
// would empty the prefetch pipeline once per K-step.  Written this way the loads are invisible
// to its wait-count bookkeeping; their completion is tracked by hand with explicit vmcnt waits
// placed before the barrier that publishes the data.  The loads have no register destination,
// so nothing can be clobbered behind the register allocator's back.
// base: wave-uniform global address; byte_off: this lane's unsigned 32-bit byte offset from it;
// lds_base + IMM: wave-uniform LDS byte address of a 1-KiB block (lane p lands at +16p).
template <int IMM>
__device__ __forceinline__ void dma_b128(const void* base, uint32_t byte_off, uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_base), "v"(byte_off), "s"(base), "n"(IMM)
               : "memory", "m0", "scc");
}
__device__ __forceinline__ uint32_t lds_addr(const bf16* p) {
  return (uint32_t)(uintptr_t)(KR_LDS const bf16*)p;
}

// ---- which 16-byte chunk a lane fetches ------------------------------------------------------
// The four waves share every operand tile: wave w issues loads i = 0..7, load i fills the 1-KiB
// block w + 4 i.  Block b of a K-major tile holds rows 8b..8b+7; block b of a transposed tile
// holds contraction rows 2b, 2b+1.  The swizzle is applied on the global side: each lane
// fetches the chunk that belongs at its LDS position.
// Returns the element offset from the K-step's base pointer.  Rows beyond the matrix are
// clamped to the last valid row; a chunk that would start beyond the contraction range
// (k_left = elements from the K-step's base to the end, >= 8) is redirected to a valid address —
// it is zeroed in LDS afterwards, so what it fetches does not matter.
// gate_up_f > 0 (K-major B of a fused SwiGLU projection, weight rows [gate: 0..F) | up: F..2F)):
// the first `half_rows` rows of the tile hold the gate rows row0 .., the next `half_rows` the up rows
// of the same output columns, so that the waves of the tile's left half end up with gate values
// and the waves of its right half with the matching up values.
// Row runs.  The rows of an operand may come in runs of 2^sh consecutive rows (stride ld) whose starts
// are `outer` elements apart: row r sits at (r >> sh) * outer + (r & (2^sh - 1)) * ld.  That is a
// nanobatch of 2^sh sequences cut out of a [s, b, h] tensor along b, read in place.  A plain matrix
// is sh = 0, outer = ld.
__device__ __forceinline__ int run_off(int r, int ld, int sh, int outer) {
  return (r >> sh) * outer + (r & ((1 << sh) - 1)) * ld;
}
template <bool TRANSPOSED>
__device__ __forceinline__ uint32_t load_offset(int i, int wave, int lane, int ld, int row0,
                                                int rows_total, int k_left, int gate_up_f = 0,
                                                int half_rows = 0, int sh = 0, int outer = 0) {
  if (!TRANSPOSED) {
    const int row = 8 * wave + (lane >> 3) + 32 * i;
    int chunk = ((lane & 7) ^ ((row >> 1) & 7)) * 8;
    int r = row0 + row;
    if (gate_up_f > 0) r = row < half_rows ? row0 + row : row0 + (row - half_rows) + gate_up_f;
    r = r < rows_total ? r : rows_total - 1;
    chunk = chunk + 8 <= k_left ? chunk : k_left - 8;
    return (uint32_t)((sh ? run_off(r, ld, sh, outer) : r * ld) + chunk);
  }
  // (the contraction rows of a K-step start at a multiple of 64, hence of the run length: the
  // position inside the K-step maps like a row of its own)
  int krow = 2 * wave + (lane >> 5) + 8 * i;
  int c = row0 + ((lane & 31) ^ transp_swz(krow)) * 8;
  c = c + 8 <= rows_total ? c : rows_total - 8;
  krow = krow < k_left ? krow : k_left - 1;
  return (uint32_t)((sh ? run_off(krow, ld, sh, outer) : krow * ld) + c);
}
// contraction index (relative to the K-step) of the chunk that load i of this lane fills
template <bool TRANSPOSED>
__device__ __forceinline__ int load_k(int i, int wave, int lane) {
  if (!TRANSPOSED) {
    const int row = 8 * wave + (lane >> 3);  // (row >> 1) & 7 does not depend on i
    return ((lane & 7) ^ ((row >> 1) & 7)) * 8;
  }
  return 2 * wave + (lane >> 5) + 8 * i;
}

// ---- LDS -> MFMA operand fragments ----------------------------------------------------------
// v_mfma_f32_16x16x32_bf16 wants from lane l the 8 contraction elements 8 (l / 16) .. + 7 of
// operand row l % 16.  Fragment (g, h): operand rows row0 + 16 g .., contraction half h (32
// elements) of the K-step.
template <bool TRANSPOSED>
struct FragReader {
  // K-major: one base per half (the swizzle XOR depends on the chunk), g is an immediate
  // transposed: one base per g (the XOR depends on the column), the half is an immediate
  static constexpr int NBASE = TRANSPOSED ? WT : 2;
  uint32_t base[NBASE];  // byte offsets inside a tile
  __device__ __forceinline__ void init(int row0, int lane) {
    if (!TRANSPOSED) {
#pragma unroll
      for (int h = 0; h < 2; ++h) base[h] = 2u * (uint32_t)kmajor_off(row0 + (lane & 15), 4 * h + (lane >> 4));
    } else {
      // transposing read: within each group of 16 lanes, lane p supplies the address of 4
      // consecutive operand rows in contraction row p / 4 and receives, for operand row p, the
      // elements of the group's 4 contraction rows
      const int p = lane & 15;
      const int krow = 8 * (lane >> 4) + (p >> 2);
#pragma unroll
      for (int g = 0; g < WT; ++g) base[g] = 2u * (uint32_t)transp_off(krow, row0 + 16 * g + (p & 3) * 4);
    }
  }
};
// slot: LDS byte address of the tile; for K-major operands `a` is slot + base[h] (opaque)
__device__ __forceinline__ bf16x8 frag_kmajor(uint32_t a, int g) {
  return *(KR_LDS const bf16x8*)(a + (uint32_t)(g * 16 * BK * 2));
}
__device__ __forceinline__ bf16x8 frag_transp(uint32_t a, int h) {
  const uint32_t a0 = a + (uint32_t)(h * 32 * 256 * 2);
  union {
    struct { s16x4 lo, hi; } s;
    bf16x8 v;
  } u;
  u.s.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a0));
  u.s.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a0 + 2u * 4 * 256));
  return u.v;
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

// Row runs of A, C and aux (see run_off): shift and distance between run starts; sh = 0 for a
// plain matrix (the distance is then unused).
struct RowRuns {
  int a_sh, a_outer, c_sh, c_outer, x_sh, x_outer;
};

// The contraction of a weight gradient over the nanobatches of a microbatch: layout NT, operands in up
// to KR_GEMM_MAX_SEGMENTS pieces (one pair per nanobatch, each `steps` K-steps of 64 rows long, all with
// the row strides lda / ldb), contracted one after the other into one sum.
constexpr int MAX_SEGMENTS = KR_GEMM_MAX_SEGMENTS;
struct Segments {
  const bf16* a[MAX_SEGMENTS];
  const bf16* b[MAX_SEGMENTS];
  int n, steps;
};

template <int WN>
struct Frags {
  bf16x8 a[WT], b[WN];
};
template <int N>
struct Count { static constexpr int value = N; };

// WN: 16-column MFMA tiles per wave along N (4..8): the workgroup's tile is 256 x 32 * WN.  Narrower
// tiles let the host avoid a mostly empty last round of workgroups or a mostly padded last tile
// column; a K-major B tile then occupies the first 32 * WN rows of its slot and takes WN loads per wave.
// EPI: the fused epilogue compiled into this instance (KR_GEMM_EPI_*).  A template parameter, not
// a run-time switch: the plain instances carry none of the extra code or registers.
// RUNS: the instance honours row runs of A, C and aux (RowRuns); the plain instances do not carry the
// extra address arithmetic or its registers.
// SEG (layout NT): A and B are the pieces named by `segs` (the A / B arguments are unused); K is their
// total length.
template <bool A_T, bool B_T, int WN, int EPI, bool RUNS = false, bool SEG = false>
__global__ __launch_bounds__(NTHREADS) void gemm_kernel(const bf16* __restrict__ A, int lda,
                                                        const bf16* __restrict__ B, int ldb,
                                                        bf16* __restrict__ C, int ldc, int M,
                                                        int N, int K, int accumulate, int k_per,
                                                        int splits, float* __restrict__ partial,
                                                        const bf16* __restrict__ aux, int ld_aux,
                                                        bf16* __restrict__ out2, int ld_out2,
                                                        RowRuns runs_arg, Segments segs) {
  static_assert(!SEG || (A_T && B_T), "operand pieces: layout NT");
  // (without RUNS every run length reads as a compile-time 1: the branches below fold away)
  const RowRuns runs = RUNS ? runs_arg : RowRuns{0, 0, 0, 0, 0, 0};
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int BN_ = 32 * WN;
  // loads per wave of a B tile: a K-major tile's unused rows are simply not fetched; in a
  // transposed tile every load spans all 256 columns
  constexpr int NB_LOADS = B_T ? 8 : WN;
  const int wm = wave >> 1, wn = wave & 1;  // wave tile: rows wm*128.., columns wn*16*WN..
  // fused epilogues: ADD: C = bf16(bf16(A.B) + aux), aux [M,N] with row stride ld_aux.
  // SWIGLU: C = x [M, N = 2F] and out2 = silu(x[:, :F]) * x[:, F:] [M, F]; a tile then covers
  // 16 * WN columns of out2: its left half (the waves with wn = 0) computes their gate columns,
  // its right half (wn = 1) the matching up columns of x, and the two meet in the epilogue.
  // TRANSPOSED_OUT (internal, layout NT only): the kernel computes the tile of C = A^T . B as
  // always but stores C^T, i.e. the caller's output is [N, M] with row stride ldc.  The host uses
  // it with the operands exchanged when the tile grid of the transposed problem fits the device
  // better (256 x 224 tiles can then be 224 rows x 256 columns of the output).
  constexpr bool trans_out = EPI == KR_GEMM_EPI_TRANSPOSED_OUT;
  // SWIGLU_BWD (layout NN, an input gradient): the product is the gradient of the activation's
  // output; the epilogue reads the activation's input x = [gate | up] for the same rows and
  // columns and stores the gradient of x instead of the product.
  constexpr bool swiglu_bwd = EPI == KR_GEMM_EPI_SWIGLU_BWD;
  static_assert(!swiglu_bwd || (!A_T && B_T), "SwiGLU backward epilogue: layout NN only");
  static_assert(EPI == KR_GEMM_EPI_NONE || trans_out || swiglu_bwd || (!A_T && !B_T),
                "residual / SwiGLU epilogues: K-major layout only");
  static_assert(!trans_out || (A_T && B_T), "transposed store: layout NT only");
  constexpr bool epi_add = EPI == KR_GEMM_EPI_ADD;
  constexpr bool swiglu = EPI == KR_GEMM_EPI_SWIGLU;
  const int gate_up_f = swiglu ? N / 2 : 0;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = swiglu ? N / BN_ : (N + BN_ - 1) / BN_;
  const int ntiles = tiles_m * tiles_n;
  const bool split_k = partial != nullptr;
  const uint32_t smem_b = lds_addr(smem);
  const uint32_t wave_blk = (uint32_t)wave * 1024u;

  // Persistent workgroups: work item v = (output tile, split-K range); this workgroup takes
  // items blockIdx.x, blockIdx.x + gridDim.x, ...  The state below describes the current item.
  // (element offsets fit 32 bits: the host checks rows * ld < 2^31 and the workspace size)
  int m0, n0, nk, k_tail, kc = K, a_off = 0, b_off = 0, p_off = 0;
  const bf16 *seg_a = A, *seg_b = B;
  int seg_left = 0, seg_next = 0;
  // elements from one K-step of A to the next (a transposed A in row runs: 64 rows are 64 / r runs)
  const int a_step = A_T ? (runs.a_sh ? (BK >> runs.a_sh) * runs.a_outer : BK * lda) : BK;
  auto select_item = [&](int v) {
    const int split = v / ntiles;
    int tile_m, tile_n;
    remap_block(v - split * ntiles, ntiles, tiles_m, tiles_n, tile_m, tile_n);
    m0 = tile_m * BM;
    n0 = swiglu ? tile_n * (16 * WN) : tile_n * BN_;
    int k0 = 0;
    if (split_k) {
      // split-K: contraction range [split*k_per, split*k_per + kc), fp32 partial tile out
      // (k_per is a multiple of 64)
      k0 = split * k_per;
      a_off = A_T ? (runs.a_sh ? (k0 >> runs.a_sh) * runs.a_outer : k0 * lda) : k0;
      b_off = B_T ? k0 * ldb : k0;
      kc = (K - k0) < k_per ? (K - k0) : k_per;
      p_off = split * M * N;
    }
    nk = (kc + BK - 1) / BK;
    k_tail = kc - (nk - 1) * BK;  // valid contraction rows of the last K-step (8..64)
    if constexpr (SEG) {
      // the request cursor goes to K-step k0 / 64 of the whole contraction
      const int g0 = k0 / BK, sg = g0 / segs.steps, within = g0 - sg * segs.steps;
      seg_a = segs.a[sg] + (int64_t)within * a_step;
      seg_b = segs.b[sg] + (int64_t)within * (BK * ldb);
      seg_left = segs.steps - within;
      seg_next = sg + 1;
    }
  };
  // SEG: K-steps are requested strictly in order (A then B of a step), so the bases are a cursor that
  // seg_advance() moves on behind the requests of a step; `t` is not needed
  auto a_base = [&](int t) {
    if constexpr (SEG) return seg_a; else return A + a_off + (int64_t)t * a_step;
  };
  auto b_base = [&](int t) {
    if constexpr (SEG) return seg_b; else return B + b_off + (int64_t)t * (B_T ? BK * ldb : BK);
  };
  auto seg_advance = [&]() {
    if constexpr (SEG) {
      seg_a += a_step;
      seg_b += BK * ldb;
      if (--seg_left == 0) {
        if (seg_next < segs.n) {
          seg_a = segs.a[seg_next];
          seg_b = segs.b[seg_next];
        }
        seg_left = segs.steps;
        ++seg_next;
      }
    }
  };

  // The ring of five 32 KB slots as LDS byte addresses, in ring order starting at A of the
  // current K-step t: r0 = A(t), r1 = B(t), r2 = A(t+1), r3 = B(t+1), r4 = A(t+2); B(t+2) goes
  // where A(t) was.  Rotated by two positions per K-step.
  uint32_t r0 = smem_b, r1 = smem_b + SLOT_BYTES, r2 = smem_b + 2 * SLOT_BYTES,
           r3 = smem_b + 3 * SLOT_BYTES, r4 = smem_b + 4 * SLOT_BYTES;
  auto rotate = [&]() {
    const uint32_t o0 = r0, o1 = r1;
    r0 = r2; r1 = r3; r2 = r4; r3 = o0; r4 = o1;
  };

  // accumulators live in the accumulation registers (the MFMAs are written as inline assembly
  // with that register class, see mfma() below); fragments in ordinary vector registers
  f32x4 acc[WT][WN];
  Frags<WN> X, Y;
  uint32_t la[8], lb[8];  // byte offsets of this lane's chunk in the 8 loads of an A / a B tile

  auto set_offsets = [&](int k_left) {
    int l2 = lane;
    asm volatile("" : "+v"(l2));
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      la[i] = 2u * load_offset<A_T>(i, wave, l2, lda, m0, M, k_left, 0, 0, runs.a_sh, runs.a_outer);
      lb[i] = 2u * load_offset<B_T>(i, wave, l2, ldb, n0, N, k_left, gate_up_f, 16 * WN);
    }
  };
  // the first `count` loads of a tile (8 for A, NB_LOADS for B)
  auto request = [&](const bf16* base, const uint32_t (&off)[8], uint32_t slot, auto count_tag) {
    constexpr int COUNT = decltype(count_tag)::value;
    const uint32_t dst = slot + wave_blk;
    dma_b128<0 * 4096>(base, off[0], dst);
    dma_b128<1 * 4096>(base, off[1], dst);
    dma_b128<2 * 4096>(base, off[2], dst);
    dma_b128<3 * 4096>(base, off[3], dst);
    dma_b128<4 * 4096>(base, off[4], dst);
    if constexpr (COUNT > 5) dma_b128<5 * 4096>(base, off[5], dst);
    if constexpr (COUNT > 6) dma_b128<6 * 4096>(base, off[6], dst);
    if constexpr (COUNT > 7) dma_b128<7 * 4096>(base, off[7], dst);
  };
  // K-steps 0 and 1 of the current item into r0..r3
  auto request_first_two = [&]() {
    set_offsets(nk == 1 ? k_tail : BK);
    request(a_base(0), la, r0, Count<8>{});
    request(b_base(0), lb, r1, Count<NB_LOADS>{});
    seg_advance();
    if (nk > 1) {
      if (nk == 2 && k_tail != BK) set_offsets(k_tail);
      request(a_base(1), la, r2, Count<8>{});
      request(b_base(1), lb, r3, Count<NB_LOADS>{});
      seg_advance();
    }
  };
  // After this wave's loads of the last K-step have landed (A in slot sa, B in slot sb): zero
  // the chunks beyond the contraction range.
  auto fix_tail = [&](uint32_t sa, uint32_t sb) {
    if (k_tail == BK) return;
    int l2 = lane;
    asm volatile("" : "+v"(l2));
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t blk = (uint32_t)(wave + 4 * i) * 1024u + (uint32_t)l2 * 16u;
      if (load_k<A_T>(i, wave, l2) >= k_tail) *(KR_LDS bf16x8*)(sa + blk) = zero8();
      if (load_k<B_T>(i, wave, l2) >= k_tail) *(KR_LDS bf16x8*)(sb + blk) = zero8();
    }
  };

  // fragment addressing, recomputed per item from an opaque copy of the lane id so that it is
  // not live through the epilogue
  FragReader<A_T> fa;
  FragReader<B_T> fb;
  // addresses for reading half h of the tiles in slots sa / sb
  auto frag_addrs = [&](uint32_t sa, uint32_t sb, int h, uint32_t (&aa)[FragReader<A_T>::NBASE],
                        uint32_t (&ba)[FragReader<B_T>::NBASE]) {
    if (!A_T) {
      aa[0] = sa + fa.base[h];
      asm volatile("" : "+v"(aa[0]));
    } else {
#pragma unroll
      for (int g = 0; g < WT; ++g) {
        aa[g] = sa + fa.base[g];
        asm volatile("" : "+v"(aa[g]));
      }
    }
    if (!B_T) {
      ba[0] = sb + fb.base[h];
      asm volatile("" : "+v"(ba[0]));
    } else {
#pragma unroll
      for (int g = 0; g < WN; ++g) {
        ba[g] = sb + fb.base[g];
        asm volatile("" : "+v"(ba[g]));
      }
    }
  };
  auto read_a = [&](const uint32_t (&aa)[FragReader<A_T>::NBASE], int g, int h) {
    if constexpr (!A_T) return frag_kmajor(aa[0], g); else return frag_transp(aa[g], h);
  };
  auto read_b = [&](const uint32_t (&ba)[FragReader<B_T>::NBASE], int g, int h) {
    if constexpr (!B_T) return frag_kmajor(ba[0], g); else return frag_transp(ba[g], h);
  };

  // One half-step: the 64 MFMAs of one 32-element half of a K-step on `cur`, with the 16
  // fragment reads of the next half-step (half h of the tiles in slots sa / sb, into `nxt`) and,
  // if DMA, the 8 requests of one operand tile woven in between in exactly this order.  The
  // operands are swapped (the B fragment feeds the instruction's A port), so a lane ends up
  // with four consecutive columns of one row of C.
  auto half = [&](Frags<WN>& cur, Frags<WN>& nxt, uint32_t sa, uint32_t sb, int h, auto dma_tag,
                  const bf16* dbase, const uint32_t (&doff)[8], uint32_t dslot) {
    constexpr int DMA = decltype(dma_tag)::value;  // how many loads to weave in (0: none)
    uint32_t aa[FragReader<A_T>::NBASE], ba[FragReader<B_T>::NBASE];
    frag_addrs(sa, sb, h, aa, ba);
    const uint32_t dst = dslot + wave_blk;
#pragma unroll
    for (int g = 0; g < WT; ++g) {
#pragma unroll
      for (int nt = 0; nt < WN; ++nt) {
        if constexpr (trans_out) {
          // operands not swapped: a lane gets four consecutive rows of one column of C, which are
          // four consecutive columns of one row of C^T
          asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                       : "+a"(acc[g][nt])
                       : "v"(cur.a[g]), "v"(cur.b[nt]));
        } else {
          asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                       : "+a"(acc[g][nt])
                       : "v"(cur.b[nt]), "v"(cur.a[g]));
        }
        if (nt == 0) nxt.a[g] = read_a(aa, g, h);
        if (nt == 2 && g < WN) nxt.b[g] = read_b(ba, g, h);
        if constexpr (DMA > 0) {
          if (nt == (WN > 4 ? 4 : 3) && g < DMA) {
            if (g == 0) dma_b128<0 * 4096>(dbase, doff[0], dst);
            if (g == 1) dma_b128<1 * 4096>(dbase, doff[1], dst);
            if (g == 2) dma_b128<2 * 4096>(dbase, doff[2], dst);
            if (g == 3) dma_b128<3 * 4096>(dbase, doff[3], dst);
            if (g == 4) dma_b128<4 * 4096>(dbase, doff[4], dst);
            if (g == 5) dma_b128<5 * 4096>(dbase, doff[5], dst);
            if (g == 6) dma_b128<6 * 4096>(dbase, doff[6], dst);
            if (g == 7) dma_b128<7 * 4096>(dbase, doff[7], dst);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  const int total_items = ntiles * (split_k ? splits : 1);
  int item = blockIdx.x;
  select_item(item);
  request_first_two();
  // the accumulators start at zero: here for the first item (behind the latency of its first
  // loads), in the epilogue for every later one (behind its LDS round trips)
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (;;) {
    {
      int lf = lane;
      asm volatile("" : "+v"(lf));
      fa.init(wm * 128, lf);
      fb.init(wn * 16 * WN, lf);
    }
    // K-step 0 complete in LDS (requested above, or before the previous item's epilogue); the
    // 16 loads of K-step 1 may still be in flight (loads retire in order)
    if (nk > 1) {
      // vmcnt(8 + NB_LOADS); lgkmcnt and expcnt untouched
      __builtin_amdgcn_s_waitcnt(0x0f70 | ((8 + NB_LOADS) & 15) | (((8 + NB_LOADS) >> 4) << 14));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      fix_tail(r0, r1);
    }
    __syncthreads();
    {
      uint32_t aa[FragReader<A_T>::NBASE], ba[FragReader<B_T>::NBASE];
      frag_addrs(r0, r1, 0, aa, ba);
#pragma unroll
      for (int g = 0; g < WT; ++g) {
        X.a[g] = read_a(aa, g, 0);
        if (g < WN) X.b[g] = read_b(ba, g, 0);
      }
    }

    // K loop.  In K-step t: first half-step computes on X (half 0) while Y is read from the
    // tiles of t (half 1) and A(t+2) is requested into r4, dead since the barrier of K-step
    // t-1; then every load but those eight must have landed (that is all of K-step t+1), one
    // barrier publishes them and retires the tiles of t; the second half-step computes on Y
    // while X is read from the tiles of t+1 and B(t+2) is requested where A(t) was.
    int t = 0;
    for (; t + 2 < nk; ++t) {
      if (t + 3 == nk && k_tail != BK) set_offsets(k_tail);
      half(X, Y, r0, r1, 1, Count<8>{}, a_base(t + 2), la, r4);
      __builtin_amdgcn_s_waitcnt(0x0f78);  // vmcnt(8)
      __syncthreads();
      half(Y, X, r2, r3, 0, Count<NB_LOADS>{}, b_base(t + 2), lb, r0);
      seg_advance();
      rotate();
    }
    for (; t < nk; ++t) {
      half(X, Y, r0, r1, 1, Count<0>{}, nullptr, la, 0u);
      __builtin_amdgcn_s_waitcnt(0x0f70);
      if (t + 2 == nk) fix_tail(r2, r3);
      __syncthreads();
      // (after the last K-step this reads tiles that do not exist: unused)
      half(Y, X, r2, r3, 0, Count<0>{}, nullptr, lb, 0u);
      rotate();
    }

    // Every LDS read of this item that matters finished before the last barrier, so slots
    // r0..r3 are free: request the first two K-steps of the next item now and let them fly
    // during the epilogue.
    const int out_m0 = m0, out_n0 = n0;
    float* const out_partial = split_k ? partial + p_off : nullptr;
    const int next = item + (int)gridDim.x;
    const bool more = next < total_items;
    if (more) {
      select_item(next);
      request_first_two();
    }
    // the compiler does not know the MFMAs' latency: let the last ones finish before their
    // results are read
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // Epilogue.  A lane holds C[m][n..n+3] for m = 16 mt + lane%16, n = 16 nt + 4 (lane/16):
    // stored from there, every instruction would scatter 64 small pieces over 16 rows.  Instead
    // each wave transposes through its own 8 KB of slot r4 (idle until K-step 2 of the next
    // item is requested, after the next workgroup barrier): a block of 16 rows x 128 columns
    // goes in as fp32 from the MFMA layout and comes out as whole rows (32 lanes per row, four
    // consecutive columns per lane), so a store instruction writes complete row segments of
    // 256 bytes (bf16 output) or 512 bytes (fp32 partial tiles); accumulation into C adds the
    // old values in fp32, so the sum is rounded once.  Only lanes of the same wave exchange
    // data: program order of its LDS instructions is all the ordering needed.  The accumulators
    // are read in one place for all three kinds of output.
    {
      const uint32_t stage = r4 + (uint32_t)wave * 8192u;
      int le = lane;  // opaque copy: nothing derived from it is kept alive through the K loop
      asm volatile("" : "+v"(le));
      const int row16 = le & 15, quad = le >> 4;
      const int hrow = le >> 5, ch = le & 31;  // read side: row 2q + hrow, columns 4 ch .. + 3
      const int m_wave = out_m0 + wm * 128, n_wave = out_n0 + wn * 16 * WN;
      auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
      };
      const bool rows_in = m_wave + 128 <= M;  // wave-uniform: no row of the wave tile is cut off
      const bool cols_in = 4 * ch < 16 * WN && n_wave + 4 * ch < N;
      const bool to_partial = out_partial != nullptr;
      const bool add_old = !to_partial && accumulate;
      const int ldo = to_partial ? N : ldc;
      uint32_t lo[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) lo[q] = (uint32_t)((2 * q + hrow) * ldo + 4 * ch);
      // accumulation into C: the old values of a 16-row block are requested one block ahead of
      // the pass that uses them (zeros otherwise).  Positions beyond the matrix read a valid
      // neighbour instead and are never stored back.
      bf16x4 oldc[2][8];
#pragma unroll
      for (int q = 0; q < 8; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) oldc[0][q][e] = oldc[1][q][e] = (bf16)0.f;
      auto fetch_old = [&](int mt) {
        const bf16* const cb = C + ((int64_t)(m_wave + mt * 16) * ldc + n_wave);
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const bool in = cols_in && (rows_in || m_wave + mt * 16 + 2 * q + hrow < M);
          oldc[mt & 1][q] = *reinterpret_cast<const bf16x4*>(in ? cb + lo[q] : C);
        }
      };
      if (add_old) fetch_old(0);
      // bf16 output without accumulation goes through the same place as bf16: 16 rows x 256 bytes
      // per block, two buffers (so one wave-level fence per block), read side row 4q + quad,
      // 16-byte chunk rch = eight consecutive columns, 16 lanes per row
      const bool narrow = !to_partial && !add_old;
      const int rch = le & 15;
      // first column the wave stores to: n_wave, or with SwiGLU column out_n0 of the gate half
      // (wn = 0) or of the up half (wn = 1) of x
      const int n_store = swiglu ? out_n0 + (wn ? gate_up_f : 0) : n_wave;
      const int ncol = 8 * rch;
      const bool ncols_in = 8 * rch < 16 * WN && (swiglu || n_wave + 8 * rch < N);
      uint32_t nlo[4];
#pragma unroll
      for (int q = 0; q < 4; ++q)   // (a 16-row block starts at a multiple of the run length: rows map inside it)
        nlo[q] = (uint32_t)((runs.c_sh ? run_off(4 * q + quad, ldc, runs.c_sh, runs.c_outer) : (4 * q + quad) * ldc) + ncol);
      // fused residual: the values to add to a 16-row block are requested one block ahead
      // SwiGLU backward: gate and up values of a 16-row block, requested one block ahead
      bf16x8 xg[swiglu_bwd ? 2 : 1][swiglu_bwd ? 4 : 1], xu[swiglu_bwd ? 2 : 1][swiglu_bwd ? 4 : 1];
      auto fetch_x = [&](int mt) {
        const bf16* const xb = aux + ((int64_t)(m_wave + mt * 16) * ld_aux + n_wave + 8 * rch);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int rr = 4 * q + quad;
          const bool in = ncols_in && (rows_in || m_wave + mt * 16 + rr < M);
          xg[mt & 1][q] = in ? ldg8(xb + (int64_t)rr * ld_aux) : zero8();
          xu[mt & 1][q] = in ? ldg8(xb + (int64_t)rr * ld_aux + N) : zero8();
        }
      };
      if constexpr (swiglu_bwd) fetch_x(0);
      bf16x8 resv[epi_add ? 2 : 1][epi_add ? 4 : 1];
      auto fetch_res = [&](int mt) {
        const int r0 = m_wave + mt * 16;
        const bf16* const rb =
            aux + ((runs.x_sh ? (int64_t)(r0 >> runs.x_sh) * runs.x_outer : (int64_t)r0 * ld_aux) + n_wave + 8 * rch);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int rr = 4 * q + quad;
          const bool in = ncols_in && (rows_in || m_wave + mt * 16 + rr < M);
          const int64_t ro = runs.x_sh ? (int64_t)run_off(rr, ld_aux, runs.x_sh, runs.x_outer) : (int64_t)rr * ld_aux;
          resv[mt & 1][q] = in ? ldg8(rb + ro) : zero8();
        }
      };
      if constexpr (epi_add) fetch_res(0);
      if constexpr (trans_out) {
        // C^T leaves in blocks of 16 of its rows (columns nt of the wave tile): the wave's eight
        // 16 x 16 tiles of that column are 16 rows x 128 columns of C^T, staged and stored like a
        // block of the plain path with the two tile indices exchanged.
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) {
          f32x4 vals[WT];
#pragma unroll
          for (int mt = 0; mt < WT; ++mt) {
            vals[mt] = acc[mt][nt];
            asm volatile("" : "+v"(vals[mt]));
            acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
          }
          const uint32_t buf = stage + (uint32_t)(nt & 1) * 4096u;
#pragma unroll
          for (int mt = 0; mt < WT; ++mt) {
            bf16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (bf16)vals[mt][e];
            *(KR_LDS bf16x4*)(buf + row16 * 256 + (((2 * mt + (quad >> 1)) ^ row16) << 4) + (quad & 1) * 8) = o;
          }
          wave_sync();
          const bool tcols_in = m_wave + 8 * rch < M;   // M is a multiple of 8: the whole chunk is in or out
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int rr = 4 * q + quad;
            const bf16x8 v = *(KR_LDS const bf16x8*)(buf + rr * 256 + ((rch ^ rr) << 4));
            const int n = n_wave + nt * 16 + rr;
            if (tcols_in && n < N) stg8_out(C + (int64_t)n * ldc + m_wave + 8 * rch, v);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
      for (int mt = 0; mt < WT; ++mt) {
        if (add_old && mt + 1 < WT) fetch_old(mt + 1);
        if constexpr (epi_add) {
          if (mt + 1 < WT) fetch_res(mt + 1);
        }
        if constexpr (swiglu_bwd) {
          if (mt + 1 < WT) fetch_x(mt + 1);
        }
        f32x4 vals[WN];  // the only place the accumulators are read
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) {
          vals[nt] = acc[mt][nt];
          asm volatile("" : "+v"(vals[nt]));  // read here, not once in each branch below
          acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        const int64_t blk = (narrow && runs.c_sh ? (int64_t)((m_wave + mt * 16) >> runs.c_sh) * runs.c_outer
                                                 : (int64_t)(m_wave + mt * 16) * ldo) +
                            (narrow ? n_store : n_wave);
        if (narrow) {
          const uint32_t buf = stage + (uint32_t)(mt & 1) * 4096u;
#pragma unroll
          for (int nt = 0; nt < WN; ++nt) {
            bf16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (bf16)vals[nt][e];
            *(KR_LDS bf16x4*)(buf + row16 * 256 + (((2 * nt + (quad >> 1)) ^ row16) << 4) + (quad & 1) * 8) = o;
          }
          if constexpr (swiglu) __syncthreads(); else wave_sync();  // SwiGLU reads the neighbour wave's block too
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int rr = 4 * q + quad;
            bf16x8 v = *(KR_LDS const bf16x8*)(buf + rr * 256 + ((rch ^ rr) << 4));
            const bool in = ncols_in && (rows_in || m_wave + mt * 16 + rr < M);
            if constexpr (epi_add) {
#pragma unroll
              for (int e = 0; e < 8; ++e) v[e] = (bf16)((float)resv[mt & 1][q][e] + (float)v[e]);
            }
            if constexpr (swiglu_bwd) {
              bf16x8 d1, d2;
#pragma unroll
              for (int e = 0; e < 8; ++e) {
                float dg, du;
                kr_swiglu_bwd_f((float)v[e], (float)xg[mt & 1][q][e], (float)xu[mt & 1][q][e], dg, du);
                d1[e] = (bf16)dg;
                d2[e] = (bf16)du;
              }
              if (in) {
                stg8_out(C + blk + nlo[q], d1);
                stg8_out(C + blk + nlo[q] + N, d2);
              }
            } else {
              if (in) stg8_out(C + blk + nlo[q], v);
            }
          }
          if constexpr (swiglu) {
            // the wave beside this one (same rows, other half of the tile) has staged the other
            // operand of the activation for the same 16 rows: this wave takes rows 4 q + quad
            // for q = 2 wn, 2 wn + 1 of the block, reads the gate chunk from the left wave's
            // buffer and the up chunk from the right wave's, and stores out2
            const uint32_t gbuf = r4 + (uint32_t)(2 * wm) * 8192u + (uint32_t)(mt & 1) * 4096u;
            const uint32_t ubuf = gbuf + 8192u;
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
              const int rr = 4 * (2 * wn + qq) + quad;
              const bf16x8 g = *(KR_LDS const bf16x8*)(gbuf + rr * 256 + ((rch ^ rr) << 4));
              const bf16x8 u = *(KR_LDS const bf16x8*)(ubuf + rr * 256 + ((rch ^ rr) << 4));
              bf16x8 y;
#pragma unroll
              for (int e = 0; e < 8; ++e) y[e] = (bf16)kr_swiglu_f((float)g[e], (float)u[e]);
              if (ncols_in && (rows_in || m_wave + mt * 16 + rr < M))
                stg8_out(out2 + (int64_t)(m_wave + mt * 16 + rr) * ld_out2 + out_n0 + 8 * rch, y);
            }
          }
        } else {
#pragma unroll
          for (int nt = 0; nt < WN; ++nt)
            *(KR_LDS f32x4*)(stage + row16 * 512 + (((4 * nt + quad) ^ row16) << 4)) = vals[nt];
          wave_sync();
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const int rr = 2 * q + hrow;
            const f32x4 v = *(KR_LDS const f32x4*)(stage + rr * 512 + ((ch ^ rr) << 4));
            const bool in = cols_in && (rows_in || m_wave + mt * 16 + rr < M);
            if (to_partial) {
              if (in) *reinterpret_cast<f32x4*>(out_partial + blk + lo[q]) = v;
            } else {
              bf16x4 o;
#pragma unroll
              for (int e = 0; e < 4; ++e) o[e] = (bf16)(v[e] + (float)oldc[mt & 1][q][e]);
              if (in) __builtin_nontemporal_store(o, reinterpret_cast<bf16x4*>(C + blk + lo[q]));
            }
          }
          wave_sync();
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the accumulator reads of later blocks below
      }
      }
    }
    if (!more) break;
    item = next;
  }
}

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

// Tile width for an output with enough tiles to occupy the GPU without a split: 32 * WN columns,
// WN in 5..8.  The estimate is the launch's own latency — rounds of tiles over the CUs times the
// cost of a tile (WN units of MFMA work plus about one unit of prologue and epilogue); ties go to
// the wider tile, which reads less from LDS per FLOP.
inline int choose_wn(int M, int N, int num_cus) {
  const int tiles_m = (M + BM - 1) / BM;
  int best = 8;
  long best_cost = 0;
  for (int wn = 8; wn >= 5; --wn) {
    const int tiles = tiles_m * ((N + 32 * wn - 1) / (32 * wn));
    const long cost = (long)((tiles + num_cus - 1) / num_cus) * (wn + 1);
    if (wn == 8 || cost < best_cost) {
      best = wn;
      best_cost = cost;
    }
  }
  return best;
}

// Tile width and number of cuts of the contraction.  An output of at least 192 full-width tiles is
// never cut and takes the width of choose_wn.  A smaller one has too few tiles to occupy the GPU:
// narrower tiles (down to 128 columns; 160 with a fused epilogue) and cuts of the contraction both
// make more work items, and the pair with the least estimated cost wins.  Two estimates, in units of one K-step of a full-width tile (~1.3 us;
// a tile of WN columns takes (WN + 2) / 10 of it):
//   latency  rounds of work items over the CUs, each item paying its K-steps plus a fixed
//            prologue/epilogue, plus the traffic of the fp32 partial tiles (written once, read
//            once by the reduce kernel at ~5 TB/s);
//   CU-time  the same work summed over the CUs it occupies, per CU of the device.
// A GEMM that has the GPU to itself wants the smallest latency (latency_weight 1); one that
// runs beside kernels of other streams, which can use the CUs it leaves idle, should mostly
// keep its CU-time small (the dispatcher uses latency_weight 0.1).  `max_splits` is what the caller's workspace holds.
struct Plan {
  int wn, splits;
};
inline Plan choose_plan(int M, int N, int K, float latency_weight, int num_cus, int max_splits,
                        int min_wn = 4) {
  constexpr int kItemOverhead = 4;
  const int tiles_m = (M + BM - 1) / BM;
  if (tiles_m * ((N + BN - 1) / BN) >= 192) return {choose_wn(M, N, num_cus), 1};
  const double w = latency_weight < 0.f ? 0.0 : (latency_weight > 1.f ? 1.0 : (double)latency_weight);
  const int nk = (K + BK - 1) / BK;
  const double reduce_per_split = (double)M * N * 8.0 / 5.0e12 / 1.3e-6;
  auto cost = [&](int wn, int sp) {
    const int tiles = tiles_m * ((N + 32 * wn - 1) / (32 * wn));
    const int items = tiles * sp, rounds = (items + num_cus - 1) / num_cus;
    const double per_item = (double)((nk + sp - 1) / sp) * (wn + 2) / 10.0 + kItemOverhead;
    const double reduce = sp > 1 ? sp * reduce_per_split : 0.0;
    const double latency = rounds * per_item + reduce;
    const double cu_time = items * per_item / num_cus + reduce;
    return w * latency + (1.0 - w) * cu_time;
  };
  Plan best{8, 1};
  double best_cost = cost(8, 1);
  for (int wn = 7; wn >= min_wn; --wn) {
    const double c = cost(wn, 1);
    if (c < best_cost) {
      best_cost = c;
      best = {wn, 1};
    }
  }
  const double unsplit = best_cost;
  for (int sp = 2; sp <= 16 && sp <= max_splits && nk / sp >= 8; ++sp)
    for (int wn = 8; wn >= min_wn; --wn) {
      const double c = cost(wn, sp);
      if (c < unsplit * 0.95 && c < best_cost) {  // a split must pay for itself clearly
        best_cost = c;
        best = {wn, sp};
      }
    }
  return best;
}

struct Fused {
  int epi = 0;              // KR_GEMM_EPI_*
  const bf16* aux = nullptr;
  int64_t ld_aux = 0;
  bf16* out2 = nullptr;
  int64_t ld_out2 = 0;
  int max_cus = 0;          // > 0: use at most this many compute units
  bool shared = false;      // other streams' kernels use the units this launch leaves idle
  RowRuns runs = {0, 0, 0, 0, 0, 0};  // row runs of A, C, aux (all plain by default)
  const Segments* segs = nullptr;     // layout NT: the operands come in these pieces (A and B are unused)
};

// Tile width for a projection with the SwiGLU epilogue: the tiles have to divide the 2F output
// columns exactly (no partly filled tile column), otherwise as choose_wn.  0: no width fits.
inline int swiglu_wn(int M, int N, int num_cus) {
  const int tiles_m = (M + BM - 1) / BM;
  int best = 0;
  long best_cost = 0;
  for (int wn = 8; wn >= 5; --wn) {
    if (N % (32 * wn)) continue;
    const int tiles = tiles_m * (N / (32 * wn));
    const long cost = (long)((tiles + num_cus - 1) / num_cus) * (wn + 1);
    if (best == 0 || cost < best_cost) {
      best = wn;
      best_cost = cost;
    }
  }
  return best;
}

using GemmKernel = void (*)(const bf16*, int, const bf16*, int, bf16*, int, int, int, int, int, int, int, float*,
                            const bf16*, int, bf16*, int, RowRuns, Segments);

// raises the dynamic-LDS limit of one kernel instance, once (thread-safe static initialisation)
template <GemmKernel FN>
hipError_t raise_lds_limit() {
  static const hipError_t status = hipFuncSetAttribute((const void*)FN, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       (int)(NSLOTS * TILE * sizeof(bf16)));
  return status;
}

template <bool A_T, bool B_T, int WN, int EPI = KR_GEMM_EPI_NONE>
int launch(const bf16* A, int64_t lda, const bf16* B, int64_t ldb, bf16* C, int64_t ldc, int M,
           int N, int K, int accumulate, float* workspace, size_t workspace_bytes,
           hipStream_t stream, int num_cus, const Fused& fu, int planned_splits = 1) {
  constexpr size_t lds_bytes = NSLOTS * TILE * sizeof(bf16);
  if (fu.max_cus > 0 && fu.max_cus < num_cus) num_cus = fu.max_cus;
  const int tiles = ((M + BM - 1) / BM) * ((N + 32 * WN - 1) / (32 * WN));
  // the planned count, which the dispatcher has already capped by what the caller's workspace holds
  int splits = planned_splits;
  const size_t one = (size_t)M * N * sizeof(float);
  if (workspace == nullptr || EPI != KR_GEMM_EPI_NONE) {
    splits = 1;  // a fused epilogue works on finished sums
  } else if ((size_t)splits * one > workspace_bytes) {
    splits = (int)(workspace_bytes / one);
  }
  if (splits < 2 || (int64_t)splits * M * N >= ((int64_t)1 << 31)) splits = 1;
  // at most one persistent workgroup per compute unit (a workgroup owns a whole CU's LDS)
  // Items are spread evenly: with r = ceil(items / CUs) rounds, ceil(items / r) workgroups (rounded
  // up to a multiple of 8, which keeps item ids and XCDs aligned) finish at the same time as one
  // workgroup per CU would, and the CUs left over are free for other streams' kernels from the
  // start of the launch instead of from the end of its first round.
  auto grid_for = [&](int items) {
    if (items <= num_cus) return items;
    const int rounds = (items + num_cus - 1) / num_cus;
    int g = (items + rounds - 1) / rounds;
    g = (g + 7) / 8 * 8;
    return g < num_cus ? g : num_cus;
  };
  const bool with_runs = fu.runs.a_sh || fu.runs.c_sh || fu.runs.x_sh;
  const bool with_segs = fu.segs != nullptr;
  // instances that honour row runs exist for what the two ends of a layer stack launch: the residual-add
  // forward (aux or C in runs), the input gradient (plain or with the SwiGLU backward) and the weight
  // gradient (A in runs); instances that contract operand pieces for the weight gradient (both forms)
  constexpr bool kRunsInstance = EPI == KR_GEMM_EPI_ADD || EPI == KR_GEMM_EPI_SWIGLU_BWD || (EPI == KR_GEMM_EPI_NONE && B_T);
  constexpr bool kSegsInstance = A_T && B_T && (EPI == KR_GEMM_EPI_NONE || EPI == KR_GEMM_EPI_TRANSPOSED_OUT);
  // (pieces in row runs: the direct store form only, A in runs)
  constexpr bool kSegsRunsInstance = kSegsInstance && EPI == KR_GEMM_EPI_NONE;
  if ((with_runs && !kRunsInstance) || (with_segs && !kSegsInstance) || (with_segs && with_runs && !kSegsRunsInstance))
    return KR_EUNSUPPORTED;
  GemmKernel fn = gemm_kernel<A_T, B_T, WN, EPI>;
  hipError_t attr_status = raise_lds_limit<gemm_kernel<A_T, B_T, WN, EPI>>();
  if constexpr (kRunsInstance) {
    if (with_runs) {
      fn = gemm_kernel<A_T, B_T, WN, EPI, true>;
      attr_status = raise_lds_limit<gemm_kernel<A_T, B_T, WN, EPI, true>>();
    }
  }
  if constexpr (kSegsInstance) {
    if (with_segs && !with_runs) {
      fn = gemm_kernel<A_T, B_T, WN, EPI, false, true>;
      attr_status = raise_lds_limit<gemm_kernel<A_T, B_T, WN, EPI, false, true>>();
    }
  }
  if constexpr (kSegsRunsInstance) {
    if (with_segs && with_runs) {
      fn = gemm_kernel<A_T, B_T, WN, EPI, true, true>;
      attr_status = raise_lds_limit<gemm_kernel<A_T, B_T, WN, EPI, true, true>>();
    }
  }
  if (attr_status != hipSuccess) return KR_ELAUNCH;
  const Segments segs = with_segs ? *fu.segs : Segments{};
  if (splits == 1) {
    hipLaunchKernelGGL(fn, dim3(grid_for(tiles)), dim3(NTHREADS), lds_bytes, stream, A, (int)lda, B, (int)ldb, C,
                       (int)ldc, M, N, K, accumulate, 0, 1, (float*)nullptr, fu.aux, (int)fu.ld_aux, fu.out2,
                       (int)fu.ld_out2, fu.runs, segs);
    return kr_launch_status();
  }
  if constexpr (EPI != KR_GEMM_EPI_NONE) return KR_EINVAL;  // (not reached: a fused launch never splits)
  int k_per = (K + splits - 1) / splits;
  k_per = (k_per + BK - 1) / BK * BK;
  splits = (K + k_per - 1) / k_per;
  const int items = tiles * splits;
  // (of the operands only A can be in runs here: an output in runs is never cut)
  hipLaunchKernelGGL(fn, dim3(grid_for(items)), dim3(NTHREADS), lds_bytes, stream, A, (int)lda, B, (int)ldb, C,
                     (int)ldc, M, N, K, 0, k_per, splits, workspace, (const bf16*)nullptr, 0, (bf16*)nullptr, 0,
                     fu.runs, segs);
  if (hipGetLastError() != hipSuccess) return KR_ELAUNCH;
  const int64_t work = (int64_t)M * (N / 8);
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, stream,
                     (const float*)workspace, C, ldc, M, N, splits, accumulate);
  return kr_launch_status();
}

int device_compute_units() {
  static const int num_cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  return num_cus;
}

}  // namespace

extern "C" size_t kr_gemm_workspace_bytes(int layout, int M, int N, int K) {
  (void)layout;
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int splits = choose_plan(M, N, K, 1.f, 256, 16).splits;
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

extern "C" size_t kr_gemm_workspace_bytes_shared(int layout, int M, int N, int K, float latency_weight) {
  (void)layout;
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int splits = choose_plan(M, N, K, latency_weight, 256, 16).splits;
  const int cap = choose_plan(M, N, K, 1.f, 256, 16).splits;
  if (splits > cap) splits = cap;
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

namespace {
int gemm_dispatch(int layout, int M, int N, int K, const void* A, int64_t lda, const void* B,
                  int64_t ldb, void* C, int64_t ldc, int accumulate, void* workspace,
                  size_t workspace_bytes, void* stream, const Fused& fu) {
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
  if (fu.max_cus < 0) return KR_EINVAL;
  // row runs: 2, 4, 8 or 16 rows per run (a 16-row block of the epilogue and a 64-row K-step start
  // at a run's first row), run starts a multiple of 8 elements apart, offsets within 32 bits
  {
    const RowRuns& rr = fu.runs;
    const int shs[3] = {rr.a_sh, rr.c_sh, rr.x_sh}, outers[3] = {rr.a_outer, rr.c_outer, rr.x_outer};
    // (A in pieces: offsets are taken from a piece's own base)
    const int64_t a_rows_in_runs = fu.segs != nullptr ? (int64_t)fu.segs->steps * BK : (layout == KR_GEMM_NT ? K : M);
    const int64_t rows_of[3] = {a_rows_in_runs, M, M};
    for (int i = 0; i < 3; ++i) {
      if (shs[i] == 0) continue;
      if (shs[i] < 0 || shs[i] > 4 || outers[i] <= 0) return KR_EINVAL;
      if (outers[i] % 8 || rows_of[i] % (1 << shs[i])) return KR_EUNSUPPORTED;
      if ((rows_of[i] >> shs[i]) * (int64_t)outers[i] >= (int64_t)1 << 31) return KR_EUNSUPPORTED;
    }
    // the output's runs are honoured by the plain bf16 store only; the second operand of the SwiGLU
    // backward (fc1's saved output) is read as a plain matrix
    if (rr.c_sh && (accumulate || fu.epi == KR_GEMM_EPI_SWIGLU || fu.epi == KR_GEMM_EPI_SWIGLU_BWD)) return KR_EUNSUPPORTED;
    if (rr.x_sh && fu.epi != KR_GEMM_EPI_ADD) return KR_EUNSUPPORTED;
  }
  if (fu.epi != KR_GEMM_EPI_NONE) {
    if (accumulate) return KR_EINVAL;
    if (fu.epi == KR_GEMM_EPI_SWIGLU_BWD) {
      if (layout != KR_GEMM_NN) return KR_EUNSUPPORTED;
      if (!fu.aux || !kr_aligned16(fu.aux) || fu.ld_aux < 2 * (int64_t)N || ldc < 2 * (int64_t)N) return KR_EINVAL;
      if (fu.ld_aux % 8 || fu.ld_aux >= (int64_t)1 << 26) return KR_EUNSUPPORTED;
    } else if (layout != KR_GEMM_TN) {
      return KR_EUNSUPPORTED;  // the other fused epilogues are built for the forward layout
    } else if (fu.epi == KR_GEMM_EPI_ADD) {
      if (!fu.aux || !kr_aligned16(fu.aux) || fu.ld_aux < N) return KR_EINVAL;
      if (fu.ld_aux % 8 || fu.ld_aux >= (int64_t)1 << 26) return KR_EUNSUPPORTED;
    } else if (fu.epi == KR_GEMM_EPI_SWIGLU) {
      if (!fu.out2 || !kr_aligned16(fu.out2) || fu.ld_out2 < N / 2) return KR_EINVAL;
      // the tiles must divide the output exactly: F a multiple of 80, 96, 112 or 128
      if (N % 2 || swiglu_wn(M, N, 256) == 0 || fu.ld_out2 % 8 || fu.ld_out2 >= (int64_t)1 << 26)
        return KR_EUNSUPPORTED;
    } else {
      return KR_EINVAL;
    }
  }
  const bf16* a = (const bf16*)A;
  const bf16* b = (const bf16*)B;
  bf16* c = (bf16*)C;
  float* ws = (float*)workspace;
  hipStream_t st = (hipStream_t)stream;
  const int num_cus = device_compute_units();
  const int cus = fu.max_cus > 0 && fu.max_cus < num_cus ? fu.max_cus : num_cus;
  // cuts of the contraction the caller's workspace can hold (a caller that wants fewer says so by
  // passing the smaller workspace kr_gemm_workspace_bytes_shared sizes); a fused epilogue works on
  // finished sums and is never cut
  int max_splits = 1;
  if (ws != nullptr && fu.epi == KR_GEMM_EPI_NONE && fu.runs.c_sh == 0) {
    const size_t held = workspace_bytes / ((size_t)M * N * sizeof(float));
    max_splits = held > 16 ? 16 : (int)held;
    if (max_splits < 1) max_splits = 1;
  }
  // beside other streams the compute-unit time of the launch counts, hardly its latency
  const Plan plan = choose_plan(M, N, K, fu.shared ? 0.1f : 1.f, cus, max_splits, fu.epi == KR_GEMM_EPI_NONE ? 4 : 5);
  const int wn = fu.epi == KR_GEMM_EPI_SWIGLU ? swiglu_wn(M, N, cus) : plan.wn;
  const int sp = plan.splits;
  if (fu.epi == KR_GEMM_EPI_SWIGLU_BWD) {
    if (lda < K || ldb < N) return KR_EINVAL;
#define KR_GEMM_SWIGLU_BWD(W) \
  return launch<false, true, W, KR_GEMM_EPI_SWIGLU_BWD>(a, lda, b, ldb, c, ldc, M, N, K, 0, ws, workspace_bytes, st, num_cus, fu)
    switch (wn) {
      case 5: KR_GEMM_SWIGLU_BWD(5);
      case 6: KR_GEMM_SWIGLU_BWD(6);
      case 7: KR_GEMM_SWIGLU_BWD(7);
      default: KR_GEMM_SWIGLU_BWD(8);
    }
#undef KR_GEMM_SWIGLU_BWD
  }
  if (fu.epi != KR_GEMM_EPI_NONE) {
    if (lda < K || ldb < K || ldc < N) return KR_EINVAL;
#define KR_GEMM_FUSED(W, E) \
  return launch<false, false, W, E>(a, lda, b, ldb, c, ldc, M, N, K, 0, ws, workspace_bytes, st, num_cus, fu)
    if (fu.epi == KR_GEMM_EPI_SWIGLU) {
      switch (wn) {
        case 5: KR_GEMM_FUSED(5, KR_GEMM_EPI_SWIGLU);
        case 6: KR_GEMM_FUSED(6, KR_GEMM_EPI_SWIGLU);
        case 7: KR_GEMM_FUSED(7, KR_GEMM_EPI_SWIGLU);
        default: KR_GEMM_FUSED(8, KR_GEMM_EPI_SWIGLU);
      }
    }
    switch (wn) {
      case 5: KR_GEMM_FUSED(5, KR_GEMM_EPI_ADD);
      case 6: KR_GEMM_FUSED(6, KR_GEMM_EPI_ADD);
      case 7: KR_GEMM_FUSED(7, KR_GEMM_EPI_ADD);
      default: KR_GEMM_FUSED(8, KR_GEMM_EPI_ADD);
    }
#undef KR_GEMM_FUSED
  }
#define KR_GEMM_LAUNCH(AT, BT)                                                                           \
  switch (wn) {                                                                                          \
    case 4: return launch<AT, BT, 4>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, ws, workspace_bytes, st, num_cus, fu, sp); \
    case 5: return launch<AT, BT, 5>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, ws, workspace_bytes, st, num_cus, fu, sp); \
    case 6: return launch<AT, BT, 6>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, ws, workspace_bytes, st, num_cus, fu, sp); \
    case 7: return launch<AT, BT, 7>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, ws, workspace_bytes, st, num_cus, fu, sp); \
    default: return launch<AT, BT, 8>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, ws, workspace_bytes, st, num_cus, fu, sp); \
  }
  switch (layout) {
    case KR_GEMM_TN:  // A [M,K], B [N,K]
      if (lda < K || ldb < K || ldc < N) return KR_EINVAL;
      KR_GEMM_LAUNCH(false, false)
    case KR_GEMM_NN:  // A [M,K], B [K,N]
      if (lda < K || ldb < N || ldc < N) return KR_EINVAL;
      KR_GEMM_LAUNCH(false, true)
    case KR_GEMM_NT: {  // A [K,M], B [K,N]
      if (lda < M || ldb < N || ldc < N) return KR_EINVAL;
      // Both operands of this layout are read the same way, so C^T = B^T . A is the same kernel
      // with the operands exchanged and a transposing store.  Take that form when its tile grid
      // needs fewer rounds of workgroups (fc1's weight gradient, 7168 x 4096: 448 tiles of
      // 256 x 256 are two rounds on 224 units; transposed, 512 tiles of 256 x 224 are two full
      // rounds of smaller tiles).  Only for a plain store: accumulation and split-K keep the
      // direct form.
      if (!accumulate && fu.runs.a_sh == 0 && fu.runs.c_sh == 0 && ((int64_t)M * lda < ((int64_t)1 << 31)) && M <= (1 << 26)) {
        auto cost = [&](int rows, int cols, int w) {
          const int tiles = ((rows + BM - 1) / BM) * ((cols + 32 * w - 1) / (32 * w));
          return (long)((tiles + cus - 1) / cus) * (w + 1);
        };
        const int wt = choose_wn(N, M, cus);
        const int tiles_direct = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
        const int tiles_trans = ((N + BM - 1) / BM) * ((M + BN - 1) / BN);
        if (tiles_direct >= 192 && tiles_trans >= 192 && cost(N, M, wt) < cost(M, N, wn)) {
          // (operand pieces change places with the operands)
          Segments exchanged{};
          Fused fut = fu;
          if (fu.segs != nullptr) {
            for (int i = 0; i < MAX_SEGMENTS; ++i) {
              exchanged.a[i] = fu.segs->b[i];
              exchanged.b[i] = fu.segs->a[i];
            }
            exchanged.n = fu.segs->n;
            exchanged.steps = fu.segs->steps;
            fut.segs = &exchanged;
          }
#define KR_GEMM_TRANS(W) \
  return launch<true, true, W, KR_GEMM_EPI_TRANSPOSED_OUT>(b, ldb, a, lda, c, ldc, N, M, K, 0, nullptr, 0, st, num_cus, fut)
          switch (wt) {
            case 5: KR_GEMM_TRANS(5);
            case 6: KR_GEMM_TRANS(6);
            case 7: KR_GEMM_TRANS(7);
            default: KR_GEMM_TRANS(8);
          }
#undef KR_GEMM_TRANS
        }
      }
      KR_GEMM_LAUNCH(true, true)
    }
    default:
      return KR_EINVAL;
  }
#undef KR_GEMM_LAUNCH
}
}  // namespace

extern "C" int kr_gemm_bf16(int layout, int M, int N, int K, const void* A, int64_t lda,
                            const void* B, int64_t ldb, void* C, int64_t ldc, int accumulate,
                            void* workspace, size_t workspace_bytes, void* stream) {
  return gemm_dispatch(layout, M, N, K, A, lda, B, ldb, C, ldc, accumulate, workspace, workspace_bytes,
                       stream, Fused{});
}

extern "C" int kr_gemm_bf16_fused(int layout, int M, int N, int K, const void* A, int64_t lda,
                                  const void* B, int64_t ldb, void* C, int64_t ldc, int accumulate,
                                  int epilogue, const void* aux, int64_t ld_aux, void* out2,
                                  int64_t ld_out2, int max_cus, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  Fused fu;
  fu.epi = epilogue & ~KR_GEMM_BESIDE_OTHER_STREAMS;
  fu.shared = (epilogue & KR_GEMM_BESIDE_OTHER_STREAMS) != 0;
  fu.aux = (const bf16*)aux;
  fu.ld_aux = ld_aux;
  fu.out2 = (bf16*)out2;
  fu.ld_out2 = ld_out2;
  fu.max_cus = max_cus;
  return gemm_dispatch(layout, M, N, K, A, lda, B, ldb, C, ldc, accumulate, workspace, workspace_bytes,
                       stream, fu);
}

// The same with row runs (see run_off): A, C and aux may each be a nanobatch of several sequences read or
// written in place in a [s, b, h] tensor.  *_run_rows: rows per run (1 = a plain matrix), a power of two up
// to 16; *_run_ld: distance between the starts of consecutive runs, in elements.
extern "C" int kr_gemm_bf16_runs(int layout, int M, int N, int K, const void* A, int64_t lda,
                                 int a_run_rows, int64_t a_run_ld, const void* B, int64_t ldb, void* C,
                                 int64_t ldc, int c_run_rows, int64_t c_run_ld, int accumulate,
                                 int epilogue, const void* aux, int64_t ld_aux, int aux_run_rows,
                                 int64_t aux_run_ld, void* out2, int64_t ld_out2, int max_cus,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  Fused fu;
  fu.epi = epilogue & ~KR_GEMM_BESIDE_OTHER_STREAMS;
  fu.shared = (epilogue & KR_GEMM_BESIDE_OTHER_STREAMS) != 0;
  fu.aux = (const bf16*)aux;
  fu.ld_aux = ld_aux;
  fu.out2 = (bf16*)out2;
  fu.ld_out2 = ld_out2;
  fu.max_cus = max_cus;
  const int run_rows[3] = {a_run_rows, c_run_rows, aux_run_rows};
  const int64_t run_ld[3] = {a_run_ld, c_run_ld, aux_run_ld};
  int sh[3];
  for (int i = 0; i < 3; ++i) {
    const int r = run_rows[i];
    if (r < 1 || (r & (r - 1))) return KR_EINVAL;
    if (r > 16) return KR_EUNSUPPORTED;
    sh[i] = r == 1 ? 0 : (r == 2 ? 1 : (r == 4 ? 2 : (r == 8 ? 3 : 4)));
    if (sh[i] && (run_ld[i] <= 0 || run_ld[i] >= (int64_t)1 << 31)) return KR_EINVAL;
  }
  fu.runs = {sh[0], sh[0] ? (int)a_run_ld : 0, sh[1], sh[1] ? (int)c_run_ld : 0, sh[2], sh[2] ? (int)aux_run_ld : 0};
  return gemm_dispatch(layout, M, N, K, A, lda, B, ldb, C, ldc, accumulate, workspace, workspace_bytes,
                       stream, fu);
}

// A weight gradient over the nanobatches of a microbatch in one launch: C[M, N] (+)= sum_i A_i^T . B_i with
// A_i [k_seg, M] (row stride lda) and B_i [k_seg, N] (row stride ldb), i < nseg <= KR_GEMM_MAX_SEGMENTS, the
// pieces anywhere in memory.  The same kernels as layout NT of kr_gemm_bf16 on K = nseg * k_seg, with the
// operand base exchanged at every piece boundary; k_seg must be a multiple of 64.  The pieces of A may be in
// row runs (a_run_rows, a_run_ld as in kr_gemm_bf16_runs; 1 = plain).
extern "C" int kr_gemm_bf16_nt_segments(int M, int N, int k_seg, int nseg, const void* const* A, int64_t lda,
                                        int a_run_rows, int64_t a_run_ld, const void* const* B, int64_t ldb,
                                        void* C, int64_t ldc, int accumulate, int flags, int max_cus,
                                        void* workspace, size_t workspace_bytes, void* stream) {
  if (!A || !B || nseg < 1 || nseg > MAX_SEGMENTS || k_seg <= 0) return KR_EINVAL;
  if (flags & ~KR_GEMM_BESIDE_OTHER_STREAMS) return KR_EINVAL;
  if (k_seg % BK) return KR_EUNSUPPORTED;
  if ((int64_t)k_seg * nseg >= (int64_t)1 << 31) return KR_EUNSUPPORTED;
  Segments segs{};
  for (int i = 0; i < nseg; ++i) {
    if (!A[i] || !B[i] || !kr_aligned16(A[i]) || !kr_aligned16(B[i])) return KR_EINVAL;
    segs.a[i] = (const bf16*)A[i];
    segs.b[i] = (const bf16*)B[i];
  }
  segs.n = nseg;
  segs.steps = k_seg / BK;
  Fused fu;
  fu.shared = (flags & KR_GEMM_BESIDE_OTHER_STREAMS) != 0;
  fu.max_cus = max_cus;
  fu.segs = &segs;
  // the pieces of A in row runs (every piece alike): rows per run a power of two up to 16 that divides 64
  if (a_run_rows < 1 || (a_run_rows & (a_run_rows - 1))) return KR_EINVAL;
  if (a_run_rows > 16) return KR_EUNSUPPORTED;
  if (a_run_rows > 1) {
    if (a_run_ld <= 0 || a_run_ld >= (int64_t)1 << 31) return KR_EINVAL;
    int sh = 0;
    while ((1 << sh) < a_run_rows) ++sh;
    fu.runs.a_sh = sh;
    fu.runs.a_outer = (int)a_run_ld;
  }
  return gemm_dispatch(KR_GEMM_NT, M, N, k_seg * nseg, A[0], lda, B[0], ldb, C, ldc, accumulate, workspace,
                       workspace_bytes, stream, fu);
}
