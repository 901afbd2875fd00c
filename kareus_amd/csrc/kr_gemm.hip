// bf16 GEMM on the gfx950 matrix cores: C[M,N] = A . B with fp32 accumulation, bf16 store.
//
// Roofline: MFMA (v_mfma_f32_32x32x16_bf16, 32768 FLOP per wave instruction).  Algorithmic
// work per launch is 2*M*N*K FLOP.
//
// Structure
//   * A workgroup owns a BM x BN tile of C and walks K in steps of 64.  Waves form a WM x WN
//     grid; each wave owns TM x TN MFMA tiles of 32x32 and keeps them in accumulator
//     registers for the whole K loop.
//   * Operand tiles are staged in LDS, double-buffered: while the matrix cores work on
//     K-step i from one buffer, the global loads of step i+1 are in flight into registers
//     and are written to the other buffer afterwards — one barrier per K-step.
//   * Global loads are 16-byte vectors along whichever dimension is contiguous in memory, so
//     every layout reads full cache lines.  An operand whose contraction dimension is the
//     contiguous one ("K-major") is fetched from LDS with ds_read_b128; an operand whose
//     contraction dimension is the row index ("transposed", the weight in dgrad and both
//     operands in wgrad) is fetched with the gfx950 transposing LDS read ds_read_b64_tr_b16,
//     which returns, per lane, four consecutive contraction elements of one output row from
//     a tile stored row-per-contraction-index.  No transposed copy of any operand is made.
//   * The MFMA is issued with the operands swapped (the B tile feeds the instruction's A
//     port), so a lane ends up with four consecutive N-columns of one C row: the epilogue
//     stores 8-byte bf16 quads contiguous along the row.
//   * LDS rows are padded (K-major: 64 -> 72 elements; transposed: +32 elements) so that the
//     16 lanes served together hit distinct banks for both the vector stores and the
//     fragment reads.
//   * Workgroup ids are remapped so that the 32 tiles resident on one XCD (ids congruent
//     mod 8) form a compact GROUP_M x n rectangle of C and share A/B panels in that XCD's L2.
#include <mutex>

#include "kr_common.h"

namespace {

constexpr int BK = 64;
constexpr int LDK = BK + 8;  // padded row length (elements) of a K-major LDS tile
constexpr int kXcds = 8;
constexpr int kGroupM = 4;

template <int ROWS>
struct TileGeom {
  // K-major:    [ROWS][LDK]
  // transposed: [BK][ROWS + 32]
  static constexpr int LDT = ROWS + 32;
  static constexpr int ELEMS = ROWS * LDK;  // == BK * LDT when ROWS == 256; take the max
  static constexpr int ELEMS_T = BK * LDT;
  static constexpr int SIZE = ELEMS > ELEMS_T ? ELEMS : ELEMS_T;
};

// ---- global -> registers -> LDS staging of one operand tile -------------------------------
template <int ROWS, bool TRANSPOSED, int NT>
struct Stager {
  static constexpr int CHUNKS = ROWS * BK / 8;
  static constexpr int PER_THREAD = CHUNKS / NT;
  static_assert(CHUNKS % NT == 0, "tile must divide evenly over the threads");
  bf16x8 regs[PER_THREAD];

  // rows_total: extent of the non-contraction dimension; k_total: contraction extent
  __device__ __forceinline__ void load(const bf16* __restrict__ base, int64_t ld, int row0, int k0,
                                       int rows_total, int k_total, int tid) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = tid + i * NT;
      if (!TRANSPOSED) {
        const int r = c >> 3, kc = (c & 7) * 8;
        const bool ok = (row0 + r < rows_total) && (k0 + kc < k_total);
        regs[i] = ok ? ldg8(base + (int64_t)(row0 + r) * ld + k0 + kc) : zero8();
      } else {
        constexpr int CPR = ROWS / 8;  // chunks per contraction row
        const int kr = c / CPR, rc = (c % CPR) * 8;
        const bool ok = (k0 + kr < k_total) && (row0 + rc < rows_total);
        regs[i] = ok ? ldg8(base + (int64_t)(k0 + kr) * ld + row0 + rc) : zero8();
      }
    }
  }
  __device__ __forceinline__ void store(bf16* tile, int tid) const {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = tid + i * NT;
      if (!TRANSPOSED) {
        const int r = c >> 3, kc = (c & 7) * 8;
        *reinterpret_cast<bf16x8*>(tile + r * LDK + kc) = regs[i];
      } else {
        constexpr int CPR = ROWS / 8;
        const int kr = c / CPR, rc = (c % CPR) * 8;
        *reinterpret_cast<bf16x8*>(tile + kr * TileGeom<ROWS>::LDT + rc) = regs[i];
      }
    }
  }
};

// ---- LDS -> MFMA operand fragment: lane gets row (row0 + lane%32), k = 16*kk + 8*(lane/32)+0..7
template <int ROWS, bool TRANSPOSED>
__device__ __forceinline__ bf16x8 read_frag(const bf16* tile, int row0, int kk, int lane) {
  if (!TRANSPOSED) {
    return *reinterpret_cast<const bf16x8*>(tile + (row0 + (lane & 31)) * LDK + kk * 16 +
                                            (lane >> 5) * 8);
  } else {
    // Transposing read: within each group of 16 lanes, lane p supplies the address of 4
    // consecutive rows-of-C elements in contraction row (p/4); lane p receives element p of
    // the 16 covered rows-of-C for the group's 4 contraction rows.
    constexpr int LDT = TileGeom<ROWS>::LDT;
    const int p = lane & 15;
    const int krow = kk * 16 + (lane >> 5) * 8 + (p >> 2);
    const int col = row0 + ((lane >> 4) & 1) * 16 + (p & 3) * 4;
    const bf16* a0 = tile + krow * LDT + col;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a0));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a0 + 4 * LDT));
    union {
      struct { s16x4 lo, hi; } s;
      bf16x8 v;
    } u;
    u.s.lo = lo;
    u.s.hi = hi;
    return u.v;
  }
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

template <bool A_T, bool B_T, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_kernel(const bf16* __restrict__ A, int64_t lda,
                                                          const bf16* __restrict__ B, int64_t ldb,
                                                          bf16* __restrict__ C, int64_t ldc, int M,
                                                          int N, int K, int accumulate) {
  constexpr int NT = WM * WN * 64;
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr int A_SIZE = TileGeom<BM>::SIZE, B_SIZE = TileGeom<BN>::SIZE;
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];
  constexpr int STAGE = A_SIZE + B_SIZE;  // buffer s: A tile at s*STAGE, B tile right after it

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  int tile_m, tile_n;
  remap_block(blockIdx.x, tiles_m * tiles_n, tiles_m, tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  f32x16 acc[TN][TM];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[j][i][e] = 0.f;

  Stager<BM, A_T, NT> sa;
  Stager<BN, B_T, NT> sb;
  const int nk = (K + BK - 1) / BK;

  sa.load(A, lda, m0, 0, M, K, tid);
  sb.load(B, ldb, n0, 0, N, K, tid);
  sa.store(smem, tid);
  sb.store(smem + A_SIZE, tid);
  __syncthreads();

  for (int ks = 0; ks < nk; ++ks) {
    const int cur = ks & 1;
    if (ks + 1 < nk) {
      sa.load(A, lda, m0, (ks + 1) * BK, M, K, tid);
      sb.load(B, ldb, n0, (ks + 1) * BK, N, K, tid);
    }
    const bf16* at = smem + cur * STAGE;
    const bf16* bt = at + A_SIZE;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = read_frag<BM, A_T>(at, (wm * TM + i) * 32, kk, lane);
#pragma unroll
      for (int j = 0; j < TN; ++j) bfr[j] = read_frag<BN, B_T>(bt, (wn * TN + j) * 32, kk, lane);
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[j][i], 0, 0, 0);
    }
    if (ks + 1 < nk) {
      sa.store(smem + (cur ^ 1) * STAGE, tid);
      sb.store(smem + (cur ^ 1) * STAGE + A_SIZE, tid);
    }
    __syncthreads();
  }

  // epilogue: lane holds C[m][n..n+3] for m = tile row (lane%32), n = 8g + 4*(lane/32)
  const int h = lane >> 5;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + (wm * TM + i) * 32 + (lane & 31);
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + (wn * TN + j) * 32 + 8 * g + 4 * h;
        if (n >= N) continue;
        bf16* dst = C + (int64_t)m * ldc + n;
        bf16x4 o;
        if (accumulate) {
          const bf16x4 old = *reinterpret_cast<const bf16x4*>(dst);
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (bf16)(acc[j][i][g * 4 + e] + (float)old[e]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (bf16)acc[j][i][g * 4 + e];
        }
        *reinterpret_cast<bf16x4*>(dst) = o;
      }
    }
  }
}

template <bool A_T, bool B_T, int WM, int WN, int TM, int TN>
int launch(const bf16* A, int64_t lda, const bf16* B, int64_t ldb, bf16* C, int64_t ldc, int M,
           int N, int K, int accumulate, hipStream_t stream) {
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr size_t lds_bytes = 2 * (TileGeom<BM>::SIZE + TileGeom<BN>::SIZE) * sizeof(bf16);
  auto kernel = gemm_kernel<A_T, B_T, WM, WN, TM, TN>;
  static std::once_flag once;
  static hipError_t attr_status = hipSuccess;
  std::call_once(once, [&] {
    attr_status = hipFuncSetAttribute((const void*)kernel,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  });
  if (attr_status != hipSuccess) return KR_ELAUNCH;
  const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  hipLaunchKernelGGL(kernel, dim3(tiles), dim3(WM * WN * 64), lds_bytes, stream, A, lda, B, ldb, C,
                     ldc, M, N, K, accumulate);
  return kr_launch_status();
}

}  // namespace

extern "C" int kr_gemm_bf16(int layout, int M, int N, int K, const void* A, int64_t lda,
                            const void* B, int64_t ldb, void* C, int64_t ldc, int accumulate,
                            void* stream) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return KR_EINVAL;
  if (!kr_aligned16(A) || !kr_aligned16(B) || !kr_aligned16(C)) return KR_EINVAL;
  if ((M | N | K) % 8 || (lda | ldb | ldc) % 8) return KR_EUNSUPPORTED;
  const bf16* a = (const bf16*)A;
  const bf16* b = (const bf16*)B;
  bf16* c = (bf16*)C;
  hipStream_t st = (hipStream_t)stream;
  switch (layout) {
    case KR_GEMM_TN:  // A [M,K], B [N,K]
      if (lda < K || ldb < K || ldc < N) return KR_EINVAL;
      return launch<false, false, 2, 4, 4, 2>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, st);
    case KR_GEMM_NN:  // A [M,K], B [K,N]
      if (lda < K || ldb < N || ldc < N) return KR_EINVAL;
      return launch<false, true, 2, 4, 4, 2>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, st);
    case KR_GEMM_NT:  // A [K,M], B [K,N]
      if (lda < M || ldb < N || ldc < N) return KR_EINVAL;
      return launch<true, true, 2, 4, 4, 2>(a, lda, b, ldb, c, ldc, M, N, K, accumulate, st);
    default:
      return KR_EINVAL;
  }
}
