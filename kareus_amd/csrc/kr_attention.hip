// Causal grouped-query flash attention for head_dim 128 on the gfx950 matrix cores.
//
// Roofline: MFMA.  Algorithmic work: forward 2*b*nq*s^2*hd FLOP (causal half of 4*s^2*hd),
// backward 2.5x that.
//
// Forward (attn_fwd_pp_kernel below).  A workgroup of 8 waves owns 128 consecutive queries of
// one (batch, query head); wave w and wave w + 4 own the same 32 of them and walk the even /
// odd 64-key tiles, in antiphase, merging their softmax partials at the end.
//   S^T = K . Q^T is computed with K rows on the MFMA A port and the wave's Q fragment (held
//   in registers for the whole kernel) on the B port, so a lane ends up with 16 scores per
//   32-key tile *of a single query row* (row = lane % 32; lanes l and l+32 split the keys).
//   The online-softmax row maximum and row sum are therefore in-lane reductions plus one
//   exchange between the two half-waves.
//   O^T += V^T . P^T: the probabilities are already laid out as the B-port operand (the
//   contraction index of an MFMA can be permuted freely as long as both operands agree), and
//   V^T fragments come out of LDS through the transposing read ds_read_b64_tr_b16.  Neither
//   P nor V is ever transposed through memory.
// Tensors are addressed through (seq, batch, head) strides, so sequence-major [s, b, h, d]
// views of the fused QKV projection are consumed in place.
#include <initializer_list>

#include "kr_common.h"

namespace {

constexpr int HD = 128;
constexpr int BQ = 128;       // queries per workgroup (4 waves x 32, twice over)
constexpr int BKV = 64;       // keys per staged tile
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// Online softmax of the MFMA forward kernels: a row's exponents are taken against a reference
// point that follows the running maximum only when the maximum has grown by more than this many
// powers of two.  In between, probabilities run up to 2^8 instead of 1 — rounding is relative in
// fp32 and in bf16, the row sum and the output carry the same factor and the final division takes
// it out — and the 64 accumulator multiplies of a rescale are skipped (with 32 rows per wave some
// row's maximum moves in most tiles; by more than 2^8 it hardly ever does after the first).
constexpr float kRescaleSlack = 8.0f;
constexpr int kXcds = 8;

__device__ __forceinline__ int xcd_contiguous_id(int pid, int nblocks) {
  const int q = nblocks / kXcds, r = nblocks % kXcds;
  const int xcd = pid % kXcds;
  return xcd * q + (xcd < r ? xcd : r) + pid / kXcds;
}

// Workgroup -> (query tile, (batch, head) pair), longest causal rows first.  With fewer than 32
// tiles per pair an XCD starts its 32 compute units on the longest tiles of `grp` pairs at once,
// and the short tiles that follow land on the units that finish first.
__device__ __forceinline__ void longest_first(int lid, int nqt, int total_pairs, int& qt, int& pair) {
  const int grp = (nqt < 32 && 32 % nqt == 0) ? 32 / nqt : 1;
  const int span = grp * nqt, base = lid / span, i = lid % span;
  if ((base + 1) * grp <= total_pairs) {
    qt = nqt - 1 - i / grp;
    pair = base * grp + i % grp;
  } else {  // a last, incomplete group keeps the plain order
    qt = nqt - 1 - (lid % nqt);
    pair = lid / nqt;
  }
}

// Output staging.  After the MFMAs a lane holds, for its row (lane % 32), groups of four
// consecutive channels; stored from there an instruction scatters 64 small pieces over 32 rows
// and the texture-address path takes them one at a time.  Each wave therefore passes its
// results through 4 KB of LDS of its own (32 rows of 128 bytes, 16-byte chunks XOR-swizzled
// against bank conflicts) and reads them back as whole rows, 8 lanes per row, so an
// instruction writes 8 contiguous 128-byte segments.  Only lanes of one wave exchange data:
// the program order of its LDS instructions is all the ordering needed.
struct RowStage {
  char* base;
  int wr, wsw, h, rrow, rch;
  __device__ __forceinline__ void init(void* lds4k, int lane) {
    base = reinterpret_cast<char*>(lds4k);
    const int r = lane & 31;
    h = lane >> 5;
    wr = r * 128;
    wsw = (r >> 1) & 7;
    rrow = lane >> 3;
    rch = lane & 7;
  }
  static __device__ __forceinline__ void sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
  }
  // bf16 pass = 32 rows x 64 channels: block j (0/1) of 32 channels, group g of the MFMA layout
  __device__ __forceinline__ void put_bf16(int j, int g, bf16x4 v) const {
    *reinterpret_cast<bf16x4*>(base + wr + (((4 * j + g) ^ wsw) << 4) + 8 * h) = v;
  }
  // read q (0..3): row 8q + lane/8 of the pass, channels 8*(lane%8) .. +7
  __device__ __forceinline__ bf16x8 get_bf16(int q, int& row, int& col) const {
    row = 8 * q + rrow;
    col = 8 * rch;
    return *reinterpret_cast<const bf16x8*>(base + row * 128 + ((rch ^ ((row >> 1) & 7)) << 4));
  }
  // fp32 pass = 32 rows x 32 channels
  __device__ __forceinline__ void put_f32(int g, f32x4 v) const {
    *reinterpret_cast<f32x4*>(base + wr + (((2 * g + h) ^ wsw) << 4)) = v;
  }
  __device__ __forceinline__ f32x4 get_f32(int q, int& row, int& col) const {
    row = 8 * q + rrow;
    col = 4 * rch;
    return *reinterpret_cast<const f32x4*>(base + row * 128 + ((rch ^ ((row >> 1) & 7)) << 4));
  }
};

// 32 rows x 128 channels of fp32 accumulators (scaled) -> bf16 rows at dst + row * row_stride
__device__ __forceinline__ void store_rows_bf16(const RowStage& st, const f32x16 (&acc)[HD / 32],
                                                float mul, bf16* dst, int64_t row_stride) {
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bf16x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (bf16)(acc[2 * pass + j][g * 4 + e] * mul);
        st.put_bf16(j, g, v);
      }
    RowStage::sync();
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int row, col;
      const bf16x8 v = st.get_bf16(q, row, col);
      stg8(dst + (int64_t)row * row_stride + pass * 64 + col, v);
    }
    RowStage::sync();
  }
}

// the same as fp32 rows (partial results for a later reduction)
__device__ __forceinline__ void store_rows_f32(const RowStage& st, const f32x16 (&acc)[HD / 32],
                                               float mul, float* dst, int64_t row_stride) {
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f32x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = acc[dt][g * 4 + e] * mul;
      st.put_f32(g, v);
    }
    RowStage::sync();
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int row, col;
      const f32x4 v = st.get_f32(q, row, col);
      *reinterpret_cast<f32x4*>(dst + (int64_t)row * row_stride + dt * 32 + col) = v;
    }
    RowStage::sync();
  }
}

}  // namespace

static int check_attn_common(int s, int b, int nq, int nkv, int hd) {
  if (s <= 0 || b <= 0 || nq <= 0 || nkv <= 0) return KR_EINVAL;
  if (hd <= 0 || hd % 8 || hd > 128 || nq % nkv) return KR_EUNSUPPORTED;
  if (b > 65535 || nq > 65535) return KR_EUNSUPPORTED;  // grid dimensions of the general kernels
  return KR_OK;
}
// The MFMA kernels take head dimension 128 and whole 128-row tiles; everything else that passes
// check_attn_common goes through the general fp32 kernels.
static bool attn_fast_path(int s, int hd) { return hd == HD && s % BQ == 0; }

static int kr_compute_units() {
  static const int num_cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  return num_cus;
}

// The kernels keep a sequence stride in 32 bits and build per-lane byte offsets of up to
// (48 * stride + 128) * 2 from it: strides must be positive and small enough for that.
template <size_t N>
inline bool attn_strides_ok(const int64_t (&seq)[N], std::initializer_list<int64_t> others) {
  for (int64_t ss : seq)
    if (ss <= 0 || 48 * ss + 128 >= ((int64_t)1 << 31)) return false;
  for (int64_t st : others)
    if (st <= 0) return false;
  return true;
}

// =============================================================================================
// Backward.  Launches: delta pre-pass, dK/dV pass, (group reduction), dQ pass — or, with 256-query
// tiles, the one-wave dQ kernel first (it computes delta itself), then dK/dV and the group
// reduction.  No atomics, deterministic.
//   1. delta[b, h, i] = sum_d dO[i, d] * O[i, d]                      (HBM-bound pre-pass)
//   2. dK, dV: a workgroup owns 128 keys of one (batch, QUERY head) — 32 per pair of waves,
//      their K and V fragments in the registers of the pair's score wave, dK and dV in those of
//      its accumulate wave — and streams every query tile at or below the diagonal through LDS.
//      Per 32x32 block:
//        S = Q.K^T, dP = dO.V^T (rows = queries on the MFMA A port, so a lane holds one key
//        column), P = exp2(S*c - lse), dS = P*(dP - delta), then dV^T += dO^T.P and
//        dK^T += Q^T.dS with the Q / dO tiles read back transposed (ds_read_b64_tr_b16).
//      With grouped-query attention several query heads share a KV head: each workgroup
//      writes an fp32 partial for its query head and a small HBM-bound kernel sums the
//      partials of a group (one query head per KV head: bf16 results are written directly).
//      Splitting by query head rather than looping over the group keeps enough workgroups in
//      flight when one GPU holds only a few KV heads (a tensor-parallel shard).
//   3. dQ: a workgroup owns 128 queries of one (batch, head) and streams the key tiles up to
//      the diagonal: S^T = K.Q^T, dP^T = V.dO^T (a lane holds one query row), dS^T, then
//      dQ^T += K^T.dS^T with the K tile read back transposed.
//   Recomputing S and dP in both passes costs 7 instead of 5 tile products but keeps every
//   accumulator in registers and every output written exactly once.
// Every K / V / Q / dO tile is staged straight from global memory into a blocked LDS tile that
// can be read both ways (as rows and transposed) without bank conflicts; see bt_request below.
// =============================================================================================
namespace {


// query-like tensors: head h of KV group g = h / per sits at g*g_ + (h % per)*h_
struct QLayout {
  int64_t s_, b_, g_, h_;
  __device__ __forceinline__ int64_t at(int bi, int head, int per) const {
    return (int64_t)bi * b_ + (head / per) * g_ + (head % per) * h_;
  }
};
struct KLayout {
  int64_t s_, b_, h_;
  __device__ __forceinline__ int64_t at(int bi, int kvh) const { return (int64_t)bi * b_ + kvh * h_; }
};

// Scalar loads return out of order, so while one is pending (a kernel argument fetched in the
// prologue and first used behind the loop is, as far as the compiler's wait-count pass knows, for
// the whole loop) every wait for an LDS read becomes lgkmcnt(0): the first MFMA of a group then
// waits for the fragments of the next group too.  An explicit lgkmcnt(0) in front of a loop ends
// that: inside, the waits count.
__device__ __forceinline__ void settle_scalar_loads() { __builtin_amdgcn_s_waitcnt(0xc07f); }

// ---- direct global -> LDS loads (see the GEMM for why they are written as inline assembly:
// the compiler must not know of them, or it drains them in front of every barrier).  The 64
// lanes of one load land contiguously: lane p at lds_byte + 16 p.
__device__ __forceinline__ void dma_b128(const void* base, uint32_t byte_off, uint32_t lds_byte) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_byte), "v"(byte_off), "s"(base)
               : "memory", "m0");
}

// 4 bytes per lane: lane p lands at lds_byte + 4 p
__device__ __forceinline__ void dma_b32(const void* base, uint32_t byte_off, uint32_t lds_byte) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(lds_byte), "v"(byte_off), "s"(base)
               : "memory", "m0");
}

// ---- blocked LDS tile: [64 rows][128 channels] bf16, filled straight from global memory ------
// A tile is 16 blocks; block B holds rows r, r+16, r+32, r+48 (r = 4 (B % 4) + B / 4), 256 bytes
// each, in the order one wave-wide request delivers them (lane p at +16 p: row r + 16 (p / 16),
// 16-byte chunk p % 16 — 16 consecutive lanes fetch one contiguous row), then 16 bytes of
// padding.  Both ways of reading fragments out of it are free of bank conflicts, and every
// fragment address is one per-lane base plus an instruction immediate.
constexpr uint32_t BT_BLK = 1024 + 16, BT_BYTES = 16 * BT_BLK;

// The four waves (wave = 0..3) of a group bring in one tile; `rows` = its first row in global
// memory.  Wave w fills blocks w, w + 4, w + 8, w + 12, which hold the tile rows 4 w + 0..3
// (+ 16, 32, 48): four consecutive rows, so a request costs one pointer increment.
__device__ __forceinline__ void bt_request(const bf16* rows, int64_t ss, uint32_t tile, int wave,
                                           int lane) {
  int l2 = lane;
  asm volatile("" : "+v"(l2));  // nothing derived from it is kept alive between requests
  const uint32_t lane_off = (uint32_t)((l2 >> 4) * 16 * (int)ss + (l2 & 15) * 8) * 2u;
  const bf16* row = rows + (int64_t)(4 * wave) * ss;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    dma_b128(row, lane_off, tile + (wave + 4 * i) * BT_BLK);
    row += ss;
  }
}
// row-major fragments: lane gets row 32 t + lane % 32, channels 16 kk + 8 (lane / 32) + 0..7
__device__ __forceinline__ uint32_t bt_rows_lane(int lane) {
  const int r = lane & 31;
  return (uint32_t)((4 * (r & 3) + ((r >> 2) & 3)) * BT_BLK + (r >> 4) * 256 + (lane >> 5) * 16);
}
__device__ __forceinline__ bf16x8 bt_rows(uint32_t base, int t, int kk) {
  return *(KR_LDS const bf16x8*)(base + t * 512 + kk * 32);
}
// transposed fragments: lane gets channel 32 dt + lane % 32, rows 16 g + {4 h + 0..3, 8 + 4 h + 0..3}
__device__ __forceinline__ uint32_t bt_cols_lane(int lane) {
  const int p = lane & 15;
  return (uint32_t)((4 * (p >> 2) + (lane >> 5)) * BT_BLK + ((lane >> 4) & 1) * 32 +
                    ((p & 3) >> 1) * 16 + (p & 1) * 8);
}
__device__ __forceinline__ bf16x8 bt_cols(uint32_t base, int g, int dt) {
  union {
    struct { s16x4 lo, hi; } s;
    bf16x8 v;
  } u;
  const uint32_t a = base + g * 256 + dt * 64;
  u.s.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a));
  u.s.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a + 2 * BT_BLK));
  return u.v;
}

// Ping-pong forward.  Two halves of four waves own the same 128 queries and walk the even / odd
// key tiles (their partial softmax results are merged at the end, half 1 handing its state to
// half 0 through LDS), but the halves run in antiphase.  Time is cut into periods by workgroup
// barriers; in every period one half only feeds the matrix pipe — P.V of its previous tile, then
// S = Q.K^T of its next one, 32 MFMAs — while the other half does everything else for its own
// tile: the softmax (exponentials, row statistics, rounding to bf16, the occasional rescale of
// the output accumulators) and the requests for the K / V tiles two steps ahead, which go
// straight from global memory into blocked [64][128] LDS tiles.  A SIMD hosts one wave of each
// half, so its matrix pipe and its vector ALU are busy at the same time instead of taking
// turns, which is what happens when co-resident waves are in the same phase.
__global__ __launch_bounds__(512, 1) void attn_fwd_pp_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k, const bf16* __restrict__ v,
    bf16* __restrict__ o, float* __restrict__ lse, int s, int nq, int nkv, float scale_log2,
    int64_t q_ss, int64_t q_sb, int64_t q_sg, int64_t q_sh, int64_t k_ss, int64_t k_sb,
    int64_t k_sh, int64_t v_ss, int64_t v_sb, int64_t v_sh, int64_t o_ss, int64_t o_sb,
    int64_t o_sg, int64_t o_sh) {
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];

  const int half = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8));
  const int tid = threadIdx.x & 255;
  const int lane = tid & 63, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nqt = s / BQ;
  const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int qt = nqt - 1 - (lid % nqt);  // longest rows first inside each (batch, head)
  const int head = (lid / nqt) % nq;
  const int bi = lid / (nqt * nq);
  const int per = nq / nkv;
  const int kvh = head / per, hj = head % per;

  const int q0 = qt * BQ;
  const int qw0 = q0 + wave * 32;
  const int qrow = qw0 + (lane & 31);
  const bf16* qp = q + (int64_t)bi * q_sb + kvh * q_sg + hj * q_sh + (int64_t)qrow * q_ss;
  const bf16* kb = k + (int64_t)bi * k_sb + (int64_t)kvh * k_sh;
  const bf16* vb = v + (int64_t)bi * v_sb + (int64_t)kvh * v_sh;

  bf16x8 qf[HD / 16];
#pragma unroll
  for (int kk = 0; kk < HD / 16; ++kk) qf[kk] = ldg8(qp + kk * 16 + h * 8);

  f32x16 oacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const int nsteps = (q0 + BQ) / (2 * BKV);  // key tiles per half
  // LDS tile = 16 blocks; block b holds rows b, b+16, b+32, b+48 of the tile, 256 bytes each, in
  // the order one wave-wide request delivers them (lane p at +16 p: row b + 16 (p / 16), chunk
  // p % 16 — 16 consecutive lanes fetch one contiguous row), followed by a little padding.  With
  // the padding chosen per operand (K: 16 bytes, V: 64) both kinds of fragment reads are free of
  // bank conflicts, and every fragment address is one per-lane base plus an instruction
  // immediate.  Per half: K tile j in kbuf + (j & 1) tiles, V tile j in vbuf + (j & 1) tiles.
  constexpr uint32_t KBLK = 1024 + 16, VBLK = 1024 + 64, KTILE = 16 * KBLK, VTILE = 16 * VBLK;
  const uint32_t kbuf = (uint32_t)(uintptr_t)(KR_LDS const bf16*)smem + half * 2 * (KTILE + VTILE);
  const uint32_t vbuf = kbuf + 2 * KTILE;
  auto key_of = [&](int j) { return (2 * j + half) * BKV; };
  // row-major fragment (K): row 32 t + lane%32, chunk 2 kk + h  ->  + 512 t + 32 kk
  const uint32_t kfrag_lane = (uint32_t)((lane & 15) * KBLK + ((lane >> 4) & 1) * 256 + h * 16);
  // transposed fragment (V): rows 16 g + 4 h + p/4 (+8), channels 32 dt + 16 (lane/16 % 2) +
  // 4 (p % 4)  ->  + 256 g + 64 dt (+ 8 blocks)
  const uint32_t vfrag_lane = (uint32_t)((4 * h + ((lane & 15) >> 2)) * VBLK + ((lane >> 4) & 1) * 32 +
                                         ((lane & 3) >> 1) * 16 + (lane & 1) * 8);

  // One wave requests 4 KiB of a tile: blocks wave + 4 i, i.e. tile rows wave + 4 i (+ 16, 32,
  // 48).  Everything a request needs is kept ready — a pointer to row `wave` of the next tile to
  // ask for, advanced by two tiles per step, the distance of four rows, the lane's byte offset —
  // so that a request costs a handful of scalar instructions: the vector period is bound by the
  // number of instructions the wave has to issue.
  const bf16* kreq = kb + (int64_t)(key_of(0) + wave) * k_ss;
  const bf16* vreq = vb + (int64_t)(key_of(0) + wave) * v_ss;
  const int64_t k_tiles2 = (int64_t)2 * BKV * k_ss, v_tiles2 = (int64_t)2 * BKV * v_ss;
  const int64_t k_rows4 = 4 * k_ss, v_rows4 = 4 * v_ss;
  const uint32_t k_lane_off = (uint32_t)((lane >> 4) * 16 * (int)k_ss + (lane & 15) * 8) * 2u;
  const uint32_t v_lane_off = (uint32_t)((lane >> 4) * 16 * (int)v_ss + (lane & 15) * 8) * 2u;
  auto request = [&](const bf16* row, int64_t rows4, uint32_t lane_off, uint32_t tile, uint32_t blk_bytes) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dma_b128(row, lane_off, tile + (wave + 4 * i) * blk_bytes);
      row += rows4;
    }
  };
  auto request_k = [&](uint32_t tile) {
    request(kreq, k_rows4, k_lane_off, tile, KBLK);
    kreq += k_tiles2;
  };
  auto request_v = [&](uint32_t tile) {
    request(vreq, v_rows4, v_lane_off, tile, VBLK);
    vreq += v_tiles2;
  };
  // one of a tile's four requests of this wave (i = 0..3); the last one moves on to the next tile
  auto request_k_part = [&](uint32_t tile, int i) {
    dma_b128(kreq + i * k_rows4, k_lane_off, tile + (wave + 4 * i) * KBLK);
    if (i == 3) kreq += k_tiles2;
  };
  auto request_v_part = [&](uint32_t tile, int i) {
    dma_b128(vreq + i * v_rows4, v_lane_off, tile + (wave + 4 * i) * VBLK);
    if (i == 3) vreq += v_tiles2;
  };

  request_k(kbuf);
  if (nsteps > 1) request_k(kbuf + KTILE);
  request_v(vbuf);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  if (half == 1) __syncthreads();  // half 1 starts one period late

  bf16x8 pb[2][2];

  // O^T += V^T . P^T for tile jj of this half (pb holds its probabilities)
  auto pv_step = [&](int jj) {
      uint32_t va = vbuf + (jj & 1) * VTILE + vfrag_lane;
      asm volatile("" : "+v"(va));  // one base register; everything else is an immediate
      auto vfrag = [&](int g, int dt) {  // keys 16 g .. 16 g + 15 of the tile, channels 32 dt ..
        union {
          struct { s16x4 lo, hi; } s;
          bf16x8 v;
        } u;
        const uint32_t a = va + g * 256 + dt * 64;
        u.s.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a));
        u.s.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a + 8 * VBLK));
        return u.v;
      };
      // fragments are fetched one group of four MFMAs ahead, by hand: left to itself the
      // scheduler hoists every read of the period to its start and runs out of registers
      bf16x8 fr[2][HD / 32];
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt) fr[0][dt] = vfrag(0, dt);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (g + 1 < 4) {
#pragma unroll
          for (int dt = 0; dt < HD / 32; ++dt) fr[(g + 1) & 1][dt] = vfrag(g + 1, dt);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
          oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[g & 1][dt], pb[g >> 1][g & 1],
                                                             oacc[dt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      };

  settle_scalar_loads();
  for (int j = 0; j < nsteps; ++j) {
    // ---- matrix period: O^T += V^T . P^T of tile j-1, then S^T = K . Q^T of tile j
    f32x16 sacc[2];
    __builtin_amdgcn_s_setprio(1);
    if (j > 0) pv_step(j - 1);
    {
      uint32_t ka = kbuf + (j & 1) * KTILE + kfrag_lane;
      asm volatile("" : "+v"(ka));
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) sacc[t][e] = 0.f;
      auto kfrag = [&](int t, int kk) { return *(KR_LDS const bf16x8*)(ka + t * 512 + kk * 32); };
      bf16x8 fr[2][4];  // group g: contraction steps 2g, 2g+1 for both 32-key blocks
#pragma unroll
      for (int u = 0; u < 4; ++u) fr[0][u] = kfrag(u & 1, u >> 1);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (g + 1 < 4) {
#pragma unroll
          for (int u = 0; u < 4; ++u) fr[(g + 1) & 1][u] = kfrag(u & 1, 2 * (g + 1) + (u >> 1));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 4; ++u)
          sacc[u & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[g & 1][u], qf[2 * g + (u >> 1)],
                                                                sacc[u & 1], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    __syncthreads();

    // ---- vector period of tile j: the softmax, and between its eight groups of exponentials
    // the eight requests for K(j+2) and V(j+1) (their buffers were last read in the matrix period
    // that just ended).  Issued back to back the requests hold the wave until the address path
    // has taken them, which is as long as the softmax itself.
    const bool want_k = j + 2 < nsteps, want_v = j + 1 < nsteps;
    const uint32_t k_dst = kbuf + (j & 1) * KTILE, v_dst = vbuf + ((j + 1) & 1) * VTILE;
    {
      const int key0 = key_of(j);
      if (key0 + BKV - 1 > qw0) {
        asm volatile("" ::: "memory");  // keeps this a branch: off the diagonal no mask code runs
        const int lim = qrow - key0 - 4 * h;  // element offsets beyond it are keys after the query
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int e = 0; e < 16; ++e)
            if (t * 32 + 8 * (e >> 2) + (e & 3) > lim) sacc[t][e] = -INFINITY;
      }
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sacc[t][e]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, KR_WAVE));
      const float m_new = fmaxf(m_run, mx);
      const bool moved = (m_new - m_run) * scale_log2 > kRescaleSlack;  // from -inf: always
      const float m_next = moved ? m_new : m_run;
      const float m_ref = m_next == -INFINITY ? 0.f : m_next;  // nothing seen yet: any finite reference
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_ref) * scale_log2);  // 1 unless moved
      m_run = m_next;
      const float neg_m = -m_ref * scale_log2;
      float psum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[t][e], scale_log2, neg_m));
          psum += pe;
          pb[t][e >> 3][e & 7] = (bf16)pe;
          // eight elements at a time: scheduled freely, all 32 exponent arguments and results
          // would be alive together
          if ((e & 7) == 7) {
            __builtin_amdgcn_sched_barrier(0);
            const int c = t * 2 + (e >> 3);   // 0..3
            if (want_k) request_k_part(k_dst, c);
            if (want_v) request_v_part(v_dst, c);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      l_run = l_run * alpha + psum;
      if (__any(moved)) {
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
          for (int e = 0; e < 16; ++e) oacc[dt][e] *= alpha;
      }
    }
    // what was requested one step ago (K(j+1), V(j)) is read in the next matrix period; exactly
    // the requests of this period (4 per tile and wave, retired in order) may stay in flight
    if (j + 2 < nsteps)
      __builtin_amdgcn_s_waitcnt(0x0f78);  // vmcnt(8): K(j+2) and V(j+1) were requested
    else if (j + 1 < nsteps)
      __builtin_amdgcn_s_waitcnt(0x0f74);  // vmcnt(4): only V(j+1)
    else
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): nothing was requested
    __syncthreads();
  }
  // last matrix period: the product of the final tile
  __builtin_amdgcn_s_setprio(1);
  pv_step(nsteps - 1);
  __builtin_amdgcn_s_setprio(0);
  __syncthreads();
  if (half == 0) __syncthreads();  // the period half 1 is behind by

  // merge the two halves' partial softmax: half 1 -> LDS -> half 0 (every buffer is idle: the
  // loop ended with a barrier and no request is in flight).  [value][wave][lane] layout.
  float* xch = reinterpret_cast<float*>(smem);
  const int slot = wave * 64 + lane;
  if (half == 1) {
    xch[slot] = m_run;
    xch[256 + slot] = l_run;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) xch[(2 + dt * 16 + e) * 256 + slot] = oacc[dt][e];
  }
  __syncthreads();
  if (half == 1) return;
  {
    const float m_b = xch[slot], l_b = xch[256 + slot];
    const float m_new = fmaxf(m_run, m_b);
    const float a_a = __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2);
    const float a_b = __builtin_amdgcn_exp2f((m_b - m_new) * scale_log2);
    m_run = m_new;
    l_run = l_run * a_a + l_b * a_b;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e)
        oacc[dt][e] = oacc[dt][e] * a_a + xch[(2 + dt * 16 + e) * 256 + slot] * a_b;
  }
  const float l_tot = l_run + __shfl_xor(l_run, 32, KR_WAVE);
  const float inv_l = 1.0f / l_tot;
  RowStage rs;  // behind the (2 + 64) KiB hand-over buffer
  rs.init(reinterpret_cast<char*>(smem) + 68 * 1024 + wave * 4096, lane);
  bf16* op = o + (int64_t)bi * o_sb + kvh * o_sg + hj * o_sh + (int64_t)qw0 * o_ss;
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[dt][e] *= inv_l;
  store_rows_bf16(rs, oacc, 1.0f, op, o_ss);
  if (h == 0)
    lse[((int64_t)bi * nq + head) * s + qrow] =
        (m_run * scale_log2 + __builtin_amdgcn_logf(l_tot)) * kLn2;
}

// Ping-pong forward over shared tiles, for launches with enough 256-query tiles to fill the GPU.
// The two halves of four waves own *different* queries (rows 0..127 and 128..255 of the tile) and
// walk the *same* 64-key tiles, half 1 one period behind half 0: a K / V tile is fetched once for
// 256 queries instead of once for 128, there are half as many workgroups to start and to finish,
// and the halves never have to merge anything.  Periods as above: in each, one half feeds the
// matrix pipe (P.V of its previous tile, S = Q.K^T of its next) and the other does its softmax;
// half 0 requests the K tiles during its softmax (K(j+2) while it works on tile j), half 1 the V
// tiles (V(j+2)).  K(j) is read in periods 2j (half 0) and 2j+1 (half 1), V(j) in 2j+2 and 2j+3;
// rings of three tiles each give every request three to four periods to land.  Half 0 needs two
// tiles fewer than half 1 (its rows end 128 earlier) and idles through the last two steps.
__global__ __launch_bounds__(512, 1) void attn_fwd_sh_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k, const bf16* __restrict__ v,
    bf16* __restrict__ o, float* __restrict__ lse, int s, int nq, int nkv, float scale_log2,
    int64_t q_ss, int64_t q_sb, int64_t q_sg, int64_t q_sh, int64_t k_ss, int64_t k_sb,
    int64_t k_sh, int64_t v_ss, int64_t v_sb, int64_t v_sh, int64_t o_ss, int64_t o_sb,
    int64_t o_sg, int64_t o_sh) {
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];
  constexpr int BQ2 = 256;

  const int half = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8));
  const int tid = threadIdx.x & 255;
  const int lane = tid & 63, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nqt = s / BQ2;
  int qt, pair;
  longest_first(xcd_contiguous_id(blockIdx.x, gridDim.x), nqt, gridDim.x / nqt, qt, pair);
  const int head = pair % nq;
  const int bi = pair / nq;
  const int per = nq / nkv;
  const int kvh = head / per, hj = head % per;

  const int q0 = qt * BQ2;
  const int qw0 = q0 + half * 128 + wave * 32;
  const int qrow = qw0 + (lane & 31);
  const bf16* qp = q + (int64_t)bi * q_sb + kvh * q_sg + hj * q_sh + (int64_t)qrow * q_ss;
  const bf16* kb = k + (int64_t)bi * k_sb + (int64_t)kvh * k_sh;
  const bf16* vb = v + (int64_t)bi * v_sb + (int64_t)kvh * v_sh;

  bf16x8 qf[HD / 16];
#pragma unroll
  for (int kk = 0; kk < HD / 16; ++kk) qf[kk] = ldg8(qp + kk * 16 + h * 8);

  f32x16 oacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const int ntiles = (q0 + BQ2) / BKV;                // tiles the workgroup walks (>= 4)
  const int nmine = (q0 + half * 128 + 128) / BKV;    // tiles with keys this half's rows see
  constexpr uint32_t KBLK = 1024 + 16, VBLK = 1024 + 64, KTILE = 16 * KBLK, VTILE = 16 * VBLK;
  const uint32_t kring = (uint32_t)(uintptr_t)(KR_LDS const bf16*)smem;
  const uint32_t vring = kring + 3 * KTILE;
  const uint32_t kfrag_lane = (uint32_t)((lane & 15) * KBLK + ((lane >> 4) & 1) * 256 + h * 16);
  const uint32_t vfrag_lane = (uint32_t)((4 * h + ((lane & 15) >> 2)) * VBLK + ((lane >> 4) & 1) * 32 +
                                         ((lane & 3) >> 1) * 16 + (lane & 1) * 8);

  // This half's requests: half 0 brings in K tiles, half 1 V tiles; block b of a tile holds its
  // rows b, b + 16, b + 32, b + 48 and wave w fills blocks w + 4 i.  `req` points at row w of the
  // next tile to ask for.
  const int64_t r_ss = half ? v_ss : k_ss;
  const uint32_t r_blk = half ? VBLK : KBLK, r_tile = half ? VTILE : KTILE;
  const uint32_t r_ring = half ? vring : kring;
  const bf16* req = (half ? vb : kb) + (int64_t)wave * r_ss;
  const int64_t r_next = (int64_t)BKV * r_ss, r_rows4 = 4 * r_ss;
  const uint32_t r_lane_off = (uint32_t)((lane >> 4) * 16 * (int)r_ss + (lane & 15) * 8) * 2u;
  auto request_part = [&](uint32_t tile, int i) {
    dma_b128(req + i * r_rows4, r_lane_off, tile + (wave + 4 * i) * r_blk);
    if (i == 3) req += r_next;
  };
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) request_part(r_ring + t * r_tile, i);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  if (half == 1) __syncthreads();  // half 1 starts one period late

  bf16x8 pb[2][2];

  // O^T += V^T . P^T for the tile in ring slot `slot` (pb holds its probabilities)
  auto pv_step = [&](int slot) {
    uint32_t va = vring + slot * VTILE + vfrag_lane;
    asm volatile("" : "+v"(va));
    auto vfrag = [&](int g, int dt) {
      union {
        struct { s16x4 lo, hi; } s;
        bf16x8 v;
      } u;
      const uint32_t a = va + g * 256 + dt * 64;
      u.s.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a));
      u.s.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((KR_LDS s16x4*)(a + 8 * VBLK));
      return u.v;
    };
    bf16x8 fr[2][HD / 32];
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt) fr[0][dt] = vfrag(0, dt);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (g + 1 < 4) {
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) fr[(g + 1) & 1][dt] = vfrag(g + 1, dt);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
        oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[g & 1][dt], pb[g >> 1][g & 1],
                                                           oacc[dt], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  int slot = 0, slot_prev = 2, slot_req = 2;  // j % 3, (j - 1) % 3, (j + 2) % 3
  settle_scalar_loads();
  for (int j = 0; j < ntiles; ++j) {
    // ---- matrix period: O^T += V^T . P^T of tile j-1, then S^T = K . Q^T of tile j
    f32x16 sacc[2];
    const bool mine = j < nmine;
    __builtin_amdgcn_s_setprio(1);
    if (j > 0 && j - 1 < nmine) pv_step(slot_prev);
    if (mine) {
      uint32_t ka = kring + slot * KTILE + kfrag_lane;
      asm volatile("" : "+v"(ka));
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) sacc[t][e] = 0.f;
      auto kfrag = [&](int t, int kk) { return *(KR_LDS const bf16x8*)(ka + t * 512 + kk * 32); };
      bf16x8 fr[2][4];
#pragma unroll
      for (int u = 0; u < 4; ++u) fr[0][u] = kfrag(u & 1, u >> 1);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (g + 1 < 4) {
#pragma unroll
          for (int u = 0; u < 4; ++u) fr[(g + 1) & 1][u] = kfrag(u & 1, 2 * (g + 1) + (u >> 1));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 4; ++u)
          sacc[u & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[g & 1][u], qf[2 * g + (u >> 1)],
                                                                sacc[u & 1], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    __syncthreads();

    // ---- vector period of tile j: the softmax, and between its four groups of exponentials
    // this wave's four requests for tile j+2 of its operand (the ring slot was last read two
    // periods ago).  Half 0 has no request left once it has run out of tiles of its own.
    const bool want = j + 2 < ntiles;
    const uint32_t r_dst = r_ring + slot_req * r_tile;
    if (mine) {
      const int key0 = j * BKV;
      if (key0 + BKV - 1 > qw0) {
        asm volatile("" ::: "memory");  // keeps this a branch: off the diagonal no mask code runs
        const int lim = qrow - key0 - 4 * h;  // element offsets beyond it are keys after the query
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int e = 0; e < 16; ++e)
            if (t * 32 + 8 * (e >> 2) + (e & 3) > lim) sacc[t][e] = -INFINITY;
      }
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sacc[t][e]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, KR_WAVE));
      const float m_new = fmaxf(m_run, mx);
      const bool moved = (m_new - m_run) * scale_log2 > kRescaleSlack;  // from -inf: always
      const float m_next = moved ? m_new : m_run;
      const float m_ref = m_next == -INFINITY ? 0.f : m_next;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_ref) * scale_log2);  // 1 unless moved
      m_run = m_next;
      const float neg_m = -m_ref * scale_log2;
      float psum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[t][e], scale_log2, neg_m));
          psum += pe;
          pb[t][e >> 3][e & 7] = (bf16)pe;
          if ((e & 7) == 7) {
            __builtin_amdgcn_sched_barrier(0);
            if (want) request_part(r_dst, t * 2 + (e >> 3));
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      l_run = l_run * alpha + psum;
      if (__any(moved)) {
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
          for (int e = 0; e < 16; ++e) oacc[dt][e] *= alpha;
      }
    } else if (want) {
#pragma unroll
      for (int i = 0; i < 4; ++i) request_part(r_dst, i);
    }
    // tile j+1 of this half's operand (requested one step ago) is read from the next period on;
    // only this period's four requests may stay in flight
    if (want)
      __builtin_amdgcn_s_waitcnt(0x0f74);  // vmcnt(4)
    else
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    __syncthreads();
    slot_prev = slot;
    slot = slot == 2 ? 0 : slot + 1;
    slot_req = slot_req == 2 ? 0 : slot_req + 1;
  }
  // last matrix period: the product of the final tile (half 1; half 0 finished two steps ago)
  if (ntiles - 1 < nmine) {
    __builtin_amdgcn_s_setprio(1);
    pv_step(slot_prev);
    __builtin_amdgcn_s_setprio(0);
  }
  if (half == 0) __syncthreads();  // the barrier half 1 spent on starting late

  // No tile is requested any more and K tiles are no longer read: each wave stages its output
  // rows through 4 KiB of the K ring.
  const float l_tot = l_run + __shfl_xor(l_run, 32, KR_WAVE);
  const float inv_l = 1.0f / l_tot;
  RowStage rs;
  rs.init(reinterpret_cast<char*>(smem) + (half * 4 + wave) * 4096, lane);
  bf16* op = o + (int64_t)bi * o_sb + kvh * o_sg + hj * o_sh + (int64_t)qw0 * o_ss;
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[dt][e] *= inv_l;
  store_rows_bf16(rs, oacc, 1.0f, op, o_ss);
  if (h == 0)
    lse[((int64_t)bi * nq + head) * s + qrow] =
        (m_run * scale_log2 + __builtin_amdgcn_logf(l_tot)) * kLn2;
}

__global__ __launch_bounds__(256) void attn_delta_kernel(const bf16* __restrict__ dout,
                                                         const bf16* __restrict__ o,
                                                         const float* __restrict__ lse,
                                                         float* __restrict__ delta,
                                                         float* __restrict__ neg_lse2, int s, int nq,
                                                         int per, int64_t total_rows, QLayout dol,
                                                         QLayout ol) {
  // 16 lanes per (batch, head, position) row of 128 channels
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 4;
  const int sub = threadIdx.x & 15;
  if (row >= total_rows) return;
  const int si = (int)(row % s);
  const int head = (int)((row / s) % nq);
  const int bi = (int)(row / ((int64_t)s * nq));
  const bf16x8 a = ldg8(dout + dol.at(bi, head, per) + (int64_t)si * dol.s_ + sub * 8);
  const bf16x8 b = ldg8(o + ol.at(bi, head, per) + (int64_t)si * ol.s_ + sub * 8);
  float acc = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) acc += (float)a[e] * (float)b[e];
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) acc += __shfl_xor(acc, off, KR_WAVE);
  if (sub == 0) {
    delta[row] = acc;
    // -lse in the log2 domain, so that the dK/dV kernel's exponent is one multiply-add and its
    // row statistics can go straight from global memory into LDS
    neg_lse2[row] = -lse[row] * kLog2e;
  }
}

// dK/dV with the waves of a SIMD specialised.  A wave issues at most one instruction every 4-5
// cycles, and one wave that does everything for its 32 keys (scores, exponentials, both
// accumulating products) needs 128 accumulator and 64 K/V-fragment registers — no room for a
// second wave on the SIMD — so it is bound by that rate: 850 instructions per 64 MFMAs.  Instead
// a workgroup has eight waves, two per SIMD, for its 128 keys:
//   waves 0-3 ("score" waves, 32 keys each, K and V fragments in registers) compute S = Q.K^T and
//     dP = dO.V^T of a 32-query block, P and dS from them, and hand P, dS (bf16, already in the
//     B-operand layout of the next products) to their partner through 4 KB of LDS;
//   waves 4-7 ("accumulate" waves, the partner on the same SIMD) hold dK and dV and issue
//     dV^T += dO^T.P and dK^T += Q^T.dS with the Q / dO tiles read transposed; they also issue
//     every global -> LDS request, which keeps the score waves' instruction stream short.
// Both run well below 256 registers, so the matrix products write plain VGPRs (no accumulator
// copies).  Two barriers per 64-query tile: after each, the accumulate waves pick up the block
// the score waves finished before it, so the two kinds of work overlap with one block of lag.
// Three LDS stages: tile it is read as rows by the score waves and transposed by the accumulate
// waves; every read of it is issued before the second barrier of iteration it, so tile it+3 is
// requested right after that barrier into the same stage and has an iteration and a half to
// land (it must be complete by the first barrier of iteration it+2: the score waves start on a
// tile one block ahead).
// PARTIAL = true: fp32 results for this query head go to part_k / part_v [b, nq, qsplit, s, 128].
template <bool PARTIAL>
__global__ __launch_bounds__(512, 1) void attn_bwd_dkdv_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k, const bf16* __restrict__ v,
    const bf16* __restrict__ dout, const float* __restrict__ neg_lse2, const float* __restrict__ delta,
    bf16* __restrict__ dk, bf16* __restrict__ dv, float* __restrict__ part_k,
    float* __restrict__ part_v, int s, int nq, int nkv, int qsplit, int hpw, float scale, float scale_log2,
    QLayout ql, KLayout kl, KLayout vl, QLayout dol, KLayout dkl, KLayout dvl) {
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];
  // stage layout: Q tile | dO tile (blocked tiles) | lse[64] fp32 | delta[64] fp32
  constexpr uint32_t STAGE = 2 * BT_BYTES + 512;  // bytes
  constexpr int NS = 3;
  // hand-over area behind the stages: [block parity][key block][slot 0..3][lane] 16 bytes each
  constexpr uint32_t XCH = NS * STAGE;

  const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5;
  const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int role = wave8 >> 2;  // 0: score wave, 1: accumulate wave
  const int wave = wave8 & 3;   // key block of the tile
  const int nkt = s / 128;
  const int lid_all = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int part = lid_all % qsplit, lid = lid_all / qsplit;
  // A workgroup takes `hpw` consecutive query heads of one KV group, one after the other: its K / V
  // fragments and its dK / dV accumulators serve them all, so a group leaves per / hpw partial
  // results instead of per (none at all when hpw = per), and the workgroup's start and end are
  // paid once for hpw heads.  The host picks hpw so that enough workgroups remain.
  const int kt = lid % nkt;  // low key tiles see the most queries: they come first
  const int nhg = nq / hpw;
  const int hgroup = (lid / nkt) % nhg;
  const int head = hgroup * hpw;  // the first of this workgroup's heads
  const int bi = lid / (nkt * nhg);
  const int per = nq / nkv;
  const int kvh = head / per;
  const int key0 = kt * 128;
  const int kw0 = key0 + wave * 32;
  const int krow = kw0 + (lane & 31);
  const int qt_first = key0 / 64;
  const int niter = (s / 64 - qt_first - part + qsplit - 1) / qsplit;  // this part's query tiles of 64, per head
  const int nit_all = niter * hpw;                                       // ... over all heads of the workgroup
  const uint32_t lds0 = (uint32_t)(uintptr_t)(KR_LDS const bf16*)smem;
  const uint32_t xch_lane = lds0 + XCH + wave * 4096 + lane * 16;  // + parity * 16384 + slot * 1024

  if (role == 0) {
    // ------------------------------------------------------------------ score waves
    const bf16* kp = k + kl.at(bi, kvh) + (int64_t)krow * kl.s_;
    const bf16* vp = v + vl.at(bi, kvh) + (int64_t)krow * vl.s_;
    bf16x8 kf[HD / 16], vf[HD / 16];
#pragma unroll
    for (int kk = 0; kk < HD / 16; ++kk) {
      kf[kk] = ldg8(kp + kk * 16 + h * 8);
      vf[kk] = ldg8(vp + kk * 16 + h * 8);
    }
    __syncthreads();  // tile 0 (and 1) requested by the accumulate waves have landed
    // S = Q.K^T and dP = dO.V^T of one 32-query block: sixteen fragments, then sixteen MFMAs
    auto issue_scores = [&](int stage, int sub, f32x16& sacc, f32x16& dpacc) {
      uint32_t q_rows = lds0 + stage * STAGE + bt_rows_lane(lane);
      uint32_t do_rows = q_rows + BT_BYTES;
      asm volatile("" : "+v"(q_rows), "+v"(do_rows));  // one base register each; the rest are immediates
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        sacc[e] = 0.f;
        dpacc[e] = 0.f;
      }
      bf16x8 qfr[HD / 16], dofr[HD / 16];
#pragma unroll
      for (int kk = 0; kk < HD / 16; ++kk) {
        qfr[kk] = bt_rows(q_rows, sub, kk);
        dofr[kk] = bt_rows(do_rows, sub, kk);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = 0; kk < HD / 16; ++kk) {
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qfr[kk], kf[kk], sacc, 0, 0, 0);
        dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dofr[kk], vf[kk], dpacc, 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    // One step: P = exp2(S c - lse), dS = P (dP - delta) of block (stage, sub), handed to the
    // partner wave, while the score products of the block after it (nstage, nsub) are issued.
    // A wave's instructions issue in order and an MFMA waits for the matrix pipe, so sixteen
    // MFMAs in a row stall the wave for as long as they take; four at a time between the four
    // groups of exponentials they cost (almost) nothing.
    auto step = [&](int stage, int sub, int qs0, f32x16& sacc, const f32x16& dpacc, int nstage, int nsub,
                    f32x16& nsacc, f32x16& ndpacc) {
      const float* stats = reinterpret_cast<const float*>(reinterpret_cast<const char*>(smem) +
                                                          stage * STAGE + 2 * BT_BYTES);
      uint32_t q_rows = lds0 + nstage * STAGE + bt_rows_lane(lane);
      uint32_t do_rows = q_rows + BT_BYTES;
      asm volatile("" : "+v"(q_rows), "+v"(do_rows));
      bf16x8 qfr[HD / 16], dofr[HD / 16];
#pragma unroll
      for (int kk = 0; kk < HD / 16; ++kk) {
        qfr[kk] = bt_rows(q_rows, nsub, kk);
        dofr[kk] = bt_rows(do_rows, nsub, kk);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        nsacc[e] = 0.f;
        ndpacc[e] = 0.f;
      }
      // lane: key column krow, query rows qs0 + 8g + 4h + e; only blocks that reach the diagonal
      // pay for the causal mask
      if (qs0 < kw0 + 31) {
        const int lim = krow - qs0 - 4 * h;  // element offsets below it are queries before the key
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          float x = 8 * (e >> 2) + (e & 3) < lim ? -INFINITY : sacc[e];
          asm volatile("" : "+v"(x));  // keeps this a branch: off the diagonal no mask code runs
          sacc[e] = x;
        }
      }
      bf16x8 pb[2], dsb[2];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(stats + sub * 32 + 8 * g + 4 * h);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(stats + 64 + sub * 32 + 8 * g + 4 * h);
#pragma unroll
        for (int kk = 2 * g; kk < 2 * g + 2; ++kk) {
          nsacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qfr[kk], kf[kk], nsacc, 0, 0, 0);
          ndpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dofr[kk], vf[kk], ndpacc, 0, 0, 0);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[g * 4 + e], scale_log2, l4[e]));
          const float ds = p * (dpacc[g * 4 + e] - d4[e]);
          pb[g >> 1][(g & 1) * 4 + e] = (bf16)p;
          dsb[g >> 1][(g & 1) * 4 + e] = (bf16)ds;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      const uint32_t xa = xch_lane + sub * 16384;
      *(KR_LDS bf16x8*)(xa) = pb[0];
      *(KR_LDS bf16x8*)(xa + 1024) = pb[1];
      *(KR_LDS bf16x8*)(xa + 2048) = dsb[0];
      *(KR_LDS bf16x8*)(xa + 3072) = dsb[1];
    };
    // The score products of a block are thus issued one block ahead of the exponentials that
    // consume them (the first block of the next tile during the second block of this one: that
    // tile is complete by the first barrier of the iteration; behind the last tile a stale
    // stage is read, unused).
    f32x16 s0, dp0, s1, dp1;
    settle_scalar_loads();
    issue_scores(0, 0, s0, dp0);
    for (int it = 0, itl = 0; it < nit_all; ++it) {
      const int stage = it % NS;
      const int q0 = (qt_first + itl * qsplit + part) * 64;
      itl = itl + 1 == niter ? 0 : itl + 1;  // the next head starts over at the diagonal
      step(stage, 0, q0, s0, dp0, stage, 1, s1, dp1);
      __syncthreads();  // hand-over of block 0
      step(stage, 1, q0 + 32, s1, dp1, (it + 1) % NS, 0, s0, dp0);
      __syncthreads();  // hand-over of block 1
    }
    return;
  }

  // -------------------------------------------------------------------- accumulate waves
  const bf16* qb = q + ql.at(bi, head, per);
  const bf16* dob = dout + dol.at(bi, head, per);
  const int64_t stat0 = ((int64_t)bi * nq + head) * s;
  // A tile is brought in by nine requests per wave (eight for waves 2 and 3): the 64 + 64 row
  // statistics, 4 bytes per lane, by waves 0 and 1, then four consecutive rows (+ 16, 32, 48
  // through the lanes) of the Q tile and four of the dO tile.  request_begin names the tile,
  // request_piece(i) issues piece i = 0..8, in this order (requests retire in order).
  uint32_t req_tile = 0, req_lane_off = 0;
  const bf16* req_row = nullptr;
  const bf16 *req_q = qb, *req_do = dob;
  int64_t req_stat = stat0;
  int req_qt = 0;
  auto request_begin = [&](int it) {
    const int hh = it / niter, itl = it - hh * niter;  // head of the workgroup, query tile of that head
    req_qt = qt_first + itl * qsplit + part;
    req_tile = lds0 + (it % NS) * STAGE;
    req_q = qb + hh * ql.h_;    // consecutive heads of one KV group
    req_do = dob + hh * dol.h_;
    req_stat = stat0 + (int64_t)hh * s;
  };
  auto request_piece = [&](int i) {
    if (i == 0) {
      if (wave < 2) {
        int l2 = lane;
        asm volatile("" : "+v"(l2));
        dma_b32((wave == 0 ? neg_lse2 : delta) + req_stat + req_qt * 64, (uint32_t)l2 * 4u,
                req_tile + 2 * BT_BYTES + wave * 256);
      }
      return;
    }
    const int j = (i - 1) & 3;
    const bool second = i > 4;
    if (j == 0) {
      int l2 = lane;
      asm volatile("" : "+v"(l2));  // the lane offset lives only across the four requests of a tile
      const int64_t ss = second ? dol.s_ : ql.s_;
      req_lane_off = (uint32_t)((l2 >> 4) * 16 * (int)ss + (l2 & 15) * 8) * 2u;
      req_row = (second ? req_do : req_q) + ((int64_t)req_qt * 64 + 4 * wave) * ss;
    }
    dma_b128(req_row, req_lane_off, req_tile + (second ? BT_BYTES : 0) + (wave + 4 * j) * BT_BLK);
    req_row += second ? dol.s_ : ql.s_;
  };
  auto request_tile = [&](int it) {
    request_begin(it);
#pragma unroll
    for (int i = 0; i < 9; ++i) request_piece(i);
  };
  // wait until at most the requests of one tile (the newest) are in flight
  auto wait_all_but_newest_tile = [&]() {
    if (wave < 2)
      __builtin_amdgcn_s_waitcnt(0x0f79);  // vmcnt(9)
    else
      __builtin_amdgcn_s_waitcnt(0x0f78);  // vmcnt(8)
  };
  f32x16 dkacc[HD / 32], dvacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      dkacc[dt][e] = 0.f;
      dvacc[dt][e] = 0.f;
    }
  request_tile(0);
  if (nit_all > 1) request_tile(1);
  if (nit_all > 2) {
    request_tile(2);
    wait_all_but_newest_tile();
  } else {
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  }
  __syncthreads();
  // The sixteen transposed fragments of a block (fr[8 k2 + 2 dt]: dO^T, fr[8 k2 + 2 dt + 1]: Q^T,
  // queries 16 k2 .. of the block, channels 32 dt ..) live in registers across blocks: each is
  // refilled for the next block right behind the MFMA that consumed it (one MFMA later), so the
  // LDS reads of the next block ride under this block's matrix work and the wave reaches the
  // next barrier with its operands already there.
  const uint32_t cols_lane = bt_cols_lane(lane);
  auto frag = [&](uint32_t stage_base, int sub, int f) {
    const uint32_t base = stage_base + ((f & 1) ? 0u : BT_BYTES);  // odd: Q tile, even: dO tile
    return bt_cols(base, 2 * sub + (f >> 3), (f >> 1) & 3);
  };
  bf16x8 fr[16];
  {
    uint32_t base = lds0 + cols_lane;
    asm volatile("" : "+v"(base));
#pragma unroll
    for (int f = 0; f < 16; ++f) fr[f] = frag(base, 0, f);
  }
  settle_scalar_loads();
  for (int it = 0; it < nit_all; ++it) {
    const int stage = it % NS;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      // tile it+1 (requested an iteration and a half ago) must have landed before this
      // iteration's first barrier: the score waves start on it right after.  Tile it+2 may still
      // be on its way.
      if (sub == 0 && it > 0) {  // (tiles 0 and 1 were awaited before the loop)
        if (it + 2 < nit_all) {
          // in flight behind tile it+1: the first five pieces of tile it+2
          if (wave < 2)
            __builtin_amdgcn_s_waitcnt(0x0f75);  // vmcnt(5)
          else
            __builtin_amdgcn_s_waitcnt(0x0f74);  // vmcnt(4)
        } else {
          __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
        }
      }
      __syncthreads();
      // After the second barrier nobody reads tile it any more (this wave fetched its last
      // fragments of it during the first block, the score waves before the first barrier):
      // tile it+3 goes into its stage, one request behind each of the first MFMAs — pieces 0-4
      // in this block, pieces 5-8 in the first block of the next iteration, so that neither
      // block of the accumulate waves outlasts the score waves' step beside it.
      const bool first_pieces = sub == 1 && it + 3 < nit_all;
      const bool last_pieces = sub == 0 && it > 0 && it + 2 < nit_all;
      if (first_pieces) request_begin(it + 3);
      const uint32_t xa = xch_lane + sub * 16384;
      bf16x8 hand[4];  // P (queries 0-15, 16-31 of the block), dS (the same)
#pragma unroll
      for (int c = 0; c < 4; ++c) hand[c] = *(KR_LDS const bf16x8*)(xa + c * 1024);
      // next block: the second of this tile, or the first of the next tile (complete since this
      // iteration's first barrier; behind the last tile a stale stage, unused)
      uint32_t next_base = lds0 + (sub == 0 ? stage : (it + 1) % NS) * STAGE + cols_lane;
      asm volatile("" : "+v"(next_base));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int f = 0; f < 16; ++f) {
        const int dt = (f >> 1) & 3;
        if (f & 1)
          dkacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[f], hand[2 + (f >> 3)], dkacc[dt], 0, 0, 0);
        else
          dvacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[f], hand[f >> 3], dvacc[dt], 0, 0, 0);
        if (f > 0) fr[f - 1] = frag(next_base, sub ^ 1, f - 1);
        if (first_pieces && f < 5) request_piece(f);
        if (last_pieces && f < 4) request_piece(5 + f);
        __builtin_amdgcn_sched_barrier(0);
      }
      fr[15] = frag(next_base, sub ^ 1, 15);
    }
  }

  // The hand-over slice this wave read last is its own: use the other one (block parity 0, read
  // one barrier earlier by this wave only) for the output transposition.
  RowStage rs;
  rs.init(reinterpret_cast<char*>(smem) + XCH + wave * 4096, lane);
  if (PARTIAL) {
    const int64_t prow = (((int64_t)bi * nhg + hgroup) * qsplit + part) * s + kw0;
    store_rows_f32(rs, dkacc, scale, part_k + prow * HD, HD);
    store_rows_f32(rs, dvacc, 1.0f, part_v + prow * HD, HD);
  } else {
    store_rows_bf16(rs, dkacc, scale, dk + dkl.at(bi, kvh) + (int64_t)kw0 * dkl.s_, dkl.s_);
    store_rows_bf16(rs, dvacc, 1.0f, dv + dvl.at(bi, kvh) + (int64_t)kw0 * dvl.s_, dvl.s_);
  }
}

// dk/dv[b, kvh, i, :] = sum over the group's query heads of the fp32 partials; one thread per
// 8 channels (two 16-byte reads per partial, one 16-byte bf16 store).
__global__ __launch_bounds__(256) void attn_group_reduce_kernel(
    const float* __restrict__ part_k, const float* __restrict__ part_v, bf16* __restrict__ dk,
    bf16* __restrict__ dv, int s, int nslots, int nkv, int qsplit, int64_t total, KLayout dkl, KLayout dvl) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // (bi, kvh, si, chunk of 8)
  if (idx >= total) return;
  const int c = (int)(idx & 15);
  const int si = (int)((idx >> 4) % s);
  const int kvh = (int)((idx >> 4) / s % nkv);
  const int bi = (int)((idx >> 4) / ((int64_t)s * nkv));
  const int per = nslots / nkv;  // partial results per KV head: one per workgroup that served the group
  float ak[8], av[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) ak[e] = av[e] = 0.f;
  for (int j = 0; j < per * qsplit; ++j) {  // (heads' workgroup, query-tile part) pairs are consecutive
    const int64_t off = (((((int64_t)bi * nslots + kvh * per) * qsplit + j) * s) + si) * HD + c * 8;
    const f32x4 k0 = *reinterpret_cast<const f32x4*>(part_k + off);
    const f32x4 k1 = *reinterpret_cast<const f32x4*>(part_k + off + 4);
    const f32x4 v0 = *reinterpret_cast<const f32x4*>(part_v + off);
    const f32x4 v1 = *reinterpret_cast<const f32x4*>(part_v + off + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ak[e] += k0[e];
      ak[4 + e] += k1[e];
      av[e] += v0[e];
      av[4 + e] += v1[e];
    }
  }
  bf16x8 ok, ov;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    ok[e] = (bf16)ak[e];
    ov[e] = (bf16)av[e];
  }
  stg8(dk + dkl.at(bi, kvh) + (int64_t)si * dkl.s_ + c * 8, ok);
  stg8(dv + dvl.at(bi, kvh) + (int64_t)si * dvl.s_ + c * 8, ov);
}

// HALVES = 2: as in the forward kernel, two halves of an 8-wave workgroup own the same 128
// queries and walk the even / odd key tiles; half 1's dQ partial is added to half 0's through
// LDS at the end.  Chosen by the host when there are few workgroups.
// When there is a 256-query tile for every compute unit (or other streams run beside the launch)
// the host takes attn_bwd_dq_w64_kernel below instead.
template <int HALVES>
__global__ __launch_bounds__(256 * HALVES, HALVES == 1 ? 2 : 1) void attn_bwd_dq_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k, const bf16* __restrict__ v,
    const bf16* __restrict__ dout, const float* __restrict__ lse, const float* __restrict__ delta,
    bf16* __restrict__ dq, int s, int nq, int nkv, float scale, float scale_log2, QLayout ql,
    KLayout kl, KLayout vl, QLayout dol, QLayout dql) {
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];
  constexpr uint32_t STAGE = 2 * BT_BYTES;  // K tile | V tile (blocked tiles), bytes

  const int half = HALVES == 1 ? 0 : __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8));
  const int tid = threadIdx.x & 255, lane = tid & 63, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int ROWS = BQ;  // queries per workgroup
  const int nqt = s / ROWS;
  const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int qt = nqt - 1 - (lid % nqt);
  const int pair = lid / nqt;
  const int head = pair % nq;
  const int bi = pair / nq;
  const int per = nq / nkv;
  const int kvh = head / per;
  const int q0 = qt * ROWS;
  const int qw0 = q0 + wave * 32;
  const int qrow = qw0 + (lane & 31);

  const bf16* qp = q + ql.at(bi, head, per) + (int64_t)qrow * ql.s_;
  const bf16* dop = dout + dol.at(bi, head, per) + (int64_t)qrow * dol.s_;
  const bf16* kb = k + kl.at(bi, kvh);
  const bf16* vb = v + vl.at(bi, kvh);
  bf16x8 qf[HD / 16], dof[HD / 16];
#pragma unroll
  for (int kk = 0; kk < HD / 16; ++kk) {
    qf[kk] = ldg8(qp + kk * 16 + h * 8);
    dof[kk] = ldg8(dop + kk * 16 + h * 8);
  }
  const int64_t stat = ((int64_t)bi * nq + head) * s + qrow;
  const float neg_lse = -lse[stat] * kLog2e;
  const float my_delta = delta[stat];

  f32x16 dqacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) dqacc[dt][e] = 0.f;

  // key tiles per half (the tile count is even), or all tiles up to the workgroup's last row
  const int ntiles = (q0 + BQ) / (HALVES * BKV);
  auto key_of = [&](int j) { return (HALVES * j + half) * BKV; };
  // K and V tiles go straight from global memory into two LDS stages: this half's own, or with
  // shared tiles the workgroup's, half 0 bringing in the K tile and half 1 the V tile
  const uint32_t area = (uint32_t)(uintptr_t)(KR_LDS const bf16*)smem + half * 2 * STAGE;
  auto stage_request = [&](int j, int buf) {
    const int key0 = key_of(j);
    bt_request(kb + (int64_t)key0 * kl.s_, kl.s_, area + buf * STAGE, wave, lane);
    bt_request(vb + (int64_t)key0 * vl.s_, vl.s_, area + buf * STAGE + BT_BYTES, wave, lane);
  };
  stage_request(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();

  settle_scalar_loads();
  for (int j = 0; j < ntiles; ++j) {
    const int cur = j & 1;
    if (j + 1 < ntiles) stage_request(j + 1, cur ^ 1);
    const int key0 = key_of(j);
    if (key0 <= qw0 + 31) {
      // one base register per tile and read direction; everything else is an immediate
      uint32_t k_rows = area + cur * STAGE + bt_rows_lane(lane);
      uint32_t v_rows = k_rows + BT_BYTES;
      uint32_t k_cols = area + cur * STAGE + bt_cols_lane(lane);
      asm volatile("" : "+v"(k_rows), "+v"(v_rows), "+v"(k_cols));
      const bool need_mask = key0 + BKV - 1 > qw0;  // wave-uniform: the tile on the diagonal
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        f32x16 sacc, dpacc;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          sacc[e] = 0.f;
          dpacc[e] = 0.f;
        }
#pragma unroll
        for (int kk = 0; kk < HD / 16; ++kk) {
          sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bt_rows(k_rows, t, kk), qf[kk], sacc, 0, 0, 0);
          dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bt_rows(v_rows, t, kk), dof[kk], dpacc, 0, 0, 0);
        }
        // lane: query row qrow, keys key0 + 32t + 8g + 4h + e
        bf16x8 dsb[2];
        if (need_mask) {
          // Off the diagonal no mask code must run.  Left alone the compiler turns the branch
          // into 16 unconditional selects; values that pass through an (empty) volatile asm can
          // only be produced where the asm executes, i.e. inside the branch.
          const int lim = qrow - key0 - t * 32 - 4 * h;
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            float v = 8 * (e >> 2) + (e & 3) > lim ? -INFINITY : sacc[e];
            asm volatile("" : "+v"(v));
            sacc[e] = v;
          }
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[e], scale_log2, neg_lse));
          dsb[e >> 3][e & 7] = (bf16)(p * (dpacc[e] - my_delta));
        }
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
          for (int dt = 0; dt < HD / 32; ++dt) {
            dqacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bt_cols(k_cols, 2 * t + k2, dt), dsb[k2],
                                                                dqacc[dt], 0, 0, 0);
          }
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's share of the next tiles has landed
    __syncthreads();
  }

  if (HALVES == 2) {  // half 1 -> LDS -> half 0 ([value][wave][lane]; the staging areas are free)
    float* xch = reinterpret_cast<float*>(smem);
    const int slot = wave * 64 + lane;
    if (half == 1) {
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) xch[(dt * 16 + e) * 256 + slot] = dqacc[dt][e];
    }
    __syncthreads();
    if (half == 1) return;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) dqacc[dt][e] += xch[(dt * 16 + e) * 256 + slot];
  }

  // output transposition through LDS (behind the 64 KiB hand-over buffer when there are two halves)
  RowStage rs;
  rs.init(reinterpret_cast<char*>(smem) + (HALVES == 2 ? 64 * 1024 : 0) + wave * 4096, lane);
  store_rows_bf16(rs, dqacc, scale, dq + dql.at(bi, head, per) + (int64_t)qw0 * dql.s_, dql.s_);
}

// ---------------------------------------------------------------------------------------------
// dQ with ONE wave per SIMD.  A wave owns 64 query rows (two blocks of 32) and all 512 registers of
// its lanes, so that every K / V fragment it reads from LDS feeds two MFMAs — a wave cannot fetch a
// 1 KB fragment faster than an MFMA takes, which is what holds the two-waves-per-SIMD kernels at
// half of the matrix pipe.  With a single instruction stream per SIMD nothing else would fill the
// pipe while the wave does its vector work, so the loop is software-pipelined by hand: behind each of
// the 32 score MFMAs (S^T, dP^T) of the NEXT 32 keys sits the multiply-add, exponential, multiplication
// and rounding of one score per lane of THIS step (dP^T comes out of its MFMAs with delta already
// subtracted), then come this step's 16 dQ MFMAs.
//
// The score MFMAs are inline assembly because their register file has to be chosen: a kernel with more
// than 256 registers gets its MFMA results in the accumulation registers, and every score would
// then pass through a copy before a vector instruction can read it.  Written by hand they land in
// ordinary VGPRs (with most Q / dO fragments in the accumulation registers, which the MFMA reads
// directly); the dQ MFMAs are ordinary builtins and keep dQ in the accumulation registers.  The
// compiler does not see an MFMA in the assembly, so the waits it would insert between such an
// instruction and a reader of its result are provided by construction:
//   * a score accumulator is read by vector instructions one step after the MFMAs that wrote it,
//     with that step's 16 dQ MFMAs in between (before the loop: explicit s_nop);
//   * score accumulators start from the instruction's zero operand or from a tuple set up before the
//     loop, never from a fresh vector write, and a result that is not also the addend is an
//     early-clobber operand (the instruction writes while it still reads).
// tests/test_attention_asm.py checks the compiled kernel for any reader that comes too early.
// Fragments come from LDS through ordinary loads, whose waits the compiler does insert.
// ---------------------------------------------------------------------------------------------
struct DqScores {
  f32x16 s[2], dp[2];  // per 32-query block: S^T and dP^T of 32 keys
};

// c = a . b / c += a . b with c in VGPRs; b in the accumulation registers or in VGPRs.  A result that
// is not also the addend must not share registers with the operands (early clobber): the
// instruction writes while it still reads.
__device__ __forceinline__ void mfma_set_v(f32x16& c, bf16x8 a, bf16x8 b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
}
__device__ __forceinline__ void mfma_acc_v(f32x16& c, bf16x8 a, bf16x8 b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
}
__device__ __forceinline__ void mfma_set_vv(f32x16& c, bf16x8 a, bf16x8 b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_acc_vv(f32x16& c, bf16x8 a, bf16x8 b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}

// c = a . b + c0 with c and c0 in VGPRs (c0 is kept)
__device__ __forceinline__ void mfma_from_v(f32x16& c, bf16x8 a, bf16x8 b, const f32x16& c0) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(c) : "v"(a), "a"(b), "v"(c0));
}
__device__ __forceinline__ void mfma_from_vv(f32x16& c, bf16x8 a, bf16x8 b, const f32x16& c0) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(c) : "v"(a), "v"(b), "v"(c0));
}

// MFMA m (0..3) of contraction step kk: S^T of block 0, block 1, dP^T of block 0, block 1.  dP^T
// starts from -delta of the lane's row (sixteen copies per block, set up once), which takes the
// subtraction out of every score's vector work.
__device__ __forceinline__ void dq_score_mfma(DqScores& x, int kk, int m, bf16x8 kf, bf16x8 vf,
                                              const bf16x8 (&qf)[2][HD / 16], const bf16x8 (&dof)[2][HD / 16],
                                              const f32x16 (&neg_delta)[2]) {
  if (kk == 0) {
    if (m == 0) mfma_set_v(x.s[0], kf, qf[0][kk]);
    if (m == 1) mfma_set_v(x.s[1], kf, qf[1][kk]);
    if (m == 2) mfma_from_v(x.dp[0], vf, dof[0][kk], neg_delta[0]);
    if (m == 3) mfma_from_vv(x.dp[1], vf, dof[1][kk], neg_delta[1]);
  } else {
    if (m == 0) mfma_acc_v(x.s[0], kf, qf[0][kk]);
    if (m == 1) mfma_acc_v(x.s[1], kf, qf[1][kk]);
    if (m == 2) mfma_acc_v(x.dp[0], vf, dof[0][kk]);
    if (m == 3) mfma_acc_vv(x.dp[1], vf, dof[1][kk]);
  }
}

// One step (32 keys).  NEXT: issue the score MFMAs of the following 32 keys (fragments of sub-tile nt
// at nk_rows / nv_rows) into `nxt`.  MASK: the step is on the causal diagonal; lim[qb] is the last
// visible key of the lane's row, relative to the lane's first key of the step.
template <bool NEXT, bool MASK>
__device__ __forceinline__ void dq_step(DqScores& nxt, const DqScores& cur, f32x16 (&dq)[2][HD / 32],
                                        uint32_t nk_rows, uint32_t nv_rows, int nt, uint32_t k_cols, int t,
                                        const bf16x8 (&qf)[2][HD / 16], const bf16x8 (&dof)[2][HD / 16],
                                        float scale_log2, const float (&neg_lse)[2],
                                        const f32x16 (&neg_delta)[2], const int (&lim)[2]) {
  bf16x8 dsb[2][2];
  auto one_score = [&](int g) {  // lane: query row of block g / 16, key 8 (e / 4) + e % 4 (+ 4 h) of the step
    const int qb = g >> 4, e = g & 15;
    float sv = cur.s[qb][e];
    if (MASK) sv = 8 * (e >> 2) + (e & 3) > lim[qb] ? -INFINITY : sv;
    const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sv, scale_log2, neg_lse[qb]));
    dsb[qb][e >> 3][e & 7] = (bf16)(p * cur.dp[qb][e]);  // dP - delta comes out of the MFMAs
  };
  // Fragments are requested from LDS well ahead of the MFMA that takes them (two contraction steps
  // = eight MFMAs for the score products, three fragments = six MFMAs for dQ): one wave per SIMD has
  // nobody to cover an LDS round trip for it.
  constexpr int NKT = 2 * (HD / 32);  // K^T fragments of the step: 2 contraction steps x 4 channel blocks
  auto kt_frag = [&](int i) { return bt_cols(k_cols, 2 * t + i / (HD / 32), i % (HD / 32)); };
  bf16x8 kt[3];
  if (NEXT) {
    bf16x8 kf[3], vf[3];
    kf[0] = bt_rows(nk_rows, nt, 0);
    vf[0] = bt_rows(nv_rows, nt, 0);
    kf[1] = bt_rows(nk_rows, nt, 1);
    vf[1] = bt_rows(nv_rows, nt, 1);
#pragma unroll
    for (int kk = 0; kk < HD / 16; ++kk) {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        if (m == 0 && kk + 2 < HD / 16) kf[(kk + 2) % 3] = bt_rows(nk_rows, nt, kk + 2);
        if (m == 2 && kk + 2 < HD / 16) vf[(kk + 2) % 3] = bt_rows(nv_rows, nt, kk + 2);
        if (m == 1 && kk >= HD / 16 - 3) kt[kk - (HD / 16 - 3)] = kt_frag(kk - (HD / 16 - 3));
        dq_score_mfma(nxt, kk, m, kf[kk % 3], vf[kk % 3], qf, dof, neg_delta);
        one_score(kk * 4 + m);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 3; ++i) kt[i] = kt_frag(i);
#pragma unroll
    for (int g = 0; g < 32; ++g) one_score(g);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 3");
  }
#pragma unroll
  for (int i = 0; i < NKT; ++i) {
    const int k2 = i / (HD / 32), dt = i % (HD / 32);
    const bf16x8 frag = kt[i % 3];
    dq[0][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag, dsb[0][k2], dq[0][dt], 0, 0, 0);
    dq[1][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag, dsb[1][k2], dq[1][dt], 0, 0, 0);
    if (i + 3 < NKT) kt[i % 3] = kt_frag(i + 3);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// The kernel also takes over the pre-pass of the backward: each wave forms delta = sum_d dO . O of its 64
// rows from the dO fragments it holds anyway, uses it, and writes it (and -lse in the log2 domain) for
// the dK/dV kernel, which the host launches behind this one.
__global__ __launch_bounds__(256, 1) void attn_bwd_dq_w64_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k, const bf16* __restrict__ v,
    const bf16* __restrict__ dout, const bf16* __restrict__ o, const float* __restrict__ lse,
    float* __restrict__ delta_out, float* __restrict__ neg_lse2_out, bf16* __restrict__ dq, int s, int nq,
    int nkv, float scale, float scale_log2, QLayout ql, KLayout kl, KLayout vl, QLayout dol, QLayout ol,
    QLayout dql) {
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];
  constexpr uint32_t STAGE = 2 * BT_BYTES;  // K tile | V tile
  constexpr int ROWS = 256;                 // queries per workgroup: 64 per wave
  constexpr int NSTAGE = 3;                 // tiles in LDS: the one in use, the next, the one after

  const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nqt = s / ROWS;
  const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  int qt, pair;
  longest_first(lid, nqt, gridDim.x / nqt, qt, pair);
  const int head = pair % nq;
  const int bi = pair / nq;
  const int per = nq / nkv;
  const int kvh = head / per;
  const int q0 = qt * ROWS;
  const int qw0 = q0 + wave * 64;

  const bf16* kb = k + kl.at(bi, kvh);
  const bf16* vb = v + vl.at(bi, kvh);
  bf16x8 qf[2][HD / 16], dof[2][HD / 16];
  float neg_lse[2];
  f32x16 neg_delta[2];
  int lim[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qrow = qw0 + 32 * qb + (lane & 31);
    const bf16* qp = q + ql.at(bi, head, per) + (int64_t)qrow * ql.s_;
    const bf16* dop = dout + dol.at(bi, head, per) + (int64_t)qrow * dol.s_;
    const bf16* op = o + ol.at(bi, head, per) + (int64_t)qrow * ol.s_;
    // delta from a second read of the dO row: the fragments kept for the MFMAs must stay values that
    // only the MFMAs read, or the compiler keeps them in VGPRs and copies them into accumulation
    // registers in front of every MFMA
    const bf16* dop2 = dop;
    asm volatile("" : "+v"(dop2));
    float dsum = 0.f;  // this lane's half of the row (channels 16 kk + 8 h ..)
#pragma unroll
    for (int kk = 0; kk < HD / 16; ++kk) {
      qf[qb][kk] = ldg8(qp + kk * 16 + h * 8);
      dof[qb][kk] = ldg8(dop + kk * 16 + h * 8);
      const bf16x8 dov = ldg8(dop2 + kk * 16 + h * 8), of = ldg8(op + kk * 16 + h * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) dsum += (float)dov[e] * (float)of[e];
    }
    dsum += __shfl_xor(dsum, 32, KR_WAVE);
    const int64_t stat = ((int64_t)bi * nq + head) * s + qrow;
    neg_lse[qb] = -lse[stat] * kLog2e;
    if (h == 0) {
      delta_out[stat] = dsum;
      neg_lse2_out[stat] = neg_lse[qb];
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) neg_delta[qb][e] = -dsum;
  }

  f32x16 dqacc[2][HD / 32];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) dqacc[qb][dt][e] = 0.f;

  const int ntiles = (q0 + ROWS) / BKV;                             // key tiles of the workgroup
  const int last = __builtin_amdgcn_readfirstlane(qw0 / BKV);       // this wave's tile on the diagonal
  const uint32_t area = (uint32_t)(uintptr_t)(KR_LDS const bf16*)smem;
  auto stage_request = [&](int j, int buf) {  // the four waves bring in the K and the V tile together
    bt_request(kb + (int64_t)(j * BKV) * kl.s_, kl.s_, area + buf * STAGE, wave, lane);
    bt_request(vb + (int64_t)(j * BKV) * vl.s_, vl.s_, area + buf * STAGE + BT_BYTES, wave, lane);
  };
  stage_request(0, 0);
  stage_request(1, 1);  // ntiles >= 4
  __builtin_amdgcn_s_waitcnt(0x0f78);  // vmcnt(8): everything but the second tile's requests has landed
  __syncthreads();
  settle_scalar_loads();

  const uint32_t rows_lane = bt_rows_lane(lane), cols_lane = bt_cols_lane(lane);
  DqScores a, b;
  {  // scores of the first 32 keys (tile 0 is below every wave's diagonal or on it)
    const uint32_t k_rows = area + rows_lane, v_rows = k_rows + BT_BYTES;
#pragma unroll
    for (int kk = 0; kk < HD / 16; ++kk) {
      const bf16x8 kf = bt_rows(k_rows, 0, kk), vf = bt_rows(v_rows, 0, kk);
#pragma unroll
      for (int m = 0; m < 4; ++m) dq_score_mfma(a, kk, m, kf, vf, qf, dof, neg_delta);
    }
    // the scores pass through the wait: no reader can be moved in front of it
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(a.s[0]), "+v"(a.s[1]), "+v"(a.dp[0]), "+v"(a.dp[1]));
  }
  // Every wave passes the same ntiles barriers and makes the same requests; what differs is how many
  // of the tiles it computes on (those up to its diagonal).  Three loops without branches inside
  // (a branch around a step would put copies of all accumulators at the merge): tiles below the
  // diagonal, the diagonal tile, the tiles only the waves further down still need.
  int buf = 0;  // stage of tile j
  auto arrive = [&](int j) {  // between the two steps of tile j
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's share of tile j + 1 has landed
    __syncthreads();                     // ... and everyone's; nobody reads tile j - 1 any more
  };
  auto turn = [&](int j) {
    arrive(j);
    if (j + NSTAGE - 1 < ntiles) stage_request(j + NSTAGE - 1, buf == 0 ? NSTAGE - 1 : buf - 1);
  };
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) lim[qb] = 0;
  for (int j = 0; j < last; ++j) {
    const int buf_next = buf == NSTAGE - 1 ? 0 : buf + 1;
    uint32_t k_rows = area + buf * STAGE + rows_lane, v_rows = k_rows + BT_BYTES;
    uint32_t k_cols = area + buf * STAGE + cols_lane;
    uint32_t nk_rows = area + buf_next * STAGE + rows_lane, nv_rows = nk_rows + BT_BYTES;
    asm volatile("" : "+v"(k_rows), "+v"(v_rows), "+v"(k_cols), "+v"(nk_rows), "+v"(nv_rows));
    dq_step<true, false>(b, a, dqacc, k_rows, v_rows, 1, k_cols, 0, qf, dof, scale_log2, neg_lse, neg_delta, lim);
    turn(j);
    dq_step<true, false>(a, b, dqacc, nk_rows, nv_rows, 0, k_cols, 1, qf, dof, scale_log2, neg_lse, neg_delta, lim);
    buf = buf_next;
  }
  {  // the diagonal tile (keys qw0 .. qw0 + 63): lim = last visible key of the lane's row, counted
     // from the lane's first key of the step
    uint32_t k_rows = area + buf * STAGE + rows_lane, v_rows = k_rows + BT_BYTES;
    uint32_t k_cols = area + buf * STAGE + cols_lane;
    asm volatile("" : "+v"(k_rows), "+v"(v_rows), "+v"(k_cols));
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) lim[qb] = 32 * qb + (lane & 31) - 4 * h;
    dq_step<true, true>(b, a, dqacc, k_rows, v_rows, 1, k_cols, 0, qf, dof, scale_log2, neg_lse, neg_delta, lim);
    turn(last);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) lim[qb] -= 32;
    dq_step<false, true>(a, b, dqacc, 0, 0, 0, k_cols, 1, qf, dof, scale_log2, neg_lse, neg_delta, lim);
    buf = buf == NSTAGE - 1 ? 0 : buf + 1;
  }
  for (int j = last + 1; j < ntiles; ++j) {
    turn(j);
    buf = buf == NSTAGE - 1 ? 0 : buf + 1;
  }

  RowStage rs;
  rs.init(reinterpret_cast<char*>(smem) + NSTAGE * STAGE + wave * 4096, lane);
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
    store_rows_bf16(rs, dqacc[qb], scale, dq + dql.at(bi, head, per) + (int64_t)(qw0 + 32 * qb) * dql.s_, dql.s_);
}

#define KR_ATTN_DQ_ARGS                                                                          \
  const bf16*, const bf16*, const bf16*, const bf16*, const float*, const float*, bf16*, int, int, \
      int, float, float, QLayout, KLayout, KLayout, QLayout, QLayout
template __global__ void attn_bwd_dq_kernel<1>(KR_ATTN_DQ_ARGS);
template __global__ void attn_bwd_dq_kernel<2>(KR_ATTN_DQ_ARGS);
#undef KR_ATTN_DQ_ARGS

#define KR_ATTN_DKDV_ARGS                                                                          \
  const bf16*, const bf16*, const bf16*, const bf16*, const float*, const float*, bf16*, bf16*, \
      float*, float*, int, int, int, int, int, float, float, QLayout, KLayout, KLayout, QLayout,      \
      KLayout, KLayout
template __global__ void attn_bwd_dkdv_kernel<false>(KR_ATTN_DKDV_ARGS);
template __global__ void attn_bwd_dkdv_kernel<true>(KR_ATTN_DKDV_ARGS);
#undef KR_ATTN_DKDV_ARGS


// =============================================================================================
// General path: any sequence length, head dimensions that are a multiple of 8 up to 128.
// The kernels above are built for head dimension 128 and sequences of whole 128-row tiles, the
// shapes of the training workloads.  Everything else (head dimension 64, ragged lengths; the
// reference's flash-attention call takes both) runs through these plain fp32 kernels: same
// interface, same tensor layouts, same results to rounding, no MFMA — they exist so that such a
// shape is computed on the device at all, not to be fast.  A workgroup of 256 threads owns 32
// query rows (forward, dQ) or 32 keys (dK/dV) and walks 32-row tiles of the other operand through
// LDS; a thread is (row r = tid / 8, part p = tid % 8): it computes the scores of row r against
// keys 4 p .. 4 p + 3 of a tile and owns channels p hd/8 .. (p + 1) hd/8 - 1 of row r's
// accumulators.  Rows beyond the sequence are loaded as zeros and never stored.  No atomics:
// grouped query heads are summed inside the dK/dV workgroup, in a fixed order.
// =============================================================================================
namespace general {

constexpr int GT = 32;          // rows per tile (queries or keys)
constexpr int GTHREADS = 256;
constexpr int GHD_MAX = 128;
constexpr int GLD = GHD_MAX + 8;  // LDS row stride in elements (rows stay 16-byte aligned)

// rows row0 .. row0 + 31 of a [s, hd] matrix with row stride ss -> LDS tile, zeros beyond s
__device__ __forceinline__ void load_tile(bf16* dst, const bf16* src, int64_t ss, int row0, int s,
                                          int hd, int tid) {
  const int vecs = hd / 8;
  for (int i = tid; i < GT * vecs; i += GTHREADS) {
    const int r = i / vecs, c = (i - r * vecs) * 8;
    const bf16x8 v = row0 + r < s ? ldg8(src + (int64_t)(row0 + r) * ss + c) : zero8();
    *reinterpret_cast<bf16x8*>(dst + r * GLD + c) = v;
  }
}

// sum / max over the 8 threads that share a row (consecutive lanes)
__device__ __forceinline__ float row_sum(float v) {
  v += __shfl_xor(v, 1, KR_WAVE);
  v += __shfl_xor(v, 2, KR_WAVE);
  v += __shfl_xor(v, 4, KR_WAVE);
  return v;
}
__device__ __forceinline__ float row_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 1, KR_WAVE));
  v = fmaxf(v, __shfl_xor(v, 2, KR_WAVE));
  v = fmaxf(v, __shfl_xor(v, 4, KR_WAVE));
  return v;
}

// dot products of row `r` of tile a with rows 4 p .. 4 p + 3 of tile b over hd channels
__device__ __forceinline__ void dot4(const bf16* a, const bf16* b, int r, int p, int hd, float (&out)[4]) {
  out[0] = out[1] = out[2] = out[3] = 0.f;
  const bf16* ar = a + r * GLD;
  const bf16* b0 = b + (4 * p) * GLD;
  for (int d = 0; d < hd; ++d) {
    const float av = (float)ar[d];
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] += av * (float)b0[j * GLD + d];
  }
}

__global__ __launch_bounds__(GTHREADS) void attn_general_fwd_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k, const bf16* __restrict__ v,
    bf16* __restrict__ o, float* __restrict__ lse, int s, int nq, int nkv, int hd, float scale,
    QLayout ql, KLayout kl, KLayout vl, QLayout ol) {
  __shared__ __attribute__((aligned(16))) bf16 sq[GT * GLD], sk[GT * GLD], sv[GT * GLD];
  __shared__ float sp[GT][GT + 1];
  const int tid = threadIdx.x, r = tid >> 3, p = tid & 7;
  const int q0 = blockIdx.x * GT, head = blockIdx.y, bi = blockIdx.z;
  const int per = nq / nkv, kvh = head / per, c = hd / 8;
  const bf16* qb = q + ql.at(bi, head, per);
  const bf16* kb = k + kl.at(bi, kvh);
  const bf16* vb = v + vl.at(bi, kvh);
  load_tile(sq, qb, ql.s_, q0, s, hd, tid);
  float acc[GHD_MAX / 8];
#pragma unroll
  for (int i = 0; i < GHD_MAX / 8; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  const int qrow = q0 + r;
  const int last_key = (q0 + GT - 1 < s ? q0 + GT - 1 : s - 1);
  for (int k0 = 0; k0 <= last_key; k0 += GT) {
    __syncthreads();  // the previous tile's K, V and probabilities are no longer read
    load_tile(sk, kb, kl.s_, k0, s, hd, tid);
    load_tile(sv, vb, vl.s_, k0, s, hd, tid);
    __syncthreads();
    float sc[4];
    dot4(sq, sk, r, p, hd, sc);
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int key = k0 + 4 * p + j;
      sc[j] = (key <= qrow && key < s) ? sc[j] * scale : -INFINITY;
      mx = fmaxf(mx, sc[j]);
    }
    mx = row_max(mx);
    const float m_new = fmaxf(m, mx);
    float pr[4], ps = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      pr[j] = sc[j] == -INFINITY ? 0.f : __expf(sc[j] - m_new);
      ps += pr[j];
      sp[r][4 * p + j] = pr[j];
    }
    ps = row_sum(ps);
    const float alpha = m == -INFINITY ? 0.f : __expf(m - m_new);
    l = l * alpha + ps;
    m = m_new;
    __syncthreads();
    for (int i = 0; i < c; ++i) acc[i] *= alpha;
    for (int kj = 0; kj < GT; ++kj) {
      const float pv = sp[r][kj];
      const bf16* vr = sv + kj * GLD + p * c;
      for (int i = 0; i < c; ++i) acc[i] += pv * (float)vr[i];
    }
  }
  if (qrow < s) {
    const float inv = 1.0f / l;
    bf16* orow = o + ol.at(bi, head, per) + (int64_t)qrow * ol.s_ + p * c;
    for (int i = 0; i < c; ++i) orow[i] = (bf16)(acc[i] * inv);
    if (p == 0) lse[((int64_t)bi * nq + head) * s + qrow] = m + __logf(l);
  }
}

// delta[b, h, i] = sum_d dO[i, d] O[i, d]
__global__ __launch_bounds__(GTHREADS) void attn_general_delta_kernel(
    const bf16* __restrict__ dout, const bf16* __restrict__ o, float* __restrict__ delta, int s,
    int nq, int nkv, int hd, QLayout dol, QLayout ol) {
  const int tid = threadIdx.x, r = tid >> 3, p = tid & 7;
  const int row = blockIdx.x * GT + r, head = blockIdx.y, bi = blockIdx.z;
  const int per = nq / nkv, c = hd / 8;
  float sum = 0.f;
  if (row < s) {
    const bf16* dr = dout + dol.at(bi, head, per) + (int64_t)row * dol.s_ + p * c;
    const bf16* orow = o + ol.at(bi, head, per) + (int64_t)row * ol.s_ + p * c;
    for (int i = 0; i < c; ++i) sum += (float)dr[i] * (float)orow[i];
  }
  sum = row_sum(sum);
  if (row < s && p == 0) delta[((int64_t)bi * nq + head) * s + row] = sum;
}

// P and dS of one 32 x 32 block: thread (r, p) handles query row r against keys 4 p .. 4 p + 3
__device__ __forceinline__ void block_p_ds(const bf16* sq, const bf16* sk, const bf16* sv, const bf16* sdo,
                                           const float* slse, const float* sdelta, int r, int p, int hd,
                                           int q0, int k0, int s, float scale, float (&pr)[4],
                                           float (&ds)[4]) {
  float sc[4], dp[4];
  dot4(sq, sk, r, p, hd, sc);
  dot4(sdo, sv, r, p, hd, dp);
  const int qrow = q0 + r;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int key = k0 + 4 * p + j;
    const bool valid = key <= qrow && key < s && qrow < s;
    pr[j] = valid ? __expf(sc[j] * scale - slse[r]) : 0.f;
    ds[j] = pr[j] * (dp[j] - sdelta[r]) * scale;
  }
}

__global__ __launch_bounds__(GTHREADS) void attn_general_dkdv_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k, const bf16* __restrict__ v,
    const bf16* __restrict__ dout, const float* __restrict__ lse, const float* __restrict__ delta,
    bf16* __restrict__ dk, bf16* __restrict__ dv, int s, int nq, int nkv, int hd, float scale,
    QLayout ql, KLayout kl, KLayout vl, QLayout dol, KLayout dkl, KLayout dvl) {
  __shared__ __attribute__((aligned(16))) bf16 sq[GT * GLD], sk[GT * GLD], sv[GT * GLD], sdo[GT * GLD];
  __shared__ float sp[GT][GT + 1], sds[GT][GT + 1], slse[GT], sdelta[GT];
  const int tid = threadIdx.x, r = tid >> 3, p = tid & 7;
  const int k0 = blockIdx.x * GT, kvh = blockIdx.y, bi = blockIdx.z;
  const int per = nq / nkv, c = hd / 8;
  load_tile(sk, k + kl.at(bi, kvh), kl.s_, k0, s, hd, tid);
  load_tile(sv, v + vl.at(bi, kvh), vl.s_, k0, s, hd, tid);
  float adk[GHD_MAX / 8], adv[GHD_MAX / 8];
#pragma unroll
  for (int i = 0; i < GHD_MAX / 8; ++i) adk[i] = adv[i] = 0.f;
  for (int hj = 0; hj < per; ++hj) {
    const int head = kvh * per + hj;
    const bf16* qb = q + ql.at(bi, head, per);
    const bf16* dob = dout + dol.at(bi, head, per);
    const int64_t stat = ((int64_t)bi * nq + head) * s;
    for (int q0 = k0; q0 < s; q0 += GT) {  // query tiles at or below the diagonal (k0 is a multiple of 32)
      __syncthreads();
      load_tile(sq, qb, ql.s_, q0, s, hd, tid);
      load_tile(sdo, dob, dol.s_, q0, s, hd, tid);
      if (tid < GT) {
        const bool in = q0 + tid < s;
        slse[tid] = in ? lse[stat + q0 + tid] : 0.f;
        sdelta[tid] = in ? delta[stat + q0 + tid] : 0.f;
      }
      __syncthreads();
      float pr[4], ds[4];
      block_p_ds(sq, sk, sv, sdo, slse, sdelta, r, p, hd, q0, k0, s, scale, pr, ds);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        sp[r][4 * p + j] = pr[j];
        sds[r][4 * p + j] = ds[j];
      }
      __syncthreads();
      // this thread now is (key r, channels p c ..): dV += P^T dO, dK += dS^T Q
      for (int qi = 0; qi < GT; ++qi) {
        const float pv = sp[qi][r], dsv = sds[qi][r];
        const bf16* dor = sdo + qi * GLD + p * c;
        const bf16* qr = sq + qi * GLD + p * c;
        for (int i = 0; i < c; ++i) {
          adv[i] += pv * (float)dor[i];
          adk[i] += dsv * (float)qr[i];
        }
      }
    }
  }
  if (k0 + r < s) {
    bf16* dkr = dk + dkl.at(bi, kvh) + (int64_t)(k0 + r) * dkl.s_ + p * c;
    bf16* dvr = dv + dvl.at(bi, kvh) + (int64_t)(k0 + r) * dvl.s_ + p * c;
    for (int i = 0; i < c; ++i) {
      dkr[i] = (bf16)adk[i];
      dvr[i] = (bf16)adv[i];
    }
  }
}

__global__ __launch_bounds__(GTHREADS) void attn_general_dq_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k, const bf16* __restrict__ v,
    const bf16* __restrict__ dout, const float* __restrict__ lse, const float* __restrict__ delta,
    bf16* __restrict__ dq, int s, int nq, int nkv, int hd, float scale, QLayout ql, KLayout kl,
    KLayout vl, QLayout dol, QLayout dql) {
  __shared__ __attribute__((aligned(16))) bf16 sq[GT * GLD], sk[GT * GLD], sv[GT * GLD], sdo[GT * GLD];
  __shared__ float sds[GT][GT + 1], slse[GT], sdelta[GT];
  const int tid = threadIdx.x, r = tid >> 3, p = tid & 7;
  const int q0 = blockIdx.x * GT, head = blockIdx.y, bi = blockIdx.z;
  const int per = nq / nkv, kvh = head / per, c = hd / 8;
  const int64_t stat = ((int64_t)bi * nq + head) * s;
  load_tile(sq, q + ql.at(bi, head, per), ql.s_, q0, s, hd, tid);
  load_tile(sdo, dout + dol.at(bi, head, per), dol.s_, q0, s, hd, tid);
  if (tid < GT) {
    const bool in = q0 + tid < s;
    slse[tid] = in ? lse[stat + q0 + tid] : 0.f;
    sdelta[tid] = in ? delta[stat + q0 + tid] : 0.f;
  }
  const bf16* kb = k + kl.at(bi, kvh);
  const bf16* vb = v + vl.at(bi, kvh);
  float adq[GHD_MAX / 8];
#pragma unroll
  for (int i = 0; i < GHD_MAX / 8; ++i) adq[i] = 0.f;
  const int last_key = (q0 + GT - 1 < s ? q0 + GT - 1 : s - 1);
  for (int k0 = 0; k0 <= last_key; k0 += GT) {
    __syncthreads();
    load_tile(sk, kb, kl.s_, k0, s, hd, tid);
    load_tile(sv, vb, vl.s_, k0, s, hd, tid);
    __syncthreads();
    float pr[4], ds[4];
    block_p_ds(sq, sk, sv, sdo, slse, sdelta, r, p, hd, q0, k0, s, scale, pr, ds);
#pragma unroll
    for (int j = 0; j < 4; ++j) sds[r][4 * p + j] = ds[j];
    __syncthreads();
    for (int kj = 0; kj < GT; ++kj) {
      const float dsv = sds[r][kj];
      const bf16* kr = sk + kj * GLD + p * c;
      for (int i = 0; i < c; ++i) adq[i] += dsv * (float)kr[i];
    }
  }
  if (q0 + r < s) {
    bf16* dqr = dq + dql.at(bi, head, per) + (int64_t)(q0 + r) * dql.s_ + p * c;
    for (int i = 0; i < c; ++i) dqr[i] = (bf16)adq[i];
  }
}

}  // namespace general

// ---- shapes outside the MFMA kernels, padded into them -----------------------------------------
// Head dimensions below 128 and sequence lengths that are not whole 128-row tiles are copied into
// dense [s_pad, b, heads, 128] buffers (zeros beyond the data), run through the MFMA kernels and
// copied back.  Zero channels add nothing to Q.K^T and give zero output channels; with the causal
// mask a query row below s never sees a key row at or beyond s, and the rows at or beyond s are
// made inert in the backward pass by a log-sum-exp so large that their probabilities are zero.
__global__ __launch_bounds__(256) void attn_pad_kernel(const bf16* __restrict__ src, bf16* __restrict__ dst,
                                                       int s, int b, int heads, int per, int hd,
                                                       int64_t total, QLayout sl) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one 16-byte vector of dst
  if (idx >= total) return;
  const int c = (int)(idx & 15) * 8;
  int64_t r = idx >> 4;
  const int head = (int)(r % heads);
  r /= heads;
  const int bi = (int)(r % b);
  const int row = (int)(r / b);
  bf16x8 v = zero8();
  if (row < s && c < hd) v = ldg8(src + (int64_t)row * sl.s_ + sl.at(bi, head, per) + c);
  stg8(dst + idx * 8, v);
}
__global__ __launch_bounds__(256) void attn_unpad_kernel(const bf16* __restrict__ src, bf16* __restrict__ dst,
                                                         int b, int heads, int per, int hd,
                                                         int64_t total, QLayout dl) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one 16-byte vector of dst
  if (idx >= total) return;
  const int vec = hd / 8;
  const int c = (int)(idx % vec) * 8;
  int64_t r = idx / vec;
  const int head = (int)(r % heads);
  r /= heads;
  const int bi = (int)(r % b);
  const int64_t row = r / b;
  const bf16x8 v = ldg8(src + (((row * b + bi) * heads + head) * HD + c));
  stg8(dst + row * dl.s_ + dl.at(bi, head, per) + c, v);
}
// rows of fp32 statistics [n, len_src] -> [n, len_dst]; positions beyond len_src get `fill`
__global__ __launch_bounds__(256) void attn_resize_rows_kernel(const float* __restrict__ src,
                                                               float* __restrict__ dst, int len_src,
                                                               int len_dst, int64_t total, float fill) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int64_t row = idx / len_dst;
  const int i = (int)(idx - row * len_dst);
  dst[idx] = i < len_src ? src[row * len_src + i] : fill;
}

}  // namespace

// Build-time cap, for measuring one form of a kernel against another: the most query heads a
// dK/dV workgroup takes.
#ifndef KR_DKDV_HPW_MAX
#define KR_DKDV_HPW_MAX 4
#endif
// The dK/dV kernel runs one workgroup per CU.  With at most two rounds of workgroups its time is
// set by the first key tiles (they see every query): two workgroups then share each key tile.
static int dkdv_query_split(int s, int b, int nq) { return (s / 128) * nq * b <= 2 * 256 ? 2 : 1; }

static int attn_padded_len(int s) { return (s + BQ - 1) / BQ * BQ; }
// bytes of one padded [s_pad, b, heads, 128] bf16 tensor / of the padded statistics [b, nq, s_pad]
static size_t attn_padded_bytes(int s, int b, int heads) {
  return (size_t)attn_padded_len(s) * b * heads * HD * sizeof(bf16);
}
static size_t attn_padded_stat_bytes(int s, int b, int nq) {
  return (size_t)attn_padded_len(s) * b * nq * sizeof(float);
}

// workspace of the MFMA backward kernels for a shape they take as it is
static size_t attn_bwd_fast_bytes(int s, int b, int nq, int nkv, int hd) {
  size_t bytes = 2 * (size_t)b * nq * s * sizeof(float);  // delta, and -lse in the log2 domain
  const int qsplit = dkdv_query_split(s, b, nq);
  if (nq != nkv || qsplit > 1)  // fp32 dK, dV partials per (query head, query-tile part)
    bytes += 2 * (size_t)b * nq * qsplit * s * hd * sizeof(float);
  return bytes;
}

extern "C" size_t kr_attn_bwd_workspace_bytes(int s, int b, int nq, int nkv, int hd) {
  if (check_attn_common(s, b, nq, nkv, hd) != KR_OK) return 0;
  if (attn_fast_path(s, hd)) return attn_bwd_fast_bytes(s, b, nq, nkv, hd);
  // padded copies of dO, q, o, dq (query-sized) and k, v, dk, dv (key-sized), the padded log-sum-exp, and
  // the MFMA kernels' own workspace at the padded shape (the general kernels, which only keep delta
  // [b, nq, s], fit in the same space)
  return 4 * attn_padded_bytes(s, b, nq) + 4 * attn_padded_bytes(s, b, nkv) + attn_padded_stat_bytes(s, b, nq) +
         attn_bwd_fast_bytes(attn_padded_len(s), b, nq, nkv, HD);
}

extern "C" size_t kr_attn_fwd_workspace_bytes(int s, int b, int nq, int nkv, int hd) {
  if (check_attn_common(s, b, nq, nkv, hd) != KR_OK || attn_fast_path(s, hd)) return 0;
  // padded copies of q, o and k, v, and the padded log-sum-exp
  return 2 * attn_padded_bytes(s, b, nq) + 2 * attn_padded_bytes(s, b, nkv) + attn_padded_stat_bytes(s, b, nq);
}

namespace {
// dense [s_pad, b, heads, 128] as the kernels' stride quadruple / triple
QLayout padded_qlayout(int b, int nq, int per) {
  return QLayout{(int64_t)b * nq * HD, (int64_t)nq * HD, (int64_t)per * HD, (int64_t)HD};
}
KLayout padded_klayout(int b, int nkv) { return KLayout{(int64_t)b * nkv * HD, (int64_t)nkv * HD, (int64_t)HD}; }

int launch_pad(const void* src, void* dst, int s, int b, int heads, int per, int hd, QLayout sl, hipStream_t st) {
  const int64_t total = (int64_t)attn_padded_len(s) * b * heads * (HD / 8);
  hipLaunchKernelGGL(attn_pad_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, (const bf16*)src,
                     (bf16*)dst, s, b, heads, per, hd, total, sl);
  return hipGetLastError() == hipSuccess ? KR_OK : KR_ELAUNCH;
}
int launch_unpad(const void* src, void* dst, int s, int b, int heads, int per, int hd, QLayout dl, hipStream_t st) {
  const int64_t total = (int64_t)s * b * heads * (hd / 8);
  hipLaunchKernelGGL(attn_unpad_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, (const bf16*)src,
                     (bf16*)dst, b, heads, per, hd, total, dl);
  return hipGetLastError() == hipSuccess ? KR_OK : KR_ELAUNCH;
}
int launch_resize_rows(const float* src, float* dst, int64_t n, int len_src, int len_dst, float fill, hipStream_t st) {
  const int64_t total = n * len_dst;
  hipLaunchKernelGGL(attn_resize_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, src, dst,
                     len_src, len_dst, total, fill);
  return hipGetLastError() == hipSuccess ? KR_OK : KR_ELAUNCH;
}
// a KV-like tensor's stride triple as the quadruple the pad kernels take (one head per group)
QLayout as_qlayout(const KLayout& l) { return QLayout{l.s_, l.b_, l.h_, 0}; }
}  // namespace

// Which form of each kernel a launch takes.  Alone on the GPU a launch wants the shortest latency:
// with few workgroups the keys of a row (forward, dQ) or the queries of a key tile (dK/dV) are split
// over two workgroups, which fills the device and costs merges, partial sums and a second pass over
// K / V.  Beside kernels of other streams (KR_ATTN_BESIDE_OTHER_STREAMS), which use the compute
// units a launch leaves idle, its compute-unit time counts instead: the unsplit forms, whatever the
// number of workgroups.
struct AttnForms {
  bool shared_fwd, shared_dq;
  int qsplit;
};
static AttnForms attn_forms(int s, int b, int nq, int flags) {
  const bool beside = (flags & KR_ATTN_BESIDE_OTHER_STREAMS) != 0;
  const int tiles256 = (s / 256) * nq * b;
  AttnForms f;
  f.shared_fwd = s % 256 == 0 && (beside || tiles256 >= kr_compute_units());
  f.shared_dq = s % 256 == 0 && (beside || tiles256 >= kr_compute_units());
  f.qsplit = beside ? 1 : dkdv_query_split(s, b, nq);
  return f;
}

static int attn_bwd_impl(const void* dout, const void* q, const void* k, const void* v,
                           const void* o, const float* lse, void* dq, void* dk, void* dv,
                           void* workspace, int s, int b, int nq, int nkv, int hd, float scale,
                           int64_t q_ss, int64_t q_sb, int64_t q_sg, int64_t q_sh, int64_t k_ss,
                           int64_t k_sb, int64_t k_sh, int64_t v_ss, int64_t v_sb, int64_t v_sh,
                           int64_t o_ss, int64_t o_sb, int64_t o_sg, int64_t o_sh, int64_t do_ss,
                           int64_t do_sb, int64_t do_sg, int64_t do_sh, int64_t dq_ss, int64_t dq_sb,
                           int64_t dq_sg, int64_t dq_sh, int64_t dk_ss, int64_t dk_sb, int64_t dk_sh,
                           int64_t dv_ss, int64_t dv_sb, int64_t dv_sh, int flags, void* stream) {
  if (flags & ~(KR_ATTN_BESIDE_OTHER_STREAMS | KR_ATTN_GENERAL_KERNELS)) return KR_EINVAL;
  if (!dout || !q || !k || !v || !o || !lse || !dq || !dk || !dv || !workspace) return KR_EINVAL;
  const int rc = check_attn_common(s, b, nq, nkv, hd);
  if (rc != KR_OK) return rc;
  const void* ptrs[] = {dout, q, k, v, o, dq, dk, dv, workspace};
  for (const void* p : ptrs)
    if (!kr_aligned16(p)) return KR_EINVAL;
  if ((q_ss | q_sb | q_sg | q_sh | k_ss | k_sb | k_sh | v_ss | v_sb | v_sh | o_ss | o_sb | o_sg |
       o_sh | do_ss | do_sb | do_sg | do_sh | dq_ss | dq_sb | dq_sg | dq_sh | dk_ss | dk_sb |
       dk_sh | dv_ss | dv_sb | dv_sh) % 8)
    return KR_EINVAL;
  {
    const int64_t seq[] = {q_ss, k_ss, v_ss, o_ss, do_ss, dq_ss, dk_ss, dv_ss};
    if (!attn_strides_ok(seq, {q_sb, q_sg, q_sh, k_sb, k_sh, v_sb, v_sh, o_sb, o_sg, o_sh, do_sb, do_sg,
                               do_sh, dq_sb, dq_sg, dq_sh, dk_sb, dk_sh, dv_sb, dv_sh}))
      return KR_EUNSUPPORTED;
  }
  hipStream_t st = (hipStream_t)stream;
  const QLayout ql{q_ss, q_sb, q_sg, q_sh}, ol{o_ss, o_sb, o_sg, o_sh}, dol{do_ss, do_sb, do_sg, do_sh},
      dql{dq_ss, dq_sb, dq_sg, dq_sh};
  const KLayout kl{k_ss, k_sb, k_sh}, vl{v_ss, v_sb, v_sh}, dkl{dk_ss, dk_sb, dk_sh},
      dvl{dv_ss, dv_sb, dv_sh};
  float* delta = (float*)workspace;
  if (!attn_fast_path(s, hd) && !(flags & KR_ATTN_GENERAL_KERNELS)) {
    // padded into the MFMA kernels: dO, q, o, k, v and the log-sum-exp go in, dq, dk, dv come back
    const int sp = attn_padded_len(s), per = nq / nkv;
    const size_t qb = attn_padded_bytes(s, b, nq), kb = attn_padded_bytes(s, b, nkv);
    char* w = (char*)workspace;
    void *do_p = w, *q_p = w + qb, *o_p = w + 2 * qb, *dq_p = w + 3 * qb;
    w += 4 * qb;
    void *k_p = w, *v_p = w + kb, *dk_p = w + 2 * kb, *dv_p = w + 3 * kb;
    w += 4 * kb;
    float* lse_p = (float*)w;
    w += attn_padded_stat_bytes(s, b, nq);
    int rc2 = launch_pad(dout, do_p, s, b, nq, per, hd, dol, st);
    if (rc2 == KR_OK) rc2 = launch_pad(q, q_p, s, b, nq, per, hd, ql, st);
    if (rc2 == KR_OK) rc2 = launch_pad(o, o_p, s, b, nq, per, hd, ol, st);
    if (rc2 == KR_OK) rc2 = launch_pad(k, k_p, s, b, nkv, 1, hd, as_qlayout(kl), st);
    if (rc2 == KR_OK) rc2 = launch_pad(v, v_p, s, b, nkv, 1, hd, as_qlayout(vl), st);
    // rows beyond s: exp2(x - 1.4e30) = 0 for every finite score, so they add nothing to dK and dV
    if (rc2 == KR_OK) rc2 = launch_resize_rows(lse, lse_p, (int64_t)b * nq, s, sp, 1e30f, st);
    if (rc2 != KR_OK) return rc2;
    const QLayout pq = padded_qlayout(b, nq, per);
    const KLayout pk = padded_klayout(b, nkv);
    rc2 = attn_bwd_impl(do_p, q_p, k_p, v_p, o_p, lse_p, dq_p, dk_p, dv_p, w, sp, b, nq, nkv, HD, scale, pq.s_, pq.b_,
                        pq.g_, pq.h_, pk.s_, pk.b_, pk.h_, pk.s_, pk.b_, pk.h_, pq.s_, pq.b_, pq.g_, pq.h_, pq.s_,
                        pq.b_, pq.g_, pq.h_, pq.s_, pq.b_, pq.g_, pq.h_, pk.s_, pk.b_, pk.h_, pk.s_, pk.b_, pk.h_,
                        flags, stream);
    if (rc2 != KR_OK) return rc2;
    rc2 = launch_unpad(dq_p, dq, s, b, nq, per, hd, dql, st);
    if (rc2 == KR_OK) rc2 = launch_unpad(dk_p, dk, s, b, nkv, 1, hd, as_qlayout(dkl), st);
    if (rc2 == KR_OK) rc2 = launch_unpad(dv_p, dv, s, b, nkv, 1, hd, as_qlayout(dvl), st);
    return rc2;
  }
  if (!attn_fast_path(s, hd)) {
    using namespace general;
    const dim3 qgrid((s + GT - 1) / GT, nq, b), kgrid((s + GT - 1) / GT, nkv, b);
    hipLaunchKernelGGL(attn_general_delta_kernel, qgrid, dim3(GTHREADS), 0, st, (const bf16*)dout,
                       (const bf16*)o, delta, s, nq, nkv, hd, dol, ol);
    if (hipGetLastError() != hipSuccess) return KR_ELAUNCH;
    hipLaunchKernelGGL(attn_general_dkdv_kernel, kgrid, dim3(GTHREADS), 0, st, (const bf16*)q,
                       (const bf16*)k, (const bf16*)v, (const bf16*)dout, lse, (const float*)delta,
                       (bf16*)dk, (bf16*)dv, s, nq, nkv, hd, scale, ql, kl, vl, dol, dkl, dvl);
    if (hipGetLastError() != hipSuccess) return KR_ELAUNCH;
    hipLaunchKernelGGL(attn_general_dq_kernel, qgrid, dim3(GTHREADS), 0, st, (const bf16*)q,
                       (const bf16*)k, (const bf16*)v, (const bf16*)dout, lse, (const float*)delta,
                       (bf16*)dq, s, nq, nkv, hd, scale, ql, kl, vl, dol, dql);
    return kr_launch_status();
  }
  const int64_t rows = (int64_t)b * nq * s;
  float* neg_lse2 = delta + rows;
  float* part_k = neg_lse2 + rows;
  const AttnForms forms = attn_forms(s, b, nq, flags);
  const int qsplit = forms.qsplit;
  float* part_v = part_k + rows * qsplit * hd;
  // query heads of a KV group per dK/dV workgroup: as many as leave two workgroups per compute
  // unit (KR_DKDV_HPW_MAX: a build-time cap, for measurements)
  int hpw = 1;
  {
    const int per_group = nq / nkv;
    const int64_t wgs = (int64_t)(s / 128) * nq * b * qsplit;
    for (int h2 = per_group < KR_DKDV_HPW_MAX ? per_group : KR_DKDV_HPW_MAX; h2 > 1; --h2)
      if (per_group % h2 == 0 && wgs / h2 >= 2 * (int64_t)kr_compute_units()) {
        hpw = h2;
        break;
      }
  }
  const bool partial = nq / hpw != nkv || qsplit > 1;
  constexpr size_t lds_dkdv = 3 * (2 * BT_BYTES + 512) + 32768;  // three stages + the hand-over area
  constexpr size_t lds_dq = 2 * (2 * BT_BYTES);  // two stages of a K and a V tile
  constexpr size_t lds_dq_w64 = 3 * (2 * BT_BYTES) + 4 * 4096;  // three stages + a 4 KB output stage per wave
  static const hipError_t attr_status = [] {
    hipError_t e = hipFuncSetAttribute((const void*)attn_bwd_dkdv_kernel<false>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dkdv);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)attn_bwd_dkdv_kernel<true>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dkdv);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)attn_bwd_dq_kernel<1>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dq);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)attn_bwd_dq_kernel<2>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)(2 * lds_dq));
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)attn_bwd_dq_w64_kernel,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dq_w64);
    return e;
  }();
  if (attr_status != hipSuccess) return KR_ELAUNCH;

  const int per = nq / nkv;
  const float scale_log2 = scale * kLog2e;
  const int dq_blocks = (s / BQ) * nq * b;
  if (forms.shared_dq) {
    // 256-query tiles (one for every compute unit, or other streams beside): one wave per SIMD, 64 rows each.
    // It comes first: it also computes delta and the log2-domain copy of lse that the dK/dV kernel reads.
    hipLaunchKernelGGL(attn_bwd_dq_w64_kernel, dim3(dq_blocks / 2), dim3(256), lds_dq_w64, st,
                       (const bf16*)q, (const bf16*)k, (const bf16*)v, (const bf16*)dout, (const bf16*)o, lse,
                       delta, neg_lse2, (bf16*)dq, s, nq, nkv, scale, scale_log2, ql, kl, vl, dol, ol, dql);
  } else {
    hipLaunchKernelGGL(attn_delta_kernel, dim3((unsigned)((rows * 16 + 255) / 256)), dim3(256), 0, st,
                       (const bf16*)dout, (const bf16*)o, lse, delta, neg_lse2, s, nq, per, rows, dol, ol);
  }
  if (hipGetLastError() != hipSuccess) return KR_ELAUNCH;
  const dim3 grid_kv((s / 128) * (nq / hpw) * b * qsplit);
#define KR_DKDV_LAUNCH(P)                                                                           \
  hipLaunchKernelGGL((attn_bwd_dkdv_kernel<P>), grid_kv, dim3(512), lds_dkdv, st, (const bf16*)q,   \
                     (const bf16*)k, (const bf16*)v, (const bf16*)dout, (const float*)neg_lse2,     \
                     (const float*)delta, (bf16*)dk, (bf16*)dv, part_k, part_v, s, nq, nkv,         \
                     partial ? qsplit : 1, hpw, scale, scale_log2, ql, kl, vl, dol, dkl, dvl)
  if (partial) {
    KR_DKDV_LAUNCH(true);
    if (hipGetLastError() != hipSuccess) return KR_ELAUNCH;
    const int64_t total = (int64_t)b * nkv * s * 16;
    hipLaunchKernelGGL(attn_group_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       st, (const float*)part_k, (const float*)part_v, (bf16*)dk, (bf16*)dv, s,
                       nq / hpw, nkv, qsplit, total, dkl, dvl);
  } else {
    KR_DKDV_LAUNCH(false);
  }
#undef KR_DKDV_LAUNCH
  if (hipGetLastError() != hipSuccess) return KR_ELAUNCH;
  if (forms.shared_dq) return kr_launch_status();  // its dQ kernel ran in front of the dK/dV kernel
  if (dq_blocks <= 4 * 256) {  // few workgroups: the longest causal rows set the time
    hipLaunchKernelGGL((attn_bwd_dq_kernel<2>), dim3(dq_blocks), dim3(512), 2 * lds_dq, st,
                       (const bf16*)q, (const bf16*)k, (const bf16*)v, (const bf16*)dout, lse,
                       (const float*)delta, (bf16*)dq, s, nq, nkv, scale, scale_log2, ql, kl, vl, dol,
                       dql);
  } else {
    hipLaunchKernelGGL((attn_bwd_dq_kernel<1>), dim3(dq_blocks), dim3(256), lds_dq, st,
                       (const bf16*)q, (const bf16*)k, (const bf16*)v, (const bf16*)dout, lse,
                       (const float*)delta, (bf16*)dq, s, nq, nkv, scale, scale_log2, ql, kl, vl, dol,
                       dql);
  }
  return kr_launch_status();
}

extern "C" int kr_attn_bwd(const void* dout, const void* q, const void* k, const void* v,
                           const void* o, const float* lse, void* dq, void* dk, void* dv,
                           void* workspace, int s, int b, int nq, int nkv, int hd, float scale,
                           int64_t q_ss, int64_t q_sb, int64_t q_sg, int64_t q_sh, int64_t k_ss,
                           int64_t k_sb, int64_t k_sh, int64_t v_ss, int64_t v_sb, int64_t v_sh,
                           int64_t o_ss, int64_t o_sb, int64_t o_sg, int64_t o_sh, int64_t do_ss,
                           int64_t do_sb, int64_t do_sg, int64_t do_sh, int64_t dq_ss, int64_t dq_sb,
                           int64_t dq_sg, int64_t dq_sh, int64_t dk_ss, int64_t dk_sb, int64_t dk_sh,
                           int64_t dv_ss, int64_t dv_sb, int64_t dv_sh, void* stream) {
  return attn_bwd_impl(dout, q, k, v, o, lse, dq, dk, dv, workspace, s, b, nq, nkv, hd, scale, q_ss, q_sb, q_sg,
                       q_sh, k_ss, k_sb, k_sh, v_ss, v_sb, v_sh, o_ss, o_sb, o_sg, o_sh, do_ss, do_sb, do_sg,
                       do_sh, dq_ss, dq_sb, dq_sg, dq_sh, dk_ss, dk_sb, dk_sh, dv_ss, dv_sb, dv_sh, 0, stream);
}

extern "C" int kr_attn_bwd_flags(const void* dout, const void* q, const void* k, const void* v,
                                 const void* o, const float* lse, void* dq, void* dk, void* dv,
                                 void* workspace, int s, int b, int nq, int nkv, int hd, float scale,
                                 int64_t q_ss, int64_t q_sb, int64_t q_sg, int64_t q_sh, int64_t k_ss,
                                 int64_t k_sb, int64_t k_sh, int64_t v_ss, int64_t v_sb, int64_t v_sh,
                                 int64_t o_ss, int64_t o_sb, int64_t o_sg, int64_t o_sh, int64_t do_ss,
                                 int64_t do_sb, int64_t do_sg, int64_t do_sh, int64_t dq_ss,
                                 int64_t dq_sb, int64_t dq_sg, int64_t dq_sh, int64_t dk_ss,
                                 int64_t dk_sb, int64_t dk_sh, int64_t dv_ss, int64_t dv_sb,
                                 int64_t dv_sh, int flags, void* stream) {
  return attn_bwd_impl(dout, q, k, v, o, lse, dq, dk, dv, workspace, s, b, nq, nkv, hd, scale, q_ss, q_sb, q_sg,
                       q_sh, k_ss, k_sb, k_sh, v_ss, v_sb, v_sh, o_ss, o_sb, o_sg, o_sh, do_ss, do_sb, do_sg,
                       do_sh, dq_ss, dq_sb, dq_sg, dq_sh, dk_ss, dk_sb, dk_sh, dv_ss, dv_sb, dv_sh, flags, stream);
}

static int attn_fwd_impl(const void* q, const void* k, const void* v, void* o, float* lse, int s,
                           int b, int nq, int nkv, int hd, float scale, int64_t q_ss, int64_t q_sb,
                           int64_t q_sg, int64_t q_sh, int64_t k_ss, int64_t k_sb, int64_t k_sh,
                           int64_t v_ss, int64_t v_sb, int64_t v_sh, int64_t o_ss, int64_t o_sb,
                           int64_t o_sg, int64_t o_sh, int flags, void* stream, void* workspace = nullptr,
                           size_t workspace_bytes = 0) {
  if (flags & ~(KR_ATTN_BESIDE_OTHER_STREAMS | KR_ATTN_GENERAL_KERNELS)) return KR_EINVAL;
  if (!q || !k || !v || !o || !lse) return KR_EINVAL;
  if (workspace && !kr_aligned16(workspace)) return KR_EINVAL;
  const int rc = check_attn_common(s, b, nq, nkv, hd);
  if (rc != KR_OK) return rc;
  if (!kr_aligned16(q) || !kr_aligned16(k) || !kr_aligned16(v) || !kr_aligned16(o)) return KR_EINVAL;
  if ((q_ss | q_sb | q_sg | q_sh | k_ss | k_sb | k_sh | v_ss | v_sb | v_sh | o_ss | o_sb | o_sg |
       o_sh) % 8)
    return KR_EINVAL;
  {
    const int64_t seq[] = {q_ss, k_ss, v_ss, o_ss};
    if (!attn_strides_ok(seq, {q_sb, q_sg, q_sh, k_sb, k_sh, v_sb, v_sh, o_sb, o_sg, o_sh}))
      return KR_EUNSUPPORTED;
  }
  // (a workspace that is there but too small is a caller's mistake, not a request for the general kernels)
  if (!attn_fast_path(s, hd) && !(flags & KR_ATTN_GENERAL_KERNELS) && workspace != nullptr &&
      workspace_bytes < kr_attn_fwd_workspace_bytes(s, b, nq, nkv, hd))
    return KR_EINVAL;
  if (!attn_fast_path(s, hd) && !(flags & KR_ATTN_GENERAL_KERNELS) && workspace != nullptr) {
    // padded into the MFMA kernels
    hipStream_t st = (hipStream_t)stream;
    const int sp = attn_padded_len(s), per = nq / nkv;
    const size_t qb = attn_padded_bytes(s, b, nq), kb = attn_padded_bytes(s, b, nkv);
    char* w = (char*)workspace;
    void *q_p = w, *o_p = w + qb, *k_p = w + 2 * qb, *v_p = w + 2 * qb + kb;
    float* lse_p = (float*)(w + 2 * qb + 2 * kb);
    const QLayout ql{q_ss, q_sb, q_sg, q_sh}, ol{o_ss, o_sb, o_sg, o_sh};
    const KLayout kl{k_ss, k_sb, k_sh}, vl{v_ss, v_sb, v_sh};
    int rc2 = launch_pad(q, q_p, s, b, nq, per, hd, ql, st);
    if (rc2 == KR_OK) rc2 = launch_pad(k, k_p, s, b, nkv, 1, hd, as_qlayout(kl), st);
    if (rc2 == KR_OK) rc2 = launch_pad(v, v_p, s, b, nkv, 1, hd, as_qlayout(vl), st);
    if (rc2 != KR_OK) return rc2;
    const QLayout pq = padded_qlayout(b, nq, per);
    const KLayout pk = padded_klayout(b, nkv);
    rc2 = attn_fwd_impl(q_p, k_p, v_p, o_p, lse_p, sp, b, nq, nkv, HD, scale, pq.s_, pq.b_, pq.g_, pq.h_, pk.s_, pk.b_,
                        pk.h_, pk.s_, pk.b_, pk.h_, pq.s_, pq.b_, pq.g_, pq.h_, flags, stream);
    if (rc2 != KR_OK) return rc2;
    rc2 = launch_unpad(o_p, o, s, b, nq, per, hd, ol, st);
    if (rc2 == KR_OK) rc2 = launch_resize_rows(lse_p, lse, (int64_t)b * nq, sp, s, 0.f, st);
    return rc2;
  }
  if (!attn_fast_path(s, hd)) {
    using namespace general;
    const QLayout ql{q_ss, q_sb, q_sg, q_sh}, ol{o_ss, o_sb, o_sg, o_sh};
    const KLayout kl{k_ss, k_sb, k_sh}, vl{v_ss, v_sb, v_sh};
    hipLaunchKernelGGL(attn_general_fwd_kernel, dim3((s + GT - 1) / GT, nq, b), dim3(GTHREADS), 0,
                       (hipStream_t)stream, (const bf16*)q, (const bf16*)k, (const bf16*)v, (bf16*)o,
                       lse, s, nq, nkv, hd, scale, ql, kl, vl, ol);
    return kr_launch_status();
  }
  if (attn_forms(s, b, nq, flags).shared_fwd) {
    // 256-query tiles (one for every compute unit, or other streams beside): the halves share their K / V tiles
    constexpr size_t lds_sh = 3 * 16 * ((1024 + 16) + (1024 + 64));  // 100 KiB
    static const hipError_t attr_sh = hipFuncSetAttribute(
        (const void*)attn_fwd_sh_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_sh);
    if (attr_sh != hipSuccess) return KR_ELAUNCH;
    hipLaunchKernelGGL(attn_fwd_sh_kernel, dim3((s / 256) * nq * b), dim3(512), lds_sh,
                       (hipStream_t)stream, (const bf16*)q, (const bf16*)k, (const bf16*)v, (bf16*)o,
                       lse, s, nq, nkv, scale * kLog2e, q_ss, q_sb, q_sg, q_sh, k_ss, k_sb, k_sh, v_ss,
                       v_sb, v_sh, o_ss, o_sb, o_sg, o_sh);
    return kr_launch_status();
  }
  // two K and two V tiles of 17 KiB (padded blocks) per half; afterwards the same memory holds
  // the hand-over of half 1 (66 KiB) and, from 68 KiB on, 4 KiB of output staging per wave
  constexpr size_t lds_pp = 2 * 2 * 16 * ((1024 + 16) + (1024 + 64));  // 133 KiB
  static_assert(lds_pp >= 84 * 1024, "hand-over and output staging must fit");
  static const hipError_t attr_status = hipFuncSetAttribute(
      (const void*)attn_fwd_pp_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_pp);
  if (attr_status != hipSuccess) return KR_ELAUNCH;
  const int blocks = (s / BQ) * nq * b;
  hipLaunchKernelGGL(attn_fwd_pp_kernel, dim3(blocks), dim3(512), lds_pp, (hipStream_t)stream,
                     (const bf16*)q, (const bf16*)k, (const bf16*)v, (bf16*)o, lse, s, nq, nkv,
                     scale * kLog2e, q_ss, q_sb, q_sg, q_sh, k_ss, k_sb, k_sh, v_ss, v_sb, v_sh, o_ss,
                     o_sb, o_sg, o_sh);
  return kr_launch_status();
}

extern "C" int kr_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, int s,
                           int b, int nq, int nkv, int hd, float scale, int64_t q_ss, int64_t q_sb,
                           int64_t q_sg, int64_t q_sh, int64_t k_ss, int64_t k_sb, int64_t k_sh,
                           int64_t v_ss, int64_t v_sb, int64_t v_sh, int64_t o_ss, int64_t o_sb,
                           int64_t o_sg, int64_t o_sh, void* stream) {
  return attn_fwd_impl(q, k, v, o, lse, s, b, nq, nkv, hd, scale, q_ss, q_sb, q_sg, q_sh, k_ss, k_sb, k_sh, v_ss,
                       v_sb, v_sh, o_ss, o_sb, o_sg, o_sh, 0, stream);
}

extern "C" int kr_attn_fwd_flags(const void* q, const void* k, const void* v, void* o, float* lse,
                                 int s, int b, int nq, int nkv, int hd, float scale, int64_t q_ss,
                                 int64_t q_sb, int64_t q_sg, int64_t q_sh, int64_t k_ss, int64_t k_sb,
                                 int64_t k_sh, int64_t v_ss, int64_t v_sb, int64_t v_sh, int64_t o_ss,
                                 int64_t o_sb, int64_t o_sg, int64_t o_sh, int flags, void* stream) {
  return attn_fwd_impl(q, k, v, o, lse, s, b, nq, nkv, hd, scale, q_ss, q_sb, q_sg, q_sh, k_ss, k_sb, k_sh, v_ss,
                       v_sb, v_sh, o_ss, o_sb, o_sg, o_sh, flags, stream);
}

// kr_attn_fwd_flags with a workspace of kr_attn_fwd_workspace_bytes(): a shape outside the MFMA kernels (head
// dimension below 128, a sequence that is not whole 128-row tiles) is padded into them through the
// workspace instead of taking the general kernels.  A shape they take as it is needs no workspace.
extern "C" int kr_attn_fwd_ws(const void* q, const void* k, const void* v, void* o, float* lse, int s, int b,
                              int nq, int nkv, int hd, float scale, int64_t q_ss, int64_t q_sb, int64_t q_sg,
                              int64_t q_sh, int64_t k_ss, int64_t k_sb, int64_t k_sh, int64_t v_ss, int64_t v_sb,
                              int64_t v_sh, int64_t o_ss, int64_t o_sb, int64_t o_sg, int64_t o_sh, int flags,
                              void* workspace, size_t workspace_bytes, void* stream) {
  return attn_fwd_impl(q, k, v, o, lse, s, b, nq, nkv, hd, scale, q_ss, q_sb, q_sg, q_sh, k_ss, k_sb, k_sh, v_ss,
                       v_sb, v_sh, o_ss, o_sb, o_sg, o_sh, flags, stream, workspace, workspace_bytes);
}
