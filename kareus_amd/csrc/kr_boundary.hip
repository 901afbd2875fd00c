// Kernels at the two ends of the layer stack: token embedding (gather forward, deterministic
// scatter-add backward) and the cross-entropy loss over the output layer's logits.  All four are
// HBM-bound; algorithmic bytes are given per kernel.
#include "kr_common.h"

namespace {

constexpr int kThreads = 256;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---- embedding forward -------------------------------------------------------------------------
// out[si, bi, :] = weight[ids[bi, si] - vocab_start, :], or zeros when the id belongs to another
// vocabulary shard.  One wave per token, 16-byte accesses.  Bytes: 2 * T * hidden * 2 (+ ids).
__global__ __launch_bounds__(kThreads) void embedding_fwd_kernel(const int64_t* __restrict__ ids,
                                                                const bf16* __restrict__ weight,
                                                                bf16* __restrict__ out, int s, int b,
                                                                int hidden, int64_t vocab_start,
                                                                int64_t vocab_rows) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t tokens = (int64_t)s * b;
  const int nvec = hidden / 8;
  for (int64_t t = (int64_t)blockIdx.x * 4 + wave; t < tokens; t += (int64_t)gridDim.x * 4) {
    const int si = (int)(t / b), bi = (int)(t % b);  // t indexes the [s, b] output order
    const int64_t row = ids[(int64_t)bi * s + si] - vocab_start;
    const bool mine = row >= 0 && row < vocab_rows;
    const bf16* src = weight + (mine ? row : 0) * hidden;
    bf16* dst = out + t * hidden;
    for (int v = lane; v < nvec; v += 64) stg8(dst + v * 8, mine ? ldg8(src + v * 8) : zero8());
  }
}

// ---- embedding backward ------------------------------------------------------------------------
// dweight[r, :] = sum over tokens t with ids[t] - vocab_start == r of dout[t, :], rows without a
// token are written as zeros.  No atomics on the result: a workgroup owns kRowsPerBlock
// consecutive vocabulary rows.  It scans all ids once (memory order, [b, s]) and collects the
// tokens that fall into its rows as (row, position) keys in LDS, sorts the keys (bitonic), then
// walks them row by row, adding each row's tokens in position order with fp32 accumulators and
// writing the row with 16-byte stores.  The result does not depend on scheduling.
// A block whose rows attract more than kListCap tokens (a heavily repeated id) falls back to
// re-scanning the ids once per row, still in position order.
// Bytes: dout read once in total (each token belongs to one row) + dweight written once + the id
// array re-read by every workgroup out of L2.
constexpr int kRowsPerBlock = 64;
constexpr int kListCap = 4096;   // keys held in LDS (a power of two, for the bitonic sort)
constexpr int kPosBits = 26;     // key = row_in_block << 26 | position; positions < 2^26
template <int VECS>              // hidden / 8 <= 256 * VECS
__global__ __launch_bounds__(kThreads) void embedding_bwd_kernel(const int64_t* __restrict__ ids,
                                                                const bf16* __restrict__ dout,
                                                                bf16* __restrict__ dweight, int s,
                                                                int b, int hidden, int64_t vocab_start,
                                                                int64_t vocab_rows) {
  __shared__ unsigned keys[kListCap];
  __shared__ int count;
  const int tid = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * kRowsPerBlock;
  const int64_t tokens = (int64_t)s * b;
  const int nvec = hidden / 8;
  if (tid == 0) count = 0;
  __syncthreads();
  for (int64_t t = tid; t < tokens; t += kThreads) {
    const int64_t d = ids[t] - vocab_start - row0;
    if (d >= 0 && d < kRowsPerBlock) {
      const int slot = atomicAdd(&count, 1);
      if (slot < kListCap) keys[slot] = ((unsigned)d << kPosBits) | (unsigned)t;
    }
  }
  __syncthreads();
  const int n = count;
  const bool listed = n <= kListCap;
  if (listed && n > 1) {  // bitonic sort of the smallest power of two >= n keys, padded with ~0
    int m = 2;
    while (m < n) m <<= 1;
    for (int i = n + tid; i < m; i += kThreads) keys[i] = 0xffffffffu;
    __syncthreads();
    for (int k = 2; k <= m; k <<= 1)
      for (int j = k >> 1; j > 0; j >>= 1) {
        for (int i = tid; i < m; i += kThreads) {
          const int p = i ^ j;
          if (p > i) {
            const unsigned a = keys[i], c = keys[p];
            if ((a > c) == ((i & k) == 0)) {
              keys[i] = c;
              keys[p] = a;
            }
          }
        }
        __syncthreads();
      }
  }

  float acc[VECS][8];
  auto add_token = [&](int64_t t) {  // t: position in ids ([b, s] order), uniform across the block
    const int64_t bi = t / s, si = t - bi * s;
    const bf16* src = dout + (si * b + bi) * hidden;
#pragma unroll
    for (int c = 0; c < VECS; ++c) {
      const int v = tid + c * kThreads;
      if (v < nvec) {
        const bf16x8 g = ldg8(src + v * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[c][e] += (float)g[e];
      }
    }
  };
  int next = 0;
  for (int r = 0; r < kRowsPerBlock && row0 + r < vocab_rows; ++r) {
#pragma unroll
    for (int c = 0; c < VECS; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[c][e] = 0.f;
    if (listed) {
      while (next < n && (int)(keys[next] >> kPosBits) == r) {
        add_token(keys[next] & ((1u << kPosBits) - 1));
        ++next;
      }
    } else {
      for (int64_t t0 = 0; t0 < tokens; t0 += kThreads) {  // one more scan, this row only
        const int64_t t = t0 + tid;
        const bool hit = t < tokens && ids[t] - vocab_start - row0 == r;
        unsigned long long mask[4];
        if (__syncthreads_count(hit) == 0) continue;
        // walk the chunk's hits in order: each wave publishes its ballot through LDS
        unsigned long long* ballots = reinterpret_cast<unsigned long long*>(keys);
        const unsigned long long bal = __ballot(hit);
        if ((tid & 63) == 0) ballots[tid >> 6] = bal;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < 4; ++w) mask[w] = ballots[w];
        __syncthreads();
        for (int w = 0; w < 4; ++w)
          while (mask[w]) {
            const int bit = __builtin_ctzll(mask[w]);
            mask[w] &= mask[w] - 1;
            add_token(t0 + w * 64 + bit);
          }
      }
    }
    bf16* dst = dweight + (row0 + r) * hidden;
#pragma unroll
    for (int c = 0; c < VECS; ++c) {
      const int v = tid + c * kThreads;
      if (v < nvec) {
        bf16x8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (bf16)acc[c][e];
        stg8(dst + v * 8, o);
      }
    }
  }
}

// ---- cross entropy -----------------------------------------------------------------------------
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// One workgroup per row of logits: lse = log sum_j exp(x_j) (online max/sum in one pass over the
// row, log2 domain), loss = lse - x[label]; a label outside [0, vocab) marks an ignored row
// (loss 0).  Bytes: rows * vocab * 2 read.
__global__ __launch_bounds__(kThreads) void xent_fwd_kernel(const bf16* __restrict__ logits,
                                                           const int64_t* __restrict__ labels,
                                                           float* __restrict__ loss,
                                                           float* __restrict__ lse, int vocab,
                                                           int64_t ld) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const bf16* x = logits + row * ld;
  const int nvec = vocab / 8;
  float m = -INFINITY, l = 0.f;
  for (int v = threadIdx.x; v < nvec; v += kThreads) {
    const bf16x8 p = ldg8_stream(x + v * 8);
    float f[8], cm = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      f[e] = (float)p[e] * kLog2e;
      cm = fmaxf(cm, f[e]);
    }
    const float mn = fmaxf(m, cm);
    float add = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) add += __builtin_amdgcn_exp2f(f[e] - mn);
    l = l * __builtin_amdgcn_exp2f(m - mn) + add;
    m = mn;
  }
  const float mx = block_max(m, red);
  const float tot = block_sum(m == -INFINITY ? 0.f : l * __builtin_amdgcn_exp2f(m - mx), red);
  if (threadIdx.x == 0) {
    const float row_lse = (mx + __builtin_amdgcn_logf(tot)) * kLn2;  // natural log
    const int64_t lab = labels[row];
    lse[row] = row_lse;
    loss[row] = (lab >= 0 && lab < vocab) ? row_lse - (float)x[lab] : 0.f;
  }
}

// dlogits[j] = (exp(x_j - lse) - [j == label]) * dloss, zeros for an ignored row; may overwrite
// the logits.  Bytes: rows * vocab * 2 read + the same written.
__global__ __launch_bounds__(kThreads) void xent_bwd_kernel(const bf16* logits,
                                                           const int64_t* __restrict__ labels,
                                                           const float* __restrict__ lse,
                                                           const float* __restrict__ dloss,
                                                           bf16* dlogits, int vocab, int64_t ld,
                                                           int64_t ld_out) {
  const int64_t row = blockIdx.x;
  const bf16* x = logits + row * ld;
  bf16* dx = dlogits + row * ld_out;
  const int64_t lab = labels[row];
  const bool live = lab >= 0 && lab < vocab;
  const float g = live ? dloss[row] : 0.f;
  const float shift = lse[row] * kLog2e;
  const int nvec = vocab / 8;
  for (int v = threadIdx.x; v < nvec; v += kThreads) {
    const bf16x8 p = ldg8_stream(x + v * 8);
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float prob = __builtin_amdgcn_exp2f((float)p[e] * kLog2e - shift);
      if (v * 8 + e == lab) prob -= 1.f;
      o[e] = (bf16)(prob * g);
    }
    stg8_stream(dx + v * 8, o);
  }
}

}  // namespace

extern "C" int kr_embedding_fwd(const int64_t* ids, const void* weight, void* out, int s, int b,
                                int hidden, int64_t vocab_start, int64_t vocab_rows, void* stream) {
  if (!ids || !weight || !out || s <= 0 || b <= 0 || hidden <= 0 || vocab_rows <= 0) return KR_EINVAL;
  if (hidden % 8) return KR_EUNSUPPORTED;
  if (!kr_aligned16(weight) || !kr_aligned16(out)) return KR_EINVAL;
  int64_t blocks = ((int64_t)s * b + 3) / 4;
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipLaunchKernelGGL(embedding_fwd_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream,
                     ids, (const bf16*)weight, (bf16*)out, s, b, hidden, vocab_start, vocab_rows);
  return kr_launch_status();
}

extern "C" int kr_embedding_bwd(const int64_t* ids, const void* dout, void* dweight, int s, int b,
                                int hidden, int64_t vocab_start, int64_t vocab_rows, void* stream) {
  if (!ids || !dout || !dweight || s <= 0 || b <= 0 || hidden <= 0 || vocab_rows <= 0) return KR_EINVAL;
  if (hidden % 8 || hidden > 8192 || (int64_t)s * b >= ((int64_t)1 << kPosBits)) return KR_EUNSUPPORTED;
  if (!kr_aligned16(dout) || !kr_aligned16(dweight)) return KR_EINVAL;
  const unsigned blocks = (unsigned)((vocab_rows + kRowsPerBlock - 1) / kRowsPerBlock);
#define KR_EMB_BWD(C)                                                                               \
  hipLaunchKernelGGL(embedding_bwd_kernel<C>, dim3(blocks), dim3(kThreads), 0, (hipStream_t)stream, \
                     ids, (const bf16*)dout, (bf16*)dweight, s, b, hidden, vocab_start, vocab_rows)
  if (hidden <= 2048) KR_EMB_BWD(1);
  else if (hidden <= 4096) KR_EMB_BWD(2);
  else KR_EMB_BWD(4);
#undef KR_EMB_BWD
  return kr_launch_status();
}

extern "C" int kr_cross_entropy_fwd(const void* logits, const int64_t* labels, float* loss, float* lse,
                                    int64_t rows, int vocab, int64_t ld, void* stream) {
  if (!logits || !labels || !loss || !lse || rows <= 0 || vocab <= 0 || ld < vocab) return KR_EINVAL;
  if (vocab % 8 || ld % 8 || rows > 0x7fffffff) return KR_EUNSUPPORTED;
  if (!kr_aligned16(logits)) return KR_EINVAL;
  hipLaunchKernelGGL(xent_fwd_kernel, dim3((unsigned)rows), dim3(kThreads), 0, (hipStream_t)stream,
                     (const bf16*)logits, labels, loss, lse, vocab, ld);
  return kr_launch_status();
}

extern "C" int kr_cross_entropy_bwd(const void* logits, const int64_t* labels, const float* lse,
                                    const float* dloss, void* dlogits, int64_t rows, int vocab,
                                    int64_t ld, int64_t ld_out, void* stream) {
  if (!logits || !labels || !lse || !dloss || !dlogits || rows <= 0 || vocab <= 0 || ld < vocab ||
      ld_out < vocab)
    return KR_EINVAL;
  if (vocab % 8 || ld % 8 || ld_out % 8 || rows > 0x7fffffff) return KR_EUNSUPPORTED;
  if (!kr_aligned16(logits) || !kr_aligned16(dlogits)) return KR_EINVAL;
  hipLaunchKernelGGL(xent_bwd_kernel, dim3((unsigned)rows), dim3(kThreads), 0, (hipStream_t)stream,
                     (const bf16*)logits, labels, lse, dloss, (bf16*)dlogits, vocab, ld, ld_out);
  return kr_launch_status();
}
