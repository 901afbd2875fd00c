// RMSNorm over the head dimension of the query and key heads of a fused QKV projection output
// (the q / k layernorm of the QKV-split operator, kareus/megatron/core/extensions/ops/
// qkv_postprocess.py:110-118 forward, :147-160 backward; the norm itself is the RMSNorm of
// kareus/transformer_engine/pytorch/ops/basic/rmsnorm.py:165-273 with the head dimension as its
// width and one weight vector for all query heads, one for all key heads).
//
// Roofline: HBM.  The fused buffer [tokens, ng, per + 2, hd] is a dense matrix of rows of hd
// channels: row (t, g, j) is query head j of group g for j < per, the group's key head for
// j = per and its value head for j = per + 1.  Forward reads every row once and writes every row
// once (query and key rows normalised, value rows copied, so that the result is again a fused
// buffer the rotary and attention kernels address as before) plus 4 bytes of 1/rms per
// normalised row; backward reads the gradient rows, the saved input rows and 1/rms and rewrites
// the query and key gradient rows in place.  A row is shared by hd / 8 lanes (16-byte vectors);
// the weight gradients are summed per lane over the rows it visits, then across the row slots of
// a workgroup through LDS, then across workgroups by a second small kernel: no atomics, a fixed
// order.
#include "kr_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kMaxBlocks = 1024;

template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, KR_WAVE);
  return v;
}

template <int LPR>  // lanes per row = hd / 8
__global__ __launch_bounds__(kThreads) void qk_norm_fwd_kernel(const bf16* __restrict__ mixed,
                                                               const bf16* __restrict__ gamma_q,
                                                               const bf16* __restrict__ gamma_k,
                                                               bf16* __restrict__ out, float* __restrict__ rstd,
                                                               int64_t rows, int per, float eps) {
  constexpr int HD = LPR * 8, RPB = kThreads / LPR;  // rows a workgroup handles at a time
  const int sub = threadIdx.x % LPR, slot = threadIdx.x / LPR;
  const bf16x8 gq = ldg8(gamma_q + sub * 8), gk = ldg8(gamma_k + sub * 8);
  for (int64_t r = (int64_t)blockIdx.x * RPB + slot; r < rows; r += (int64_t)gridDim.x * RPB) {
    const int j = (int)(r % (per + 2));
    const bf16x8 x = ldg8(mixed + r * HD + sub * 8);
    if (j == per + 1) {  // a value head: carried along
      stg8_stream(out + r * HD + sub * 8, x);
      continue;          // (all lanes of a row take the same branch)
    }
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += (float)x[e] * (float)x[e];
    ss = row_sum<LPR>(ss);
    const float rs = __builtin_amdgcn_rsqf(ss * (1.0f / HD) + eps);
    const bf16x8 g = j < per ? gq : gk;
    bf16x8 y;
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (bf16)((float)x[e] * rs * (float)g[e]);
    stg8_stream(out + r * HD + sub * 8, y);
    if (sub == 0) rstd[(r / (per + 2)) * (per + 1) + j] = rs;
  }
}

// dmixed rows of query and key heads: dx = rstd * (dy * gamma - xhat * mean(dy * gamma * xhat)), in place;
// partial weight gradients of this workgroup to part[blockIdx.x][2][HD] (query weights, key weights)
template <int LPR>
__global__ __launch_bounds__(kThreads) void qk_norm_bwd_kernel(bf16* dmixed, const bf16* __restrict__ mixed,
                                                               const float* __restrict__ rstd,
                                                               const bf16* __restrict__ gamma_q,
                                                               const bf16* __restrict__ gamma_k,
                                                               float* __restrict__ part, int64_t rows, int per) {
  constexpr int HD = LPR * 8, RPB = kThreads / LPR;
  __shared__ float red[2][RPB][HD];
  const int sub = threadIdx.x % LPR, slot = threadIdx.x / LPR;
  const bf16x8 gq = ldg8(gamma_q + sub * 8), gk = ldg8(gamma_k + sub * 8);
  float dgq[8], dgk[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) dgq[e] = dgk[e] = 0.f;
  for (int64_t r = (int64_t)blockIdx.x * RPB + slot; r < rows; r += (int64_t)gridDim.x * RPB) {
    const int j = (int)(r % (per + 2));
    if (j == per + 1) continue;
    const bf16x8 x = ldg8(mixed + r * HD + sub * 8), dy = ldg8(dmixed + r * HD + sub * 8);
    const float rs = rstd[(r / (per + 2)) * (per + 1) + j];
    const bf16x8 g = j < per ? gq : gk;
    float xh[8], dyg[8], dot = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      xh[e] = (float)x[e] * rs;
      dyg[e] = (float)dy[e] * (float)g[e];
      dot += dyg[e] * xh[e];
    }
    dot = row_sum<LPR>(dot) * (1.0f / HD);
    bf16x8 dx;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      dx[e] = (bf16)(rs * (dyg[e] - xh[e] * dot));
      const float dgam = (float)dy[e] * xh[e];
      if (j < per)
        dgq[e] += dgam;
      else
        dgk[e] += dgam;
    }
    stg8(dmixed + r * HD + sub * 8, dx);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    red[0][slot][sub * 8 + e] = dgq[e];
    red[1][slot][sub * 8 + e] = dgk[e];
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 2 * HD; i += kThreads) {
    const int which = i / HD, c = i % HD;
    float acc = 0.f;
#pragma unroll 4
    for (int s2 = 0; s2 < RPB; ++s2) acc += red[which][s2][c];
    part[((int64_t)blockIdx.x * 2 + which) * HD + c] = acc;
  }
}

// Sums the workgroups' partial rows: a workgroup takes 16 of the 2 * hd columns (query weights, then key
// weights); its 64 x 16 threads each walk every 64th partial row of one column, then the 64 walkers of a
// column are summed through LDS, always in the same order.
constexpr int kWalkers = 64;
__global__ __launch_bounds__(16 * kWalkers) void qk_norm_dgamma_kernel(const float* __restrict__ part, int nblocks,
                                                                       int hd, bf16* __restrict__ dgamma_q,
                                                                       bf16* __restrict__ dgamma_k) {
  __shared__ float red[kWalkers][17];
  const int c = threadIdx.x % 16, walker = threadIdx.x / 16;
  const int col = blockIdx.x * 16 + c;  // < 2 * hd: hd is a multiple of 16
  float acc = 0.f;
#pragma unroll 8
  for (int b = walker; b < nblocks; b += kWalkers) acc += part[(int64_t)b * 2 * hd + col];
  red[walker][c] = acc;
  __syncthreads();
  if (walker == 0) {
    float sum = 0.f;
#pragma unroll 8
    for (int w = 0; w < kWalkers; ++w) sum += red[w][c];
    (col < hd ? dgamma_q : dgamma_k)[col % hd] = (bf16)sum;
  }
}

int qk_blocks(int64_t rows, int hd) {
  const int rpb = kThreads / (hd / 8);
  const int64_t want = (rows + rpb - 1) / rpb;
  return (int)(want < kMaxBlocks ? want : kMaxBlocks);
}

bool qk_shape_ok(int64_t tokens, int ng, int per) {
  return tokens > 0 && ng > 0 && per > 0;
}

}  // namespace

extern "C" size_t kr_qk_norm_bwd_workspace_bytes(int64_t tokens, int ng, int per, int hd) {
  if (!qk_shape_ok(tokens, ng, per) || (hd != 64 && hd != 128 && hd != 256)) return 0;
  return (size_t)qk_blocks(tokens * ng * (per + 2), hd) * 2 * hd * sizeof(float);
}

extern "C" int kr_qk_norm_fwd(const void* mixed, const void* gamma_q, const void* gamma_k, void* out, float* rstd,
                              int64_t tokens, int ng, int per, int hd, float eps, void* stream) {
  if (!mixed || !gamma_q || !gamma_k || !out || !rstd || out == mixed || !qk_shape_ok(tokens, ng, per))
    return KR_EINVAL;
  if (hd != 64 && hd != 128 && hd != 256) return KR_EUNSUPPORTED;
  if (!kr_aligned16(mixed) || !kr_aligned16(gamma_q) || !kr_aligned16(gamma_k) || !kr_aligned16(out))
    return KR_EINVAL;
  const int64_t rows = tokens * ng * (per + 2);
  const dim3 grid(qk_blocks(rows, hd));
#define KR_QK_FWD(L)                                                                                   \
  hipLaunchKernelGGL(qk_norm_fwd_kernel<L>, grid, dim3(kThreads), 0, (hipStream_t)stream,            \
                     (const bf16*)mixed, (const bf16*)gamma_q, (const bf16*)gamma_k, (bf16*)out, rstd, rows, \
                     per, eps)
  if (hd == 64)
    KR_QK_FWD(8);
  else if (hd == 128)
    KR_QK_FWD(16);
  else
    KR_QK_FWD(32);
#undef KR_QK_FWD
  return kr_launch_status();
}

extern "C" int kr_qk_norm_bwd(void* dmixed, const void* mixed, const float* rstd, const void* gamma_q,
                              const void* gamma_k, void* dgamma_q, void* dgamma_k, void* workspace,
                              int64_t tokens, int ng, int per, int hd, void* stream) {
  if (!dmixed || !mixed || !rstd || !gamma_q || !gamma_k || !dgamma_q || !dgamma_k || !workspace ||
      !qk_shape_ok(tokens, ng, per))
    return KR_EINVAL;
  if (hd != 64 && hd != 128 && hd != 256) return KR_EUNSUPPORTED;
  if (!kr_aligned16(dmixed) || !kr_aligned16(mixed) || !kr_aligned16(gamma_q) || !kr_aligned16(gamma_k) ||
      !kr_aligned16(workspace))
    return KR_EINVAL;
  const int64_t rows = tokens * ng * (per + 2);
  const int nblocks = qk_blocks(rows, hd);
#define KR_QK_BWD(L)                                                                                   \
  hipLaunchKernelGGL(qk_norm_bwd_kernel<L>, dim3(nblocks), dim3(kThreads), 0, (hipStream_t)stream,    \
                     (bf16*)dmixed, (const bf16*)mixed, rstd, (const bf16*)gamma_q, (const bf16*)gamma_k,   \
                     (float*)workspace, rows, per)
  if (hd == 64)
    KR_QK_BWD(8);
  else if (hd == 128)
    KR_QK_BWD(16);
  else
    KR_QK_BWD(32);
#undef KR_QK_BWD
  if (hipGetLastError() != hipSuccess) return KR_ELAUNCH;
  hipLaunchKernelGGL(qk_norm_dgamma_kernel, dim3(2 * hd / 16), dim3(16 * kWalkers), 0,
                     (hipStream_t)stream, (const float*)workspace, nblocks, hd, (bf16*)dgamma_q, (bf16*)dgamma_k);
  return kr_launch_status();
}
