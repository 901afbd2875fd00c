// HBM-bound passes: residual add, SwiGLU forward/backward, rotary embedding.
// Each thread moves 16-byte vectors (8 bf16); the math is fp32 with one rounding on store.
// Roofline for all of them is HBM bandwidth: bytes moved = inputs read once + outputs
// written once.
#include "kr_common.h"

namespace {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void add_kernel(const bf16* a, const bf16* b, bf16* out,
                                                       int64_t nvec,
                                                       int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < nvec; i += stride) {
    bf16x8 x = ldg8_stream(a + i * 8), y = ldg8_stream(b + i * 8), r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (bf16)((float)x[e] + (float)y[e]);
    stg8_stream(out + i * 8, r);
  }
  // tail (n not a multiple of 8)
  if (blockIdx.x == 0) {
    for (int64_t i = nvec * 8 + threadIdx.x; i < n; i += kThreads)
      out[i] = (bf16)((float)a[i] + (float)b[i]);
  }
}

// row-strided operands: element (r, c) of a at a[r*lda + c]; cols a multiple of 8
__global__ __launch_bounds__(kThreads) void add_rows_kernel(const bf16* a, int64_t lda, const bf16* b,
                                                            int64_t ldb, bf16* out, int64_t ldo,
                                                            int64_t rows, int cols) {
  const int nv = cols / 8;
  const int64_t total = rows * nv, stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / nv;
    const int c = (int)(i - r * nv) * 8;
    bf16x8 x = ldg8_stream(a + r * lda + c), y = ldg8_stream(b + r * ldb + c), o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)((float)x[e] + (float)y[e]);
    stg8_stream(out + r * ldo + c, o);
  }
}

// ---- hidden dropout in front of the residual add ------------------------------------------------
// Philox-4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3"): a counter-based
// generator, so element i of a call gets the same bits whatever the launch shape.  One call of the
// generator (128 bits) serves 8 elements, 16 bits each: an element is kept when its 16 bits are at
// or above p * 65536.
__device__ __forceinline__ void philox4x32_10(uint32_t (&ctr)[4], uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * ctr[0], p1 = (uint64_t)0xCD9E8D57u * ctr[2];
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ ctr[1] ^ k0, n2 = (uint32_t)(p0 >> 32) ^ ctr[3] ^ k1;
    ctr[1] = (uint32_t)p1;
    ctr[3] = (uint32_t)p0;
    ctr[0] = n0;
    ctr[2] = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

// out = residual + bf16(x * mask / (1 - p)); mask [rows, cols] bytes (1 = kept), dense.  The product
// is rounded to bf16 before the add, as the reference's dropout output is.
__global__ __launch_bounds__(kThreads) void dropout_add_kernel(const bf16* x, int64_t ldx, const bf16* res,
                                                               int64_t ldr, bf16* out, int64_t ldo,
                                                               uint8_t* __restrict__ mask, int64_t rows, int cols,
                                                               uint32_t threshold, float scale, uint64_t seed,
                                                               uint64_t offset) {
  const int nv = cols / 8;
  const int64_t total = rows * nv, stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / nv;
    const int c = (int)(i - r * nv) * 8;
    const uint64_t index = offset + (uint64_t)i;  // one generator call per 8 elements
    uint32_t ctr[4] = {(uint32_t)index, (uint32_t)(index >> 32), 0u, 0u};
    philox4x32_10(ctr, (uint32_t)seed, (uint32_t)(seed >> 32));
    const bf16x8 xv = ldg8_stream(x + r * ldx + c), rv = ldg8_stream(res + r * ldr + c);
    bf16x8 o;
    uint64_t m = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t bits = (ctr[e >> 1] >> (16 * (e & 1))) & 0xffffu;
      const bool keep = bits >= threshold;
      const bf16 d = (bf16)(keep ? (float)xv[e] * scale : 0.f);
      o[e] = (bf16)((float)rv[e] + (float)d);
      m |= (uint64_t)(keep ? 1 : 0) << (8 * e);
    }
    stg8_stream(out + r * ldo + c, o);
    *reinterpret_cast<uint64_t*>(mask + r * cols + c) = m;
  }
}

// dx = bf16(dy * mask * scale)
__global__ __launch_bounds__(kThreads) void dropout_bwd_kernel(const bf16* dy, int64_t lddy,
                                                               const uint8_t* __restrict__ mask, bf16* dx,
                                                               int64_t lddx, int64_t rows, int cols, float scale) {
  const int nv = cols / 8;
  const int64_t total = rows * nv, stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / nv;
    const int c = (int)(i - r * nv) * 8;
    const bf16x8 g = ldg8_stream(dy + r * lddy + c);
    const uint64_t m = *reinterpret_cast<const uint64_t*>(mask + r * cols + c);
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)(((m >> (8 * e)) & 1) ? (float)g[e] * scale : 0.f);
    stg8_stream(dx + r * lddx + c, o);
  }
}

__device__ __forceinline__ float sigmoidf_(float x) { return kr_sigmoidf(x); }

// x [rows, 2F] -> y [rows, F]; one thread per 8 output columns.
__global__ __launch_bounds__(kThreads) void swiglu_fwd_kernel(const bf16* __restrict__ x,
                                                              bf16* __restrict__ y, int64_t rows,
                                                              int F) {
  const int fv = F / 8;
  const int64_t total = rows * fv;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / fv;
    const int c = (int)(i - r * fv) * 8;
    const bf16* xr = x + r * 2 * F;
    bf16x8 g = ldg8_stream(xr + c), u = ldg8_stream(xr + F + c), o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x1 = (float)g[e], x2 = (float)u[e];
      o[e] = (bf16)kr_swiglu_f(x1, x2);
    }
    stg8_stream(y + r * F + c, o);
  }
}

__global__ __launch_bounds__(kThreads) void swiglu_bwd_kernel(const bf16* __restrict__ dy,
                                                              const bf16* __restrict__ x,
                                                              bf16* __restrict__ dx, int64_t rows,
                                                              int F) {
  const int fv = F / 8;
  const int64_t total = rows * fv;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / fv;
    const int c = (int)(i - r * fv) * 8;
    const bf16* xr = x + r * 2 * F;
    bf16x8 g = ldg8_stream(xr + c), u = ldg8_stream(xr + F + c), d = ldg8_stream(dy + r * F + c), d1, d2;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float dg, du;
      kr_swiglu_bwd_f((float)d[e], (float)g[e], (float)u[e], dg, du);
      d1[e] = (bf16)dg;
      d2[e] = (bf16)du;
    }
    stg8_stream(dx + r * 2 * F + c, d1);
    stg8_stream(dx + r * 2 * F + F + c, d2);
  }
}

// One block per sequence position: the hd/2 (cos, sin) pairs of that position are computed
// once into LDS, then the block streams all (batch, head) rows of the position.
// A thread owns 8 consecutive channels of the first half and the matching 8 of the second.
__global__ __launch_bounds__(kThreads) void rope_kernel(
    const bf16* t, bf16* out, const float* __restrict__ freqs, int b,
    int heads, int hd, int64_t ts, int64_t tb, int64_t th, int64_t os, int64_t ob, int64_t oh,
    float sin_sign, int group_size, int group_rotate) {
  __shared__ float cs[128], sn[128];
  const int pos = blockIdx.x;
  const int half = hd / 2;
  for (int i = threadIdx.x; i < half; i += kThreads) {
    float s_, c_;
    sincosf(freqs[(int64_t)pos * hd + i], &s_, &c_);
    cs[i] = c_;
    sn[i] = s_ * sin_sign;
  }
  __syncthreads();
  const int vec_per_row = half / 8;
  const int rows = b * heads;
  const int total = rows * vec_per_row;
  for (int i = threadIdx.x; i < total; i += kThreads) {
    const int row = i / vec_per_row;
    const int c = (i - row * vec_per_row) * 8;
    const int bi = row / heads, h = row - bi * heads;
    const bf16* src = t + pos * ts + bi * tb + h * th;
    bf16* dst = out + pos * os + bi * ob + h * oh;
    bf16x8 lo = ldg8(src + c), hi = ldg8(src + half + c), olo, ohi;
    if (h % group_size >= group_rotate) {  // a head that is carried along unrotated
      if (dst != src) {
        stg8(dst + c, lo);
        stg8(dst + half + c, hi);
      }
      continue;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float a = (float)lo[e], bb = (float)hi[e];
      float co = cs[c + e], si = sn[c + e];
      olo[e] = (bf16)(a * co - bb * si);
      ohi[e] = (bf16)(bb * co + a * si);
    }
    stg8(dst + c, olo);
    stg8(dst + half + c, ohi);
  }
}

inline int grid_for(int64_t work_items, int per_block) {
  int64_t blocks = (work_items + per_block - 1) / per_block;
  const int64_t cap = 256 * 16;  // 256 CUs, enough resident blocks to cover HBM latency
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

}  // namespace

extern "C" int kr_add(const void* a, const void* b, void* out, int64_t n, void* stream) {
  if (!a || !b || !out || n <= 0) return KR_EINVAL;
  if (!kr_aligned16(a) || !kr_aligned16(b) || !kr_aligned16(out)) return KR_EINVAL;
  const int64_t nvec = n / 8;
  hipLaunchKernelGGL(add_kernel, dim3(grid_for(nvec, kThreads)), dim3(kThreads), 0,
                     (hipStream_t)stream, (const bf16*)a, (const bf16*)b, (bf16*)out, nvec, n);
  return kr_launch_status();
}

extern "C" int kr_add_rows(const void* a, int64_t lda, const void* b, int64_t ldb, void* out,
                           int64_t ldo, int64_t rows, int cols, void* stream) {
  if (!a || !b || !out || rows <= 0 || cols <= 0 || lda < cols || ldb < cols || ldo < cols)
    return KR_EINVAL;
  if (cols % 8 || lda % 8 || ldb % 8 || ldo % 8) return KR_EUNSUPPORTED;
  if (!kr_aligned16(a) || !kr_aligned16(b) || !kr_aligned16(out)) return KR_EINVAL;
  hipLaunchKernelGGL(add_rows_kernel, dim3(grid_for(rows * (cols / 8), kThreads)), dim3(kThreads), 0,
                     (hipStream_t)stream, (const bf16*)a, lda, (const bf16*)b, ldb, (bf16*)out, ldo,
                     rows, cols);
  return kr_launch_status();
}

extern "C" int kr_dropout_add(const void* x, int64_t ldx, const void* residual, int64_t ldr, void* out,
                              int64_t ldo, void* mask, int64_t rows, int cols, float p, uint64_t seed,
                              uint64_t offset, void* stream) {
  if (!x || !residual || !out || !mask || rows <= 0 || cols <= 0 || ldx < cols || ldr < cols || ldo < cols)
    return KR_EINVAL;
  if (!(p >= 0.f) || !(p < 1.f)) return KR_EINVAL;
  if (cols % 8 || ldx % 8 || ldr % 8 || ldo % 8) return KR_EUNSUPPORTED;
  if (!kr_aligned16(x) || !kr_aligned16(residual) || !kr_aligned16(out) ||
      (reinterpret_cast<uintptr_t>(mask) & 7u))
    return KR_EINVAL;
  const uint32_t threshold = (uint32_t)(p * 65536.0f + 0.5f);  // kept: 16 random bits >= threshold
  hipLaunchKernelGGL(dropout_add_kernel, dim3(grid_for(rows * (cols / 8), kThreads)), dim3(kThreads), 0,
                     (hipStream_t)stream, (const bf16*)x, ldx, (const bf16*)residual, ldr, (bf16*)out, ldo,
                     (uint8_t*)mask, rows, cols, threshold, 1.0f / (1.0f - p), seed, offset);
  return kr_launch_status();
}

extern "C" int kr_dropout_bwd(const void* dy, int64_t lddy, const void* mask, void* dx, int64_t lddx,
                              int64_t rows, int cols, float scale, void* stream) {
  if (!dy || !mask || !dx || rows <= 0 || cols <= 0 || lddy < cols || lddx < cols) return KR_EINVAL;
  if (cols % 8 || lddy % 8 || lddx % 8) return KR_EUNSUPPORTED;
  if (!kr_aligned16(dy) || !kr_aligned16(dx) || (reinterpret_cast<uintptr_t>(mask) & 7u)) return KR_EINVAL;
  hipLaunchKernelGGL(dropout_bwd_kernel, dim3(grid_for(rows * (cols / 8), kThreads)), dim3(kThreads), 0,
                     (hipStream_t)stream, (const bf16*)dy, lddy, (const uint8_t*)mask, (bf16*)dx, lddx, rows,
                     cols, scale);
  return kr_launch_status();
}

extern "C" int kr_swiglu_fwd(const void* x, void* y, int64_t rows, int F, void* stream) {
  if (!x || !y || rows <= 0 || F <= 0) return KR_EINVAL;
  if (F % 8) return KR_EUNSUPPORTED;
  if (!kr_aligned16(x) || !kr_aligned16(y)) return KR_EINVAL;
  hipLaunchKernelGGL(swiglu_fwd_kernel, dim3(grid_for(rows * (F / 8), kThreads)), dim3(kThreads),
                     0, (hipStream_t)stream, (const bf16*)x, (bf16*)y, rows, F);
  return kr_launch_status();
}

extern "C" int kr_swiglu_bwd(const void* dy, const void* x, void* dx, int64_t rows, int F,
                             void* stream) {
  if (!dy || !x || !dx || rows <= 0 || F <= 0) return KR_EINVAL;
  if (F % 8) return KR_EUNSUPPORTED;
  if (!kr_aligned16(x) || !kr_aligned16(dy) || !kr_aligned16(dx)) return KR_EINVAL;
  hipLaunchKernelGGL(swiglu_bwd_kernel, dim3(grid_for(rows * (F / 8), kThreads)), dim3(kThreads),
                     0, (hipStream_t)stream, (const bf16*)dy, (const bf16*)x, (bf16*)dx, rows, F);
  return kr_launch_status();
}

extern "C" int kr_rope(const void* t, void* out, const float* freqs, int s, int b, int heads,
                       int hd, int64_t ts, int64_t tb, int64_t th, int64_t os, int64_t ob,
                       int64_t oh, int backward, int group_size, int group_rotate, void* stream) {
  if (!t || !out || !freqs || s <= 0 || b <= 0 || heads <= 0 || hd <= 0) return KR_EINVAL;
  if (group_size <= 0 || group_rotate <= 0 || group_rotate > group_size || heads % group_size)
    return KR_EINVAL;
  if (hd % 16 || hd > 256) return KR_EUNSUPPORTED;
  if (!kr_aligned16(t) || !kr_aligned16(out)) return KR_EINVAL;
  if ((ts | tb | th | os | ob | oh) % 8) return KR_EINVAL;
  if (ts <= 0 || tb <= 0 || th <= 0 || os <= 0 || ob <= 0 || oh <= 0) return KR_EUNSUPPORTED;
  hipLaunchKernelGGL(rope_kernel, dim3(s), dim3(kThreads), 0, (hipStream_t)stream,
                     (const bf16*)t, (bf16*)out, freqs, b, heads, hd, ts, tb, th, os, ob, oh,
                     backward ? -1.0f : 1.0f, group_size, group_rotate);
  return kr_launch_status();
}
