// RMSNorm forward and backward.  HBM-bound: forward reads x and writes y (+4 B/row of rstd),
// backward reads dy and x and writes dx; gamma stays in cache.  One wavefront owns one row at
// a time and keeps it in registers (NCHUNK 16-byte vectors per lane), so each element is read
// from HBM exactly once.  Row statistics are wave shuffle reductions in fp32.
//
// The weight gradient is a column sum over all rows: every wave accumulates its rows' dy*xhat
// in registers (a lane always owns the same columns), the waves of a block combine through
// LDS, each block writes one fp32 partial row into the workspace, and a second small kernel
// sums the partial rows and rounds to bf16.
#include <mutex>

#include "kr_common.h"

namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * KR_WAVE;
constexpr int kMaxBwdBlocks = 512;

// Row runs: the rows of a tensor may come in runs of 2^sh consecutive rows (stride ld) whose starts are
// `outer` elements apart — a nanobatch of 2^sh sequences cut out of a [s, b, h] tensor along b, used in
// place.  A plain matrix has sh = 0 (outer unused).
struct Runs {
  int sh;
  int64_t outer;
};
__device__ __forceinline__ int64_t row_at(int64_t row, int64_t ld, Runs r) {
  return r.sh ? (row >> r.sh) * r.outer + (row & ((1 << r.sh) - 1)) * ld : row * ld;
}

template <int NCHUNK>
__global__ __launch_bounds__(kThreads) void rmsnorm_fwd_kernel(const bf16* __restrict__ x,
                                                               const bf16* __restrict__ gamma,
                                                               bf16* __restrict__ y,
                                                               float* __restrict__ rstd, int rows,
                                                               int cols, int64_t x_ld, float eps,
                                                               Runs x_runs) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nvec = cols / 8;
  const float inv_cols = 1.0f / (float)cols;
  bf16x8 g[NCHUNK];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const int v = lane + c * 64;
    g[c] = v < nvec ? ldg8(gamma + v * 8) : zero8();
  }
  for (int row = blockIdx.x * kWaves + wave; row < rows; row += gridDim.x * kWaves) {
    const bf16* xr = x + row_at(row, x_ld, x_runs);
    bf16x8 xv[NCHUNK];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int v = lane + c * 64;
      xv[c] = v < nvec ? ldg8(xr + v * 8) : zero8();
    }
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float f = (float)xv[c][e];
        ss += f * f;
      }
    ss = wave_sum(ss);
    const float rs = rsqrtf(ss * inv_cols + eps);
    if (lane == 0) rstd[row] = rs;
    bf16* yr = y + (int64_t)row * cols;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int v = lane + c * 64;
      if (v < nvec) {
        bf16x8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (bf16)(((float)xv[c][e] * rs) * (float)g[c][e]);
        stg8_stream(yr + v * 8, o);
      }
    }
  }
}

// ADD: the residual fork that follows the norm in the backward pass is folded in: the input
// gradient of the norm is rounded to bf16 exactly as the stand-alone kernel rounds it and then
// the gradient of the residual branch is added, so the fused result is bit-identical to the
// two kernels run one after the other while one write and one read of the tensor disappear.
// FULL: the row is exactly SPLIT * NCHUNK * 64 vectors long (hidden sizes 512 * k).  No lane is
// ever idle, so the loop body is straight-line code and every load of a row — x, dy and the
// residual gradient — is issued before the first wait; with per-chunk bounds checks each chunk of
// the output pass paid its own round trip to memory.
// SPLIT = 2: two waves share a row (rows of more than 4096 elements), each holding half of it, so
// that a wave's registers still hold its part; the halves of the row's dot product meet in LDS.
template <int NCHUNK, bool ADD, bool FULL, int SPLIT>
__global__ __launch_bounds__(kThreads) void rmsnorm_bwd_kernel(
    const bf16* __restrict__ dy, const bf16* __restrict__ x, const float* __restrict__ rstd,
    const bf16* __restrict__ gamma, const bf16* __restrict__ dres, bf16* __restrict__ dx,
    float* __restrict__ partial, int rows, int cols, int64_t dy_ld, int64_t x_ld, int64_t dres_ld,
    int64_t dx_ld, Runs x_runs, Runs dres_runs, Runs dx_runs) {
  constexpr int kRowsPerBlock = kWaves / SPLIT;
  __shared__ float red[kWaves - 1][64 * 8];
  __shared__ float halves[2][kRowsPerBlock][2];  // [iteration parity][row of the block][half]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int part = SPLIT == 2 ? (wave & 1) : 0;      // which half of the row this wave holds
  const int slot = SPLIT == 2 ? (wave >> 1) : wave;  // which of the block's rows
  const int nvec = cols / 8;
  const float inv_cols = 1.0f / (float)cols;
  // this lane's vectors of a row: v0, v0 + 64, ...
  const int v0 = part * NCHUNK * 64 + lane;
  bf16x8 g[NCHUNK];
  float dg[NCHUNK][8];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const int v = v0 + c * 64;
    g[c] = (FULL || v < nvec) ? ldg8(gamma + v * 8) : zero8();
#pragma unroll
    for (int e = 0; e < 8; ++e) dg[c][e] = 0.f;
  }
  int parity = 0;
  // (with two waves per row every wave of the block makes the same number of trips: the loop
  // holds a workgroup barrier)
  for (int base = blockIdx.x * kRowsPerBlock; base < rows; base += gridDim.x * kRowsPerBlock) {
    const int row = base + slot;
    const bool active = SPLIT == 1 || row < rows;  // SPLIT == 1: the loop bound is the wave's own
    if (SPLIT == 1 && row >= rows) break;
    const int64_t r64 = active ? row : 0;
    const bf16* xr = x + row_at(r64, x_ld, x_runs);
    const bf16* dr = dy + r64 * dy_ld;
    const bf16* rr = ADD ? dres + row_at(r64, dres_ld, dres_runs) : nullptr;
    const float rs = active ? rstd[r64] : 0.f;
    bf16x8 xv[NCHUNK], dv[NCHUNK], rv[ADD && FULL ? NCHUNK : 1];
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int v = v0 + c * 64;
      xv[c] = (active && (FULL || v < nvec)) ? ldg8_stream(xr + v * 8) : zero8();
      dv[c] = (active && (FULL || v < nvec)) ? ldg8_stream(dr + v * 8) : zero8();
    }
    if (ADD && FULL) {
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) rv[c] = active ? ldg8_stream(rr + (v0 + c * 64) * 8) : zero8();
    }
    float dot = 0.f;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xh = (float)xv[c][e] * rs;
        const float d = (float)dv[c][e];
        dot += d * (float)g[c][e] * xh;
        dg[c][e] += d * xh;
      }
    dot = wave_sum(dot);
    if (SPLIT == 2) {
      if (lane == 0) halves[parity][slot][part] = dot;
      __syncthreads();
      dot = halves[parity][slot][0] + halves[parity][slot][1];
      parity ^= 1;  // the next row uses the other buffer: one barrier per row is enough
    }
    dot *= inv_cols;
    bf16* oxr = dx + row_at(r64, dx_ld, dx_runs);
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int v = v0 + c * 64;
      if (active && (FULL || v < nvec)) {
        bf16x8 o, r;
        if (ADD) r = FULL ? rv[c] : ldg8_stream(rr + v * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xh = (float)xv[c][e] * rs;
          o[e] = (bf16)(rs * ((float)dv[c][e] * (float)g[c][e] - xh * dot));
          if (ADD) o[e] = (bf16)((float)o[e] + (float)r[e]);
        }
        stg8_stream(oxr + v * 8, o);
      }
    }
  }
  // combine the waves that hold the same columns chunk by chunk, then publish the block's
  // partial row
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (slot > 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e) red[(slot - 1) * SPLIT + part][e * 64 + lane] = dg[c][e];
    }
    __syncthreads();
    if (slot == 0) {
      const int v = v0 + c * 64;
      if (v < nvec) {
        float* pr = partial + (int64_t)blockIdx.x * cols + v * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float sum = dg[c][e];
#pragma unroll
          for (int w = 1; w < kRowsPerBlock; ++w) sum += red[(w - 1) * SPLIT + part][e * 64 + lane];
          pr[e] = sum;
        }
      }
    }
    __syncthreads();
  }
}

// dgamma[col] = sum over partial rows.  A block of 16 waves owns 32 columns; half-waves take
// different partial rows (128-byte coalesced reads), 32 row-lanes in all, each summing every
// 32nd row into four independent accumulators so that many loads are in flight; the row-lanes
// are combined through LDS in a fixed order.
constexpr int kDgammaThreads = 1024;
__global__ __launch_bounds__(kDgammaThreads) void rmsnorm_dgamma_kernel(const float* __restrict__ partial,
                                                                        bf16* __restrict__ dgamma,
                                                                        int nparts, int cols) {
  __shared__ float red[32][33];
  const int c = threadIdx.x & 31, rl = threadIdx.x >> 5;  // column in block, row-lane 0..31
  const int col = blockIdx.x * 32 + c;
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  if (col < cols) {
    const float* src = partial + col;
    int p = rl;
    for (; p + 96 < nparts; p += 128) {
      a0 += src[(int64_t)p * cols];
      a1 += src[(int64_t)(p + 32) * cols];
      a2 += src[(int64_t)(p + 64) * cols];
      a3 += src[(int64_t)(p + 96) * cols];
    }
    for (; p < nparts; p += 32) a0 += src[(int64_t)p * cols];
  }
  red[rl][c] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (rl == 0 && col < cols) {
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 32; ++r) sum += red[r][c];
    dgamma[col] = (bf16)sum;
  }
}

// Rows wider than this are shared by two waves (half the registers per wave, twice the waves per
// SIMD to hide the latency of a row's loads behind)
#ifndef KR_RMS_SPLIT_ABOVE
#define KR_RMS_SPLIT_ABOVE 2048
#endif
inline int bwd_split(int cols) { return cols > KR_RMS_SPLIT_ABOVE ? 2 : 1; }

inline int bwd_blocks(int rows, int cols) {
  const int rows_per_block = kWaves / bwd_split(cols);
  int blocks = (rows + rows_per_block - 1) / rows_per_block;
  return blocks > kMaxBwdBlocks ? kMaxBwdBlocks : blocks;
}

inline int chunks_for(int cols) { return (cols / 8 + 63) / 64; }

}  // namespace

// at most 8 vectors per lane (backward: wider rows are shared by two waves)
#define KR_DISPATCH_CHUNKS8(NC, CALL) \
  switch (NC) {                       \
    case 1: { constexpr int C_ = 1; CALL; } break;   \
    case 2: { constexpr int C_ = 2; CALL; } break;   \
    case 3: { constexpr int C_ = 3; CALL; } break;   \
    case 4: { constexpr int C_ = 4; CALL; } break;   \
    case 5: case 6: { constexpr int C_ = 6; CALL; } break;   \
    case 7: case 8: { constexpr int C_ = 8; CALL; } break;   \
    default: return KR_EUNSUPPORTED;  \
  }

#define KR_DISPATCH_CHUNKS(NC, CALL) \
  switch (NC) {                      \
    case 1: { constexpr int C_ = 1; CALL; } break;   \
    case 2: { constexpr int C_ = 2; CALL; } break;   \
    case 3: { constexpr int C_ = 3; CALL; } break;   \
    case 4: { constexpr int C_ = 4; CALL; } break;   \
    case 5: case 6: { constexpr int C_ = 6; CALL; } break;   \
    case 7: case 8: { constexpr int C_ = 8; CALL; } break;   \
    default: { constexpr int C_ = 16; CALL; } break; \
  }

namespace {
// rows per run (a power of two, 1 = plain) and distance between run starts -> Runs; false if invalid
bool make_runs(int run_rows, int64_t run_ld, int rows, Runs* out, int* rc) {
  *out = Runs{0, 0};
  if (run_rows == 1) return true;
  if (run_rows < 1 || (run_rows & (run_rows - 1)) || run_ld <= 0) { *rc = KR_EINVAL; return false; }
  if (run_rows > 1024 || run_ld % 8 || rows % run_rows) { *rc = KR_EUNSUPPORTED; return false; }
  int sh = 0;
  while ((1 << sh) < run_rows) ++sh;
  *out = Runs{sh, run_ld};
  return true;
}
int rmsnorm_fwd_impl(const void* x, const void* gamma, void* y, float* rstd, int rows, int cols,
                     int64_t x_ld, Runs x_runs, float eps, void* stream);
}  // namespace

extern "C" int kr_rmsnorm_fwd(const void* x, const void* gamma, void* y, float* rstd, int rows,
                              int cols, int64_t x_ld, float eps, void* stream) {
  return rmsnorm_fwd_impl(x, gamma, y, rstd, rows, cols, x_ld, Runs{0, 0}, eps, stream);
}

// kr_rmsnorm_fwd on an input whose rows come in runs (a nanobatch of several sequences read in place)
extern "C" int kr_rmsnorm_fwd_runs(const void* x, const void* gamma, void* y, float* rstd, int rows,
                                   int cols, int64_t x_ld, int x_run_rows, int64_t x_run_ld, float eps,
                                   void* stream) {
  Runs xr;
  int rc = KR_OK;
  if (rows <= 0 || !make_runs(x_run_rows, x_run_ld, rows, &xr, &rc)) return rc == KR_OK ? KR_EINVAL : rc;
  return rmsnorm_fwd_impl(x, gamma, y, rstd, rows, cols, x_ld, xr, eps, stream);
}

namespace {
int rmsnorm_fwd_impl(const void* x, const void* gamma, void* y, float* rstd, int rows, int cols,
                     int64_t x_ld, Runs x_runs, float eps, void* stream) {
  if (!x || !gamma || !y || !rstd || rows <= 0 || cols <= 0 || x_ld < cols) return KR_EINVAL;
  if (cols % 8 || x_ld % 8 || cols > 8192) return KR_EUNSUPPORTED;
  if (!kr_aligned16(x) || !kr_aligned16(y) || !kr_aligned16(gamma)) return KR_EINVAL;
  int blocks = (rows + kWaves - 1) / kWaves;
  if (blocks > 256 * 8) blocks = 256 * 8;
  const int nc = chunks_for(cols);
  KR_DISPATCH_CHUNKS(nc, hipLaunchKernelGGL(rmsnorm_fwd_kernel<C_>, dim3(blocks), dim3(kThreads), 0,
                                           (hipStream_t)stream, (const bf16*)x, (const bf16*)gamma,
                                           (bf16*)y, rstd, rows, cols, x_ld, eps, x_runs));
  return kr_launch_status();
}
}  // namespace

extern "C" size_t kr_rmsnorm_bwd_workspace_bytes(int rows, int cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return (size_t)bwd_blocks(rows, cols) * (size_t)cols * sizeof(float);
}

namespace {
struct BwdRuns {
  Runs x{0, 0}, dres{0, 0}, dx{0, 0};
};
int rmsnorm_bwd_impl(const void* dy, const void* x, const float* rstd, const void* gamma,
                     const void* dres, void* dx, void* dgamma, void* workspace, int rows, int cols,
                     int64_t dy_ld, int64_t x_ld, int64_t dres_ld, int64_t dx_ld, void* stream,
                     const BwdRuns& runs = BwdRuns());
}

extern "C" int kr_rmsnorm_bwd_add(const void* dy, const void* x, const float* rstd,
                                  const void* gamma, const void* dres, void* dx, void* dgamma,
                                  void* workspace, int rows, int cols, int64_t dy_ld, int64_t x_ld,
                                  int64_t dres_ld, int64_t dx_ld, void* stream) {
  return rmsnorm_bwd_impl(dy, x, rstd, gamma, dres, dx, dgamma, workspace, rows, cols, dy_ld, x_ld,
                          dres_ld, dx_ld, stream);
}

// kr_rmsnorm_bwd_add where the saved input, the residual gradient and / or the result are nanobatches
// of several sequences used in place: rows in runs of *_run_rows (1 = plain), run starts *_run_ld apart
extern "C" int kr_rmsnorm_bwd_add_runs(const void* dy, const void* x, const float* rstd,
                                       const void* gamma, const void* dres, void* dx, void* dgamma,
                                       void* workspace, int rows, int cols, int64_t dy_ld,
                                       int64_t x_ld, int x_run_rows, int64_t x_run_ld,
                                       int64_t dres_ld, int dres_run_rows, int64_t dres_run_ld,
                                       int64_t dx_ld, int dx_run_rows, int64_t dx_run_ld,
                                       void* stream) {
  BwdRuns runs;
  int rc = KR_OK;
  if (rows <= 0) return KR_EINVAL;
  if (!make_runs(x_run_rows, x_run_ld, rows, &runs.x, &rc)) return rc;
  if (dres && !make_runs(dres_run_rows, dres_run_ld, rows, &runs.dres, &rc)) return rc;
  if (!make_runs(dx_run_rows, dx_run_ld, rows, &runs.dx, &rc)) return rc;
  return rmsnorm_bwd_impl(dy, x, rstd, gamma, dres, dx, dgamma, workspace, rows, cols, dy_ld, x_ld,
                          dres_ld, dx_ld, stream, runs);
}

// ---- the variant that allocates nothing --------------------------------------------------------
// The partial rows of the weight gradient (at most kMaxBwdBlocks rows of at most 8192 columns,
// fp32: 16 MiB) live in a file-scope device array instead of a caller workspace.  Each GPU holds
// its own copy of the array at its own address; the address is looked up once per device.
namespace {
constexpr int kScratchCols = 8192;
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) float scratch[(size_t)kMaxBwdBlocks * kScratchCols];
namespace {
std::mutex scratch_mutex;
float* scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, null until looked up

// The device address of `scratch` on the current device (never the array's name: in host code that
// is a host-side stand-in, not a device address).
float* scratch_on_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    scratch_ptr[dev] = (float*)p;
  }
  return scratch_ptr[dev];
}
}  // namespace

extern "C" int kr_rmsnorm_bwd_add_noalloc(const void* dy, const void* x, const float* rstd,
                                          const void* gamma, const void* dres, void* dx,
                                          void* dgamma, int rows, int cols, int64_t dy_ld,
                                          int64_t x_ld, int64_t dres_ld, int64_t dx_ld, void* stream) {
  // the partial rows stay in the library's private array, which no caller can read: without a
  // place for the reduced weight gradient the call could not hand it over at all
  if (rows <= 0 || cols <= 0 || !dgamma) return KR_EINVAL;
  if (cols > kScratchCols) return KR_EUNSUPPORTED;  // beyond what the device array holds
  float* const ws = scratch_on_current_device();
  if (ws == nullptr) return KR_ELAUNCH;
  return rmsnorm_bwd_impl(dy, x, rstd, gamma, dres, dx, dgamma, ws, rows, cols, dy_ld, x_ld, dres_ld,
                          dx_ld, stream);
}

namespace {
int rmsnorm_bwd_impl(const void* dy, const void* x, const float* rstd, const void* gamma,
                     const void* dres, void* dx, void* dgamma, void* workspace, int rows, int cols,
                     int64_t dy_ld, int64_t x_ld, int64_t dres_ld, int64_t dx_ld, void* stream,
                     const BwdRuns& runs) {
  if (!dy || !x || !rstd || !gamma || !dx || !workspace || rows <= 0 || cols <= 0 ||
      dy_ld < cols || x_ld < cols || dx_ld < cols || (dres && dres_ld < cols))
    return KR_EINVAL;
  if (cols % 8 || dy_ld % 8 || x_ld % 8 || dx_ld % 8 || (dres && dres_ld % 8) || cols > 8192)
    return KR_EUNSUPPORTED;
  if (!kr_aligned16(x) || !kr_aligned16(dy) || !kr_aligned16(dx) || !kr_aligned16(gamma) ||
      !kr_aligned16(workspace) || (dres && !kr_aligned16(dres)))
    return KR_EINVAL;
  const int blocks = bwd_blocks(rows, cols);
  const int split = bwd_split(cols);
  const int nc = (cols / 8 + 64 * split - 1) / (64 * split);  // 16-byte vectors per lane
#define KR_RMS_BWD(ADDV, FULLV, SPLITV)                                                             \
  KR_DISPATCH_CHUNKS8(nc, hipLaunchKernelGGL((rmsnorm_bwd_kernel<C_, ADDV, FULLV, SPLITV>),         \
                                           dim3(blocks), dim3(kThreads), 0, (hipStream_t)stream,    \
                                           (const bf16*)dy, (const bf16*)x, rstd,                   \
                                           (const bf16*)gamma, (const bf16*)dres, (bf16*)dx,        \
                                           (float*)workspace, rows, cols, dy_ld, x_ld,              \
                                           dres ? dres_ld : (int64_t)0, dx_ld, runs.x, runs.dres,  \
                                           runs.dx))
  // rows of exactly 1, 2, 3, 4, 6 or 8 times 512 elements per wave take the straight-line kernel
  const bool full = cols % (512 * split) == 0 && cols / (512 * split) == nc && nc <= 8 && nc != 5 && nc != 7;
  if (split == 2) {
    if (dres) {
      if (full) { KR_RMS_BWD(true, true, 2); } else { KR_RMS_BWD(true, false, 2); }
    } else {
      if (full) { KR_RMS_BWD(false, true, 2); } else { KR_RMS_BWD(false, false, 2); }
    }
  } else if (dres) {
    if (full) { KR_RMS_BWD(true, true, 1); } else { KR_RMS_BWD(true, false, 1); }
  } else {
    if (full) { KR_RMS_BWD(false, true, 1); } else { KR_RMS_BWD(false, false, 1); }
  }
#undef KR_RMS_BWD
  if (hipGetLastError() != hipSuccess) return KR_ELAUNCH;
  if (dgamma == nullptr) return KR_OK;  // the caller sums the partial rows later (kr_rmsnorm_dgamma)
  hipLaunchKernelGGL(rmsnorm_dgamma_kernel, dim3((cols + 31) / 32), dim3(kDgammaThreads), 0,
                     (hipStream_t)stream, (const float*)workspace, (bf16*)dgamma, blocks, cols);
  return kr_launch_status();
}
}  // namespace

extern "C" int kr_rmsnorm_bwd_partial_rows(int rows, int cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return bwd_blocks(rows, cols);
}

extern "C" int kr_rmsnorm_dgamma(const float* partial, int nparts, int cols, void* dgamma,
                                 void* stream) {
  if (!partial || !dgamma || nparts <= 0 || cols <= 0) return KR_EINVAL;
  if (!kr_aligned16(partial)) return KR_EINVAL;
  hipLaunchKernelGGL(rmsnorm_dgamma_kernel, dim3((cols + 31) / 32), dim3(kDgammaThreads), 0,
                     (hipStream_t)stream, partial, (bf16*)dgamma, nparts, cols);
  return kr_launch_status();
}

extern "C" int kr_rmsnorm_bwd(const void* dy, const void* x, const float* rstd, const void* gamma,
                              void* dx, void* dgamma, void* workspace, int rows, int cols,
                              int64_t dy_ld, int64_t x_ld, void* stream) {
  return kr_rmsnorm_bwd_add(dy, x, rstd, gamma, nullptr, dx, dgamma, workspace, rows, cols, dy_ld,
                            x_ld, 0, cols, stream);
}
