// Shared device helpers for the gfx950 kernels: vector types, bf16 packing, wave reductions,
// argument checks.  CDNA4 only: 64-wide wavefronts, MFMA builtins, no portability layer.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/kareus_hip.h"

typedef __bf16 bf16;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;

#define KR_WAVE 64
#define KR_LDS __attribute__((address_space(3)))

// One 16-byte global access = 8 bf16.
struct __attribute__((aligned(16))) Pack8 {
  bf16x8 v;
};

__device__ __forceinline__ bf16x8 ldg8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ void stg8(bf16* p, bf16x8 v) { *reinterpret_cast<bf16x8*>(p) = v; }
// The same for data that streams through a kernel: operands it reads once and results it does not read
// back, with the non-temporal hint.  Results stored with it: every kernel that writes a tensor it did not read
// (RMSNorm forward 42.9 -> 40.7 us at 16384 tokens of the 8B shard, 12.6 -> 10.6 us at 4096).  Operands loaded
// with it: only where a kernel reads two or three streams for each one it writes (residual add 5.2 -> 6.1 TB/s,
// RMSNorm backward with the residual gradient 5.1 -> 6.0, SwiGLU 5.4 -> 6.1, dropout 5.2 -> 6.2, 10-17 % less
// time at 16384 tokens); kernels that read one stream got 7-39 % slower with the hint on their loads, kernels
// that rewrite what they read (rotary, the per-head norm's backward) gained nothing either way, and loads that
// lanes or workgroups share (norm weights, rotary angles) keep the default policy.
__device__ __forceinline__ bf16x8 ldg8_stream(const bf16* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p));
}
__device__ __forceinline__ void stg8_stream(bf16* p, bf16x8 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<bf16x8*>(p));
}
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.0f;
  return z;
}

// Sum / max across the 64 lanes of a wave; every lane gets the result.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, KR_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, KR_WAVE));
  return v;
}

// SwiGLU on one element, fp32: silu(gate) * up.  One definition for the stand-alone kernel and the
// GEMM epilogue that fuses it, so that the two produce the same bits.
// one v_exp_f32 and one v_rcp_f32 (1 ulp each): an IEEE division here is ten instructions per
// element, which is what a GEMM epilogue that applies the activation spends its time on
__device__ __forceinline__ float kr_sigmoidf(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
__device__ __forceinline__ float kr_swiglu_f(float gate, float up) { return gate * kr_sigmoidf(gate) * up; }

// SwiGLU backward on one element: upstream gradient gy, forward inputs (gate, up) -> gradients.
__device__ __forceinline__ void kr_swiglu_bwd_f(float gy, float gate, float up, float& d_gate, float& d_up) {
  const float sg = kr_sigmoidf(gate);
  d_gate = gy * sg * (1.0f + gate * (1.0f - sg)) * up;
  d_up = gy * gate * sg;
}

static inline bool kr_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static inline int kr_launch_status() {
  return hipGetLastError() == hipSuccess ? KR_OK : KR_ELAUNCH;
}
