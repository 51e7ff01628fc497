// Storage-type helpers for kernels that run in either bf16 or fp32 storage
// with fp32 math (gfx950).  `bf16s` is a 2-byte POD so the same template
// body serves both; all arithmetic happens on the float returned by ld().
#pragma once

#include "common.h"

struct bf16s {
  uint16_t v;
};

LIG_DEVICE float ld(const float* p) { return *p; }
LIG_DEVICE float ld(const bf16s* p) { return bf16_to_f32(p->v); }
LIG_DEVICE void st(float* p, float x) { *p = x; }
LIG_DEVICE void st(bf16s* p, float x) { p->v = f32_to_bf16(x); }

// Accurate logistic (expf, not the fast intrinsic): the recurrent gates and
// the fp32 serving mode need full single precision.
LIG_DEVICE float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// Block-wide sum over `blockDim.x` threads (multiple of 64, <= 1024).
// `lds` must hold 17 floats.  Result replicated in every thread.
LIG_DEVICE float block_reduce_sum(float v, float* lds) {
  v = wave_reduce_sum(v);
  const int wave = threadIdx.x / WAVE_SIZE;
  const int lane = threadIdx.x % WAVE_SIZE;
  const int nwaves = blockDim.x / WAVE_SIZE;
  __syncthreads();  // protect lds reuse across consecutive reductions
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  float total = 0.0f;
  for (int w = 0; w < nwaves; ++w) total += lds[w];
  return total;
}
