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

// 8 consecutive elements <-> 8 floats (16-byte accesses; the pointer must be
// 16-byte aligned for bf16 and for fp32).
LIG_DEVICE void ld8(const bf16s* p, float* o) {
  const u16x8 h = *reinterpret_cast<const u16x8*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = bf16_to_f32(h[i]);
}
LIG_DEVICE void ld8(const float* p, float* o) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p);
  const f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[i] = a[i];
    o[4 + i] = b[i];
  }
}
LIG_DEVICE void st8(bf16s* p, const float* v) {
  u16x8 h;
#pragma unroll
  for (int i = 0; i < 8; ++i) h[i] = f32_to_bf16(v[i]);
  *reinterpret_cast<u16x8*>(p) = h;
}
LIG_DEVICE void st8(float* p, const float* v) {
  f32x4 a, b;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = v[i];
    b[i] = v[4 + i];
  }
  *reinterpret_cast<f32x4*>(p) = a;
  *reinterpret_cast<f32x4*>(p + 4) = b;
}

static inline bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// Accurate logistic (expf, not the fast intrinsic): the recurrent gates and
// the fp32 serving mode need full single precision.
LIG_DEVICE float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// Hardware exp2/rcp based logistic (about 1e-6 relative): for bf16 storage,
// where the inputs carry 8 bits of mantissa anyway.  Still fp32 arithmetic.
LIG_DEVICE float sigmoid_fast(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}
template <typename T>
LIG_DEVICE float sigmoid_for(float x);
template <>
LIG_DEVICE float sigmoid_for<float>(float x) { return sigmoid_f32(x); }
template <>
LIG_DEVICE float sigmoid_for<bf16s>(float x) { return sigmoid_fast(x); }

// N consecutive elements (N = 1 or 4) <-> floats; N = 4 needs 8-byte (bf16)
// or 16-byte (fp32) alignment.
template <int N>
LIG_DEVICE void ldn(const bf16s* p, float* o) {
  if (N == 4) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    o[0] = bf16_to_f32((uint16_t)(w.x & 0xffffu));
    o[1] = bf16_to_f32((uint16_t)(w.x >> 16));
    o[2] = bf16_to_f32((uint16_t)(w.y & 0xffffu));
    o[3] = bf16_to_f32((uint16_t)(w.y >> 16));
  } else {
    o[0] = ld(p);
  }
}
template <int N>
LIG_DEVICE void ldn(const float* p, float* o) {
  if (N == 4) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = a[i];
  } else {
    o[0] = *p;
  }
}
template <int N>
LIG_DEVICE void stn(bf16s* p, const float* v) {
  if (N == 4) {
    uint2 w;
    w.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
    w.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
    *reinterpret_cast<uint2*>(p) = w;
  } else {
    st(p, v[0]);
  }
}
template <int N>
LIG_DEVICE void stn(float* p, const float* v) {
  if (N == 4) {
    f32x4 a;
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = v[i];
    *reinterpret_cast<f32x4*>(p) = a;
  } else {
    *p = v[0];
  }
}

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
