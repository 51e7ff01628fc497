// Elementwise activations of the hybrid models, bf16 or fp32 storage with
// fp32 math, gfx950.
//
// xIELU with two coefficients a_pos > 0, a_neg > 1/2 (the caller passes the
// softplus-transformed learnable scalars):
//   z > 0 : a_pos * z^2 + z/2
//   z <= 0: a_neg * (exp(z) - 1 - z) + z/2
// expm1f keeps the negative branch accurate near zero.
//
// sigmoid_gate_mul: x[r, c] *= sigmoid(g[r, c]) with a strided gate view
// (the gate is a column block of a fused projection output).

#include "elem_types.h"

template <typename T>
__global__ void xielu_kernel(T* __restrict__ out, const T* __restrict__ x,
                             float a_pos, float a_neg, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += gridDim.x * (long)blockDim.x) {
    const float z = ld(x + i);
    const float y = z > 0.f ? a_pos * z * z + 0.5f * z
                            : a_neg * (expm1f(z) - z) + 0.5f * z;
    st(out + i, y);
  }
}

// 8 elements per thread (16-byte accesses for bf16): n8 = n / 8 vectors.
template <typename T>
__global__ void xielu_vec_kernel(T* __restrict__ out, const T* __restrict__ x,
                                 float a_pos, float a_neg, long n8) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n8;
       i += gridDim.x * (long)blockDim.x) {
    float v[8];
    ld8(x + i * 8, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float z = v[k];
      v[k] = z > 0.f ? a_pos * z * z + 0.5f * z
                     : a_neg * (expm1f(z) - z) + 0.5f * z;
    }
    st8(out + i * 8, v);
  }
}

template <typename T>
__global__ void sigmoid_gate_mul_vec_kernel(T* __restrict__ x,
                                            const T* __restrict__ g, long g_stride,
                                            int C8, long n8) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n8;
       i += gridDim.x * (long)blockDim.x) {
    const long r = i / C8;
    const int c = (int)(i - r * C8) * 8;
    float xv[8], gv[8];
    ld8(x + i * 8, xv);
    ld8(g + r * g_stride + c, gv);
#pragma unroll
    for (int k = 0; k < 8; ++k) xv[k] *= sigmoid_f32(gv[k]);
    st8(x + i * 8, xv);
  }
}

template <typename T>
__global__ void sigmoid_gate_mul_kernel(T* __restrict__ x,  // [R, C] contiguous
                                        const T* __restrict__ g, long g_stride,
                                        int C, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += gridDim.x * (long)blockDim.x) {
    const long r = i / C;
    const int c = (int)(i - r * C);
    st(x + i, ld(x + i) * sigmoid_f32(ld(g + r * g_stride + c)));
  }
}

static inline int ew_grid(long n) {
  long g = (n + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 65535 ? 65535 : g));
}

extern "C" {

void lig_xielu(void* out, const void* x, float a_pos, float a_neg, long n,
               int is_f32, hipStream_t s) {
  if (n <= 0) return;
  if (n % 8 == 0 && aligned16(out) && aligned16(x)) {
    const long n8 = n / 8;
    if (is_f32)
      hipLaunchKernelGGL(xielu_vec_kernel<float>, dim3(ew_grid(n8)), dim3(256),
                         0, s, (float*)out, (const float*)x, a_pos, a_neg, n8);
    else
      hipLaunchKernelGGL(xielu_vec_kernel<bf16s>, dim3(ew_grid(n8)), dim3(256),
                         0, s, (bf16s*)out, (const bf16s*)x, a_pos, a_neg, n8);
    return;
  }
  if (is_f32)
    hipLaunchKernelGGL(xielu_kernel<float>, dim3(ew_grid(n)), dim3(256), 0, s,
                       (float*)out, (const float*)x, a_pos, a_neg, n);
  else
    hipLaunchKernelGGL(xielu_kernel<bf16s>, dim3(ew_grid(n)), dim3(256), 0, s,
                       (bf16s*)out, (const bf16s*)x, a_pos, a_neg, n);
}

void lig_sigmoid_gate_mul(void* x, const void* g, long g_stride, int rows,
                          int C, int is_f32, hipStream_t s) {
  const long n = (long)rows * C;
  if (n <= 0) return;
  if (C % 8 == 0 && g_stride % 8 == 0 && aligned16(x) && aligned16(g)) {
    const long n8 = n / 8;
    if (is_f32)
      hipLaunchKernelGGL(sigmoid_gate_mul_vec_kernel<float>, dim3(ew_grid(n8)),
                         dim3(256), 0, s, (float*)x, (const float*)g, g_stride,
                         C / 8, n8);
    else
      hipLaunchKernelGGL(sigmoid_gate_mul_vec_kernel<bf16s>, dim3(ew_grid(n8)),
                         dim3(256), 0, s, (bf16s*)x, (const bf16s*)g, g_stride,
                         C / 8, n8);
    return;
  }
  if (is_f32)
    hipLaunchKernelGGL(sigmoid_gate_mul_kernel<float>, dim3(ew_grid(n)),
                       dim3(256), 0, s, (float*)x, (const float*)g, g_stride,
                       C, n);
  else
    hipLaunchKernelGGL(sigmoid_gate_mul_kernel<bf16s>, dim3(ew_grid(n)),
                       dim3(256), 0, s, (bf16s*)x, (const bf16s*)g, g_stride,
                       C, n);
}

}  // extern "C"
