// Grouped RMS norm over an fp32 residual stream, gfx950.
//
// A row of width H is split into `groups` equal consecutive parts; each part
// is divided by its own sqrt(mean(part^2) + eps) and the row is multiplied
// by a weight.  groups == 1 is the ordinary RMS norm.  The residual stream
// is kept in fp32 whatever the storage type T (bf16 or fp32) of the
// activations that feed the matrix products.
//
// Three entry points, one workgroup per (row, group):
//   embed_norm   : residual = norm(table[token]) * w            (T  -> f32)
//   norm         : out      = norm(residual) * w                (f32 -> T)
//   post_add_pre : residual += norm(y) * w_post;                (T  -> f32)
//                  out = norm(residual) * w_pre                 (f32 -> T)
// The last one fuses a sub-layer's output norm, the residual add and the
// next sub-layer's input norm: one pass over y and the residual instead of
// three kernels.

#include "elem_types.h"

template <typename T>
__global__ void embed_group_norm_kernel(float* __restrict__ residual,   // [R, H]
                                        const T* __restrict__ table,    // [V, H]
                                        const int64_t* __restrict__ tokens,
                                        const T* __restrict__ w, float eps,
                                        int H, int P) {
  __shared__ float lds[17];
  const int row = blockIdx.x, g = blockIdx.y;
  const T* src = table + (size_t)tokens[row] * H + (size_t)g * P;
  float ss = 0.f;
  for (int i = threadIdx.x; i < P; i += blockDim.x) {
    const float v = ld(src + i);
    ss += v * v;
  }
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / (float)P + eps);
  float* dst = residual + (size_t)row * H + (size_t)g * P;
  const T* wg = w + (size_t)g * P;
  for (int i = threadIdx.x; i < P; i += blockDim.x)
    dst[i] = ld(src + i) * inv * ld(wg + i);
}

template <typename T>
__global__ void group_norm_kernel(T* __restrict__ out,                 // [R, H]
                                  const float* __restrict__ residual,  // [R, H]
                                  const T* __restrict__ w, float eps, int H,
                                  int P) {
  __shared__ float lds[17];
  const int row = blockIdx.x, g = blockIdx.y;
  const float* src = residual + (size_t)row * H + (size_t)g * P;
  float ss = 0.f;
  for (int i = threadIdx.x; i < P; i += blockDim.x) {
    const float v = src[i];
    ss += v * v;
  }
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / (float)P + eps);
  T* dst = out + (size_t)row * H + (size_t)g * P;
  const T* wg = w + (size_t)g * P;
  for (int i = threadIdx.x; i < P; i += blockDim.x)
    st(dst + i, src[i] * inv * ld(wg + i));
}

template <typename T>
__global__ void post_add_pre_norm_kernel(T* __restrict__ out,          // [R, H]
                                         float* __restrict__ residual, // [R, H]
                                         const T* __restrict__ y,      // [R, H]
                                         const T* __restrict__ w_post,
                                         const T* __restrict__ w_pre,
                                         float eps, int H, int P) {
  __shared__ float lds[17];
  const int row = blockIdx.x, g = blockIdx.y;
  const size_t base = (size_t)row * H + (size_t)g * P;
  const T* ysrc = y + base;
  float* res = residual + base;
  float ss = 0.f;
  for (int i = threadIdx.x; i < P; i += blockDim.x) {
    const float v = ld(ysrc + i);
    ss += v * v;
  }
  ss = block_reduce_sum(ss, lds);
  const float inv_y = 1.0f / sqrtf(ss / (float)P + eps);
  const T* wp = w_post + (size_t)g * P;
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < P; i += blockDim.x) {
    // each thread re-reads below only what it wrote itself here
    const float r = res[i] + ld(ysrc + i) * inv_y * ld(wp + i);
    res[i] = r;
    ss2 += r * r;
  }
  if (out == nullptr) return;  // uniform across the block
  ss2 = block_reduce_sum(ss2, lds);
  const float inv_r = 1.0f / sqrtf(ss2 / (float)P + eps);
  const T* wn = w_pre + (size_t)g * P;
  T* dst = out + base;
  for (int i = threadIdx.x; i < P; i += blockDim.x)
    st(dst + i, res[i] * inv_r * ld(wn + i));
}

static inline int norm_block(int P) { return P <= 128 ? 64 : (P <= 1024 ? 128 : 256); }

extern "C" {

void lig_embed_group_norm(float* residual, const void* table,
                          const int64_t* tokens, const void* w, float eps,
                          int rows, int H, int groups, int is_f32,
                          hipStream_t s) {
  if (rows <= 0) return;
  const int P = H / groups;
  dim3 grid(rows, groups), block(norm_block(P));
  if (is_f32)
    hipLaunchKernelGGL(embed_group_norm_kernel<float>, grid, block, 0, s,
                       residual, (const float*)table, tokens, (const float*)w,
                       eps, H, P);
  else
    hipLaunchKernelGGL(embed_group_norm_kernel<bf16s>, grid, block, 0, s,
                       residual, (const bf16s*)table, tokens, (const bf16s*)w,
                       eps, H, P);
}

void lig_group_norm(void* out, const float* residual, const void* w, float eps,
                    int rows, int H, int groups, int is_f32, hipStream_t s) {
  if (rows <= 0) return;
  const int P = H / groups;
  dim3 grid(rows, groups), block(norm_block(P));
  if (is_f32)
    hipLaunchKernelGGL(group_norm_kernel<float>, grid, block, 0, s,
                       (float*)out, residual, (const float*)w, eps, H, P);
  else
    hipLaunchKernelGGL(group_norm_kernel<bf16s>, grid, block, 0, s,
                       (bf16s*)out, residual, (const bf16s*)w, eps, H, P);
}

// out may be null: then only the residual update is done.
void lig_post_add_pre_norm(void* out, float* residual, const void* y,
                           const void* w_post, const void* w_pre, float eps,
                           int rows, int H, int groups, int is_f32,
                           hipStream_t s) {
  if (rows <= 0) return;
  const int P = H / groups;
  dim3 grid(rows, groups), block(norm_block(P));
  if (is_f32)
    hipLaunchKernelGGL(post_add_pre_norm_kernel<float>, grid, block, 0, s,
                       (float*)out, residual, (const float*)y,
                       (const float*)w_post, (const float*)w_pre, eps, H, P);
  else
    hipLaunchKernelGGL(post_add_pre_norm_kernel<bf16s>, grid, block, 0, s,
                       (bf16s*)out, residual, (const bf16s*)y,
                       (const bf16s*)w_post, (const bf16s*)w_pre, eps, H, P);
}

}  // extern "C"
