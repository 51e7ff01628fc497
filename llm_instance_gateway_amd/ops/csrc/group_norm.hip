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
//
// Memory-bound: when a part is a multiple of 8 elements (and at most 8192)
// each thread keeps its 16-byte vectors of the part in registers between the
// reduction and the scaling pass, so every operand crosses HBM once.  Other
// shapes take the scalar kernels.

#include "elem_types.h"

// ---- vector path: part P = 8 * nvec, thread t owns vectors t, t+B, ... ------

template <typename TIn, typename TOut, typename TW, int VPT>
__global__ void norm_vec_kernel(TOut* __restrict__ out, const TIn* __restrict__ in,
                                const int64_t* __restrict__ gather,
                                const TW* __restrict__ w, float eps, int H, int P) {
  __shared__ float lds[17];
  const int row = blockIdx.x, g = blockIdx.y, nvec = P / 8;
  const size_t src_row = gather ? (size_t)gather[row] : (size_t)row;
  const TIn* src = in + src_row * H + (size_t)g * P;
  float v[VPT][8];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int idx = threadIdx.x + k * blockDim.x;
    if (idx < nvec) {
      ld8(src + idx * 8, v[k]);
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[k][i] * v[k][i];
    }
  }
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / (float)P + eps);
  TOut* dst = out + (size_t)row * H + (size_t)g * P;
  const TW* wg = w + (size_t)g * P;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int idx = threadIdx.x + k * blockDim.x;
    if (idx < nvec) {
      float wv[8];
      ld8(wg + idx * 8, wv);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[k][i] = v[k][i] * inv * wv[i];
      st8(dst + idx * 8, v[k]);
    }
  }
}

template <typename T, int VPT>
__global__ void post_add_pre_norm_vec_kernel(T* __restrict__ out,
                                             float* __restrict__ residual,
                                             const T* __restrict__ y,
                                             const T* __restrict__ w_post,
                                             const T* __restrict__ w_pre,
                                             float eps, int H, int P) {
  __shared__ float lds[17];
  const int row = blockIdx.x, g = blockIdx.y, nvec = P / 8;
  const size_t base = (size_t)row * H + (size_t)g * P;
  float v[VPT][8];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int idx = threadIdx.x + k * blockDim.x;
    if (idx < nvec) {
      ld8(y + base + idx * 8, v[k]);
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[k][i] * v[k][i];
    }
  }
  ss = block_reduce_sum(ss, lds);
  const float inv_y = 1.0f / sqrtf(ss / (float)P + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int idx = threadIdx.x + k * blockDim.x;
    if (idx < nvec) {
      float wv[8], r[8];
      ld8(w_post + (size_t)g * P + idx * 8, wv);
      ld8(residual + base + idx * 8, r);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        v[k][i] = r[i] + v[k][i] * inv_y * wv[i];
        ss2 += v[k][i] * v[k][i];
      }
      st8(residual + base + idx * 8, v[k]);
    }
  }
  if (out == nullptr) return;  // uniform across the block
  ss2 = block_reduce_sum(ss2, lds);
  const float inv_r = 1.0f / sqrtf(ss2 / (float)P + eps);
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int idx = threadIdx.x + k * blockDim.x;
    if (idx < nvec) {
      float wv[8];
      ld8(w_pre + (size_t)g * P + idx * 8, wv);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[k][i] = v[k][i] * inv_r * wv[i];
      st8(out + base + idx * 8, v[k]);
    }
  }
}

// ---- scalar path: any part size ----------------------------------------------

template <typename TIn, typename TOut, typename TW>
__global__ void norm_scalar_kernel(TOut* __restrict__ out, const TIn* __restrict__ in,
                                   const int64_t* __restrict__ gather,
                                   const TW* __restrict__ w, float eps, int H, int P) {
  __shared__ float lds[17];
  const int row = blockIdx.x, g = blockIdx.y;
  const size_t src_row = gather ? (size_t)gather[row] : (size_t)row;
  const TIn* src = in + src_row * H + (size_t)g * P;
  float ss = 0.f;
  for (int i = threadIdx.x; i < P; i += blockDim.x) {
    const float v = ld(src + i);
    ss += v * v;
  }
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / (float)P + eps);
  TOut* dst = out + (size_t)row * H + (size_t)g * P;
  const TW* wg = w + (size_t)g * P;
  for (int i = threadIdx.x; i < P; i += blockDim.x)
    st(dst + i, ld(src + i) * inv * ld(wg + i));
}

template <typename T>
__global__ void post_add_pre_norm_scalar_kernel(T* __restrict__ out,
                                                float* __restrict__ residual,
                                                const T* __restrict__ y,
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

// ---- launch -------------------------------------------------------------------

static inline int norm_block(int P) { return P <= 128 ? 64 : (P <= 1024 ? 128 : 256); }

// Vector-path geometry for a part of P elements: block size and vectors per
// thread (1, 2 or 4); vpt == 0 means "use the scalar path".
static inline void vec_geometry(int H, int P, int* block, int* vpt) {
  *vpt = 0;
  if (P % 8 != 0 || H % 8 != 0 || P > 8192) return;
  const int nvec = P / 8;
  int b = (nvec + 63) / 64 * 64;
  if (b > 256) b = 256;
  const int need = (nvec + b - 1) / b;
  *block = b;
  *vpt = need <= 1 ? 1 : (need <= 2 ? 2 : 4);
}

template <typename TIn, typename TOut, typename TW>
static void launch_norm(TOut* out, const TIn* in, const int64_t* gather,
                        const TW* w, float eps, int rows, int H, int groups,
                        hipStream_t s) {
  const int P = H / groups;
  int b = 0, vpt = 0;
  vec_geometry(H, P, &b, &vpt);
  if (!(aligned16(out) && aligned16(in) && aligned16(w))) vpt = 0;
  dim3 grid(rows, groups);
  if (vpt == 1)
    hipLaunchKernelGGL((norm_vec_kernel<TIn, TOut, TW, 1>), grid, dim3(b), 0, s, out, in, gather, w, eps, H, P);
  else if (vpt == 2)
    hipLaunchKernelGGL((norm_vec_kernel<TIn, TOut, TW, 2>), grid, dim3(b), 0, s, out, in, gather, w, eps, H, P);
  else if (vpt == 4)
    hipLaunchKernelGGL((norm_vec_kernel<TIn, TOut, TW, 4>), grid, dim3(b), 0, s, out, in, gather, w, eps, H, P);
  else
    hipLaunchKernelGGL((norm_scalar_kernel<TIn, TOut, TW>), grid, dim3(norm_block(P)), 0, s, out, in, gather, w, eps, H, P);
}

template <typename T>
static void launch_post_add_pre(T* out, float* residual, const T* y,
                                const T* w_post, const T* w_pre, float eps,
                                int rows, int H, int groups, hipStream_t s) {
  const int P = H / groups;
  int b = 0, vpt = 0;
  vec_geometry(H, P, &b, &vpt);
  if (!(aligned16(out) && aligned16(residual) && aligned16(y) &&
        aligned16(w_post) && aligned16(w_pre)))
    vpt = 0;
  dim3 grid(rows, groups);
  if (vpt == 1)
    hipLaunchKernelGGL((post_add_pre_norm_vec_kernel<T, 1>), grid, dim3(b), 0, s, out, residual, y, w_post, w_pre, eps, H, P);
  else if (vpt == 2)
    hipLaunchKernelGGL((post_add_pre_norm_vec_kernel<T, 2>), grid, dim3(b), 0, s, out, residual, y, w_post, w_pre, eps, H, P);
  else if (vpt == 4)
    hipLaunchKernelGGL((post_add_pre_norm_vec_kernel<T, 4>), grid, dim3(b), 0, s, out, residual, y, w_post, w_pre, eps, H, P);
  else
    hipLaunchKernelGGL((post_add_pre_norm_scalar_kernel<T>), grid, dim3(norm_block(P)), 0, s, out, residual, y, w_post, w_pre, eps, H, P);
}

extern "C" {

void lig_embed_group_norm(float* residual, const void* table,
                          const int64_t* tokens, const void* w, float eps,
                          int rows, int H, int groups, int is_f32,
                          hipStream_t s) {
  if (rows <= 0) return;
  if (is_f32)
    launch_norm<float, float, float>(residual, (const float*)table, tokens,
                                     (const float*)w, eps, rows, H, groups, s);
  else
    launch_norm<bf16s, float, bf16s>(residual, (const bf16s*)table, tokens,
                                     (const bf16s*)w, eps, rows, H, groups, s);
}

void lig_group_norm(void* out, const float* residual, const void* w, float eps,
                    int rows, int H, int groups, int is_f32, hipStream_t s) {
  if (rows <= 0) return;
  if (is_f32)
    launch_norm<float, float, float>((float*)out, residual, nullptr,
                                     (const float*)w, eps, rows, H, groups, s);
  else
    launch_norm<float, bf16s, bf16s>((bf16s*)out, residual, nullptr,
                                     (const bf16s*)w, eps, rows, H, groups, s);
}

// out may be null: then only the residual update is done.
void lig_post_add_pre_norm(void* out, float* residual, const void* y,
                           const void* w_post, const void* w_pre, float eps,
                           int rows, int H, int groups, int is_f32,
                           hipStream_t s) {
  if (rows <= 0) return;
  if (is_f32)
    launch_post_add_pre<float>((float*)out, residual, (const float*)y,
                               (const float*)w_post, (const float*)w_pre, eps,
                               rows, H, groups, s);
  else
    launch_post_add_pre<bf16s>((bf16s*)out, residual, (const bf16s*)y,
                               (const bf16s*)w_post, (const bf16s*)w_pre, eps,
                               rows, H, groups, s);
}

}  // extern "C"
