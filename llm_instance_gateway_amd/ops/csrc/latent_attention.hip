// Front end of latent (low-rank key/value) attention, gfx950.
//
// One fused projection gives, per token, a query latent, a key/value latent
// and one rotated key part shared by all heads.  `latent_kv_prep` RMS-norms
// both latents (plain weights), rotates the shared key part and writes the
// token's cache row [normed key/value latent | rotated key part] straight
// into the paged cache; only that row is ever cached.  `rotate_pack_queries`
// rotates the rotated part of every query head into the tail of the packed
// per-head query [latent-space part | rotated part]; the latent-space part
// is filled by a batched GEMM with the per-head key up-projection.
//
// Rotation: interleaved pairs (2i, 2i+1), angle = position * inv_freq[i] in
// fp32, accurate sinf/cosf.  Entries past 2 * n_freq pass unchanged.

#include "elem_types.h"

#define LA_THREADS 256

template <typename T>
__global__ __launch_bounds__(LA_THREADS) void latent_kv_prep_kernel(
    T* __restrict__ cq_out,                 // [R, q_rank]
    const T* __restrict__ proj, long proj_stride,
    const T* __restrict__ w_q, const T* __restrict__ w_kv,
    const float* __restrict__ inv_freq, int n_freq,
    const int64_t* __restrict__ positions, const int64_t* __restrict__ slot_mapping,
    T* __restrict__ cache,                  // rows of kv_rank + rot_dim
    float eps, int q_rank, int kv_rank, int rot_dim) {
  __shared__ float red[2][17];
  const int r = blockIdx.x, tid = threadIdx.x;
  const T* row = proj + (size_t)r * proj_stride;
  const T* lat = row + q_rank;
  const T* kr = lat + kv_rank;
  float a = 0.f, b = 0.f;
  for (int d = tid; d < q_rank; d += LA_THREADS) {
    const float v = ld(row + d);
    a += v * v;
  }
  for (int d = tid; d < kv_rank; d += LA_THREADS) {
    const float v = ld(lat + d);
    b += v * v;
  }
  a = block_reduce_sum(a, red[0]);
  b = block_reduce_sum(b, red[1]);
  const float inv_q = 1.0f / sqrtf(a / (float)q_rank + eps);
  const float inv_c = 1.0f / sqrtf(b / (float)kv_rank + eps);
  for (int d = tid; d < q_rank; d += LA_THREADS)
    st(cq_out + (size_t)r * q_rank + d, ld(row + d) * inv_q * ld(w_q + d));
  const int64_t slot = slot_mapping[r];
  if (slot < 0) return;
  T* crow = cache + (size_t)slot * (kv_rank + rot_dim);
  for (int d = tid; d < kv_rank; d += LA_THREADS)
    st(crow + d, ld(lat + d) * inv_c * ld(w_kv + d));
  const float pos = (float)positions[r];
  const int pairs = (rot_dim + 1) / 2;
  for (int i = tid; i < pairs; i += LA_THREADS) {
    const int d = 2 * i;
    const float u = ld(kr + d);
    if (d + 1 >= rot_dim) {
      st(crow + kv_rank + d, u);
    } else {
      const float v = ld(kr + d + 1);
      if (i < n_freq) {
        const float ang = pos * inv_freq[i];
        const float c = cosf(ang), s = sinf(ang);
        st(crow + kv_rank + d, u * c - v * s);
        st(crow + kv_rank + d + 1, v * c + u * s);
      } else {
        st(crow + kv_rank + d, u);
        st(crow + kv_rank + d + 1, v);
      }
    }
  }
}


// Vector path: one wave per row (4 rows per workgroup), 16-byte accesses,
// wave-shuffle reductions only.  q_rank, kv_rank and rot_dim multiples of 8
// (every row and part starts 16-byte aligned).
template <typename T>
__global__ __launch_bounds__(LA_THREADS) void latent_kv_prep_vec_kernel(
    T* __restrict__ cq_out, const T* __restrict__ proj, long proj_stride,
    const T* __restrict__ w_q, const T* __restrict__ w_kv,
    const float* __restrict__ inv_freq, int n_freq,
    const int64_t* __restrict__ positions, const int64_t* __restrict__ slot_mapping,
    T* __restrict__ cache, float eps, int R, int q_rank, int kv_rank, int rot_dim) {
  const int lane = threadIdx.x % WAVE_SIZE;
  const int r = blockIdx.x * (LA_THREADS / WAVE_SIZE) + threadIdx.x / WAVE_SIZE;
  if (r >= R) return;  // whole waves leave; no workgroup barrier below
  const T* row = proj + (size_t)r * proj_stride;
  const T* lat = row + q_rank;
  const T* kr = lat + kv_rank;
  float a = 0.f, b = 0.f;
  float v[8], w[8];
  for (int d = lane * 8; d < q_rank; d += WAVE_SIZE * 8) {
    ld8(row + d, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) a += v[e] * v[e];
  }
  for (int d = lane * 8; d < kv_rank; d += WAVE_SIZE * 8) {
    ld8(lat + d, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) b += v[e] * v[e];
  }
  a = wave_reduce_sum(a);
  b = wave_reduce_sum(b);
  const float inv_q = 1.0f / sqrtf(a / (float)q_rank + eps);
  const float inv_c = 1.0f / sqrtf(b / (float)kv_rank + eps);
  for (int d = lane * 8; d < q_rank; d += WAVE_SIZE * 8) {
    ld8(row + d, v);
    ld8(w_q + d, w);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = v[e] * inv_q * w[e];
    st8(cq_out + (size_t)r * q_rank + d, v);
  }
  const int64_t slot = slot_mapping[r];
  if (slot < 0) return;
  T* crow = cache + (size_t)slot * (kv_rank + rot_dim);
  for (int d = lane * 8; d < kv_rank; d += WAVE_SIZE * 8) {
    ld8(lat + d, v);
    ld8(w_kv + d, w);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = v[e] * inv_c * w[e];
    st8(crow + d, v);
  }
  const float pos = (float)positions[r];
  for (int i = lane; i < rot_dim / 2; i += WAVE_SIZE) {
    const float u = ld(kr + 2 * i), t = ld(kr + 2 * i + 1);
    float c = 1.f, sn = 0.f;
    if (i < n_freq) {
      const float ang = pos * inv_freq[i];
      c = cosf(ang);
      sn = sinf(ang);
    }
    st(crow + kv_rank + 2 * i, u * c - t * sn);
    st(crow + kv_rank + 2 * i + 1, t * c + u * sn);
  }
}

template <typename T>
__global__ void rotate_pack_queries_kernel(
    T* __restrict__ out,       // [R, heads, lead + rot_dim]
    const T* __restrict__ q,   // [R, heads, dim + rot_dim]
    const float* __restrict__ inv_freq, int n_freq,
    const int64_t* __restrict__ positions, int heads, int dim, int rot_dim,
    int lead, long total) {  // total = R * heads * pairs
  const int pairs = (rot_dim + 1) / 2;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += gridDim.x * (long)blockDim.x) {
    const int i = (int)(idx % pairs);
    const long rh = idx / pairs;
    const long r = rh / heads;
    const T* src = q + rh * (dim + rot_dim) + dim;
    T* dst = out + rh * (lead + rot_dim) + lead;
    const int d = 2 * i;
    const float u = ld(src + d);
    if (d + 1 >= rot_dim) {
      st(dst + d, u);
      continue;
    }
    const float v = ld(src + d + 1);
    if (i < n_freq) {
      const float ang = (float)positions[r] * inv_freq[i];
      const float c = cosf(ang), s = sinf(ang);
      st(dst + d, u * c - v * s);
      st(dst + d + 1, v * c + u * s);
    } else {
      st(dst + d, u);
      st(dst + d + 1, v);
    }
  }
}


// 8 entries (4 pairs) per thread, 16-byte accesses: dim, rot_dim and lead
// multiples of 8.
template <typename T>
__global__ void rotate_pack_queries_vec_kernel(
    T* __restrict__ out, const T* __restrict__ q, const float* __restrict__ inv_freq,
    int n_freq, const int64_t* __restrict__ positions, int heads, int dim,
    int rot_dim, int lead, long total) {  // total = R * heads * rot_dim / 8
  const int chunks = rot_dim / 8;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += gridDim.x * (long)blockDim.x) {
    const int c = (int)(idx % chunks);
    const long rh = idx / chunks;
    const long r = rh / heads;
    float v[8];
    ld8(q + rh * (dim + rot_dim) + dim + c * 8, v);
    const float pos = (float)positions[r];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int i = c * 4 + k;
      if (i < n_freq) {
        const float ang = pos * inv_freq[i];
        const float cs = cosf(ang), sn = sinf(ang);
        const float u = v[2 * k], t = v[2 * k + 1];
        v[2 * k] = u * cs - t * sn;
        v[2 * k + 1] = t * cs + u * sn;
      }
    }
    st8(out + rh * (lead + rot_dim) + lead + c * 8, v);
  }
}

// out[i, :] = w[i] * x[idx[i], :] (fp32 product); idx < 0 gives a zero row.
// The routed feed-forward scales an expert's INPUT by the router weight.
template <typename T>
__global__ void scale_gather_rows_kernel(T* __restrict__ out, const T* __restrict__ x,
                                         const int64_t* __restrict__ idx,
                                         const float* __restrict__ w, int H, long total) {
  for (long e = blockIdx.x * (long)blockDim.x + threadIdx.x; e < total;
       e += gridDim.x * (long)blockDim.x) {
    const long i = e / H;
    const int d = (int)(e - i * H);
    const int64_t src = idx[i];
    st(out + e, src < 0 ? 0.f : w[i] * ld(x + src * H + d));
  }
}

extern "C" {

void lig_latent_kv_prep(void* cq_out, const void* proj, long proj_stride,
                        const void* w_q, const void* w_kv, const float* inv_freq,
                        int n_freq, const int64_t* positions,
                        const int64_t* slot_mapping, void* cache, float eps,
                        int R, int q_rank, int kv_rank, int rot_dim, int is_f32,
                        hipStream_t s) {
  if (R <= 0) return;
  if (q_rank % 8 == 0 && kv_rank % 8 == 0 && rot_dim % 8 == 0 && proj_stride % 8 == 0 &&
      aligned16(cq_out) && aligned16(proj) && aligned16(w_q) && aligned16(w_kv) &&
      aligned16(cache)) {
    const int per = LA_THREADS / WAVE_SIZE;
    const dim3 grid((R + per - 1) / per);
    if (is_f32)
      hipLaunchKernelGGL(latent_kv_prep_vec_kernel<float>, grid, dim3(LA_THREADS), 0, s,
                         (float*)cq_out, (const float*)proj, proj_stride,
                         (const float*)w_q, (const float*)w_kv, inv_freq, n_freq,
                         positions, slot_mapping, (float*)cache, eps, R, q_rank,
                         kv_rank, rot_dim);
    else
      hipLaunchKernelGGL(latent_kv_prep_vec_kernel<bf16s>, grid, dim3(LA_THREADS), 0, s,
                         (bf16s*)cq_out, (const bf16s*)proj, proj_stride,
                         (const bf16s*)w_q, (const bf16s*)w_kv, inv_freq, n_freq,
                         positions, slot_mapping, (bf16s*)cache, eps, R, q_rank,
                         kv_rank, rot_dim);
    return;
  }
  if (is_f32)
    hipLaunchKernelGGL(latent_kv_prep_kernel<float>, dim3(R), dim3(LA_THREADS), 0, s,
                       (float*)cq_out, (const float*)proj, proj_stride,
                       (const float*)w_q, (const float*)w_kv, inv_freq, n_freq,
                       positions, slot_mapping, (float*)cache, eps, q_rank,
                       kv_rank, rot_dim);
  else
    hipLaunchKernelGGL(latent_kv_prep_kernel<bf16s>, dim3(R), dim3(LA_THREADS), 0, s,
                       (bf16s*)cq_out, (const bf16s*)proj, proj_stride,
                       (const bf16s*)w_q, (const bf16s*)w_kv, inv_freq, n_freq,
                       positions, slot_mapping, (bf16s*)cache, eps, q_rank,
                       kv_rank, rot_dim);
}

void lig_rotate_pack_queries(void* out, const void* q, const float* inv_freq,
                             int n_freq, const int64_t* positions, int R,
                             int heads, int dim, int rot_dim, int lead,
                             int is_f32, hipStream_t s) {
  if (dim % 8 == 0 && rot_dim % 8 == 0 && lead % 8 == 0 && aligned16(out) && aligned16(q)) {
    const long total8 = (long)R * heads * (rot_dim / 8);
    if (total8 <= 0) return;
    long g8 = (total8 + 255) / 256;
    const int grid8 = (int)(g8 > 65535 ? 65535 : g8);
    if (is_f32)
      hipLaunchKernelGGL(rotate_pack_queries_vec_kernel<float>, dim3(grid8), dim3(256), 0, s,
                         (float*)out, (const float*)q, inv_freq, n_freq, positions,
                         heads, dim, rot_dim, lead, total8);
    else
      hipLaunchKernelGGL(rotate_pack_queries_vec_kernel<bf16s>, dim3(grid8), dim3(256), 0, s,
                         (bf16s*)out, (const bf16s*)q, inv_freq, n_freq, positions,
                         heads, dim, rot_dim, lead, total8);
    return;
  }
  const long total = (long)R * heads * ((rot_dim + 1) / 2);
  if (total <= 0) return;
  long g = (total + 255) / 256;
  const int grid = (int)(g > 65535 ? 65535 : g);
  if (is_f32)
    hipLaunchKernelGGL(rotate_pack_queries_kernel<float>, dim3(grid), dim3(256), 0, s,
                       (float*)out, (const float*)q, inv_freq, n_freq, positions,
                       heads, dim, rot_dim, lead, total);
  else
    hipLaunchKernelGGL(rotate_pack_queries_kernel<bf16s>, dim3(grid), dim3(256), 0, s,
                       (bf16s*)out, (const bf16s*)q, inv_freq, n_freq, positions,
                       heads, dim, rot_dim, lead, total);
}

void lig_scale_gather_rows(void* out, const void* x, const int64_t* idx,
                           const float* w, long rows, int H, int is_f32,
                           hipStream_t s) {
  const long total = rows * H;
  if (total <= 0) return;
  long g = (total + 255) / 256;
  const int grid = (int)(g > 65535 ? 65535 : g);
  if (is_f32)
    hipLaunchKernelGGL(scale_gather_rows_kernel<float>, dim3(grid), dim3(256), 0, s,
                       (float*)out, (const float*)x, idx, w, H, total);
  else
    hipLaunchKernelGGL(scale_gather_rows_kernel<bf16s>, dim3(grid), dim3(256), 0, s,
                       (bf16s*)out, (const bf16s*)x, idx, w, H, total);
}

}  // extern "C"
