// minGRU recurrence over a flat token batch with per-sequence state slots,
// gfx950.
//
// Per channel c and token t of a sequence:
//   z_t = sigmoid(zpre_t)            cand_t = u_t >= 0 ? u_t + 1/2 : sigmoid(u_t)
//   S_t = (1 - z_t) * S_{t-1} + z_t * cand_t
//   out_t = S_t * silu(g_t)
// The gates read only the current token, so the recurrence is linear in S:
// S_t = a_t S_{t-1} + b_t.  A segment (the tokens one sequence brings in
// this step) is cut into NW consecutive time ranges, one per wave; every
// wave first reduces its range to (prod a, local b), the carries are chained
// through LDS, then every wave replays its range from its carry and writes
// the outputs.  A single-token segment (decode) runs with one wave and no
// LDS pass.  State is fp32 in `state[slot, W]`; a segment that starts a
// sequence ignores what the slot held before (slots are reused).
//
// Grid: (ceil(W / 64), segments); block: 64 * NW threads; lane = channel.

#include "elem_types.h"

#define MINGRU_MAX_WAVES 16

template <typename T>
__global__ void mingru_scan_kernel(
    T* __restrict__ out,       // [R, W]
    const T* __restrict__ zp,  // row stride `stride`
    const T* __restrict__ up, const T* __restrict__ gp, long stride,
    float* __restrict__ state,           // [slots, W]
    const int* __restrict__ seg_start,   // [S] first row of the segment
    const int* __restrict__ seg_len,     // [S]
    const int* __restrict__ seg_slot,    // [S]
    const int* __restrict__ seg_fresh,   // [S] 1: sequence starts here
    int W) {
  __shared__ float lds_a[MINGRU_MAX_WAVES][WAVE_SIZE];
  __shared__ float lds_b[MINGRU_MAX_WAVES][WAVE_SIZE];
  const int s = blockIdx.y;
  const int len = seg_len[s];
  if (len <= 0) return;
  const int lane = threadIdx.x % WAVE_SIZE;
  const int wave = threadIdx.x / WAVE_SIZE;
  const int nw = blockDim.x / WAVE_SIZE;
  const int c = blockIdx.x * WAVE_SIZE + lane;
  const bool active = c < W;
  const long row0 = seg_start[s];
  const int cl = (len + nw - 1) / nw;
  const int t0 = min(len, wave * cl);
  const int t1 = min(len, t0 + cl);

  float* st_ptr = state + (size_t)seg_slot[s] * W + c;
  float carry = 0.f;
  if (active && !seg_fresh[s]) carry = *st_ptr;

  if (nw > 1) {
    float a = 1.f, b = 0.f;
    if (active) {
      for (int t = t0; t < t1; ++t) {
        const long r = (row0 + t) * stride + c;
        const float z = sigmoid_f32(ld(zp + r));
        const float u = ld(up + r);
        const float cand = u >= 0.f ? u + 0.5f : sigmoid_f32(u);
        const float keep = 1.f - z;
        b = keep * b + z * cand;
        a *= keep;
      }
    }
    lds_a[wave][lane] = a;
    lds_b[wave][lane] = b;
    __syncthreads();
    for (int j = 0; j < wave; ++j) carry = lds_a[j][lane] * carry + lds_b[j][lane];
  }

  if (!active) return;
  float S = carry;
  for (int t = t0; t < t1; ++t) {
    const long r = (row0 + t) * stride + c;
    const float z = sigmoid_f32(ld(zp + r));
    const float u = ld(up + r);
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_f32(u);
    S = (1.f - z) * S + z * cand;
    const float g = ld(gp + r);
    st(out + (row0 + t) * (long)W + c, S * (g * sigmoid_f32(g)));
  }
  if (t1 == len && t0 < t1) *st_ptr = S;
}

extern "C" void lig_mingru_scan(void* out, const void* zp, const void* up,
                                const void* gp, long stride, float* state,
                                const int* seg_start, const int* seg_len,
                                const int* seg_slot, const int* seg_fresh,
                                int num_segs, int max_len, int W, int is_f32,
                                hipStream_t s) {
  if (num_segs <= 0 || W <= 0) return;
  int nw = 1;
  if (max_len >= 512) nw = 16;
  else if (max_len >= 64) nw = 8;
  else if (max_len >= 8) nw = 4;
  dim3 grid((W + WAVE_SIZE - 1) / WAVE_SIZE, num_segs), block(WAVE_SIZE * nw);
  if (is_f32)
    hipLaunchKernelGGL(mingru_scan_kernel<float>, grid, block, 0, s,
                       (float*)out, (const float*)zp, (const float*)up,
                       (const float*)gp, stride, state, seg_start, seg_len,
                       seg_slot, seg_fresh, W);
  else
    hipLaunchKernelGGL(mingru_scan_kernel<bf16s>, grid, block, 0, s,
                       (bf16s*)out, (const bf16s*)zp, (const bf16s*)up,
                       (const bf16s*)gp, stride, state, seg_start, seg_len,
                       seg_slot, seg_fresh, W);
}
