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
// Long segments (a step with prompt portions of 128 tokens or more) take a
// three-pass variant further down that spreads the time chunks over many
// workgroups.
//
// Grid: (ceil(W / (64 * CH)), segments); block: 64 * NW threads; a lane owns
// CH adjacent channels (CH = 4 when W and the row stride allow 8/16-byte
// accesses, else 1).  Time is walked four steps at a time so the loads of
// the next steps are in flight while the recurrence, which is the only
// serial dependency, advances.  Arithmetic is fp32 throughout; with bf16
// storage the logistic uses the hardware exp2/rcp (about 1e-6 relative),
// with fp32 storage the accurate expf.

#include "elem_types.h"

#define MINGRU_MAX_WAVES 16
#define MINGRU_TU 4  // time steps staged per iteration

// Reduce the time range [t0, t1) of one lane's CH channels to (a, b) with
// S_{t1-1} = a * S_{t0-1} + b.
template <typename T, int CH>
LIG_DEVICE void range_reduce(const T* __restrict__ zp, const T* __restrict__ up,
                             long stride, long row0, int c, int t0, int t1,
                             float* a, float* b) {
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    a[i] = 1.f;
    b[i] = 0.f;
  }
  int t = t0;
  for (; t + MINGRU_TU <= t1; t += MINGRU_TU) {
    float zv[MINGRU_TU][CH], uv[MINGRU_TU][CH];
#pragma unroll
    for (int k = 0; k < MINGRU_TU; ++k) {
      const long r = (row0 + t + k) * stride + c;
      ldn<CH>(zp + r, zv[k]);
      ldn<CH>(up + r, uv[k]);
    }
#pragma unroll
    for (int k = 0; k < MINGRU_TU; ++k)
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const float z = sigmoid_for<T>(zv[k][i]);
        const float u = uv[k][i];
        const float cand = u >= 0.f ? u + 0.5f : sigmoid_for<T>(u);
        const float keep = 1.f - z;
        b[i] = keep * b[i] + z * cand;
        a[i] *= keep;
      }
  }
  for (; t < t1; ++t) {
    float zv[CH], uv[CH];
    const long r = (row0 + t) * stride + c;
    ldn<CH>(zp + r, zv);
    ldn<CH>(up + r, uv);
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const float z = sigmoid_for<T>(zv[i]);
      const float cand = uv[i] >= 0.f ? uv[i] + 0.5f : sigmoid_for<T>(uv[i]);
      const float keep = 1.f - z;
      b[i] = keep * b[i] + z * cand;
      a[i] *= keep;
    }
  }
}

// Walk [t0, t1) from state S (updated in place) and write the gated outputs.
template <typename T, int CH>
LIG_DEVICE void range_replay(T* __restrict__ out, const T* __restrict__ zp,
                             const T* __restrict__ up, const T* __restrict__ gp,
                             long stride, int W, long row0, int c, int t0, int t1,
                             float* S) {
  int t = t0;
  for (; t + MINGRU_TU <= t1; t += MINGRU_TU) {
    float zv[MINGRU_TU][CH], uv[MINGRU_TU][CH], gv[MINGRU_TU][CH];
#pragma unroll
    for (int k = 0; k < MINGRU_TU; ++k) {
      const long r = (row0 + t + k) * stride + c;
      ldn<CH>(zp + r, zv[k]);
      ldn<CH>(up + r, uv[k]);
      ldn<CH>(gp + r, gv[k]);
    }
#pragma unroll
    for (int k = 0; k < MINGRU_TU; ++k) {
      float o[CH];
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const float z = sigmoid_for<T>(zv[k][i]);
        const float u = uv[k][i];
        const float cand = u >= 0.f ? u + 0.5f : sigmoid_for<T>(u);
        S[i] = (1.f - z) * S[i] + z * cand;
        const float g = gv[k][i];
        o[i] = S[i] * (g * sigmoid_for<T>(g));
      }
      stn<CH>(out + (row0 + t + k) * (long)W + c, o);
    }
  }
  for (; t < t1; ++t) {
    float zv[CH], uv[CH], gv[CH], o[CH];
    const long r = (row0 + t) * stride + c;
    ldn<CH>(zp + r, zv);
    ldn<CH>(up + r, uv);
    ldn<CH>(gp + r, gv);
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const float z = sigmoid_for<T>(zv[i]);
      const float cand = uv[i] >= 0.f ? uv[i] + 0.5f : sigmoid_for<T>(uv[i]);
      S[i] = (1.f - z) * S[i] + z * cand;
      o[i] = S[i] * (gv[i] * sigmoid_for<T>(gv[i]));
    }
    stn<CH>(out + (row0 + t) * (long)W + c, o);
  }
}

// ---- one kernel per step: short segments and decode ---------------------------

template <typename T, int CH>
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
  __shared__ float lds_a[MINGRU_MAX_WAVES][WAVE_SIZE * CH];
  __shared__ float lds_b[MINGRU_MAX_WAVES][WAVE_SIZE * CH];
  const int s = blockIdx.y;
  const int len = seg_len[s];
  if (len <= 0) return;
  const int lane = threadIdx.x % WAVE_SIZE;
  const int wave = threadIdx.x / WAVE_SIZE;
  const int nw = blockDim.x / WAVE_SIZE;
  const int c = (blockIdx.x * WAVE_SIZE + lane) * CH;
  const bool active = c < W;  // W % CH == 0: a lane is wholly in or out
  const long row0 = seg_start[s];
  const int cl = (len + nw - 1) / nw;
  const int t0 = min(len, wave * cl);
  const int t1 = min(len, t0 + cl);

  float* st_ptr = state + (size_t)seg_slot[s] * W + c;
  float S[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) S[i] = 0.f;
  if (active && !seg_fresh[s]) ldn<CH>(st_ptr, S);

  if (nw > 1) {
    float a[CH], b[CH];
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      a[i] = 1.f;
      b[i] = 0.f;
    }
    if (active) range_reduce<T, CH>(zp, up, stride, row0, c, t0, t1, a, b);
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      lds_a[wave][lane * CH + i] = a[i];
      lds_b[wave][lane * CH + i] = b[i];
    }
    __syncthreads();
    for (int j = 0; j < wave; ++j)
#pragma unroll
      for (int i = 0; i < CH; ++i)
        S[i] = lds_a[j][lane * CH + i] * S[i] + lds_b[j][lane * CH + i];
  }

  if (!active) return;
  range_replay<T, CH>(out, zp, up, gp, stride, W, row0, c, t0, t1, S);
  if (t1 == len && t0 < t1) stn<CH>(st_ptr, S);
}

// ---- three passes: long segments -------------------------------------------------
// Time is cut into chunks of MINGRU_TC steps; pass 1 reduces every chunk to
// (a, b) in a scratch, pass 2 chains the carries per (segment, channel) and
// updates the state slot, pass 3 replays every chunk from its carry.  Passes
// 1 and 3 have one wave per (chunk, 64*CH channels): enough waves to hide
// the load latency that the serial walk of a chunk cannot.

#define MINGRU_TC 32
#define MINGRU_CB 4  // chunks (waves) per block

template <typename T, int CH>
__global__ void mingru_chunk_reduce_kernel(
    const T* __restrict__ zp, const T* __restrict__ up, long stride,
    float* __restrict__ sa, float* __restrict__ sb,  // [S, nchunk, W]
    const int* __restrict__ seg_start, const int* __restrict__ seg_len,
    int nchunk, int W) {
  const int s = blockIdx.z;
  const int len = seg_len[s];
  const int j = blockIdx.y * MINGRU_CB + threadIdx.x / WAVE_SIZE;
  const int c = (blockIdx.x * WAVE_SIZE + threadIdx.x % WAVE_SIZE) * CH;
  const int t0 = j * MINGRU_TC;
  if (j >= nchunk || t0 >= len || c >= W) return;
  const int t1 = min(len, t0 + MINGRU_TC);
  float a[CH], b[CH];
  range_reduce<T, CH>(zp, up, stride, seg_start[s], c, t0, t1, a, b);
  const size_t o = ((size_t)s * nchunk + j) * W + c;
  stn<CH>(sa + o, a);
  stn<CH>(sb + o, b);
}

// After this pass sb[s, j] holds the state entering chunk j.
__global__ void mingru_chunk_carry_kernel(
    float* __restrict__ sa, float* __restrict__ sb, float* __restrict__ state,
    const int* __restrict__ seg_len, const int* __restrict__ seg_slot,
    const int* __restrict__ seg_fresh, int nchunk, int W) {
  const int s = blockIdx.y;
  const int len = seg_len[s];
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (len <= 0 || c >= W) return;
  float* st_ptr = state + (size_t)seg_slot[s] * W + c;
  float carry = seg_fresh[s] ? 0.f : *st_ptr;
  const int n = (len + MINGRU_TC - 1) / MINGRU_TC;
  for (int j = 0; j < n; ++j) {
    const size_t o = ((size_t)s * nchunk + j) * W + c;
    const float a = sa[o], b = sb[o];
    sb[o] = carry;
    carry = a * carry + b;
  }
  *st_ptr = carry;
}

template <typename T, int CH>
__global__ void mingru_chunk_replay_kernel(
    T* __restrict__ out, const T* __restrict__ zp, const T* __restrict__ up,
    const T* __restrict__ gp, long stride, const float* __restrict__ sb,
    const int* __restrict__ seg_start, const int* __restrict__ seg_len,
    int nchunk, int W) {
  const int s = blockIdx.z;
  const int len = seg_len[s];
  const int j = blockIdx.y * MINGRU_CB + threadIdx.x / WAVE_SIZE;
  const int c = (blockIdx.x * WAVE_SIZE + threadIdx.x % WAVE_SIZE) * CH;
  const int t0 = j * MINGRU_TC;
  if (j >= nchunk || t0 >= len || c >= W) return;
  const int t1 = min(len, t0 + MINGRU_TC);
  float S[CH];
  ldn<CH>(sb + ((size_t)s * nchunk + j) * W + c, S);
  range_replay<T, CH>(out, zp, up, gp, stride, W, seg_start[s], c, t0, t1, S);
}

template <typename T>
static void launch_mingru(T* out, const T* zp, const T* up, const T* gp,
                          long stride, float* state, float* scratch,
                          const int* seg_start, const int* seg_len,
                          const int* seg_slot, const int* seg_fresh,
                          int num_segs, int max_len, int W, hipStream_t s) {
  const uintptr_t al = sizeof(T) * 4 - 1;  // 4-element accesses
  const bool vec = W % 4 == 0 && stride % 4 == 0 &&
                   ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(zp) |
                     reinterpret_cast<uintptr_t>(up) | reinterpret_cast<uintptr_t>(gp)) & al) == 0 &&
                   (reinterpret_cast<uintptr_t>(state) & 15u) == 0 &&
                   (reinterpret_cast<uintptr_t>(scratch) & 15u) == 0;
  const int ch = vec ? 4 : 1;
  const int gx = (W + WAVE_SIZE * ch - 1) / (WAVE_SIZE * ch);
  if (scratch != nullptr) {
    const int nchunk = (max_len + MINGRU_TC - 1) / MINGRU_TC;
    float* sa = scratch;
    float* sb = scratch + (size_t)num_segs * nchunk * W;
    dim3 grid(gx, (nchunk + MINGRU_CB - 1) / MINGRU_CB, num_segs), block(WAVE_SIZE * MINGRU_CB);
    if (vec)
      hipLaunchKernelGGL((mingru_chunk_reduce_kernel<T, 4>), grid, block, 0, s, zp, up, stride, sa, sb, seg_start, seg_len, nchunk, W);
    else
      hipLaunchKernelGGL((mingru_chunk_reduce_kernel<T, 1>), grid, block, 0, s, zp, up, stride, sa, sb, seg_start, seg_len, nchunk, W);
    hipLaunchKernelGGL(mingru_chunk_carry_kernel, dim3((W + 255) / 256, num_segs), dim3(256), 0, s,
                       sa, sb, state, seg_len, seg_slot, seg_fresh, nchunk, W);
    if (vec)
      hipLaunchKernelGGL((mingru_chunk_replay_kernel<T, 4>), grid, block, 0, s, out, zp, up, gp, stride, sb, seg_start, seg_len, nchunk, W);
    else
      hipLaunchKernelGGL((mingru_chunk_replay_kernel<T, 1>), grid, block, 0, s, out, zp, up, gp, stride, sb, seg_start, seg_len, nchunk, W);
    return;
  }
  int nw = 1;
  if (max_len >= 512) nw = 16;
  else if (max_len >= 64) nw = 8;
  else if (max_len >= 8) nw = 4;
  dim3 grid(gx, num_segs), block(WAVE_SIZE * nw);
  if (vec)
    hipLaunchKernelGGL((mingru_scan_kernel<T, 4>), grid, block, 0, s, out, zp, up,
                       gp, stride, state, seg_start, seg_len, seg_slot, seg_fresh, W);
  else
    hipLaunchKernelGGL((mingru_scan_kernel<T, 1>), grid, block, 0, s, out, zp, up,
                       gp, stride, state, seg_start, seg_len, seg_slot, seg_fresh, W);
}

// scratch: null for the one-kernel path, else 2 * num_segs *
// ceil(max_len / 32) * W floats for the three-pass path.
extern "C" void lig_mingru_scan(void* out, const void* zp, const void* up,
                                const void* gp, long stride, float* state,
                                float* scratch, const int* seg_start, const int* seg_len,
                                const int* seg_slot, const int* seg_fresh,
                                int num_segs, int max_len, int W, int is_f32,
                                hipStream_t s) {
  if (num_segs <= 0 || W <= 0) return;
  if (is_f32)
    launch_mingru<float>((float*)out, (const float*)zp, (const float*)up,
                         (const float*)gp, stride, state, scratch, seg_start, seg_len,
                         seg_slot, seg_fresh, num_segs, max_len, W, s);
  else
    launch_mingru<bf16s>((bf16s*)out, (const bf16s*)zp, (const bf16s*)up,
                         (const bf16s*)gp, stride, state, scratch, seg_start, seg_len,
                         seg_slot, seg_fresh, num_segs, max_len, W, s);
}
