// Multi-query attention over a paged latent cache on MFMA tiles, bf16, gfx950:
// every query head of a token reads the SAME cache rows, keys being the whole
// row (D entries) and values its leading Dv entries.
//
// Because all heads share the keys, the query rows of a tile are (token,
// head) pairs: row rho = token * H + head inside a sequence's segment of the
// step, 64 consecutive rho per workgroup (4 waves x 16 rows).  A key/value
// tile is read from HBM/L2 once per workgroup and serves every head in it,
// so a decode step (one token, H heads) is one pass over the sequence's cache
// and a prompt portion moves H times fewer key bytes than a per-head grid.
// Prompt portions and single tokens go through the same kernel: a segment is
// (first row, token count, context length after the step), and a row's
// causal bound is its token's position.
//
// Per 32-key tile: each 16-byte chunk of a cache row is loaded once and
// stored twice in LDS, row-major for S^T = K Q^T and transposed for O += P V
// (mfma_f32_16x16x32_bf16, zero padding to the template's DKP / DVP).
// Consecutive lanes stage consecutive KEYS of one chunk column, so the
// transposed 2-byte stores of a wave fall into consecutive LDS words; LDS
// rows are padded by 16 bytes so that the 16-byte fragment reads of 16
// different rows spread over all banks.  The loads of the next tile are
// issued before the current tile's arithmetic (one tile in registers).
// Scores, running max and sum are fp32; an optional per-head sink starts a
// row's running max at sink_h and its sum at one.
//
// Grid = (ceil(max segment rows / 64), segments, splits); workgroups past a
// segment's last row exit at once.  With splits > 1 (few rows, long
// contexts) each z-slice walks an equal share of the tile's visible keys and
// leaves its unnormalised sum with its running max and sum in an fp32
// scratch; a second kernel merges the slices.  The sink is counted by slice
// zero only.

#include "elem_types.h"

typedef __bf16 lr_bf16x8 __attribute__((ext_vector_type(8)));
typedef float lr_f32x4 __attribute__((ext_vector_type(4)));

#define LR_KVBLK 32
#define LR_ROWS 64
#define LR_PAD 8
#define LR_PART_PAD 4  // a slice row is Dv values, running max, running sum, 2 unused

// NCH 16-byte chunks of one cache row (columns sd0, sd0 + 64, ...) into
// registers; zeros for a key past the visible range (blk < 0) and for
// columns at or past D.
template <int NCH>
LIG_DEVICE void lr_load_chunks(u16x8* stage, const uint16_t* __restrict__ cache, int blk,
                               int t, int block_size, int D, int sd0) {
  const uint16_t* rowp =
      cache + ((size_t)(blk < 0 ? 0 : blk) * block_size + (t % block_size)) * D;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int d0 = sd0 + j * 64;
    if (blk >= 0 && d0 < D) {
      stage[j] = *reinterpret_cast<const u16x8*>(rowp + d0);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) stage[j][e] = 0;
    }
  }
}

template <int DKP, int DVP>
__global__ __launch_bounds__(256) void latent_attention_rows_kernel(
    uint16_t* __restrict__ out,          // [R, H * Dv]
    const uint16_t* __restrict__ q,      // [R, H * D] contiguous
    const uint16_t* __restrict__ cache,  // [blocks, 1, BS, D]
    const float* __restrict__ sink,      // nullable, [H]
    const int* __restrict__ seg_start, const int* __restrict__ seg_len,
    const int* __restrict__ seg_ctx,     // tokens of the sequence after this step
    const int* __restrict__ block_tables, int max_blocks, float scale, int H,
    int D, int Dv, int block_size, int nsplit,
    float* __restrict__ partial) {  // [R * H, nsplit, Dv + 4] when nsplit > 1
  static_assert(DVP <= DKP, "values are a prefix of the key row");
  constexpr int DB = DVP / 16;
  constexpr int KB = DKP / 32;

  struct Shared {
    uint16_t K[LR_KVBLK][DKP + LR_PAD];
    uint16_t VT[DVP][LR_KVBLK + LR_PAD];
    uint16_t P[4][16][LR_KVBLK + LR_PAD];
  };
  __shared__ Shared sm;

  const int s = blockIdx.y;
  const int n = seg_len[s];
  const long nrows = (long)n * H;
  const long rho0 = (long)blockIdx.x * LR_ROWS;
  if (rho0 >= nrows) return;
  const long lo = seg_start[s];
  const int ctx = seg_ctx[s];
  const int* bt = block_tables + (size_t)s * max_blocks;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 15;
  const int lg = lane >> 4;

  const long rho = rho0 + wave * 16 + li;
  const bool row_valid = rho < nrows;
  // a wave whose 16 rows all lie past the segment only helps staging
  const bool wave_active = rho0 + wave * 16 < nrows;
  const int tok = (int)((row_valid ? rho : rho0) / H);
  const int head = (int)((row_valid ? rho : rho0) - (long)tok * H);
  const int qpos = ctx - n + tok;

  lr_bf16x8 q_frag[KB];
  {
    const uint16_t* qp = q + ((size_t)lo * H + (row_valid ? rho : rho0)) * D;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int d0 = kb * 32 + lg * 8;
      u16x8 raw;
      if (d0 < D) {
        raw = *reinterpret_cast<const u16x8*>(qp + d0);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) raw[e] = 0;
      }
      q_frag[kb] = *reinterpret_cast<lr_bf16x8*>(&raw);
    }
  }

  const int z = blockIdx.z;
  const bool with_sink = sink != nullptr && z == 0;
  float m = with_sink ? sink[head] : -INFINITY;
  float l = with_sink ? 1.0f : 0.0f;
  lr_f32x4 acc_o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) acc_o[db] = lr_f32x4{0.f, 0.f, 0.f, 0.f};

  const long last_rho = (rho0 + LR_ROWS < nrows ? rho0 + LR_ROWS : nrows) - 1;
  const int kv_end = ctx - n + (int)(last_rho / H) + 1;  // keys any row of the tile sees

  int kv_lo = 0, kv_hi = kv_end;
  if (nsplit > 1) {
    const int nt = (kv_end + LR_KVBLK - 1) / LR_KVBLK;
    const int per = (nt + nsplit - 1) / nsplit;
    kv_lo = min(kv_end, z * per * LR_KVBLK);
    kv_hi = min(kv_end, kv_lo + per * LR_KVBLK);
  }

  // Staging is software-pipelined: a thread always stages the same key row of
  // a tile (256 threads = 8 chunk columns x 32 keys, NCH column groups), so it
  // needs ONE block-table entry per tile.  The chunks of tile i+1 are loaded
  // into registers, and the table entry of tile i+2 is fetched, while tile i
  // is being multiplied; they are written to LDS at the top of the next turn.
  constexpr int NCH = DKP / 64;
  const int srow = tid % LR_KVBLK;
  const int sd0 = (tid / LR_KVBLK) * 8;
  u16x8 stage[NCH];
  int blk_next;
  {
    const int t = kv_lo + srow;
    const int blk = (kv_lo < kv_hi && t < kv_end) ? bt[t / block_size] : -1;
    lr_load_chunks<NCH>(stage, cache, blk, t, block_size, D, sd0);
    const int t2 = t + LR_KVBLK;
    blk_next = (kv_lo + LR_KVBLK < kv_hi && t2 < kv_end) ? bt[t2 / block_size] : -1;
  }

  for (int kv0 = kv_lo; kv0 < kv_hi; kv0 += LR_KVBLK) {
    // ---- registers -> LDS: row-major for S^T = K Q^T, transposed for O += P V ----
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int d0 = sd0 + j * 64;
      const u16x8 kval = stage[j];
      *reinterpret_cast<u16x8*>(&sm.K[srow][d0]) = kval;
      if (d0 < DVP) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sm.VT[d0 + e][srow] = (d0 + e < Dv) ? kval[e] : (uint16_t)0;
      }
    }
    __syncthreads();
    {  // prefetch the next tile (loads stay in flight through the arithmetic below)
      const int kvn = kv0 + LR_KVBLK;
      if (kvn < kv_hi) {
        const int t = kvn + srow;
        lr_load_chunks<NCH>(stage, cache, blk_next, t, block_size, D, sd0);
        const int t2 = t + LR_KVBLK;
        blk_next = (kvn + LR_KVBLK < kv_hi && t2 < kv_end) ? bt[t2 / block_size] : -1;
      }
    }

    if (wave_active) {
    // ---- S^T = K Q^T ----------------------------------------------------------
    lr_f32x4 acc_s[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      acc_s[kt] = lr_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        u16x8 raw =
            *reinterpret_cast<const u16x8*>(&sm.K[kt * 16 + li][kb * 32 + lg * 8]);
        lr_bf16x8 a_frag = *reinterpret_cast<lr_bf16x8*>(&raw);
        acc_s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            a_frag, q_frag[kb], acc_s[kt], 0, 0, 0);
      }
    }

    // ---- mask + online softmax (this lane owns row rho) -------------------------
    float sc[8];
    float rowmax = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = kv0 + kt * 16 + lg * 4 + r;
        float v = acc_s[kt][r] * scale;
        if (!row_valid || key > qpos) v = -INFINITY;
        sc[kt * 4 + r] = v;
        rowmax = fmaxf(rowmax, v);
      }
    }
    rowmax = stride_reduce_max<16, 4>(rowmax);
    const float m_new = fmaxf(m, rowmax);
    float alpha;
    float psum = 0.0f;
    float p[8];
    if (m_new == -INFINITY) {
      alpha = 1.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = 0.0f;
    } else {
      alpha = (m == -INFINITY) ? 0.0f : __expf(m - m_new);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        p[i] = (sc[i] == -INFINITY) ? 0.0f : __expf(sc[i] - m_new);
        psum += p[i];
      }
      m = m_new;
    }
    psum = stride_reduce_sum<16, 4>(psum);
    l = l * alpha + psum;
    // acc_o rows follow the MFMA C layout (row = lg*4 + r); the softmax stats
    // of row x live in lane x (replicated over the lg groups)
    float alpha_r[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) alpha_r[r] = __shfl(alpha, lg * 4 + r, 64);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int r = 0; r < 4; ++r) acc_o[db][r] *= alpha_r[r];
    }

    // ---- P: C layout -> A-fragment layout through the wave's LDS slab ---------
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        sm.P[wave][li][kt * 16 + lg * 4 + r] = f32_to_bf16(p[kt * 4 + r]);
      }
    }
    u16x8 praw = *reinterpret_cast<const u16x8*>(&sm.P[wave][li][lg * 8]);
    lr_bf16x8 p_frag = *reinterpret_cast<lr_bf16x8*>(&praw);

    // ---- O += P V -----------------------------------------------------------------
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      u16x8 vraw =
          *reinterpret_cast<const u16x8*>(&sm.VT[db * 16 + li][lg * 8]);
      lr_bf16x8 v_frag = *reinterpret_cast<lr_bf16x8*>(&vraw);
      acc_o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_frag, v_frag,
                                                          acc_o[db], 0, 0, 0);
    }
    }  // wave_active
    __syncthreads();
  }

  if (nsplit > 1) {
    // ---- partial result: unnormalised sums, running max and sum -------------------
    const size_t stride = (size_t)Dv + LR_PART_PAD;
    if (row_valid && lg == 0) {
      float* pp = partial + (((size_t)lo * H + rho) * nsplit + z) * stride;
      pp[Dv] = m;
      pp[Dv + 1] = l;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const long orho = rho0 + wave * 16 + lg * 4 + r;
      if (orho >= nrows) continue;
      float* pp = partial + (((size_t)lo * H + orho) * nsplit + z) * stride;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int d = db * 16 + li;
        if (d < Dv) pp[d] = acc_o[db][r];
      }
    }
    return;
  }

  // ---- epilogue: normalise and store ------------------------------------------------
  float inv_l[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float lr = __shfl(l, lg * 4 + r, 64);  // all lanes active here
    inv_l[r] = lr > 0.f ? 1.0f / lr : 0.0f;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const long orho = rho0 + wave * 16 + lg * 4 + r;
    if (orho >= nrows) continue;
    uint16_t* op = out + ((size_t)lo * H + orho) * Dv;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int d = db * 16 + li;
      if (d < Dv) op[d] = f32_to_bf16(acc_o[db][r] * inv_l[r]);
    }
  }
}


// Merge the z-slices of every row: m* = max m_z, out = sum_z e^(m_z - m*) acc_z
// / sum_z e^(m_z - m*) l_z.  One wave per row.  Lane z holds slice z's weight
// (up to 64 slices); the lanes then own float4 columns of the value row and
// add up the slices with independent 16-byte loads (slice rows are padded
// to Dv + 4 floats so that they stay 16-byte aligned).
__global__ __launch_bounds__(256) void latent_attention_rows_combine_kernel(
    uint16_t* __restrict__ out, const float* __restrict__ partial,
    const int* __restrict__ seg_start, const int* __restrict__ seg_len, int H,
    int Dv, int nsplit) {
  const int s = blockIdx.y;
  const long nrows = (long)seg_len[s] * H;
  const long rho = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (rho >= nrows) return;  // whole waves leave; no workgroup barrier below
  const int lane = threadIdx.x & 63;
  const size_t g = (size_t)seg_start[s] * H + rho;
  const size_t stride = (size_t)Dv + LR_PART_PAD;
  const float* pp = partial + g * nsplit * stride;
  float mz = -INFINITY, lz = 0.f;
  if (lane < nsplit) {
    mz = pp[lane * stride + Dv];
    lz = pp[lane * stride + Dv + 1];
  }
  const float mstar = wave_reduce_max(mz);
  const float wz = (mz == -INFINITY) ? 0.f : __expf(mz - mstar);
  const float lsum = wave_reduce_sum(wz * lz);
  const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
  for (int d0 = 0; d0 < Dv; d0 += 256) {  // uniform trip count: every lane feeds the shuffles
    const int d = d0 + lane * 4;
    const bool act = d < Dv;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    const float* col = pp + (act ? d : 0);
    int zz = 0;
    for (; zz + 4 <= nsplit; zz += 4) {  // four slices' loads in flight at a time
      f32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const f32x4*>(col + (zz + u) * stride);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float w = __shfl(wz, zz + u, 64);
        a0 += w * v[u][0];
        a1 += w * v[u][1];
        a2 += w * v[u][2];
        a3 += w * v[u][3];
      }
    }
    for (; zz < nsplit; ++zz) {
      const float w = __shfl(wz, zz, 64);
      const f32x4 v = *reinterpret_cast<const f32x4*>(col + zz * stride);
      a0 += w * v[0];
      a1 += w * v[1];
      a2 += w * v[2];
      a3 += w * v[3];
    }
    if (!act) continue;
    uint2 packed;
    packed.x = (uint32_t)f32_to_bf16(a0 * inv) | ((uint32_t)f32_to_bf16(a1 * inv) << 16);
    packed.y = (uint32_t)f32_to_bf16(a2 * inv) | ((uint32_t)f32_to_bf16(a3 * inv) << 16);
    *reinterpret_cast<uint2*>(out + g * Dv + d) = packed;
  }
}

// Returns 0 when launched, 1 when the shape is not served (the caller then
// uses another kernel).
extern "C" int lig_latent_attention_rows(
    void* out, const void* q, const void* cache, const float* sink,
    const int* seg_start, const int* seg_len, const int* seg_ctx,
    const int* block_tables, int max_blocks, float scale, int num_segs,
    int max_seg_len, int H, int D, int Dv, int block_size, int nsplit,
    float* partial, hipStream_t stream) {
  if (D % 8 != 0 || Dv % 8 != 0 || D <= 0 || Dv <= 0 || Dv > D || D > 576 ||
      Dv > 512 || !aligned16(q) || !aligned16(cache) || H <= 0)
    return 1;
  if (num_segs <= 0 || max_seg_len <= 0) return 0;
  const long tiles = ((long)max_seg_len * H + LR_ROWS - 1) / LR_ROWS;
  if (tiles > 2147483647L || num_segs > 65535) return 1;
  if (nsplit < 1 || nsplit > 64 || (nsplit > 1 && partial == nullptr)) return 1;
  dim3 grid((unsigned)tiles, num_segs, nsplit);
  dim3 block(256);
#define LAUNCH_LR(DKP, DVP)                                                    \
  hipLaunchKernelGGL((latent_attention_rows_kernel<DKP, DVP>), grid, block, 0, \
                     stream, (uint16_t*)out, (const uint16_t*)q,               \
                     (const uint16_t*)cache, sink, seg_start, seg_len,         \
                     seg_ctx, block_tables, max_blocks, scale, H, D, Dv,       \
                     block_size, nsplit, partial)
  if (D <= 64 && Dv <= 64) LAUNCH_LR(64, 64);
  else if (D <= 128 && Dv <= 64) LAUNCH_LR(128, 64);
  else if (D <= 128) LAUNCH_LR(128, 128);
  else if (D <= 192 && Dv <= 128) LAUNCH_LR(192, 128);
  else if (D <= 320 && Dv <= 256) LAUNCH_LR(320, 256);
  else LAUNCH_LR(576, 512);
#undef LAUNCH_LR
  if (nsplit > 1) {
    const long rows4 = ((long)max_seg_len * H + 3) / 4;
    hipLaunchKernelGGL(latent_attention_rows_combine_kernel,
                       dim3((unsigned)rows4, num_segs), dim3(256), 0, stream,
                       (uint16_t*)out, partial, seg_start, seg_len, H, Dv, nsplit);
  }
  return 0;
}
