// Paged-attention prefill on MFMA tiles for head sizes the 64/128 kernel does
// not take: key size D and value size Dv independent, each a multiple of 8
// and at most 128, bf16, gfx950.
//
// Same tiling as the fixed-size flash-prefill kernel: grid = (64-row query
// tiles, q heads), 4 waves per workgroup, wave w owns rows [16w, 16w+16) and
// walks the sequence's pages 32 keys at a time with
// mfma_f32_16x16x32_bf16: S^T = K Q^T (so a lane ends up holding 8 scores of
// ONE query row and the row softmax needs two xor-shuffles), online softmax
// in fp32, P through a wave-private LDS slab into the A-fragment layout,
// then O += P V against V staged transposed.
//
// Differences: the head sizes are run-time values padded with zeros in LDS
// to the template's DKP (multiple of 32) and DVP (multiple of 16); q is read
// from a strided view (a column block of the fused projection); the
// per-position query temperature tau(p) = 1 + c ln(floor((p+1)/e) + 1)
// multiplies the fp32 scores of row p; the sigmoid output gate is applied in
// the epilogue.  K and V are staged separately since their rows differ in
// length.  An optional per-head sink starts every row's running max at
// sink_h and its running sum at one (a key with that unscaled score and no
// value).  chunk > 0 restricts a row at position p to keys j with
// floor(j / chunk) == floor(p / chunk); window > 0 to keys j with
// p - j < window.  sigmoid_weights replaces the softmax by unnormalised
// weights sigmoid(score + score_bias[h]); gate_per_head reads one gate entry
// per (row, head).  A value row is the first Dv entries of a cache row of v_row
// entries, so a latent cache can pass its key rows as values.

#include "elem_types.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define PT_KVBLK 32
#define PT_TQ 64

template <int DKP, int DVP>
__global__ __launch_bounds__(256) void paged_attention_prefill_tiles_kernel(
    uint16_t* __restrict__ out,            // [R, Hq * Dv]
    const uint16_t* __restrict__ q, long q_stride,
    const uint16_t* __restrict__ k_cache,  // [B, Hkv, BS, D]
    const uint16_t* __restrict__ v_cache,  // [B, Hkv, BS, Dv]
    const uint16_t* __restrict__ gate, long gate_stride,  // nullable
    const float* __restrict__ sink,                       // nullable, [Hq]
    const int* __restrict__ tile_seq, const int* __restrict__ tile_qstart,
    const int* __restrict__ query_start_locs,  // [S+1]
    const int* __restrict__ context_lens,      // [S] after this step's tokens
    const int* __restrict__ block_tables, float scale, float temp_coef,
    float temp_every, int temp_every_int, int num_q_heads, int num_kv_heads,
    int D, int Dv, int v_row, int block_size, int max_blocks, int chunk,
    int window, const float* __restrict__ score_bias, int sigmoid_weights,
    int gate_per_head) {
  constexpr int DB = DVP / 16;
  constexpr int KB = DKP / 32;

  struct Shared {
    uint16_t K[PT_KVBLK][DKP];
    uint16_t VT[DVP][PT_KVBLK];
    uint16_t P[4][16][PT_KVBLK];
  };
  __shared__ Shared sm;

  const int tile = blockIdx.x;
  const int h = blockIdx.y;
  const int s = tile_seq[tile];
  const int qt = tile_qstart[tile];
  const int group = num_q_heads / num_kv_heads;
  const int kvh = h / group;

  const int lo = query_start_locs[s];
  const int n = query_start_locs[s + 1] - lo;
  const int ctx = context_lens[s];
  const int* bt = block_tables + (size_t)s * max_blocks;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 15;
  const int lg = lane >> 4;

  const int qrow_sm = qt + wave * 16 + li;
  const bool row_valid = qrow_sm < n;
  const int qpos = ctx - n + qrow_sm;

  float row_scale = scale;
  if (temp_coef != 0.f && row_valid) {
    const float m = temp_every_int > 0
                        ? (float)((qpos + 1) / temp_every_int)
                        : floorf((float)(qpos + 1) / temp_every);
    row_scale = scale * (1.f + temp_coef * logf(m + 1.f));
  }

  // Q fragments; 8-element chunks at or past D are zero (D % 8 == 0)
  bf16x8_t q_frag[KB];
  {
    const int qr = row_valid ? qrow_sm : 0;
    const uint16_t* qp = q + (size_t)(lo + qr) * q_stride + (size_t)h * D;
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
      q_frag[kb] = *reinterpret_cast<bf16x8_t*>(&raw);
    }
  }

  float m = sink ? sink[h] : -INFINITY;
  float l = sink ? 1.0f : 0.0f;
  f32x4_t acc_o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) acc_o[db] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int kv_end_tile = min(ctx, ctx - n + qt + PT_TQ);

  // chunked visibility: a row at position p sees keys from floor(p / chunk)
  // * chunk on; the tile's walk starts at its first row's chunk
  const int qpos0 = ctx - n + qt;
  int kv_begin = chunk > 0 ? (qpos0 / chunk) * chunk : 0;
  int key_lo = (chunk > 0 && row_valid) ? (qpos / chunk) * chunk : 0;
  if (window > 0) {
    kv_begin = max(kv_begin, qpos0 - window + 1);
    if (row_valid) key_lo = max(key_lo, qpos - window + 1);
  }
  const float sb = score_bias ? score_bias[h] : 0.f;

  for (int kv0 = kv_begin; kv0 < kv_end_tile; kv0 += PT_KVBLK) {
    // ---- staging: K rows [32][DKP], V transposed [DVP][32]; zero padding ----
    for (int c = tid; c < PT_KVBLK * (DKP / 8); c += 256) {
      const int row = c / (DKP / 8);
      const int d0 = (c % (DKP / 8)) * 8;
      const int t = kv0 + row;
      u16x8 kval;
      if (t < ctx && d0 < D) {
        const size_t base =
            (((size_t)bt[t / block_size] * num_kv_heads + kvh) * block_size +
             (t % block_size)) * D + d0;
        kval = *reinterpret_cast<const u16x8*>(k_cache + base);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) kval[e] = 0;
      }
      *reinterpret_cast<u16x8*>(&sm.K[row][d0]) = kval;
    }
    for (int c = tid; c < PT_KVBLK * (DVP / 8); c += 256) {
      const int row = c / (DVP / 8);
      const int d0 = (c % (DVP / 8)) * 8;
      const int t = kv0 + row;
      u16x8 vval;
      if (t < ctx && d0 < Dv) {
        const size_t base =
            (((size_t)bt[t / block_size] * num_kv_heads + kvh) * block_size +
             (t % block_size)) * v_row + d0;
        vval = *reinterpret_cast<const u16x8*>(v_cache + base);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) vval[e] = 0;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) sm.VT[d0 + e][row] = vval[e];
    }
    __syncthreads();

    // ---- S^T = K Q^T ----------------------------------------------------------
    f32x4_t acc_s[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      acc_s[kt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        u16x8 raw =
            *reinterpret_cast<const u16x8*>(&sm.K[kt * 16 + li][kb * 32 + lg * 8]);
        bf16x8_t a_frag = *reinterpret_cast<bf16x8_t*>(&raw);
        acc_s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            a_frag, q_frag[kb], acc_s[kt], 0, 0, 0);
      }
    }

    // ---- mask + online softmax (this lane owns row qrow_sm) --------------------
    float sc[8];
    float rowmax = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = kv0 + kt * 16 + lg * 4 + r;
        float v = acc_s[kt][r] * row_scale;
        if (!row_valid || key > qpos || key >= ctx || key < key_lo) v = -INFINITY;
        sc[kt * 4 + r] = v;
        rowmax = fmaxf(rowmax, v);
      }
    }
    rowmax = stride_reduce_max<16, 4>(rowmax);
    const float m_new = fmaxf(m, rowmax);
    float alpha;
    float psum = 0.0f;
    float p[8];
    if (sigmoid_weights) {
      alpha = 1.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        p[i] = (sc[i] == -INFINITY) ? 0.0f : sigmoid_fast(sc[i] + sb);
    } else if (m_new == -INFINITY) {
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
    bf16x8_t p_frag = *reinterpret_cast<bf16x8_t*>(&praw);

    // ---- O += P V -----------------------------------------------------------------
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      u16x8 vraw =
          *reinterpret_cast<const u16x8*>(&sm.VT[db * 16 + li][lg * 8]);
      bf16x8_t v_frag = *reinterpret_cast<bf16x8_t*>(&vraw);
      acc_o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_frag, v_frag,
                                                          acc_o[db], 0, 0, 0);
    }
    __syncthreads();
  }

  // ---- epilogue: normalise, gate, store -------------------------------------------
  float inv_l[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float lr = __shfl(l, lg * 4 + r, 64);  // all lanes active here
    inv_l[r] = sigmoid_weights ? 1.0f : (lr > 0.f ? 1.0f / lr : 0.0f);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int orow = qt + wave * 16 + lg * 4 + r;
    if (orow >= n) continue;
    uint16_t* op = out + ((size_t)(lo + orow) * num_q_heads + h) * Dv;
    const uint16_t* gp =
        (gate && !gate_per_head)
            ? gate + (size_t)(lo + orow) * gate_stride + (size_t)h * Dv : nullptr;
    const float hg =
        (gate && gate_per_head)
            ? sigmoid_fast(bf16_to_f32(gate[(size_t)(lo + orow) * gate_stride + h])) : 1.0f;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int d = db * 16 + li;
      if (d < Dv) {
        float o = acc_o[db][r] * inv_l[r];
        if (gp) o *= sigmoid_fast(bf16_to_f32(gp[d]));
        o *= hg;
        op[d] = f32_to_bf16(o);
      }
    }
  }
}

// Returns 0 when launched, 1 when the shape is not served (the caller then
// uses the any-shape kernel).
extern "C" int lig_paged_attention_prefill_tiles(
    void* out, const void* q, long q_stride, const void* k_cache,
    const void* v_cache, const void* gate, long gate_stride, const float* sink,
    const int* tile_seq, const int* tile_qstart, const int* query_start_locs,
    const int* context_lens, const int* block_tables, float scale,
    float temp_coef, float temp_every, int temp_every_int, int ntiles,
    int num_q_heads, int num_kv_heads, int D, int Dv, int v_row, int block_size,
    int max_blocks, int chunk, int window, const float* score_bias,
    int sigmoid_weights, int gate_per_head, hipStream_t stream) {
  if (D % 8 != 0 || Dv % 8 != 0 || D > 128 || Dv > 128 || D <= 0 || Dv <= 0 ||
      v_row % 8 != 0 || v_row < Dv ||
      q_stride % 8 != 0 || !aligned16(q) || !aligned16(k_cache) ||
      !aligned16(v_cache) || num_q_heads % num_kv_heads != 0)
    return 1;
  if (ntiles <= 0) return 0;
  dim3 grid(ntiles, num_q_heads);
  dim3 block(256);
#define LAUNCH_PT(DKP, DVP)                                                   \
  hipLaunchKernelGGL((paged_attention_prefill_tiles_kernel<DKP, DVP>), grid,  \
                     block, 0, stream, (uint16_t*)out, (const uint16_t*)q,    \
                     q_stride, (const uint16_t*)k_cache,                      \
                     (const uint16_t*)v_cache, (const uint16_t*)gate,         \
                     gate_stride, sink, tile_seq, tile_qstart,                \
                     query_start_locs,                                        \
                     context_lens, block_tables, scale, temp_coef, temp_every, \
                     temp_every_int, num_q_heads, num_kv_heads, D, Dv, v_row, \
                     block_size, max_blocks, chunk, window, score_bias,       \
                     sigmoid_weights, gate_per_head)
  const int dkp = D <= 32 ? 32 : (D <= 64 ? 64 : 128);
  const int dvp = Dv <= 32 ? 32 : (Dv <= 64 ? 64 : 128);
  if (dkp == 32 && dvp == 32) LAUNCH_PT(32, 32);
  else if (dkp == 32 && dvp == 64) LAUNCH_PT(32, 64);
  else if (dkp == 32 && dvp == 128) LAUNCH_PT(32, 128);
  else if (dkp == 64 && dvp == 32) LAUNCH_PT(64, 32);
  else if (dkp == 64 && dvp == 64) LAUNCH_PT(64, 64);
  else if (dkp == 64 && dvp == 128) LAUNCH_PT(64, 128);
  else if (dkp == 128 && dvp == 32) LAUNCH_PT(128, 32);
  else if (dkp == 128 && dvp == 64) LAUNCH_PT(128, 64);
  else LAUNCH_PT(128, 128);
#undef LAUNCH_PT
  return 0;
}
