// Head-mixed paged attention for prompt rows on MFMA tiles, bf16, gfx950.
//
// Same mathematics as the any-shape head-mixing kernel: for a query at
// position p and a visible key j (j <= p, in p's chunk when chunk > 0)
//     a_g = (q_g . k_j) * scale + dist_bias[min(p - j, N - 1)][g]
//     s_h = sum_g talk[h][g] * a_g
// and an ordinary softmax of s_h per head.  Since a head's weights need every
// head's raw score of the same (query, key) pair, one workgroup serves 16
// query rows of ALL heads, one wave per head up to 16 heads and two heads per
// wave (h and h + 16) up to 32:
//
//   per 32 keys: all waves stage the K rows and transposed V rows of every
//   key/value head in LDS; wave h computes S_h^T = K_g Q_h^T with
//   mfma_f32_16x16x32_bf16, scales, adds the bias and writes its fp32 raw
//   scores to LDS; after a barrier it mixes the raw scores of all heads for
//   its own (fp32 FMAs) into registers; after another barrier (the raw rows
//   are now free) it masks, runs the online softmax, turns P into an A
//   fragment through the LDS rows its own raw scores occupied and accumulates
//   O_h += P V_g.
//
// Head sizes are run-time values, multiples of 8 up to 128, zero-padded in
// LDS to the template's DKP (multiple of 32) and DVP (multiple of 16).  The
// grid walks the runner's 64-row query tiles in four 16-row parts.

#include "elem_types.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define MT_KVBLK 32
#define MT_ROWS 16
#define MT_RS 36  // floats per raw-score row (32 + padding against bank conflicts)

template <int DKP, int DVP, int HPW>
__global__ __launch_bounds__(1024) void paged_attention_mixed_heads_tiles_kernel(
    uint16_t* __restrict__ out,            // [R, H * Dv]
    const uint16_t* __restrict__ q, long q_stride,
    const uint16_t* __restrict__ k_cache,  // [B, G, BS, D]
    const uint16_t* __restrict__ v_cache,  // [B, G, BS, Dv]
    const float* __restrict__ dist_bias, int n_dist,  // nullable, [N, H]
    const float* __restrict__ talk,                   // nullable, [H, H]
    const int* __restrict__ tile_seq, const int* __restrict__ tile_qstart,
    const int* __restrict__ query_start_locs,  // [S+1]
    const int* __restrict__ context_lens,      // [S] after this step's tokens
    const int* __restrict__ block_tables, float scale, int chunk, int H, int G,
    int D, int Dv, int block_size, int max_blocks) {
  constexpr int DB = DVP / 16;
  constexpr int KB = DKP / 32;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint16_t* Ks = reinterpret_cast<uint16_t*>(smem_raw);          // [G][32][DKP]
  uint16_t* VTs = Ks + (size_t)G * MT_KVBLK * DKP;               // [G][DVP][32]
  // raw scores [H][16][MT_RS] fp32; once mixed, head h's rows hold its P
  // slab [16][32] bf16
  float* raw_s = reinterpret_cast<float*>(VTs + (size_t)G * DVP * MT_KVBLK);
  float* talk_s = raw_s + (size_t)H * MT_ROWS * MT_RS;           // [H][H]

  const int tile = blockIdx.x >> 2;
  const int s = tile_seq[tile];
  const int qt = tile_qstart[tile] + (blockIdx.x & 3) * MT_ROWS;
  const int lo = query_start_locs[s];
  const int n = query_start_locs[s + 1] - lo;
  if (qt >= n) return;  // the whole workgroup
  const int ctx = context_lens[s];
  const int* bt = block_tables + (size_t)s * max_blocks;

  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int wave = tid >> 6;  // heads wave, wave + 16
  const int lane = tid & 63;
  const int li = lane & 15;
  const int lg = lane >> 4;
  const int group = H / G;

  const int qrow_sm = qt + li;
  const bool row_valid = qrow_sm < n;
  const int qpos = ctx - n + qrow_sm;

  for (int c = tid; c < H * H; c += nthreads)
    talk_s[c] = talk != nullptr ? talk[c] : ((c / H) == (c % H) ? 1.f : 0.f);

  bf16x8_t q_frag[HPW][KB];
  float m[HPW], l[HPW];
  f32x4_t acc_o[HPW][DB];
#pragma unroll
  for (int hp = 0; hp < HPW; ++hp) {
    const int h = wave + hp * 16;
    const int qr = row_valid ? qrow_sm : 0;
    const uint16_t* qp = q + (size_t)(lo + qr) * q_stride + (size_t)(h < H ? h : 0) * D;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int d0 = kb * 32 + lg * 8;
      u16x8 rawq;
      if (d0 < D) {
        rawq = *reinterpret_cast<const u16x8*>(qp + d0);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) rawq[e] = 0;
      }
      q_frag[hp][kb] = *reinterpret_cast<bf16x8_t*>(&rawq);
    }
    m[hp] = -INFINITY;
    l[hp] = 0.0f;
#pragma unroll
    for (int db = 0; db < DB; ++db) acc_o[hp][db] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  const int qpos0 = ctx - n + qt;
  const int kv_begin = chunk > 0 ? (qpos0 / chunk) * chunk : 0;
  const int key_lo = (chunk > 0 && row_valid) ? (qpos / chunk) * chunk : 0;
  const int kv_end_tile = min(ctx, qpos0 + MT_ROWS);

  for (int kv0 = kv_begin; kv0 < kv_end_tile; kv0 += MT_KVBLK) {
    // ---- staging: every key/value head's K rows and transposed V rows ----------
    for (int c = tid; c < G * MT_KVBLK * (DKP / 8); c += nthreads) {
      const int g = c / (MT_KVBLK * (DKP / 8));
      const int rem = c - g * (MT_KVBLK * (DKP / 8));
      const int row = rem / (DKP / 8);
      const int d0 = (rem % (DKP / 8)) * 8;
      const int t = kv0 + row;
      u16x8 kval;
      if (t < ctx && d0 < D) {
        const size_t base =
            (((size_t)bt[t / block_size] * G + g) * block_size + (t % block_size)) * D + d0;
        kval = *reinterpret_cast<const u16x8*>(k_cache + base);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) kval[e] = 0;
      }
      *reinterpret_cast<u16x8*>(Ks + ((size_t)g * MT_KVBLK + row) * DKP + d0) = kval;
    }
    for (int c = tid; c < G * MT_KVBLK * (DVP / 8); c += nthreads) {
      const int g = c / (MT_KVBLK * (DVP / 8));
      const int rem = c - g * (MT_KVBLK * (DVP / 8));
      const int row = rem / (DVP / 8);
      const int d0 = (rem % (DVP / 8)) * 8;
      const int t = kv0 + row;
      u16x8 vval;
      if (t < ctx && d0 < Dv) {
        const size_t base =
            (((size_t)bt[t / block_size] * G + g) * block_size + (t % block_size)) * Dv + d0;
        vval = *reinterpret_cast<const u16x8*>(v_cache + base);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) vval[e] = 0;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) VTs[((size_t)g * DVP + d0 + e) * MT_KVBLK + row] = vval[e];
    }
    __syncthreads();

    // ---- raw scores of this wave's heads: S^T = K Q^T, scale, bias ----------------
#pragma unroll
    for (int hp = 0; hp < HPW; ++hp) {
      const int h = wave + hp * 16;
      if (h < H) {  // uniform per wave
        const uint16_t* Kg = Ks + (size_t)(h / group) * MT_KVBLK * DKP;
        float* raw_w = raw_s + ((size_t)h * MT_ROWS + li) * MT_RS;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
          f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            u16x8 rawk = *reinterpret_cast<const u16x8*>(Kg + (size_t)(kt * 16 + li) * DKP + kb * 32 + lg * 8);
            bf16x8_t a_frag = *reinterpret_cast<bf16x8_t*>(&rawk);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_frag, q_frag[hp][kb], acc, 0, 0, 0);
          }
          f32x4_t a4;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int key = kv0 + kt * 16 + lg * 4 + r;
            float a = acc[r] * scale;
            if (dist_bias != nullptr) {
              const int dist = min(max(qpos - key, 0), n_dist - 1);
              a += dist_bias[(size_t)dist * H + h];
            }
            a4[r] = a;
          }
          *reinterpret_cast<f32x4_t*>(raw_w + kt * 16 + lg * 4) = a4;
        }
      }
    }
    __syncthreads();

    // ---- mix the heads' scores into registers -----------------------------------------
    float sc[HPW][8];
#pragma unroll
    for (int hp = 0; hp < HPW; ++hp)
#pragma unroll
      for (int i = 0; i < 8; ++i) sc[hp][i] = 0.f;
    for (int g2 = 0; g2 < H; ++g2) {
      const float* rr = raw_s + ((size_t)g2 * MT_ROWS + li) * MT_RS + lg * 4;
      const f32x4_t x0 = *reinterpret_cast<const f32x4_t*>(rr);
      const f32x4_t x1 = *reinterpret_cast<const f32x4_t*>(rr + 16);
#pragma unroll
      for (int hp = 0; hp < HPW; ++hp) {
        const int h = wave + hp * 16;
        const float tw = h < H ? talk_s[h * H + g2] : 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          sc[hp][r] += tw * x0[r];
          sc[hp][4 + r] += tw * x1[r];
        }
      }
    }
    __syncthreads();  // every wave has read the raw rows: they may hold P now

#pragma unroll
    for (int hp = 0; hp < HPW; ++hp) {
      const int h = wave + hp * 16;
      if (h < H) {  // uniform per wave
        // ---- mask, online softmax ---------------------------------------------------
        float rowmax = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int key = kv0 + kt * 16 + lg * 4 + r;
            if (!row_valid || key > qpos || key >= ctx || key < key_lo) sc[hp][kt * 4 + r] = -INFINITY;
            rowmax = fmaxf(rowmax, sc[hp][kt * 4 + r]);
          }
        }
        rowmax = stride_reduce_max<16, 4>(rowmax);
        const float m_new = fmaxf(m[hp], rowmax);
        float alpha;
        float psum = 0.0f;
        float p[8];
        if (m_new == -INFINITY) {
          alpha = 1.0f;
#pragma unroll
          for (int i = 0; i < 8; ++i) p[i] = 0.0f;
        } else {
          alpha = (m[hp] == -INFINITY) ? 0.0f : __expf(m[hp] - m_new);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            p[i] = (sc[hp][i] == -INFINITY) ? 0.0f : __expf(sc[hp][i] - m_new);
            psum += p[i];
          }
          m[hp] = m_new;
        }
        psum = stride_reduce_sum<16, 4>(psum);
        l[hp] = l[hp] * alpha + psum;
        float alpha_r[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) alpha_r[r] = __shfl(alpha, lg * 4 + r, 64);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#pragma unroll
          for (int r = 0; r < 4; ++r) acc_o[hp][db][r] *= alpha_r[r];
        }

        // ---- P: C layout -> A-fragment layout through this head's LDS rows ------------
        uint16_t* Pw = reinterpret_cast<uint16_t*>(raw_s + (size_t)h * MT_ROWS * MT_RS);
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            Pw[li * MT_KVBLK + kt * 16 + lg * 4 + r] = f32_to_bf16(p[kt * 4 + r]);
        }
        u16x8 praw = *reinterpret_cast<const u16x8*>(Pw + li * MT_KVBLK + lg * 8);
        bf16x8_t p_frag = *reinterpret_cast<bf16x8_t*>(&praw);

        // ---- O += P V -------------------------------------------------------------------
        const uint16_t* VTg = VTs + (size_t)(h / group) * DVP * MT_KVBLK;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          u16x8 vraw = *reinterpret_cast<const u16x8*>(VTg + (size_t)(db * 16 + li) * MT_KVBLK + lg * 8);
          bf16x8_t v_frag = *reinterpret_cast<bf16x8_t*>(&vraw);
          acc_o[hp][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_frag, v_frag, acc_o[hp][db], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }

  // ---- epilogue: normalise, store ------------------------------------------------------
#pragma unroll
  for (int hp = 0; hp < HPW; ++hp) {
    const int h = wave + hp * 16;
    if (h >= H) continue;
    float inv_l[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float lr = __shfl(l[hp], lg * 4 + r, 64);
      inv_l[r] = lr > 0.f ? 1.0f / lr : 0.0f;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int orow = qt + lg * 4 + r;
      if (orow >= n) continue;
      uint16_t* op = out + ((size_t)(lo + orow) * H + h) * Dv;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int d = db * 16 + li;
        if (d < Dv) op[d] = f32_to_bf16(acc_o[hp][db][r] * inv_l[r]);
      }
    }
  }
}

static size_t mt_smem_bytes(int H, int G, int dkp, int dvp) {
  return (size_t)G * MT_KVBLK * dkp * 2 + (size_t)G * dvp * MT_KVBLK * 2 +
         (size_t)H * MT_ROWS * MT_RS * 4 + (size_t)H * H * 4;
}

// Returns 0 when launched, 1 when the shape is not served (the caller then
// uses the any-shape kernel).
extern "C" int lig_paged_attention_mixed_heads_tiles(
    void* out, const void* q, long q_stride, const void* k_cache, const void* v_cache,
    const float* dist_bias, int n_dist, const float* talk, const int* tile_seq,
    const int* tile_qstart, const int* query_start_locs, const int* context_lens,
    const int* block_tables, float scale, int chunk, int ntiles, int H, int G, int D,
    int Dv, int block_size, int max_blocks, hipStream_t stream) {
  if (D % 8 != 0 || Dv % 8 != 0 || D > 128 || Dv > 128 || D <= 0 || Dv <= 0 ||
      q_stride % 8 != 0 || !aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) ||
      H < 1 || H > 32 || G < 1 || H % G != 0)
    return 1;
  const int dkp = D <= 32 ? 32 : (D <= 64 ? 64 : 128);
  const int dvp = Dv <= 32 ? 32 : (Dv <= 64 ? 64 : 128);
  const size_t smem = mt_smem_bytes(H, G, dkp, dvp);
  if (smem > 150 * 1024) return 1;
  if (ntiles <= 0) return 0;
  dim3 grid(ntiles * 4), block((H < 16 ? H : 16) * WAVE_SIZE);
#define LAUNCH_MT(DKP, DVP)                                                          \
  do {                                                                               \
    auto kern = H <= 16 ? paged_attention_mixed_heads_tiles_kernel<DKP, DVP, 1>      \
                        : paged_attention_mixed_heads_tiles_kernel<DKP, DVP, 2>;     \
    if (smem > 48 * 1024 &&                                                          \
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                     \
                            hipFuncAttributeMaxDynamicSharedMemorySize,              \
                            (int)smem) != hipSuccess)                                \
      return 1;                                                                      \
    hipLaunchKernelGGL(kern, grid, block, smem, stream, (uint16_t*)out,              \
                       (const uint16_t*)q, q_stride, (const uint16_t*)k_cache,       \
                       (const uint16_t*)v_cache, dist_bias, n_dist, talk, tile_seq,  \
                       tile_qstart, query_start_locs, context_lens, block_tables,    \
                       scale, chunk, H, G, D, Dv, block_size, max_blocks);           \
  } while (0)
  if (dkp == 32 && dvp == 32) LAUNCH_MT(32, 32);
  else if (dkp == 32 && dvp == 64) LAUNCH_MT(32, 64);
  else if (dkp == 32 && dvp == 128) LAUNCH_MT(32, 128);
  else if (dkp == 64 && dvp == 32) LAUNCH_MT(64, 32);
  else if (dkp == 64 && dvp == 64) LAUNCH_MT(64, 64);
  else if (dkp == 64 && dvp == 128) LAUNCH_MT(64, 128);
  else if (dkp == 128 && dvp == 32) LAUNCH_MT(128, 32);
  else if (dkp == 128 && dvp == 64) LAUNCH_MT(128, 64);
  else LAUNCH_MT(128, 128);
#undef LAUNCH_MT
  return 0;
}
