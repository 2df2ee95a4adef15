// Paged causal attention whose heads are coupled before the softmax, gfx950:
// any head sizes, bf16 or fp32 storage, fp32 scores and softmax.
//
// For a query at position p and a visible key j (j <= p, and in p's chunk
// when chunk > 0):
//     a_g = (q_g . k_j) * scale + dist_bias[min(p - j, N - 1)][g]   per head g
//     s_h = sum_g talk[h][g] * a_g                                  (heads mixed)
//     weights = softmax over the visible keys of s_h, per head h
// so one head's weights need every head's raw score of the same key.  One
// workgroup per token holds all heads: wave w serves heads w, w + NW, ...; for
// a tile of 64 keys every wave writes its heads' raw scores (lane = key) to
// LDS, after a barrier mixes them for its own heads, keeps a running max and
// sum per head (online softmax), then its lanes switch to value columns and
// accumulate sum_j p_j V[j, :].  Prompt rows and single decoded tokens take
// the same path.  dist_bias and talk are optional (nullptr: no bias / heads
// independent).
//
// Cache layout: K [blocks, G, BS, D], V [blocks, G, BS, Dv].

#include "elem_types.h"

#define MH_MAX_HPW 4     // heads per wave: H <= 16 * 4
#define MH_MAX_DVL 4     // value columns per lane: Dv <= 256

template <typename T, bool VEC>
__global__ void paged_attention_mixed_heads_kernel(
    T* __restrict__ out, const T* __restrict__ q, long q_stride,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ tok_seq, const int64_t* __restrict__ positions,
    const float* __restrict__ dist_bias, int n_dist, const float* __restrict__ talk,
    float scale, int chunk, int H, int G, int D, int Dv, int BS) {
  extern __shared__ __align__(16) float sm[];
  float* q_s = sm;                       // [H*D]
  float* raw_s = q_s + H * D;            // [H][64]
  float* p_s = raw_s + H * WAVE_SIZE;    // [H][64]
  float* talk_s = p_s + H * WAVE_SIZE;   // [H*H]
  long* base_s = reinterpret_cast<long*>(talk_s + ((H * H + 1) & ~1));  // [64]

  const int r = blockIdx.x;
  const int tid = threadIdx.x, nt = blockDim.x;
  const int wave = tid / WAVE_SIZE, lane = tid % WAVE_SIZE, nw = nt / WAVE_SIZE;
  const int seq = tok_seq[r];
  T* orow = out + (size_t)r * H * Dv;
  if (seq < 0) {
    for (int c = tid; c < H * Dv; c += nt) st(orow + c, 0.f);
    return;
  }
  const int pos = (int)positions[r];
  const int ctx = pos + 1;
  const int first_key = chunk > 0 ? (pos / chunk) * chunk : 0;
  const int* bt = block_tables + (size_t)seq * max_blocks;
  const int group = H / G;

  const T* qrow = q + (size_t)r * q_stride;
  for (int c = tid; c < H * D; c += nt) q_s[c] = ld(qrow + c);
  for (int c = tid; c < H * H; c += nt)
    talk_s[c] = talk != nullptr ? talk[c] : ((c / H) == (c % H) ? 1.f : 0.f);

  float m[MH_MAX_HPW], l[MH_MAX_HPW], acc[MH_MAX_HPW][MH_MAX_DVL];
#pragma unroll
  for (int t = 0; t < MH_MAX_HPW; ++t) {
    m[t] = -INFINITY;
    l[t] = 0.f;
#pragma unroll
    for (int i = 0; i < MH_MAX_DVL; ++i) acc[t][i] = 0.f;
  }

  for (int j0 = first_key; j0 < ctx; j0 += WAVE_SIZE) {
    const int j = j0 + lane;
    const bool valid = j < ctx;
    __syncthreads();  // q_s / talk_s ready; the previous tile's readers are done
    long kbase = 0;   // row index of (block, kv head 0, offset)
    if (valid) kbase = ((long)bt[j / BS] * G) * BS + (j % BS);
    if (wave == 0) base_s[lane] = kbase;
    // raw scores of this wave's heads, lane = key
#pragma unroll
    for (int t = 0; t < MH_MAX_HPW; ++t) {
      const int h = wave + t * nw;
      if (h < H) {
        float a = 0.f;
        if (valid) {
          const int g = h / group;
          const T* krow = k_cache + (kbase + (long)g * BS) * D;
          const float* qh = q_s + h * D;
          float dot = 0.f;
          if (VEC) {  // D % 8 == 0 and 16-byte aligned rows
            for (int d = 0; d < D; d += 8) {
              float kv[8];
              ld8(krow + d, kv);
#pragma unroll
              for (int i = 0; i < 8; ++i) dot += qh[d + i] * kv[i];
            }
          } else {
            for (int d = 0; d < D; ++d) dot += qh[d] * ld(krow + d);
          }
          a = dot * scale;
          if (dist_bias != nullptr) a += dist_bias[(long)min(pos - j, n_dist - 1) * H + h];
        }
        raw_s[h * WAVE_SIZE + lane] = a;
      }
    }
    __syncthreads();
    const int nv = min(WAVE_SIZE, ctx - j0);
#pragma unroll
    for (int t = 0; t < MH_MAX_HPW; ++t) {
      const int h = wave + t * nw;
      if (h < H) {  // uniform per wave
        float sc = -INFINITY;
        if (valid) {
          sc = 0.f;
          for (int g = 0; g < H; ++g) sc += talk_s[h * H + g] * raw_s[g * WAVE_SIZE + lane];
        }
        const float m_new = fmaxf(m[t], wave_reduce_max(sc));  // finite: key j0 is valid
        const float p = valid ? expf(sc - m_new) : 0.f;
        const float alpha = expf(m[t] - m_new);  // 0 on the first tile
        l[t] = l[t] * alpha + wave_reduce_sum(p);
        m[t] = m_new;
        p_s[h * WAVE_SIZE + lane] = p;  // read back by this wave only
        __builtin_amdgcn_wave_barrier();
        const int g = h / group;
#pragma unroll
        for (int i = 0; i < MH_MAX_DVL; ++i) {
          const int d = lane + i * WAVE_SIZE;
          if (d < Dv) {
            float a = acc[t][i] * alpha;
            for (int jj = 0; jj < nv; ++jj)
              a += p_s[h * WAVE_SIZE + jj] * ld(v_cache + (base_s[jj] + (long)g * BS) * Dv + d);
            acc[t][i] = a;
          }
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < MH_MAX_HPW; ++t) {
    const int h = wave + t * nw;
    if (h < H) {
      const float inv_l = 1.f / l[t];
#pragma unroll
      for (int i = 0; i < MH_MAX_DVL; ++i) {
        const int d = lane + i * WAVE_SIZE;
        if (d < Dv) st(orow + (size_t)h * Dv + d, acc[t][i] * inv_l);
      }
    }
  }
}

// Returns 0 when launched, 1 when the shape is not served.
extern "C" int lig_paged_attention_mixed_heads(
    void* out, const void* q, long q_stride, const void* k_cache, const void* v_cache,
    const int* block_tables, int max_blocks, const int* tok_seq,
    const int64_t* positions, const float* dist_bias, int n_dist, const float* talk,
    float scale, int chunk, int R, int H, int G, int D, int Dv, int BS, int is_f32,
    hipStream_t s) {
  if (H > 16 * MH_MAX_HPW || Dv > WAVE_SIZE * MH_MAX_DVL || H % G != 0) return 1;
  if (R <= 0) return 0;
  const int nw = H < 16 ? H : 16;
  const size_t smem =
      (size_t)(H * D + 2 * H * WAVE_SIZE + ((H * H + 1) & ~1)) * sizeof(float) +
      WAVE_SIZE * sizeof(long);
  if (smem > 64 * 1024) return 1;
  const bool vec = D % 8 == 0 && aligned16(k_cache);
#define LIG_MH(T, VEC)                                                              \
  hipLaunchKernelGGL((paged_attention_mixed_heads_kernel<T, VEC>), dim3(R),         \
                     dim3(nw * WAVE_SIZE), smem, s, (T*)out, (const T*)q, q_stride, \
                     (const T*)k_cache, (const T*)v_cache, block_tables,            \
                     max_blocks, tok_seq, positions, dist_bias, n_dist, talk,       \
                     scale, chunk, H, G, D, Dv, BS)
  if (is_f32) {
    if (vec) LIG_MH(float, true); else LIG_MH(float, false);
  } else {
    if (vec) LIG_MH(bf16s, true); else LIG_MH(bf16s, false);
  }
#undef LIG_MH
  return 0;
}
