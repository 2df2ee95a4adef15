// Paged causal attention for any head sizes, bf16 or fp32 storage, fp32
// scores and softmax, gfx950.
//
// Serves the shapes the MFMA kernels do not: key size != value size, sizes
// that are not 64/128, fp32 caches.  One wave per (token, query head part) walks
// the sequence's pages 64 keys at a time: lane j scores key j against the
// query held in LDS, the wave keeps a running max / sum (online softmax),
// then the lanes switch to value columns and accumulate sum_j p_j V[j, :].
// Prompt portions and single decoded tokens go through the same walk: a
// token at position p sees keys 0..p of its own sequence, whatever else is
// in the flat batch.
//
// Optional per-position query temperature
//   tau(p) = 1 + coef * ln(floor((p + 1) / every) + 1)
// multiplies the score (same as scaling q), and an optional output gate
// multiplies the result element-wise by sigmoid(gate) before it is stored.
//
// An optional per-head sink adds exp(sink_h) to the softmax denominator: a
// key with that (unscaled) score and no value, counted once per row.  The
// running max starts at the sink and the running sum at one.
//
// chunk > 0 restricts a query at position p to the keys of its own chunk,
// floor(j / chunk) == floor(p / chunk), chunks counted from position 0 of the
// sequence.
//
// window > 0 restricts a query at position p to keys j with p - j < window
// (itself and the window - 1 tokens before it).
//
// sigmoid_weights: instead of a softmax every visible key weighs
// sigmoid(score + score_bias[h]) (score_bias nullable, fp32 per head); the
// weights are not normalised over the keys.  gate_per_head: the output gate
// holds ONE entry per (token, head) instead of one per output element.
//
// Cache layout: K [blocks, G, BS, D], V [blocks, G, BS, v_row] of which the
// first Dv entries of a row are the value (v_row == Dv for a cache of its
// own; a latent cache passes the key rows themselves, v_row == D).

#include "elem_types.h"

#define ATT_MAX_DV_PER_LANE 8  // Dv <= 512

// A wave serves HB query heads of one key/value head at once (HB divides the
// group size): a key row is loaded once and multiplied with HB queries held in
// LDS, a value element once and weighted HB times, so grouped-query layers
// read their cache rows once per group part instead of once per head.
//
// NW waves of a workgroup share one (token, head part): wave w takes the
// 64-key tiles w, w + NW, ... of the walk and keeps its own running max / sum
// / accumulator; wave 0 merges them through LDS at the end.  Small batches of
// single tokens, which would otherwise leave most of the chip idle behind one
// serial walk per wave, run with NW = 4.  Every wave makes the same number of
// loop trips (a trip without a tile only meets the barriers).
template <typename T, bool VEC, int NW, int HB>
__global__ __launch_bounds__(WAVE_SIZE * NW) void paged_attention_general_kernel(
    T* __restrict__ out,  // [R, H * Dv]
    const T* __restrict__ q, long q_stride,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ tok_seq,        // [R], -1 = padding row
    const int64_t* __restrict__ positions,  // [R]
    const T* __restrict__ gate, long gate_stride, const float* __restrict__ sink,
    float scale, float temp_coef, float temp_every, int temp_every_int, int H,
    int G, int D, int Dv, int v_row, int BS, int chunk, int window,
    const float* __restrict__ score_bias, int sigmoid_weights, int gate_per_head) {
  extern __shared__ __align__(16) float smem[];
  const int Dpad = (D + 1) & ~1;
  float* q_s = smem;                                   // [HB][Dpad]
  float* p_all = smem + HB * Dpad;                     // [NW][HB][64]
  long* voff_all = reinterpret_cast<long*>(p_all + NW * HB * WAVE_SIZE);  // [NW][64]
  float* ml_s = reinterpret_cast<float*>(voff_all + NW * WAVE_SIZE);      // [NW][HB][2]
  float* acc_s = ml_s + 2 * NW * HB;                   // [NW][HB][Dv]

  const int r = blockIdx.x, h0 = blockIdx.y * HB;
  const int lane = threadIdx.x % WAVE_SIZE, wave = threadIdx.x / WAVE_SIZE;
  float* p_s = p_all + wave * HB * WAVE_SIZE;
  long* voff_s = voff_all + wave * WAVE_SIZE;
  const int seq = tok_seq[r];
  T* orow = out + (size_t)r * H * Dv + (size_t)h0 * Dv;  // HB heads side by side
  if (seq < 0) {
    for (int d = threadIdx.x; d < HB * Dv; d += WAVE_SIZE * NW) st(orow + d, 0.f);
    return;
  }
  const long pos = positions[r];
  const int ctx = (int)pos + 1;
  const int g = h0 / (H / G);
  const int* bt = block_tables + (size_t)seq * max_blocks;

  float tau = 1.f;
  if (temp_coef != 0.f) {
    const float n = temp_every_int > 0
                        ? (float)((pos + 1) / temp_every_int)
                        : floorf((float)(pos + 1) / temp_every);
    tau = 1.f + temp_coef * logf(n + 1.f);
  }
  const float sc = scale * tau;

  const T* qrow = q + (size_t)r * q_stride + (size_t)h0 * D;
  for (int idx = threadIdx.x; idx < HB * D; idx += WAVE_SIZE * NW) {
    const int hh = idx / D;
    q_s[hh * Dpad + (idx - hh * D)] = ld(qrow + idx);
  }
  __syncthreads();

  float m[HB], l[HB], sb[HB];
  float acc[HB][ATT_MAX_DV_PER_LANE];
#pragma unroll
  for (int hh = 0; hh < HB; ++hh) {
    m[hh] = -INFINITY;
    l[hh] = 0.f;
    if (sink != nullptr && wave == 0) {  // the sink is counted once
      m[hh] = sink[h0 + hh];
      l[hh] = 1.f;
    }
    sb[hh] = score_bias != nullptr ? score_bias[h0 + hh] : 0.f;
#pragma unroll
    for (int i = 0; i < ATT_MAX_DV_PER_LANE; ++i) acc[hh][i] = 0.f;
  }

  // chunked visibility: the walk starts at the first key of the query's chunk
  int first_key = chunk > 0 ? (int)(pos / chunk) * chunk : 0;
  if (window > 0) first_key = max(first_key, (int)pos - window + 1);
  const int ntiles = (ctx - first_key + WAVE_SIZE - 1) / WAVE_SIZE;
  const int trips = (ntiles + NW - 1) / NW;
  for (int it = 0; it < trips; ++it) {
    const int tile = it * NW + wave;
    const bool active = tile < ntiles;  // uniform over the wave
    const int j0 = first_key + tile * WAVE_SIZE;
    const int j = j0 + lane;
    const bool valid = active && j < ctx;
    float dot[HB];
#pragma unroll
    for (int hh = 0; hh < HB; ++hh) dot[hh] = 0.f;
    long voff = 0;
    if (valid) {
      const long blk = bt[j / BS];
      const int off = j % BS;
      const T* krow = k_cache + ((blk * G + g) * BS + off) * (long)D;
      voff = ((blk * G + g) * BS + off) * (long)v_row;
      if (VEC) {  // D % 8 == 0 and 16-byte aligned rows: whole 8-element vectors
        for (int d = 0; d < D; d += 8) {
          float kv[8];
          ld8(krow + d, kv);
#pragma unroll
          for (int hh = 0; hh < HB; ++hh) {
#pragma unroll
            for (int i = 0; i < 8; ++i) dot[hh] += q_s[hh * Dpad + d + i] * kv[i];
          }
        }
      } else {
        for (int d = 0; d < D; ++d) {
          const float kv = ld(krow + d);
#pragma unroll
          for (int hh = 0; hh < HB; ++hh) dot[hh] += q_s[hh * Dpad + d] * kv;
        }
      }
    }
    float p[HB], alpha[HB];
#pragma unroll
    for (int hh = 0; hh < HB; ++hh) {
      p[hh] = 0.f;
      alpha[hh] = 1.f;
      if (active) {
        const float score = valid ? dot[hh] * sc : -INFINITY;
        if (sigmoid_weights) {
          p[hh] = valid ? sigmoid_f32(score + sb[hh]) : 0.f;
        } else {
          const float m_new = fmaxf(m[hh], wave_reduce_max(score));  // finite: key j0 is valid
          p[hh] = valid ? expf(score - m_new) : 0.f;
          alpha[hh] = expf(m[hh] - m_new);                           // 0 on the wave's first tile
          l[hh] = l[hh] * alpha[hh] + wave_reduce_sum(p[hh]);
          m[hh] = m_new;
        }
      }
    }
    __syncthreads();  // previous tile's readers are done
#pragma unroll
    for (int hh = 0; hh < HB; ++hh) p_s[hh * WAVE_SIZE + lane] = p[hh];
    voff_s[lane] = voff;
    __syncthreads();
    if (active) {
      const int nv = min(WAVE_SIZE, ctx - j0);
#pragma unroll
      for (int i = 0; i < ATT_MAX_DV_PER_LANE; ++i) {
        const int d = lane + i * WAVE_SIZE;
        if (d < Dv) {
          float a[HB];
#pragma unroll
          for (int hh = 0; hh < HB; ++hh) a[hh] = acc[hh][i] * alpha[hh];
          for (int jj = 0; jj < nv; ++jj) {
            const float v = ld(v_cache + voff_s[jj] + d);
#pragma unroll
            for (int hh = 0; hh < HB; ++hh) a[hh] += p_s[hh * WAVE_SIZE + jj] * v;
          }
#pragma unroll
          for (int hh = 0; hh < HB; ++hh) acc[hh][i] = a[hh];
        }
      }
    }
  }
  if (NW > 1) {
    // wave 0 gathers the other waves' partial results
#pragma unroll
    for (int hh = 0; hh < HB; ++hh) {
      if (lane == 0) {
        ml_s[2 * (wave * HB + hh)] = m[hh];
        ml_s[2 * (wave * HB + hh) + 1] = l[hh];
      }
#pragma unroll
      for (int i = 0; i < ATT_MAX_DV_PER_LANE; ++i) {
        const int d = lane + i * WAVE_SIZE;
        if (d < Dv) acc_s[(wave * HB + hh) * Dv + d] = acc[hh][i];
      }
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int hh = 0; hh < HB; ++hh) {
      if (sigmoid_weights) {
#pragma unroll
        for (int i = 0; i < ATT_MAX_DV_PER_LANE; ++i) {
          const int d = lane + i * WAVE_SIZE;
          if (d < Dv)
            for (int w = 1; w < NW; ++w) acc[hh][i] += acc_s[(w * HB + hh) * Dv + d];
        }
      } else {
        float M = m[hh];  // finite: wave 0 always has the walk's first key
        for (int w = 1; w < NW; ++w) M = fmaxf(M, ml_s[2 * (w * HB + hh)]);
        const float f0 = expf(m[hh] - M);
        l[hh] *= f0;
#pragma unroll
        for (int i = 0; i < ATT_MAX_DV_PER_LANE; ++i) acc[hh][i] *= f0;
        for (int w = 1; w < NW; ++w) {
          const float fw = expf(ml_s[2 * (w * HB + hh)] - M);  // 0 for a wave without tiles
          l[hh] += ml_s[2 * (w * HB + hh) + 1] * fw;
#pragma unroll
          for (int i = 0; i < ATT_MAX_DV_PER_LANE; ++i) {
            const int d = lane + i * WAVE_SIZE;
            if (d < Dv) acc[hh][i] += acc_s[(w * HB + hh) * Dv + d] * fw;
          }
        }
      }
    }
  }
#pragma unroll
  for (int hh = 0; hh < HB; ++hh) {
    const int h = h0 + hh;
    const float inv_l = sigmoid_weights ? 1.f : 1.f / l[hh];
    float head_gate = 1.f;
    if (gate != nullptr && gate_per_head)
      head_gate = sigmoid_f32(ld(gate + (size_t)r * gate_stride + h));
#pragma unroll
    for (int i = 0; i < ATT_MAX_DV_PER_LANE; ++i) {
      const int d = lane + i * WAVE_SIZE;
      if (d < Dv) {
        float o = acc[hh][i] * inv_l;
        if (gate_per_head)
          o *= head_gate;
        else if (gate != nullptr)
          o *= sigmoid_f32(ld(gate + (size_t)r * gate_stride + (size_t)h * Dv + d));
        st(orow + (size_t)hh * Dv + d, o);
      }
    }
  }
}

// Scatter this step's K and V rows (column blocks of a fused projection
// output, row stride `src_stride`) into the paged caches.
template <typename T>
__global__ void kv_scatter_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                  long src_stride, T* __restrict__ k_cache,
                                  T* __restrict__ v_cache,
                                  const int64_t* __restrict__ slot_mapping,
                                  int R, int G, int D, int Dv, int BS) {
  const int per_row = G * (D + Dv);
  const long total = (long)R * per_row;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += gridDim.x * (long)blockDim.x) {
    const long t = idx / per_row;
    const int e = (int)(idx - t * per_row);
    const int64_t slot = slot_mapping[t];
    if (slot < 0) continue;
    const long blk = slot / BS;
    const int off = (int)(slot % BS);
    if (e < G * D) {
      const int g = e / D, d = e % D;
      k_cache[((blk * G + g) * BS + off) * (long)D + d] = k[t * src_stride + e];
    } else {
      const int e2 = e - G * D;
      const int g = e2 / Dv, d = e2 % Dv;
      v_cache[((blk * G + g) * BS + off) * (long)Dv + d] = v[t * src_stride + e2];
    }
  }
}

// 16-byte chunks: every head row (D and Dv multiples of 8) is moved as whole
// 8-element vectors, one thread per chunk.
template <typename T>
__global__ void kv_scatter_vec_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                      long src_stride, T* __restrict__ k_cache,
                                      T* __restrict__ v_cache,
                                      const int64_t* __restrict__ slot_mapping,
                                      int R, int G, int D, int Dv, int BS) {
  const int kc = G * D / 8, per_row = G * (D + Dv) / 8;
  const long total = (long)R * per_row;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += gridDim.x * (long)blockDim.x) {
    const long t = idx / per_row;
    const int c = (int)(idx - t * per_row);
    const int64_t slot = slot_mapping[t];
    if (slot < 0) continue;
    const long blk = slot / BS;
    const int off = (int)(slot % BS);
    float tmp[8];
    if (c < kc) {
      const int e = c * 8, g = e / D, d = e % D;
      ld8(k + t * src_stride + e, tmp);
      st8(k_cache + ((blk * G + g) * BS + off) * (long)D + d, tmp);
    } else {
      const int e = (c - kc) * 8, g = e / Dv, d = e % Dv;
      ld8(v + t * src_stride + e, tmp);
      st8(v_cache + ((blk * G + g) * BS + off) * (long)Dv + d, tmp);
    }
  }
}

template <typename T>
__global__ void temperature_scale_rows_vec_kernel(T* __restrict__ out,
                                                  const T* __restrict__ q, long q_stride,
                                                  const int64_t* __restrict__ positions,
                                                  float temp_coef, float temp_every,
                                                  int temp_every_int, int C8, long n8) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n8;
       i += gridDim.x * (long)blockDim.x) {
    const long r = i / C8;
    const int c = (int)(i - r * C8) * 8;
    float tau = 1.f;
    if (temp_coef != 0.f) {
      const long pos = positions[r];
      const float m = temp_every_int > 0
                          ? (float)((pos + 1) / temp_every_int)
                          : floorf((float)(pos + 1) / temp_every);
      tau = 1.f + temp_coef * logf(m + 1.f);
    }
    float v[8];
    ld8(q + r * q_stride + c, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] *= tau;
    st8(out + i * 8, v);
  }
}

// q_out[r, :] = q[r, :] * tau(position r): the query temperature applied
// ahead of an attention kernel that takes one scalar scale.  Also packs the
// strided q view (a column block of the fused projection) contiguously.
template <typename T>
__global__ void temperature_scale_rows_kernel(T* __restrict__ out,  // [R, C]
                                              const T* __restrict__ q, long q_stride,
                                              const int64_t* __restrict__ positions,
                                              float temp_coef, float temp_every,
                                              int temp_every_int, int C, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += gridDim.x * (long)blockDim.x) {
    const long r = i / C;
    const int c = (int)(i - r * C);
    float tau = 1.f;
    if (temp_coef != 0.f) {
      const long pos = positions[r];
      const float m = temp_every_int > 0
                          ? (float)((pos + 1) / temp_every_int)
                          : floorf((float)(pos + 1) / temp_every);
      tau = 1.f + temp_coef * logf(m + 1.f);
    }
    st(out + i, ld(q + r * q_stride + c) * tau);
  }
}

extern "C" {

void lig_temperature_scale_rows(void* out, const void* q, long q_stride,
                                const int64_t* positions, float temp_coef,
                                float temp_every, int temp_every_int, int R,
                                int C, int is_f32, hipStream_t s) {
  const long n = (long)R * C;
  if (n <= 0) return;
  if (C % 8 == 0 && q_stride % 8 == 0 && aligned16(out) && aligned16(q)) {
    const long n8 = n / 8;
    long g8 = (n8 + 255) / 256;
    const int grid8 = (int)(g8 > 65535 ? 65535 : g8);
    if (is_f32)
      hipLaunchKernelGGL(temperature_scale_rows_vec_kernel<float>, dim3(grid8),
                         dim3(256), 0, s, (float*)out, (const float*)q,
                         q_stride, positions, temp_coef, temp_every,
                         temp_every_int, C / 8, n8);
    else
      hipLaunchKernelGGL(temperature_scale_rows_vec_kernel<bf16s>, dim3(grid8),
                         dim3(256), 0, s, (bf16s*)out, (const bf16s*)q,
                         q_stride, positions, temp_coef, temp_every,
                         temp_every_int, C / 8, n8);
    return;
  }
  long gl = (n + 255) / 256;
  const int grid = (int)(gl > 65535 ? 65535 : gl);
  if (is_f32)
    hipLaunchKernelGGL(temperature_scale_rows_kernel<float>, dim3(grid),
                       dim3(256), 0, s, (float*)out, (const float*)q, q_stride,
                       positions, temp_coef, temp_every, temp_every_int, C, n);
  else
    hipLaunchKernelGGL(temperature_scale_rows_kernel<bf16s>, dim3(grid),
                       dim3(256), 0, s, (bf16s*)out, (const bf16s*)q, q_stride,
                       positions, temp_coef, temp_every, temp_every_int, C, n);
}

void lig_paged_attention_general(
    void* out, const void* q, long q_stride, const void* k_cache,
    const void* v_cache, const int* block_tables, int max_blocks,
    const int* tok_seq, const int64_t* positions, const void* gate,
    long gate_stride, const float* sink, float scale, float temp_coef,
    float temp_every, int temp_every_int, int R, int H, int G, int D, int Dv,
    int v_row, int BS, int chunk, int window, const float* score_bias,
    int sigmoid_weights, int gate_per_head, int is_f32, hipStream_t s) {
  if (R <= 0) return;
  // heads of one key/value head that a wave serves together: as many as
  // divide the group, but fewer while that would leave the chip short of
  // waves (a small batch of single tokens wants parallel walks first)
  const int gs = H / G;
  int hb = gs % 4 == 0 ? 4 : (gs % 2 == 0 ? 2 : 1);
  while (hb > 1 && (long)R * (H / hb) * 4 < 2048) hb /= 2;
  // few workgroups: four waves share each of them and split the walk
  const int nw = (long)R * (H / hb) <= 2048 ? 4 : 1;
  dim3 grid(R, H / hb), block(WAVE_SIZE * nw);
  const size_t smem = (size_t)(hb * ((D + 1) & ~1) + nw * hb * WAVE_SIZE) * sizeof(float) +
                      (size_t)nw * WAVE_SIZE * sizeof(long) +
                      (size_t)nw * hb * (2 + Dv) * sizeof(float);
  const bool vec = D % 8 == 0 && aligned16(k_cache);
#define LIG_LAUNCH_ATT(T, VEC, NW, HB)                                          \
  hipLaunchKernelGGL((paged_attention_general_kernel<T, VEC, NW, HB>), grid,    \
                     block, smem, s, (T*)out, (const T*)q, q_stride,            \
                     (const T*)k_cache, (const T*)v_cache, block_tables,        \
                     max_blocks, tok_seq, positions, (const T*)gate,            \
                     gate_stride, sink, scale, temp_coef, temp_every,           \
                     temp_every_int, H, G, D, Dv, v_row, BS, chunk, window,      \
                     score_bias, sigmoid_weights, gate_per_head)
#define LIG_LAUNCH_ATT_H(T, VEC, NW)                    \
  if (hb == 4) LIG_LAUNCH_ATT(T, VEC, NW, 4);           \
  else if (hb == 2) LIG_LAUNCH_ATT(T, VEC, NW, 2);      \
  else LIG_LAUNCH_ATT(T, VEC, NW, 1)
#define LIG_LAUNCH_ATT_W(T, VEC) \
  if (nw == 4) { LIG_LAUNCH_ATT_H(T, VEC, 4); } else { LIG_LAUNCH_ATT_H(T, VEC, 1); }
  if (is_f32) {
    if (vec) { LIG_LAUNCH_ATT_W(float, true) } else { LIG_LAUNCH_ATT_W(float, false) }
  } else {
    if (vec) { LIG_LAUNCH_ATT_W(bf16s, true) } else { LIG_LAUNCH_ATT_W(bf16s, false) }
  }
#undef LIG_LAUNCH_ATT_H
#undef LIG_LAUNCH_ATT_W
#undef LIG_LAUNCH_ATT
}

void lig_kv_scatter(const void* k, const void* v, long src_stride,
                    void* k_cache, void* v_cache, const int64_t* slot_mapping,
                    int R, int G, int D, int Dv, int BS, int is_f32,
                    hipStream_t s) {
  const long total = (long)R * G * (D + Dv);
  if (total <= 0) return;
  if (D % 8 == 0 && Dv % 8 == 0 && src_stride % 8 == 0 && aligned16(k) &&
      aligned16(v) && aligned16(k_cache) && aligned16(v_cache)) {
    long g8 = (total / 8 + 255) / 256;
    const int grid8 = (int)(g8 > 65535 ? 65535 : g8);
    if (is_f32)
      hipLaunchKernelGGL(kv_scatter_vec_kernel<float>, dim3(grid8), dim3(256),
                         0, s, (const float*)k, (const float*)v, src_stride,
                         (float*)k_cache, (float*)v_cache, slot_mapping, R, G,
                         D, Dv, BS);
    else
      hipLaunchKernelGGL(kv_scatter_vec_kernel<bf16s>, dim3(grid8), dim3(256),
                         0, s, (const bf16s*)k, (const bf16s*)v, src_stride,
                         (bf16s*)k_cache, (bf16s*)v_cache, slot_mapping, R, G,
                         D, Dv, BS);
    return;
  }
  long gl = (total + 255) / 256;
  const int grid = (int)(gl > 65535 ? 65535 : gl);
  if (is_f32)
    hipLaunchKernelGGL(kv_scatter_kernel<float>, dim3(grid), dim3(256), 0, s,
                       (const float*)k, (const float*)v, src_stride,
                       (float*)k_cache, (float*)v_cache, slot_mapping, R, G, D,
                       Dv, BS);
  else
    hipLaunchKernelGGL(kv_scatter_kernel<bf16s>, dim3(grid), dim3(256), 0, s,
                       (const bf16s*)k, (const bf16s*)v, src_stride,
                       (bf16s*)k_cache, (bf16s*)v_cache, slot_mapping, R, G, D,
                       Dv, BS);
}

}  // extern "C"
