// Everything between an attention layer's fused input projection and its
// attention kernel, one workgroup per token row, gfx950.  fp32 arithmetic,
// bf16 or fp32 storage.
//
//   * q and k RMS norms: over the whole projection (weights of that size),
//     per head (one weight of size D shared by the heads), or none;
//   * rotation of the first 2*n_freq entries of every q and k head, angle =
//     float(pos) * f_i, accurate sincosf; rotate-half pairs entry i with
//     entry i + n_freq, the interleaved layout pairs entry 2i with 2i + 1;
//   * norm mode 3: q and k divided per head by their root mean square AFTER
//     the rotation, without a weight;
//   * values from their own columns or, v_from_key, the keys as projected
//     (before the norm); optionally divided per head by their root mean
//     square; optionally blended with another layer's values of the same
//     token, (1 - lam) v + lam v_first;
//   * keys and values stored into the paged caches at the row's slot, the
//     values optionally also exported in fp32; q written contiguously.
//
// Row layout of proj: [q (H*D) | k (G*D) | v (G*Dv)] (no v with v_from_key).

#include "elem_types.h"

// VEC: every block of the row (q, k, v) and every head is a multiple of 8
// entries and 16-byte aligned, so global loads and stores move 8 at a time.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void qkv_norm_rope_cache_kernel(
    T* __restrict__ q_out, float* __restrict__ v_out, const T* __restrict__ proj,
    long proj_stride, const T* __restrict__ w_q, const T* __restrict__ w_k,
    const float* __restrict__ inv_freq, int n_freq,
    const int64_t* __restrict__ positions, const float* __restrict__ v_first,
    float lam, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, float eps, int H, int G, int D,
    int Dv, int norm_mode, int v_from_key, int v_unit_norm, int BS,
    int rot_interleaved) {
  extern __shared__ __align__(16) float sm[];
  __shared__ float red[17];
  const int nq = H * D, nk = G * D, nv = G * Dv;
  float* q_s = sm;             // [nq]
  float* k_s = sm + nq;        // [nk]
  float* v_s = sm + nq + nk;   // [nv]
  const long r = blockIdx.x;
  const T* row = proj + r * proj_stride;
  const int tid = threadIdx.x, nt = blockDim.x;
  const int wave = tid / WAVE_SIZE, lane = tid % WAVE_SIZE, nwaves = nt / WAVE_SIZE;

  if (VEC) {
    // q_s, k_s, v_s are contiguous in LDS just as q | k | v are in the row
    const int n_in = nq + nk + (v_from_key ? 0 : nv);
    for (int c = tid * 8; c < n_in; c += nt * 8) {
      float t[8];
      ld8(row + c, t);
      st8(sm + c, t);
      if (v_from_key && c >= nq) st8(v_s + (c - nq), t);  // Dv == D
    }
  } else {
    for (int c = tid; c < nq; c += nt) q_s[c] = ld(row + c);
    for (int c = tid; c < nk; c += nt) {
      const float kv = ld(row + nq + c);
      k_s[c] = kv;
      if (v_from_key) v_s[c] = kv;  // Dv == D
    }
    if (!v_from_key)
      for (int c = tid; c < nv; c += nt) v_s[c] = ld(row + nq + nk + c);
  }
  __syncthreads();

  if (norm_mode == 1) {
    float sq = 0.f, sk = 0.f;
    for (int c = tid; c < nq; c += nt) sq += q_s[c] * q_s[c];
    for (int c = tid; c < nk; c += nt) sk += k_s[c] * k_s[c];
    sq = block_reduce_sum(sq, red);
    sk = block_reduce_sum(sk, red);
    const float iq = 1.0f / sqrtf(sq / (float)nq + eps);
    const float ik = 1.0f / sqrtf(sk / (float)nk + eps);
    for (int c = tid; c < nq; c += nt) q_s[c] = q_s[c] * iq * ld(w_q + c);
    for (int c = tid; c < nk; c += nt) k_s[c] = k_s[c] * ik * ld(w_k + c);
  } else if (norm_mode == 2) {
    for (int hh = wave; hh < H + G; hh += nwaves) {
      float* v = hh < H ? q_s + hh * D : k_s + (hh - H) * D;
      const T* w = hh < H ? w_q : w_k;
      float ss = 0.f;
      for (int d = lane; d < D; d += WAVE_SIZE) ss += v[d] * v[d];
      ss = wave_reduce_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)D + eps);
      for (int d = lane; d < D; d += WAVE_SIZE) v[d] = v[d] * inv * ld(w + d);
    }
  }
  // values: unit RMS per head, blend
  if (v_unit_norm || v_first != nullptr) {
    for (int g = wave; g < G; g += nwaves) {
      float* v = v_s + g * Dv;
      float inv = 1.f;
      if (v_unit_norm) {
        float ss = 0.f;
        for (int d = lane; d < Dv; d += WAVE_SIZE) ss += v[d] * v[d];
        ss = wave_reduce_sum(ss);
        inv = 1.0f / sqrtf(ss / (float)Dv + eps);
      }
      for (int d = lane; d < Dv; d += WAVE_SIZE) {
        float t = v[d] * inv;
        if (v_first != nullptr) t = (1.0f - lam) * t + lam * v_first[r * nv + g * Dv + d];
        v[d] = t;
      }
    }
  }
  __syncthreads();

  const int64_t pos = positions[r];
  if (n_freq > 0) {
    const float fp = (float)pos;
    for (int idx = tid; idx < (H + G) * n_freq; idx += nt) {
      const int hh = idx / n_freq, i = idx - hh * n_freq;
      float* v = hh < H ? q_s + hh * D : k_s + (hh - H) * D;
      float sn, cs;
      sincosf(fp * inv_freq[i], &sn, &cs);
      const int ia = rot_interleaved ? 2 * i : i;
      const int ib = rot_interleaved ? 2 * i + 1 : i + n_freq;
      const float a = v[ia], b = v[ib];
      v[ia] = a * cs - b * sn;
      v[ib] = b * cs + a * sn;
    }
    __syncthreads();
  }
  if (norm_mode == 3) {
    for (int hh = wave; hh < H + G; hh += nwaves) {
      float* v = hh < H ? q_s + hh * D : k_s + (hh - H) * D;
      float ss = 0.f;
      for (int d = lane; d < D; d += WAVE_SIZE) ss += v[d] * v[d];
      ss = wave_reduce_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)D + eps);
      for (int d = lane; d < D; d += WAVE_SIZE) v[d] *= inv;
    }
    __syncthreads();
  }

  if (VEC) {
    for (int c = tid * 8; c < nq; c += nt * 8) {
      float t[8];
      ld8(q_s + c, t);
      st8(q_out + r * nq + c, t);
    }
  } else {
    for (int c = tid; c < nq; c += nt) st(q_out + r * nq + c, q_s[c]);
  }
  if (v_out != nullptr)
    for (int c = tid; c < nv; c += nt) v_out[r * nv + c] = v_s[c];
  const int64_t slot = slot_mapping[r];
  if (slot < 0) return;
  const long blk = slot / BS;
  const int off = (int)(slot % BS);
  if (VEC) {
    for (int c = tid * 8; c < nk + nv; c += nt * 8) {
      float t[8];
      if (c < nk) {
        const int g = c / D, d = c - g * D;
        ld8(k_s + c, t);
        st8(k_cache + ((blk * G + g) * BS + off) * (long)D + d, t);
      } else {
        const int e = c - nk, g = e / Dv, d = e - g * Dv;
        ld8(v_s + e, t);
        st8(v_cache + ((blk * G + g) * BS + off) * (long)Dv + d, t);
      }
    }
    return;
  }
  for (int c = tid; c < nk; c += nt) {
    const int g = c / D, d = c - g * D;
    st(k_cache + ((blk * G + g) * BS + off) * (long)D + d, k_s[c]);
  }
  for (int c = tid; c < nv; c += nt) {
    const int g = c / Dv, d = c - g * Dv;
    st(v_cache + ((blk * G + g) * BS + off) * (long)Dv + d, v_s[c]);
  }
}

extern "C" void lig_qkv_norm_rope_cache(
    void* q_out, float* v_out, const void* proj, long proj_stride, const void* w_q,
    const void* w_k, const float* inv_freq, int n_freq, const int64_t* positions,
    const float* v_first, float lam, void* k_cache, void* v_cache,
    const int64_t* slot_mapping, float eps, int R, int H, int G, int D, int Dv,
    int norm_mode, int v_from_key, int v_unit_norm, int BS, int rot_interleaved,
    int is_f32, hipStream_t s) {
  if (R <= 0) return;
  const size_t smem = (size_t)(H * D + G * D + G * Dv) * sizeof(float);
  const bool vec = D % 8 == 0 && Dv % 8 == 0 && proj_stride % 8 == 0 && aligned16(proj) &&
                   aligned16(q_out) && aligned16(k_cache) && aligned16(v_cache);
#define LIG_QP(T, VEC)                                                              \
  hipLaunchKernelGGL((qkv_norm_rope_cache_kernel<T, VEC>), dim3(R), dim3(256), smem, \
                     s, (T*)q_out, v_out, (const T*)proj, proj_stride,              \
                     (const T*)w_q, (const T*)w_k, inv_freq, n_freq, positions,     \
                     v_first, lam, (T*)k_cache, (T*)v_cache, slot_mapping, eps, H,  \
                     G, D, Dv, norm_mode, v_from_key, v_unit_norm, BS, rot_interleaved)
  if (is_f32) {
    if (vec) LIG_QP(float, true); else LIG_QP(float, false);
  } else {
    if (vec) LIG_QP(bf16s, true); else LIG_QP(bf16s, false);
  }
#undef LIG_QP
}
