// Linear recurrences with a matrix state per head, gfx950: one [D, Dv] fp32
// matrix S per (sequence, head), scanned token by token in fp32.
//
//   bonus form (u, per-token per-channel decay):
//       o_t = (S + diag(u) k_t v_t^T)^T q_t
//       S  <- diag(w_t) S + k_t v_t^T,   w_t = exp(-exp(decay_pre_t))
//   constant-decay form (one d per head):
//       S  <- d S + k_t v_t^T
//       o_t = S^T q_t
//   optional silu on q, k, v as they are read.
//
// One workgroup per (segment, head).  A thread owns value column j and one
// quarter of the key channels (lane = 4 j + s, keys s*KPT .. s*KPT + KPT-1),
// keeps its KPT state entries in registers for the whole segment, and the
// four partial outputs of a column are summed with two lane shuffles.  The
// segment is walked serially, TT tokens staged into LDS at a time (q, k, the
// decay already exponentiated, v), so a prompt portion and a single decoded
// token take the same arithmetic path in the same order: results do not
// depend on how a sequence is cut into steps.
//
// The state row of a sequence is stored in the order the threads hold it,
// [head][ii][thread] with D padded to 4*KPT: loads and stores are coalesced.
// A segment that starts its sequence ignores what the slot held.

#include "elem_types.h"

#define MS_SPLIT 4

// EXACT: kpt == KMAX and a multiple of 4, so the per-token loop has constant
// bounds and reads q, k and the decay from LDS four entries at a time.
template <typename T, int KMAX, bool BONUS, bool EXACT>
__global__ void matrix_state_scan_kernel(
    float* __restrict__ out,  // [R, H*Dv]
    const T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride,
    const T* __restrict__ v, long v_stride,
    const float* __restrict__ decay_pre,   // [R, H*D]   (BONUS)
    const float* __restrict__ head_decay,  // [H]        (!BONUS)
    const float* __restrict__ bonus,       // [H*D]      (BONUS)
    float* __restrict__ state, long state_stride, const int* __restrict__ seg_start,
    const int* __restrict__ seg_len, const int* __restrict__ seg_slot,
    const int* __restrict__ seg_fresh, int H, int D, int Dv, int kpt, int TT,
    int act_silu) {
  extern __shared__ __align__(16) float sm[];
  const int Dp = MS_SPLIT * kpt;
  float* q_s = sm;                 // [TT][Dp]
  float* k_s = q_s + TT * Dp;      // [TT][Dp]
  float* w_s = k_s + TT * Dp;      // [TT][Dp] (BONUS only)
  float* v_s = BONUS ? w_s + TT * Dp : w_s;  // [TT][Dv]

  const int seg = blockIdx.x, h = blockIdx.y;
  const int n = seg_len[seg];
  if (n <= 0) return;
  const int r0 = seg_start[seg];
  const int tid = threadIdx.x, nt = blockDim.x;
  const int j = tid / MS_SPLIT, s = tid % MS_SPLIT;
  const bool owner = j < Dv;
  const int nthr = Dv * MS_SPLIT;  // threads that own state

  float S[KMAX], U[KMAX];
  float* srow = state + (long)seg_slot[seg] * state_stride + (long)h * kpt * nthr;
  const bool fresh = seg_fresh[seg] != 0;
#pragma unroll
  for (int ii = 0; ii < KMAX; ++ii) {
    S[ii] = 0.f;
    U[ii] = 0.f;
    if (ii < kpt && owner) {
      if (!fresh) S[ii] = srow[(long)ii * nthr + tid];
      const int i = s * kpt + ii;
      if (BONUS && i < D) U[ii] = bonus[h * D + i];
    }
  }
  const float dconst = BONUS ? 0.f : head_decay[h];

  for (int t0 = 0; t0 < n; t0 += TT) {
    const int nt_tok = min(TT, n - t0);
    __syncthreads();  // the previous tile's readers are done
    for (int e = tid; e < nt_tok * Dp; e += nt) {
      const int t = e / Dp, i = e - t * Dp;
      const long r = r0 + t0 + t;
      float qv = 0.f, kv = 0.f, wv = 0.f;
      if (i < D) {
        qv = ld(q + r * q_stride + h * D + i);
        kv = ld(k + r * k_stride + h * D + i);
        if (act_silu) {
          qv = qv * sigmoid_f32(qv);
          kv = kv * sigmoid_f32(kv);
        }
        if (BONUS) wv = expf(-expf(decay_pre[r * (long)(H * D) + h * D + i]));
      }
      q_s[e] = qv;
      k_s[e] = kv;
      if (BONUS) w_s[e] = wv;
    }
    for (int e = tid; e < nt_tok * Dv; e += nt) {
      const int t = e / Dv, c = e - t * Dv;
      float vv = ld(v + (long)(r0 + t0 + t) * v_stride + h * Dv + c);
      if (act_silu) vv = vv * sigmoid_f32(vv);
      v_s[e] = vv;
    }
    __syncthreads();
    if (tid < ((nthr + WAVE_SIZE - 1) / WAVE_SIZE) * WAVE_SIZE) {  // whole waves: shuffles below
      for (int t = 0; t < nt_tok; ++t) {
        const float vj = owner ? v_s[t * Dv + j] : 0.f;
        const float* qt = q_s + t * Dp + s * kpt;
        const float* kt = k_s + t * Dp + s * kpt;
        const float* wt = w_s + t * Dp + s * kpt;
        float o = 0.f;
        if (EXACT) {
#pragma unroll
          for (int i4 = 0; i4 < KMAX; i4 += 4) {
            const f32x4 k4 = *reinterpret_cast<const f32x4*>(kt + i4);
            const f32x4 q4 = *reinterpret_cast<const f32x4*>(qt + i4);
            f32x4 w4 = {0.f, 0.f, 0.f, 0.f};
            if (BONUS) w4 = *reinterpret_cast<const f32x4*>(wt + i4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int ii = i4 + e;
              const float kv = k4[e] * vj;
              if (BONUS) {
                o += q4[e] * (S[ii] + U[ii] * kv);
                S[ii] = w4[e] * S[ii] + kv;
              } else {
                S[ii] = dconst * S[ii] + kv;
                o += q4[e] * S[ii];
              }
            }
          }
        } else {
#pragma unroll
          for (int ii = 0; ii < KMAX; ++ii) {
            if (ii < kpt) {
              const float kv = kt[ii] * vj;
              if (BONUS) {
                o += qt[ii] * (S[ii] + U[ii] * kv);
                S[ii] = wt[ii] * S[ii] + kv;
              } else {
                S[ii] = dconst * S[ii] + kv;
                o += qt[ii] * S[ii];
              }
            }
          }
        }
        o += __shfl_xor(o, 1, WAVE_SIZE);
        o += __shfl_xor(o, 2, WAVE_SIZE);
        if (owner && s == 0) out[(long)(r0 + t0 + t) * (H * Dv) + h * Dv + j] = o;
      }
    }
  }
  if (owner) {
#pragma unroll
    for (int ii = 0; ii < KMAX; ++ii)
      if (ii < kpt) srow[(long)ii * nthr + tid] = S[ii];
  }
}

// Returns 0 when launched, 1 when a head is wider than the kernel holds.
extern "C" int lig_matrix_state_scan(
    float* out, const void* q, long q_stride, const void* k, long k_stride,
    const void* v, long v_stride, const float* decay_pre, const float* head_decay,
    const float* bonus, float* state, long state_stride, const int* seg_start,
    const int* seg_len, const int* seg_slot, const int* seg_fresh, int S, int H,
    int D, int Dv, int act_silu, int is_f32, hipStream_t stream) {
  if (D <= 0 || Dv <= 0 || D > 256 || Dv > 256) return 1;
  if (S <= 0) return 0;
  const int kpt = (D + MS_SPLIT - 1) / MS_SPLIT;
  const int Dp = kpt * MS_SPLIT;
  const bool has_bonus = bonus != nullptr;
  const int per_tok = (has_bonus ? 3 : 2) * Dp + Dv;
  const int TT = per_tok * 16 * 4 <= 48 * 1024 ? 16 : 8;
  const size_t smem = (size_t)per_tok * TT * sizeof(float);
  const int threads = ((Dv * MS_SPLIT + WAVE_SIZE - 1) / WAVE_SIZE) * WAVE_SIZE;
  dim3 grid(S, H), block(threads);
#define LIG_MS(T, KMAX, B, E)                                                   \
  hipLaunchKernelGGL((matrix_state_scan_kernel<T, KMAX, B, E>), grid, block,    \
                     smem, stream, out, (const T*)q, q_stride, (const T*)k,     \
                     k_stride, (const T*)v, v_stride, decay_pre, head_decay,    \
                     bonus, state, state_stride, seg_start, seg_len, seg_slot,  \
                     seg_fresh, H, D, Dv, kpt, TT, act_silu)
#define LIG_MS_K(T, B)                                    \
  do {                                                    \
    if (kpt == 8) LIG_MS(T, 8, B, true);                  \
    else if (kpt < 8) LIG_MS(T, 8, B, false);             \
    else if (kpt == 16) LIG_MS(T, 16, B, true);           \
    else if (kpt < 16) LIG_MS(T, 16, B, false);           \
    else if (kpt == 32) LIG_MS(T, 32, B, true);           \
    else if (kpt < 32) LIG_MS(T, 32, B, false);           \
    else if (kpt == 64) LIG_MS(T, 64, B, true);           \
    else LIG_MS(T, 64, B, false);                         \
  } while (0)
  if (is_f32) {
    if (has_bonus) LIG_MS_K(float, true); else LIG_MS_K(float, false);
  } else {
    if (has_bonus) LIG_MS_K(bf16s, true); else LIG_MS_K(bf16s, false);
  }
#undef LIG_MS_K
#undef LIG_MS
  return 0;
}
