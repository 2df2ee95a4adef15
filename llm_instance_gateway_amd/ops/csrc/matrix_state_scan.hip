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
// SPLIT-th of the key channels (lane = SPLIT j + s, keys s*KPT .. s*KPT +
// KPT-1, KPT one of a few size classes; SPLIT is 8 for heads of 32 or more
// key channels when 8 Dv threads fit a workgroup, else 4), keeps its KPT
// state entries in registers for the whole segment, and the partial outputs
// of a column are summed with lane shuffles.  The
// segment is walked serially, TT (8 to 32) tokens staged into LDS at a time (q, k, the
// decay already exponentiated, v), so a prompt portion and a single decoded
// token take the same arithmetic path in the same order: results do not
// depend on how a sequence is cut into steps.
//
// The state row of a sequence is stored in the order the threads hold it,
// [head][ii][thread] with D padded to SPLIT*KPT: loads and stores are
// coalesced (a row holds H * SPLIT * KPT * Dv entries; ops.matrix_state_width
// mirrors this).
// A segment that starts its sequence ignores what the slot held.

#include "elem_types.h"


// Sum over the 4 or 8 neighbouring lanes that share a value column, through
// the data-parallel lane permutes of the vector ALU (no trip through LDS):
// swaps inside pairs, then pairs inside quads, then the two quads of a group
// of 8 mirrored onto each other.
template <int CTRL>
LIG_DEVICE float lane_permute(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int SPLIT>
LIG_DEVICE float split_sum(float o) {
  o += lane_permute<0xB1>(o);   // quad_perm [1, 0, 3, 2]
  o += lane_permute<0x4E>(o);   // quad_perm [2, 3, 0, 1]
  if (SPLIT == 8) o += lane_permute<0x141>(o);  // row_half_mirror: lane i <-> 7 - i
  return o;
}

// KPT: key channels per thread (D is padded to SPLIT * KPT; padded channels carry
// q = k = w = 0 and stay zero).  MAXT bounds the workgroup size (4 * Dv
// rounded up to whole waves) so the compiler may use the register file a
// small workgroup leaves it.
template <typename T, int MS_SPLIT, int KPT, bool BONUS, int MAXT>
__global__ __launch_bounds__(MAXT) void matrix_state_scan_kernel(
    float* __restrict__ out,  // [R, H*Dv]
    const T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride,
    const T* __restrict__ v, long v_stride,
    const float* __restrict__ decay_pre,   // [R, H*D]   (BONUS)
    const float* __restrict__ head_decay,  // [H]        (!BONUS)
    const float* __restrict__ bonus,       // [H*D]      (BONUS)
    float* __restrict__ state, long state_stride, const int* __restrict__ seg_start,
    const int* __restrict__ seg_len, const int* __restrict__ seg_slot,
    const int* __restrict__ seg_fresh, int H, int D, int Dv, int TT, int act_silu) {
  extern __shared__ __align__(16) float sm[];
  constexpr int Dp = MS_SPLIT * KPT;
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

  float S[KPT], U[KPT];
  float* srow = state + (long)seg_slot[seg] * state_stride + (long)h * KPT * nthr;
  const bool load_state = owner && seg_fresh[seg] == 0;
#pragma unroll
  for (int ii = 0; ii < KPT; ++ii) {
    S[ii] = load_state ? srow[(long)ii * nthr + tid] : 0.f;
    const int i = s * KPT + ii;
    U[ii] = (BONUS && i < D) ? bonus[h * D + i] : 0.f;
  }
  const float dconst = BONUS ? 0.f : head_decay[h];

#pragma nounroll
  for (int t0 = 0; t0 < n; t0 += TT) {
    const int nt_tok = min(TT, n - t0);
    __syncthreads();  // the previous tile's readers are done
#pragma nounroll
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
#pragma nounroll
    for (int e = tid; e < nt_tok * Dv; e += nt) {
      const int t = e / Dv, c = e - t * Dv;
      float vv = ld(v + (long)(r0 + t0 + t) * v_stride + h * Dv + c);
      if (act_silu) vv = vv * sigmoid_f32(vv);
      v_s[e] = vv;
    }
    __syncthreads();
    // every wave of the workgroup walks the tile (idle lanes of the last
    // wave take part in the lane permutes with zeros)
    // one token: read its q, k, decay and v from LDS, output, state update
    auto step = [&](int t) __attribute__((always_inline)) {
      const float vj = owner ? v_s[t * Dv + j] : 0.f;
      const float* qt = q_s + t * Dp + s * KPT;
      const float* kt = k_s + t * Dp + s * KPT;
      const float* wt = w_s + t * Dp + s * KPT;
      float o = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < KPT; i4 += 4) {
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
      o = split_sum<MS_SPLIT>(o);
      if (owner && s == 0) out[(long)(r0 + t0 + t) * (H * Dv) + h * Dv + j] = o;
    };
    // two tokens per trip: the second token's LDS reads overlap the first
    // token's arithmetic (the state update itself stays in order)
    int t = 0;
#pragma nounroll
    for (; t + 1 < nt_tok; t += 2) {
      step(t);
      step(t + 1);
    }
    if (t < nt_tok) step(t);
  }
  if (owner) {
#pragma unroll
    for (int ii = 0; ii < KPT; ++ii) srow[(long)ii * nthr + tid] = S[ii];
  }
}

// Key split and key channels per thread for a head of D key channels and Dv
// value channels: the smallest size class that holds ceil(D / split); kpt 0
// when D is too wide.
static void ms_shape(int D, int Dv, int* split, int* kpt) {
  static const int classes[] = {4, 8, 12, 16, 24, 32, 48, 64};
  *split = (D >= 32 && Dv * 8 <= 1024) ? 8 : 4;
  const int need = (D + *split - 1) / *split;
  *kpt = 0;
  for (int c : classes)
    if (c >= need) {
      *kpt = c;
      break;
    }
}

// Returns 0 when launched, 1 when a head is wider than the kernel holds.
extern "C" int lig_matrix_state_scan(
    float* out, const void* q, long q_stride, const void* k, long k_stride,
    const void* v, long v_stride, const float* decay_pre, const float* head_decay,
    const float* bonus, float* state, long state_stride, const int* seg_start,
    const int* seg_len, const int* seg_slot, const int* seg_fresh, int S, int H,
    int D, int Dv, int act_silu, int is_f32, hipStream_t stream) {
  int split = 4, kpt = 0;
  if (D > 0) ms_shape(D, Dv, &split, &kpt);
  if (kpt == 0 || Dv <= 0 || Dv > 256) return 1;
  if (S <= 0) return 0;
  const int Dp = kpt * split;
  const bool has_bonus = bonus != nullptr;
  const int per_tok = (has_bonus ? 3 : 2) * Dp + Dv;
  // tokens staged per tile: as many as 40 KB of LDS hold, 8 to 32
  const int TT = per_tok * 32 * 4 <= 40 * 1024 ? 32 : (per_tok * 16 * 4 <= 48 * 1024 ? 16 : 8);
  const size_t smem = (size_t)per_tok * TT * sizeof(float);
  const int threads = ((Dv * split + WAVE_SIZE - 1) / WAVE_SIZE) * WAVE_SIZE;
  dim3 grid(S, H), block(threads);
#define LIG_MS_T(T, SP, KPT, B, MAXT)                                           \
  hipLaunchKernelGGL((matrix_state_scan_kernel<T, SP, KPT, B, MAXT>), grid,     \
                     block, smem, stream, out, (const T*)q, q_stride,           \
                     (const T*)k, k_stride, (const T*)v, v_stride, decay_pre,   \
                     head_decay, bonus, state, state_stride, seg_start,         \
                     seg_len, seg_slot, seg_fresh, H, D, Dv, TT, act_silu)
#define LIG_MS(T, SP, KPT, B)                             \
  do {                                                    \
    if (threads <= 256) LIG_MS_T(T, SP, KPT, B, 256);     \
    else LIG_MS_T(T, SP, KPT, B, 1024);                   \
  } while (0)
#define LIG_MS_K(T, B)                                    \
  if (split == 8) {                                       \
    switch (kpt) {                                        \
      case 4: LIG_MS(T, 8, 4, B); break;                  \
      case 8: LIG_MS(T, 8, 8, B); break;                  \
      case 12: LIG_MS(T, 8, 12, B); break;                \
      case 16: LIG_MS(T, 8, 16, B); break;                \
      case 24: LIG_MS(T, 8, 24, B); break;                \
      default: LIG_MS(T, 8, 32, B); break;                \
    }                                                     \
  } else {                                                \
    switch (kpt) {                                        \
      case 4: LIG_MS(T, 4, 4, B); break;                  \
      case 8: LIG_MS(T, 4, 8, B); break;                  \
      case 12: LIG_MS(T, 4, 12, B); break;                \
      case 16: LIG_MS(T, 4, 16, B); break;                \
      case 24: LIG_MS(T, 4, 24, B); break;                \
      case 32: LIG_MS(T, 4, 32, B); break;                \
      case 48: LIG_MS(T, 4, 48, B); break;                \
      default: LIG_MS(T, 4, 64, B); break;                \
    }                                                     \
  }
  if (is_f32) {
    if (has_bonus) { LIG_MS_K(float, true) } else { LIG_MS_K(float, false) }
  } else {
    if (has_bonus) { LIG_MS_K(bf16s, true) } else { LIG_MS_K(bf16s, false) }
  }
#undef LIG_MS_K
#undef LIG_MS
#undef LIG_MS_T
  return 0;
}
