// Norms that FOLLOW a sum or a recurrence, gfx950.  fp32 arithmetic; the
// residual and the recurrence outputs are fp32, weights / branch outputs /
// gates are bf16 or fp32 storage.
//
// scaled_add_rms_norm: the norm after the residual sum,
//     x <- rms(alpha * x + s1 * y1 + s2 * y2) * w
// one workgroup per row; the sum is held in LDS between the reduction and
// the scaling so every operand crosses HBM once.  The normed row is written
// twice: fp32 back into the residual and rounded to the storage type as the
// next GEMM's input.  Without y1 the row is only normed (x untouched).
//
// group_rms_norm_gate: every `group` consecutive entries of an fp32 row are
// divided by their root mean square (group == C: the whole row), times a
// weight, times silu(gate) or sigmoid(gate).

#include "elem_types.h"

template <typename T>
__global__ __launch_bounds__(256) void scaled_add_rms_norm_kernel(
    float* __restrict__ x, T* __restrict__ h, const T* __restrict__ y1,
    const T* __restrict__ y2, const T* __restrict__ w, float alpha, float s1,
    float s2, float eps, int H) {
  extern __shared__ __align__(16) float row_s[];  // [H]
  __shared__ float red[17];
  const long base = (long)blockIdx.x * H;
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    float t = x[base + c];
    if (y1 != nullptr) {
      t = alpha * t + s1 * ld(y1 + base + c);
      if (y2 != nullptr) t += s2 * ld(y2 + base + c);
    }
    row_s[c] = t;
    ss += t * t;
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    const float v = row_s[c] * inv * ld(w + c);
    if (y1 != nullptr) x[base + c] = v;
    st(h + base + c, v);
  }
}

// 8 elements per thread and access: H % 8 == 0, 16-byte aligned rows.
template <typename T>
__global__ __launch_bounds__(256) void scaled_add_rms_norm_vec_kernel(
    float* __restrict__ x, T* __restrict__ h, const T* __restrict__ y1,
    const T* __restrict__ y2, const T* __restrict__ w, float alpha, float s1,
    float s2, float eps, int H) {
  extern __shared__ __align__(16) float row_s[];  // [H]
  __shared__ float red[17];
  const long base = (long)blockIdx.x * H;
  float ss = 0.f;
  for (int c = threadIdx.x * 8; c < H; c += blockDim.x * 8) {
    float t[8];
    ld8(x + base + c, t);
    if (y1 != nullptr) {
      float a[8];
      ld8(y1 + base + c, a);
#pragma unroll
      for (int i = 0; i < 8; ++i) t[i] = alpha * t[i] + s1 * a[i];
      if (y2 != nullptr) {
        ld8(y2 + base + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] += s2 * a[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += t[i] * t[i];
    st8(row_s + c, t);
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  for (int c = threadIdx.x * 8; c < H; c += blockDim.x * 8) {
    float t[8], ww[8];
    ld8(row_s + c, t);  // this thread's own chunk
    ld8(w + c, ww);
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = t[i] * inv * ww[i];
    if (y1 != nullptr) st8(x + base + c, t);
    st8(h + base + c, t);
  }
}

// 4 elements per thread: a group of `group` entries (a multiple of 4 whose
// quarter is a power of two up to 64, or the whole row) is spread over
// group/4 neighbouring lanes and reduced with xor shuffles.
template <typename T>
__global__ __launch_bounds__(256) void group_rms_norm_gate_vec_kernel(
    T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ gate,
    long gate_stride, const T* __restrict__ w, int group, int gate_silu, float eps,
    int C) {
  __shared__ float red[17];
  const long r = blockIdx.x;
  const float* orow = o + r * C;
  const T* grow = gate + r * gate_stride;
  T* out_row = out + r * C;
  const bool whole = group == C;
  float inv_whole = 0.f;
  if (whole) {
    float ss = 0.f;
    for (int c = threadIdx.x * 4; c < C; c += blockDim.x * 4) {
      float t[4];
      ldn<4>(orow + c, t);
      ss += t[0] * t[0] + t[1] * t[1] + t[2] * t[2] + t[3] * t[3];
    }
    ss = block_reduce_sum(ss, red);
    inv_whole = 1.0f / sqrtf(ss / (float)C + eps);
  }
  const int lanes = group / 4;  // lanes per group (power of two) when !whole
  const int span = (C + 3) / 4;
  for (int c4 = threadIdx.x; c4 < ((span + 63) / 64) * 64; c4 += blockDim.x) {
    const int c = c4 * 4;
    const bool live = c < C;
    float t[4] = {0.f, 0.f, 0.f, 0.f};
    if (live) ldn<4>(orow + c, t);
    float inv = inv_whole;
    if (!whole) {
      float ss = t[0] * t[0] + t[1] * t[1] + t[2] * t[2] + t[3] * t[3];
      for (int m = 1; m < lanes; m <<= 1) ss += __shfl_xor(ss, m, WAVE_SIZE);
      inv = 1.0f / sqrtf(ss / (float)group + eps);
    }
    if (live) {
      float g[4], ww[4];
      ldn<4>(grow + c, g);
      ldn<4>(w + c, ww);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a = gate_silu ? g[i] * sigmoid_f32(g[i]) : sigmoid_f32(g[i]);
        t[i] = t[i] * inv * ww[i] * a;
      }
      stn<4>(out_row + c, t);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void group_rms_norm_gate_kernel(
    T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ gate,
    long gate_stride, const T* __restrict__ w, int group, int gate_silu, float eps,
    int C) {
  __shared__ float red[17];
  const long r = blockIdx.x;
  const float* orow = o + r * C;
  const T* grow = gate + r * gate_stride;
  T* out_row = out + r * C;
  if (group == C) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
      const float t = orow[c];
      ss += t * t;
    }
    ss = block_reduce_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)C + eps);
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
      const float g = ld(grow + c);
      const float a = gate_silu ? g * sigmoid_f32(g) : sigmoid_f32(g);
      st(out_row + c, orow[c] * inv * ld(w + c) * a);
    }
    return;
  }
  // one wave per group at a time
  const int wave = threadIdx.x / WAVE_SIZE, lane = threadIdx.x % WAVE_SIZE;
  const int nwaves = blockDim.x / WAVE_SIZE;
  for (int g0 = wave; g0 < C / group; g0 += nwaves) {
    const int c0 = g0 * group;
    float ss = 0.f;
    for (int d = lane; d < group; d += WAVE_SIZE) {
      const float t = orow[c0 + d];
      ss += t * t;
    }
    ss = wave_reduce_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)group + eps);
    for (int d = lane; d < group; d += WAVE_SIZE) {
      const float g = ld(grow + c0 + d);
      const float a = gate_silu ? g * sigmoid_f32(g) : sigmoid_f32(g);
      st(out_row + c0 + d, orow[c0 + d] * inv * ld(w + c0 + d) * a);
    }
  }
}

extern "C" {

void lig_scaled_add_rms_norm(float* x, void* h, const void* y1, const void* y2,
                             const void* w, float alpha, float s1, float s2,
                             float eps, int R, int H, int is_f32, hipStream_t s) {
  if (R <= 0 || H <= 0) return;
  const size_t smem = (size_t)H * sizeof(float);
  const bool vec = H % 8 == 0 && aligned16(x) && aligned16(h) && aligned16(w) &&
                   (y1 == nullptr || aligned16(y1)) && (y2 == nullptr || aligned16(y2));
  if (vec) {
    if (is_f32)
      hipLaunchKernelGGL(scaled_add_rms_norm_vec_kernel<float>, dim3(R), dim3(256), smem,
                         s, x, (float*)h, (const float*)y1, (const float*)y2,
                         (const float*)w, alpha, s1, s2, eps, H);
    else
      hipLaunchKernelGGL(scaled_add_rms_norm_vec_kernel<bf16s>, dim3(R), dim3(256), smem,
                         s, x, (bf16s*)h, (const bf16s*)y1, (const bf16s*)y2,
                         (const bf16s*)w, alpha, s1, s2, eps, H);
    return;
  }
  if (is_f32)
    hipLaunchKernelGGL(scaled_add_rms_norm_kernel<float>, dim3(R), dim3(256), smem, s,
                       x, (float*)h, (const float*)y1, (const float*)y2,
                       (const float*)w, alpha, s1, s2, eps, H);
  else
    hipLaunchKernelGGL(scaled_add_rms_norm_kernel<bf16s>, dim3(R), dim3(256), smem, s,
                       x, (bf16s*)h, (const bf16s*)y1, (const bf16s*)y2,
                       (const bf16s*)w, alpha, s1, s2, eps, H);
}

void lig_group_rms_norm_gate(void* out, const float* o, const void* gate,
                             long gate_stride, const void* w, int group,
                             int gate_silu, float eps, int R, int C, int is_f32,
                             hipStream_t s) {
  if (R <= 0 || C <= 0) return;
  const int esz = is_f32 ? 4 : 2;
  const int lanes = group / 4;
  const bool vec = C % 4 == 0 && group % 4 == 0 &&
                   (group == C || (lanes <= 64 && (lanes & (lanes - 1)) == 0)) &&
                   aligned16(o) && gate_stride % 4 == 0 &&
                   (reinterpret_cast<uintptr_t>(gate) % (4 * esz)) == 0 &&
                   (reinterpret_cast<uintptr_t>(out) % (4 * esz)) == 0 &&
                   (reinterpret_cast<uintptr_t>(w) % (4 * esz)) == 0;
  if (vec) {
    if (is_f32)
      hipLaunchKernelGGL(group_rms_norm_gate_vec_kernel<float>, dim3(R), dim3(256), 0, s,
                         (float*)out, o, (const float*)gate, gate_stride,
                         (const float*)w, group, gate_silu, eps, C);
    else
      hipLaunchKernelGGL(group_rms_norm_gate_vec_kernel<bf16s>, dim3(R), dim3(256), 0, s,
                         (bf16s*)out, o, (const bf16s*)gate, gate_stride,
                         (const bf16s*)w, group, gate_silu, eps, C);
    return;
  }
  if (is_f32)
    hipLaunchKernelGGL(group_rms_norm_gate_kernel<float>, dim3(R), dim3(256), 0, s,
                       (float*)out, o, (const float*)gate, gate_stride,
                       (const float*)w, group, gate_silu, eps, C);
  else
    hipLaunchKernelGGL(group_rms_norm_gate_kernel<bf16s>, dim3(R), dim3(256), 0, s,
                       (bf16s*)out, o, (const bf16s*)gate, gate_stride,
                       (const bf16s*)w, group, gate_silu, eps, C);
}

}  // extern "C"
