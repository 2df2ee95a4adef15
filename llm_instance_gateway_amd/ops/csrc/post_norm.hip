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
