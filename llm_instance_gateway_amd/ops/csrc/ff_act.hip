// Feed-forward activations between the two GEMMs, gfx950: squared ReLU, the
// gated SiLU (silu(gate) * up over a fused [gate | up] projection), the exact
// (erf) gelu, tanh, and the tanh soft cap of fp32 logits.
// fp32 arithmetic, bf16 or fp32 storage; 4-element vectors when the row
// width allows.

#include "elem_types.h"

template <typename T, int N>
__global__ void relu_squared_kernel(T* __restrict__ out, const T* __restrict__ x, long n) {
  for (long i = (blockIdx.x * (long)blockDim.x + threadIdx.x) * N; i < n;
       i += gridDim.x * (long)blockDim.x * N) {
    float v[N];
    ldn<N>(x + i, v);
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const float z = fmaxf(v[k], 0.f);
      v[k] = z * z;
    }
    stn<N>(out + i, v);
  }
}

template <typename T, int N>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ x,
                                int F, long n) {  // x [rows, 2F], out [rows, F]
  for (long i = (blockIdx.x * (long)blockDim.x + threadIdx.x) * N; i < n;
       i += gridDim.x * (long)blockDim.x * N) {
    const long r = i / F;
    const int c = (int)(i - r * F);
    float g[N], u[N];
    ldn<N>(x + r * 2 * F + c, g);
    ldn<N>(x + r * 2 * F + F + c, u);
#pragma unroll
    for (int k = 0; k < N; ++k) g[k] = g[k] * sigmoid_for<T>(g[k]) * u[k];
    stn<N>(out + i, g);
  }
}

// Element-wise maps: 0 = exact gelu 0.5 z (1 + erf(z / sqrt 2)), 1 = tanh.
template <typename T, int N, int OP>
__global__ void unary_act_kernel(T* __restrict__ out, const T* __restrict__ x, long n) {
  for (long i = (blockIdx.x * (long)blockDim.x + threadIdx.x) * N; i < n;
       i += gridDim.x * (long)blockDim.x * N) {
    float v[N];
    ldn<N>(x + i, v);
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const float z = v[k];
      v[k] = OP == 0 ? 0.5f * z * (1.0f + erff(z * 0.70710678118654752440f)) : tanhf(z);
    }
    stn<N>(out + i, v);
  }
}

__global__ void tanh_softcap_kernel(float* __restrict__ x, float cap, float inv_cap, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += gridDim.x * (long)blockDim.x)
    x[i] = cap * tanhf(x[i] * inv_cap);
}

template <int OP>
static void launch_unary(void* out, const void* x, long n, int is_f32, hipStream_t s) {
  if (n <= 0) return;
  const bool v4 = n % 4 == 0 && aligned16(out) && aligned16(x);
  long g = ((v4 ? n / 4 : n) + 255) / 256;
  const int grid = (int)(g > 65535 ? 65535 : g);
#define LIG_UA(T, N)                                                             \
  hipLaunchKernelGGL((unary_act_kernel<T, N, OP>), dim3(grid), dim3(256), 0, s,  \
                     (T*)out, (const T*)x, n)
  if (is_f32) {
    if (v4) LIG_UA(float, 4); else LIG_UA(float, 1);
  } else {
    if (v4) LIG_UA(bf16s, 4); else LIG_UA(bf16s, 1);
  }
#undef LIG_UA
}

extern "C" {

void lig_gelu_erf(void* out, const void* x, long n, int is_f32, hipStream_t s) {
  launch_unary<0>(out, x, n, is_f32, s);
}

void lig_tanh_act(void* out, const void* x, long n, int is_f32, hipStream_t s) {
  launch_unary<1>(out, x, n, is_f32, s);
}

void lig_tanh_softcap(float* x, float cap, long n, hipStream_t s) {
  if (n <= 0) return;
  long g = (n + 255) / 256;
  const int grid = (int)(g > 65535 ? 65535 : g);
  hipLaunchKernelGGL(tanh_softcap_kernel, dim3(grid), dim3(256), 0, s, x, cap, 1.0f / cap, n);
}

void lig_relu_squared(void* out, const void* x, long n, int is_f32, hipStream_t s) {
  if (n <= 0) return;
  const bool v4 = n % 4 == 0 && aligned16(out) && aligned16(x);
  long g = ((v4 ? n / 4 : n) + 255) / 256;
  const int grid = (int)(g > 65535 ? 65535 : g);
#define LIG_R2(T, N)                                                           \
  hipLaunchKernelGGL((relu_squared_kernel<T, N>), dim3(grid), dim3(256), 0, s, \
                     (T*)out, (const T*)x, n)
  if (is_f32) {
    if (v4) LIG_R2(float, 4); else LIG_R2(float, 1);
  } else {
    if (v4) LIG_R2(bf16s, 4); else LIG_R2(bf16s, 1);
  }
#undef LIG_R2
}

void lig_silu_mul(void* out, const void* x, long rows, int F, int is_f32,
                  hipStream_t s) {
  const long n = rows * F;
  if (n <= 0) return;
  const bool v4 = F % 4 == 0 && aligned16(out) && aligned16(x);
  long g = ((v4 ? n / 4 : n) + 255) / 256;
  const int grid = (int)(g > 65535 ? 65535 : g);
#define LIG_SM(T, N)                                                        \
  hipLaunchKernelGGL((silu_mul_kernel<T, N>), dim3(grid), dim3(256), 0, s,  \
                     (T*)out, (const T*)x, F, n)
  if (is_f32) {
    if (v4) LIG_SM(float, 4); else LIG_SM(float, 1);
  } else {
    if (v4) LIG_SM(bf16s, 4); else LIG_SM(bf16s, 1);
  }
#undef LIG_SM
}

}  // extern "C"
