// A residual kept as S parallel streams that sub-layers read through a
// weighted sum and write through a mixing matrix ("hyper-connections"),
// gfx950.  fp32 streams and arithmetic; branch outputs and the normed read
// are bf16 or fp32 storage.
//
// Layout: xs [R, S, W] fp32, a token's streams side by side.
//
// hyper_step does, per token row and in one pass over HBM,
//   1. the WRITE of the sub-layer that just ran (y non-null), all streams at
//      once from the old ones:
//          x_t <- sum_s mix[s, t] x_s + m * out[t] * y
//   2. the READ of the next sub-layer (in non-null):
//          u = sum_t in[t] x_t;   h = u / sqrt(mean(u^2) + eps) * g
//      with ONE weight g for all coordinates (a pointer to a single fp32, so
//      nothing is copied to the host); h is stored in the activation type.
// u waits in LDS between the reduction and the scaling.  S == 1 with mix =
// out = in = 1 is the ordinary pre-norm residual.  The coefficients are
// small fp32 device vectors staged in LDS.

#include "elem_types.h"

#define HS_MAX_STREAMS 16

template <typename T, int SC, int N>  // SC: compile-time stream count, 0 = run time
__global__ __launch_bounds__(256) void hyper_step_kernel(
    float* __restrict__ xs, const T* __restrict__ y, const float* __restrict__ mix,
    const float* __restrict__ outw, float m, const float* __restrict__ inw,
    const float* __restrict__ g, float eps, T* __restrict__ h, int S_rt, int W) {
  extern __shared__ __align__(16) float row_s[];  // [W]
  __shared__ float red[17];
  __shared__ float mix_s[HS_MAX_STREAMS * HS_MAX_STREAMS];
  __shared__ float out_s[HS_MAX_STREAMS], in_s[HS_MAX_STREAMS];
  constexpr int SA = SC ? SC : HS_MAX_STREAMS;
  const int S = SC ? SC : S_rt;
  const bool write = y != nullptr, read = inw != nullptr;
  for (int i = threadIdx.x; i < S * S; i += blockDim.x) mix_s[i] = write ? mix[i] : 0.f;
  for (int i = threadIdx.x; i < S; i += blockDim.x) {
    out_s[i] = write ? m * outw[i] : 0.f;
    in_s[i] = read ? inw[i] : 0.f;
  }
  __syncthreads();
  float* xrow = xs + (long)blockIdx.x * S * W;
  const long ybase = (long)blockIdx.x * W;
  float ss = 0.f;
  for (int c = threadIdx.x * N; c < W; c += blockDim.x * N) {
    float x[SA][N], yv[N], u[N];
#pragma unroll
    for (int s = 0; s < SA; ++s)
      if (s < S) ldn<N>(xrow + (long)s * W + c, x[s]);
    if (write) {
      ldn<N>(y + ybase + c, yv);
      float nx[SA][N];
#pragma unroll
      for (int t = 0; t < SA; ++t) {
        if (t < S) {
#pragma unroll
          for (int k = 0; k < N; ++k) nx[t][k] = out_s[t] * yv[k];
#pragma unroll
          for (int s = 0; s < SA; ++s)
            if (s < S) {
#pragma unroll
              for (int k = 0; k < N; ++k) nx[t][k] += mix_s[s * S + t] * x[s][k];
            }
        }
      }
#pragma unroll
      for (int t = 0; t < SA; ++t)
        if (t < S) {
#pragma unroll
          for (int k = 0; k < N; ++k) x[t][k] = nx[t][k];
          stn<N>(xrow + (long)t * W + c, x[t]);
        }
    }
    if (read) {
#pragma unroll
      for (int k = 0; k < N; ++k) u[k] = 0.f;
#pragma unroll
      for (int t = 0; t < SA; ++t)
        if (t < S) {
#pragma unroll
          for (int k = 0; k < N; ++k) u[k] += in_s[t] * x[t][k];
        }
#pragma unroll
      for (int k = 0; k < N; ++k) ss += u[k] * u[k];
      stn<N>(row_s + c, u);
    }
  }
  if (!read) return;
  ss = block_reduce_sum(ss, red);
  const float sc = g[0] / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x * N; c < W; c += blockDim.x * N) {
    float u[N];
    ldn<N>(row_s + c, u);  // this thread's own chunk
#pragma unroll
    for (int k = 0; k < N; ++k) u[k] *= sc;
    stn<N>(h + ybase + c, u);
  }
}

// Returns 0 when launched, 1 when the shape is not served.
extern "C" int lig_hyper_step(float* xs, const void* y, const float* mix,
                              const float* outw, float m, const float* inw,
                              const float* g, float eps, void* h, int R, int S,
                              int W, int is_f32, hipStream_t st) {
  if (S < 1 || S > HS_MAX_STREAMS || W < 1) return 1;
  if (R <= 0) return 0;
  const size_t smem = (size_t)W * sizeof(float);
  const bool v4 = W % 4 == 0 && aligned16(xs) && aligned16(h) && (y == nullptr || aligned16(y));
  const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
#define LIG_HS(T, SC, N)                                                          \
  hipLaunchKernelGGL((hyper_step_kernel<T, SC, N>), dim3(R), dim3(threads), smem, \
                     st, xs, (const T*)y, mix, outw, m, inw, g, eps, (T*)h, S, W)
#define LIG_HS_S(T, N)                                   \
  switch (S) {                                           \
    case 1: LIG_HS(T, 1, N); break;                      \
    case 2: LIG_HS(T, 2, N); break;                      \
    case 4: LIG_HS(T, 4, N); break;                      \
    default: LIG_HS(T, 0, N); break;                     \
  }
  if (is_f32) {
    if (v4) { LIG_HS_S(float, 4) } else { LIG_HS_S(float, 1) }
  } else {
    if (v4) { LIG_HS_S(bf16s, 4) } else { LIG_HS_S(bf16s, 1) }
  }
#undef LIG_HS_S
#undef LIG_HS
  return 0;
}
