// Routed feed-forward pieces, gfx950: a softmax router with correction
// offsets and group-limited choice, the weighted combine of the chosen
// experts' outputs, and gated activations between the expert GEMMs.
// fp32 arithmetic; bf16 or fp32 storage for activations.
//
// grouped_topk_route, one wave per token over N router logits (fp32):
//   s = softmax(z);  c = s + correction   (choice scores)
//   the N outputs form `groups` equal groups of neighbours; a group scores
//   its largest c; only outputs of the `keep` best groups can be chosen;
//   the `top` largest c among them are chosen (ties: the lower index);
//   weights = chosen s / (their sum + 1e-20).
//
// routed_combine: out[t] = sum_k w[t, k] * src_k, src_k = ye[row[t, k]] or,
// for row < 0, the token's own input x[t] (an identity expert).  Rows come
// as a table, or are computed from the choices themselves when every expert
// saw every token (ye = [experts, T, W]): row = idx * T + t, idx >= experts
// being an identity expert.
//
// glu_act over a fused [gate | up] projection:
//   0: relu(gate) * up
//   1: g = min(gate, limit), u = clamp(up, -limit, limit),
//      g * sigmoid(alpha * g) * (u + 1)

#include "elem_types.h"

struct BestPair {
  float v;
  int i;
};

LIG_DEVICE BestPair wave_argmax(BestPair b) {
#pragma unroll
  for (int off = WAVE_SIZE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(b.v, off, WAVE_SIZE);
    const int oi = __shfl_xor(b.i, off, WAVE_SIZE);
    if (ov > b.v || (ov == b.v && oi < b.i)) {
      b.v = ov;
      b.i = oi;
    }
  }
  return b;
}

__global__ __launch_bounds__(WAVE_SIZE) void grouped_topk_route_kernel(
    const float* __restrict__ z, const float* __restrict__ corr, int N, int groups,
    int keep, int top, int* __restrict__ idx_out, float* __restrict__ w_out) {
  extern __shared__ __align__(16) float sm[];
  float* s_s = sm;           // [N] scores
  float* c_s = sm + N;       // [N] choice scores, -inf once taken or barred
  float* g_s = sm + 2 * N;   // [groups]
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* zr = z + (long)t * N;
  float mx = -INFINITY;
  for (int i = lane; i < N; i += WAVE_SIZE) mx = fmaxf(mx, zr[i]);
  mx = wave_reduce_max(mx);
  float sum = 0.f;
  for (int i = lane; i < N; i += WAVE_SIZE) {
    const float e = expf(zr[i] - mx);
    s_s[i] = e;
    sum += e;
  }
  sum = wave_reduce_sum(sum);
  const float inv = 1.0f / sum;
  for (int i = lane; i < N; i += WAVE_SIZE) {
    const float s = s_s[i] * inv;
    s_s[i] = s;
    c_s[i] = s + (corr != nullptr ? corr[i] : 0.f);
  }
  __syncthreads();
  if (groups > 1 && keep < groups) {
    const int per = N / groups;
    for (int g = lane; g < groups; g += WAVE_SIZE) {
      float gm = -INFINITY;
      for (int i = g * per; i < (g + 1) * per; ++i) gm = fmaxf(gm, c_s[i]);
      g_s[g] = gm;
    }
    __syncthreads();
    // the kept groups are marked with NaN-free +inf
    for (int k = 0; k < keep; ++k) {
      BestPair b{-INFINITY, 0x7fffffff};
      for (int g = lane; g < groups; g += WAVE_SIZE) {
        const float v = g_s[g];
        if (v != INFINITY && (v > b.v || (v == b.v && g < b.i))) b = BestPair{v, g};
      }
      b = wave_argmax(b);
      __syncthreads();
      if (lane == 0 && b.i < groups) g_s[b.i] = INFINITY;
      __syncthreads();
    }
    for (int i = lane; i < N; i += WAVE_SIZE)
      if (g_s[i / per] != INFINITY) c_s[i] = -INFINITY;
    __syncthreads();
  }
  float wsum = 0.f;
  for (int k = 0; k < top; ++k) {
    BestPair b{-INFINITY, 0x7fffffff};
    for (int i = lane; i < N; i += WAVE_SIZE) {
      const float v = c_s[i];
      if (v > b.v || (v == b.v && i < b.i)) b = BestPair{v, i};
    }
    b = wave_argmax(b);
    const int pick = b.i < N ? b.i : 0;
    const float w = s_s[pick];
    wsum += w;
    __syncthreads();
    if (lane == 0) {
      idx_out[(long)t * top + k] = pick;
      w_out[(long)t * top + k] = w;
      c_s[pick] = -INFINITY;
    }
    __syncthreads();
  }
  const float winv = 1.0f / (wsum + 1e-20f);
  for (int k = lane; k < top; k += WAVE_SIZE) w_out[(long)t * top + k] *= winv;
}

template <typename T, int N>
__global__ void routed_combine_kernel(T* __restrict__ out, const T* __restrict__ ye,
                                      const T* __restrict__ x,
                                      const long* __restrict__ rows,
                                      const int* __restrict__ idx, int experts,
                                      const float* __restrict__ w, int top, int W) {
  const long t = blockIdx.x;
  const long ntok = gridDim.x;
  for (int c = threadIdx.x * N; c < W; c += blockDim.x * N) {
    float acc[N];
#pragma unroll
    for (int i = 0; i < N; ++i) acc[i] = 0.f;
    for (int k = 0; k < top; ++k) {
      long r;
      if (idx != nullptr) {
        const int e = idx[t * top + k];
        r = e < experts ? (long)e * ntok + t : -1;
      } else {
        r = rows[t * top + k];
      }
      const float wk = w[t * top + k];
      float v[N];
      ldn<N>(r >= 0 ? ye + r * W + c : x + t * W + c, v);
#pragma unroll
      for (int i = 0; i < N; ++i) acc[i] += wk * v[i];
    }
    stn<N>(out + t * W + c, acc);
  }
}

template <typename T, int N, int KIND>
__global__ void glu_act_kernel(T* __restrict__ out, const T* __restrict__ x, int F,
                               long n, float limit, float alpha) {
  for (long i = (blockIdx.x * (long)blockDim.x + threadIdx.x) * N; i < n;
       i += gridDim.x * (long)blockDim.x * N) {
    const long r = i / F;
    const int c = (int)(i - r * F);
    float g[N], u[N];
    ldn<N>(x + r * 2 * F + c, g);
    ldn<N>(x + r * 2 * F + F + c, u);
#pragma unroll
    for (int k = 0; k < N; ++k) {
      if (KIND == 0) {
        g[k] = fmaxf(g[k], 0.f) * u[k];
      } else {
        const float gg = fminf(g[k], limit);
        const float uu = fminf(fmaxf(u[k], -limit), limit);
        g[k] = gg * sigmoid_for<T>(alpha * gg) * (uu + 1.0f);
      }
    }
    stn<N>(out + i, g);
  }
}

extern "C" {

int lig_grouped_topk_route(const float* z, const float* corr, int T, int N,
                           int groups, int keep, int top, int* idx_out,
                           float* w_out, hipStream_t s) {
  if (N < 1 || top < 1 || top > N || groups < 1 || N % groups != 0 || keep < 1 ||
      keep > groups || top > keep * (N / groups) || N > 8192)
    return 1;
  if (T <= 0) return 0;
  const size_t smem = (size_t)(2 * N + groups) * sizeof(float);
  hipLaunchKernelGGL(grouped_topk_route_kernel, dim3(T), dim3(WAVE_SIZE), smem, s, z,
                     corr, N, groups, keep, top, idx_out, w_out);
  return 0;
}

void lig_routed_combine(void* out, const void* ye, const void* x, const long* rows,
                        const int* idx, int experts, const float* w, int T, int top,
                        int W, int is_f32, hipStream_t s) {
  if (T <= 0) return;
  const bool v4 = W % 4 == 0 && aligned16(out) && aligned16(ye) && aligned16(x);
  const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
#define LIG_RC(T_, N)                                                             \
  hipLaunchKernelGGL((routed_combine_kernel<T_, N>), dim3(T), dim3(threads), 0, s, \
                     (T_*)out, (const T_*)ye, (const T_*)x, rows, idx, experts, w, top, W)
  if (is_f32) {
    if (v4) LIG_RC(float, 4); else LIG_RC(float, 1);
  } else {
    if (v4) LIG_RC(bf16s, 4); else LIG_RC(bf16s, 1);
  }
#undef LIG_RC
}

void lig_glu_act(void* out, const void* x, long rows, int F, int kind, float limit,
                 float alpha, int is_f32, hipStream_t s) {
  const long n = rows * F;
  if (n <= 0) return;
  const bool v4 = F % 4 == 0 && aligned16(out) && aligned16(x);
  long g = ((v4 ? n / 4 : n) + 255) / 256;
  const int grid = (int)(g > 65535 ? 65535 : g);
#define LIG_GA(T, N, K)                                                         \
  hipLaunchKernelGGL((glu_act_kernel<T, N, K>), dim3(grid), dim3(256), 0, s,    \
                     (T*)out, (const T*)x, F, n, limit, alpha)
#define LIG_GA_K(T, N) \
  if (kind == 0) LIG_GA(T, N, 0); else LIG_GA(T, N, 1)
  if (is_f32) {
    if (v4) { LIG_GA_K(float, 4); } else { LIG_GA_K(float, 1); }
  } else {
    if (v4) { LIG_GA_K(bf16s, 4); } else { LIG_GA_K(bf16s, 1); }
  }
#undef LIG_GA_K
#undef LIG_GA
}

}  // extern "C"
