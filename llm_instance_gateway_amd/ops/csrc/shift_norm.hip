// Offset-weight RMS norms over an fp32 residual with a token shift, and the
// residual add that goes with a parallel (mixer + feed-forward) layer, gfx950.
//
//   n      = x / sqrt(mean(x^2) + eps)              (one statistic per row)
//   h      = n * (1 + w_mix)                        mixer branch
//   h_mix  = h + (h_prev - h) * mu                  token shift
//   h_ff   = n * (1 + w_ff)                         feed-forward branch
//
// h_prev is the same quantity of the previous token of the sequence: the row
// before inside a step's segment (recomputed here from that row, so nothing
// is exchanged between workgroups), the sequence's state row at a segment's
// first token (zeros when the sequence starts there).  The workgroup of a
// segment's FIRST row also refreshes the state with the segment's LAST
// unblended h after it has read the old one: reader and writer of a state
// element are the same thread, so a segment of any length needs no second
// launch.  All arithmetic is fp32; T is the storage type of the weights and
// of the outputs.
//
// The previous layer's two branch outputs can be added on the way in
// (x_new = x + (a + b), written to a second buffer so that neighbouring
// workgroups still read the old rows): the residual add and the next layer's
// norms are then one pass.

#include "elem_types.h"

#define SN_THREADS 256

template <typename T>
__global__ __launch_bounds__(SN_THREADS) void offset_norm_shift_kernel(
    T* __restrict__ h_mix, T* __restrict__ h_ff,  // [R, H]; h_ff nullable
    const float* __restrict__ x,                  // [R, H]
    const T* __restrict__ w_mix, const T* __restrict__ w_ff,
    const T* __restrict__ mu,                     // nullable: no shift
    float* __restrict__ state,                    // [slots, H]
    const int* __restrict__ tok_seq, const int* __restrict__ seg_start,
    const int* __restrict__ seg_len, const int* __restrict__ seg_slot,
    const int* __restrict__ seg_fresh, float eps, int H) {
  __shared__ float red[3][17];
  const int r = blockIdx.x, tid = threadIdx.x;
  const int s = tok_seq[r];
  T* om = h_mix + (size_t)r * H;
  T* of = h_ff ? h_ff + (size_t)r * H : nullptr;
  if (s < 0) {  // padding row
    for (int d = tid; d < H; d += SN_THREADS) {
      st(om + d, 0.f);
      if (of) st(of + d, 0.f);
    }
    return;
  }
  const int s0 = seg_start[s], cnt = seg_len[s];
  const bool first = r == s0;
  const int r_last = s0 + cnt - 1;
  const bool shift = mu != nullptr;
  const bool need_prev = shift && !first;
  const bool need_last = shift && first && r_last != r;
  const float* xr = x + (size_t)r * H;
  const float* xp = x + (size_t)(need_prev ? r - 1 : r) * H;
  const float* xl = x + (size_t)(need_last ? r_last : r) * H;

  float a = 0.f, b = 0.f, c = 0.f;
  for (int d = tid; d < H; d += SN_THREADS) {
    const float v = xr[d];
    a += v * v;
    if (need_prev) {
      const float u = xp[d];
      b += u * u;
    }
    if (need_last) {
      const float u = xl[d];
      c += u * u;
    }
  }
  a = block_reduce_sum(a, red[0]);
  if (need_prev) b = block_reduce_sum(b, red[1]);  // uniform per workgroup
  if (need_last) c = block_reduce_sum(c, red[2]);
  const float inv = 1.0f / sqrtf(a / (float)H + eps);
  const float inv_p = need_prev ? 1.0f / sqrtf(b / (float)H + eps) : 0.f;
  const float inv_l = need_last ? 1.0f / sqrtf(c / (float)H + eps) : 0.f;
  float* st_row = shift ? state + (size_t)seg_slot[s] * H : nullptr;
  const bool fresh = seg_fresh[s] != 0;

  for (int d = tid; d < H; d += SN_THREADS) {
    const float n = xr[d] * inv;
    const float g = 1.0f + ld(w_mix + d);
    const float h = n * g;
    float o = h;
    if (shift) {
      float prev;
      if (first) {
        prev = fresh ? 0.f : st_row[d];
        st_row[d] = need_last ? xl[d] * inv_l * g : h;
      } else {
        prev = xp[d] * inv_p * g;
      }
      o = h + (prev - h) * ld(mu + d);
    }
    st(om + d, o);
    if (of) st(of + d, n * (1.0f + ld(w_ff + d)));
  }
}


// Vector path: H % 4 == 0 and H <= 4 * SN_THREADS * VPT.  Every thread keeps
// its float4 chunks of the row (and of the neighbouring row it needs) in
// registers between the reduction and the scaling, so each operand crosses
// the memory system once; the three sums share one LDS exchange.
template <typename T, int VPT>
__global__ __launch_bounds__(SN_THREADS) void offset_norm_shift_vec_kernel(
    T* __restrict__ h_mix, T* __restrict__ h_ff, const float* __restrict__ x,
    const T* __restrict__ add_a, const T* __restrict__ add_b,  // nullable addends
    float* __restrict__ x_out,                                 // x + (a + b) when add_a
    const T* __restrict__ w_mix, const T* __restrict__ w_ff, const T* __restrict__ mu,
    float* __restrict__ state, const int* __restrict__ tok_seq,
    const int* __restrict__ seg_start, const int* __restrict__ seg_len,
    const int* __restrict__ seg_slot, const int* __restrict__ seg_fresh, float eps,
    int H) {
  __shared__ float red[3][SN_THREADS / WAVE_SIZE];
  const int r = blockIdx.x, tid = threadIdx.x;
  const int s = tok_seq[r];
  const int nvec = H / 4;
  T* om = h_mix + (size_t)r * H;
  T* of = h_ff ? h_ff + (size_t)r * H : nullptr;
  if (s < 0) {  // padding row
    const float z[4] = {0.f, 0.f, 0.f, 0.f};
    for (int v = tid; v < nvec; v += SN_THREADS) {
      stn<4>(om + 4 * v, z);
      if (of) stn<4>(of + 4 * v, z);
      if (add_a) stn<4>(x_out + (size_t)r * H + 4 * v, z);
    }
    return;
  }
  const int s0 = seg_start[s], cnt = seg_len[s];
  const bool first = r == s0;
  const int r_last = s0 + cnt - 1;
  const bool shift = mu != nullptr;
  const bool need_prev = shift && !first;
  const bool need_last = shift && first && r_last != r;
  const bool need_other = need_prev || need_last;  // never both
  const size_t r_other = (size_t)(need_prev ? r - 1 : (need_last ? r_last : r));
  const float* xr = x + (size_t)r * H;
  const float* xo = x + r_other * H;

  float a[VPT][4], b[VPT][4];
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int v = tid + k * SN_THREADS;
    if (v < nvec) {
      ldn<4>(xr + 4 * v, a[k]);
      if (add_a) {
        float p[4], q[4] = {0.f, 0.f, 0.f, 0.f};
        ldn<4>(add_a + (size_t)r * H + 4 * v, p);
        if (add_b) ldn<4>(add_b + (size_t)r * H + 4 * v, q);
#pragma unroll
        for (int e = 0; e < 4; ++e) a[k][e] += p[e] + q[e];
        stn<4>(x_out + (size_t)r * H + 4 * v, a[k]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) sa += a[k][e] * a[k][e];
      if (need_other) {
        ldn<4>(xo + 4 * v, b[k]);
        if (add_a) {  // the same sum the other row's workgroup stores
          float p[4], q[4] = {0.f, 0.f, 0.f, 0.f};
          ldn<4>(add_a + r_other * H + 4 * v, p);
          if (add_b) ldn<4>(add_b + r_other * H + 4 * v, q);
#pragma unroll
          for (int e = 0; e < 4; ++e) b[k][e] += p[e] + q[e];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) sb += b[k][e] * b[k][e];
      }
    }
  }
  sa = wave_reduce_sum(sa);
  sb = wave_reduce_sum(sb);
  const int wave = tid / WAVE_SIZE, lane = tid % WAVE_SIZE;
  if (lane == 0) {
    red[0][wave] = sa;
    red[1][wave] = sb;
  }
  __syncthreads();
  sa = 0.f;
  sb = 0.f;
#pragma unroll
  for (int w = 0; w < SN_THREADS / WAVE_SIZE; ++w) {
    sa += red[0][w];
    sb += red[1][w];
  }
  const float inv = 1.0f / sqrtf(sa / (float)H + eps);
  const float inv_o = need_other ? 1.0f / sqrtf(sb / (float)H + eps) : 0.f;
  float* st_row = shift ? state + (size_t)seg_slot[s] * H : nullptr;
  const bool fresh = seg_fresh[s] != 0;

#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int v = tid + k * SN_THREADS;
    if (v >= nvec) continue;
    float g[4], o[4], f[4];
    ldn<4>(w_mix + 4 * v, g);
    if (shift) {
      float m4[4], prev[4];
      ldn<4>(mu + 4 * v, m4);
      if (first) {
        if (fresh) {
#pragma unroll
          for (int e = 0; e < 4; ++e) prev[e] = 0.f;
        } else {
          ldn<4>(st_row + 4 * v, prev);
        }
        float keep[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          keep[e] = need_last ? b[k][e] * inv_o * (1.0f + g[e]) : a[k][e] * inv * (1.0f + g[e]);
        stn<4>(st_row + 4 * v, keep);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) prev[e] = b[k][e] * inv_o * (1.0f + g[e]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float h = a[k][e] * inv * (1.0f + g[e]);
        o[e] = h + (prev[e] - h) * m4[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = a[k][e] * inv * (1.0f + g[e]);
    }
    stn<4>(om + 4 * v, o);
    if (of) {
      ldn<4>(w_ff + 4 * v, f);
#pragma unroll
      for (int e = 0; e < 4; ++e) f[e] = a[k][e] * inv * (1.0f + f[e]);
      stn<4>(of + 4 * v, f);
    }
  }
}

// out = x / sqrt(mean(x^2) + eps) * (1 + w), fp32 rows -> storage type
template <typename T>
__global__ __launch_bounds__(SN_THREADS) void offset_rms_norm_kernel(
    T* __restrict__ out, const float* __restrict__ x, const T* __restrict__ w,
    float eps, int H) {
  __shared__ float red[17];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* xr = x + (size_t)r * H;
  float a = 0.f;
  for (int d = tid; d < H; d += SN_THREADS) a += xr[d] * xr[d];
  a = block_reduce_sum(a, red);
  const float inv = 1.0f / sqrtf(a / (float)H + eps);
  for (int d = tid; d < H; d += SN_THREADS)
    st(out + (size_t)r * H + d, xr[d] * inv * (1.0f + ld(w + d)));
}

// out = x + (a + b): the fp32 residual takes both branch outputs in one pass
// (out may be x itself)
template <typename T, int N>
__global__ void residual_add_kernel(float* out, const float* x, const T* __restrict__ a,
                                    const T* __restrict__ b, long n) {
  for (long i = (blockIdx.x * (long)blockDim.x + threadIdx.x) * N; i < n;
       i += gridDim.x * (long)blockDim.x * N) {
    float xv[N], av[N], bv[N];
    ldn<N>(x + i, xv);
    ldn<N>(a + i, av);
    if (b) ldn<N>(b + i, bv);
#pragma unroll
    for (int k = 0; k < N; ++k) xv[k] += b ? av[k] + bv[k] : av[k];
    stn<N>(out + i, xv);
  }
}

static void launch_residual_add(float* out, const float* x, const void* a, const void* b,
                                long n, int is_f32, hipStream_t s) {
  if (n <= 0) return;
  const bool v4 = n % 4 == 0 && aligned16(out) && aligned16(x) && aligned16(a) &&
                  (!b || aligned16(b));
  const long items = v4 ? n / 4 : n;
  long g = (items + 255) / 256;
  const int grid = (int)(g > 65535 ? 65535 : g);
#define LIG_RA(T, N)                                                            \
  hipLaunchKernelGGL((residual_add_kernel<T, N>), dim3(grid), dim3(256), 0, s,  \
                     out, x, (const T*)a, (const T*)b, n)
  if (is_f32) {
    if (v4) LIG_RA(float, 4); else LIG_RA(float, 1);
  } else {
    if (v4) LIG_RA(bf16s, 4); else LIG_RA(bf16s, 1);
  }
#undef LIG_RA
}

extern "C" {

// add_a (and add_b) non-null: x_out = x + (add_a + add_b) and the norms read
// x_out; x_out must be a buffer of its own.  add_a null: x_out is unused.
void lig_offset_norm_shift(void* h_mix, void* h_ff, const float* x,
                           const void* add_a, const void* add_b, float* x_out,
                           const void* w_mix, const void* w_ff, const void* mu,
                           float* state, const int* tok_seq, const int* seg_start,
                           const int* seg_len, const int* seg_slot,
                           const int* seg_fresh, float eps, int R, int H,
                           int is_f32, hipStream_t s) {
  if (R <= 0) return;
  const bool al = aligned16(h_mix) && aligned16(x) && aligned16(w_mix) && aligned16(state) &&
                  (!h_ff || (aligned16(h_ff) && aligned16(w_ff))) && (!mu || aligned16(mu)) &&
                  (!add_a || (aligned16(add_a) && aligned16(x_out))) && (!add_b || aligned16(add_b));
  if (H % 4 == 0 && H <= 4 * SN_THREADS * 8 && al) {
    const int vpt = (H / 4 + SN_THREADS - 1) / SN_THREADS;
#define LIG_SNV(T, V)                                                            \
  hipLaunchKernelGGL((offset_norm_shift_vec_kernel<T, V>), dim3(R),              \
                     dim3(SN_THREADS), 0, s, (T*)h_mix, (T*)h_ff, x,             \
                     (const T*)add_a, (const T*)add_b, x_out, (const T*)w_mix,   \
                     (const T*)w_ff, (const T*)mu, state, tok_seq, seg_start,    \
                     seg_len, seg_slot, seg_fresh, eps, H)
#define LIG_SNV_PICK(T)                                                          \
  do {                                                                           \
    if (vpt <= 1) LIG_SNV(T, 1);                                                 \
    else if (vpt <= 2) LIG_SNV(T, 2);                                            \
    else if (vpt <= 4) LIG_SNV(T, 4);                                            \
    else LIG_SNV(T, 8);                                                          \
  } while (0)
    if (is_f32) LIG_SNV_PICK(float); else LIG_SNV_PICK(bf16s);
#undef LIG_SNV_PICK
#undef LIG_SNV
    return;
  }
  // any width: the add as a pass of its own, then the scalar kernel
  if (add_a) {
    launch_residual_add(x_out, x, add_a, add_b, (long)R * H, is_f32, s);
    x = x_out;
  }
  if (is_f32)
    hipLaunchKernelGGL(offset_norm_shift_kernel<float>, dim3(R), dim3(SN_THREADS), 0, s,
                       (float*)h_mix, (float*)h_ff, x, (const float*)w_mix,
                       (const float*)w_ff, (const float*)mu, state, tok_seq,
                       seg_start, seg_len, seg_slot, seg_fresh, eps, H);
  else
    hipLaunchKernelGGL(offset_norm_shift_kernel<bf16s>, dim3(R), dim3(SN_THREADS), 0, s,
                       (bf16s*)h_mix, (bf16s*)h_ff, x, (const bf16s*)w_mix,
                       (const bf16s*)w_ff, (const bf16s*)mu, state, tok_seq,
                       seg_start, seg_len, seg_slot, seg_fresh, eps, H);
}

void lig_offset_rms_norm(void* out, const float* x, const void* w, float eps,
                         int R, int H, int is_f32, hipStream_t s) {
  if (R <= 0) return;
  if (is_f32)
    hipLaunchKernelGGL(offset_rms_norm_kernel<float>, dim3(R), dim3(SN_THREADS), 0, s,
                       (float*)out, x, (const float*)w, eps, H);
  else
    hipLaunchKernelGGL(offset_rms_norm_kernel<bf16s>, dim3(R), dim3(SN_THREADS), 0, s,
                       (bf16s*)out, x, (const bf16s*)w, eps, H);
}

void lig_residual_add(float* x, const void* a, const void* b, long n, int is_f32,
                      hipStream_t s) {
  launch_residual_add(x, x, a, b, n, is_f32, s);
}

}  // extern "C"

// Several blends of a row with the row before it in one pass over the fp32
// rows: out[m][r] = x[r] + (x_prev - x[r]) * mu[m].  Ahead of a segment's
// first row stands the sequence's state row (zeros when the sequence starts
// here).  The workgroup of a segment's FIRST row is the only one that touches
// the state: it reads it, and then stores the segment's last row there, so
// no other workgroup races with it.  Rows of no segment come out zero.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(
    T* __restrict__ out, const float* __restrict__ x, const T* __restrict__ mu,
    float* __restrict__ state, const int* __restrict__ tok_seq,
    const int* __restrict__ seg_start, const int* __restrict__ seg_len,
    const int* __restrict__ seg_slot, const int* __restrict__ seg_fresh,
    int n_mix, int R, int W) {
  const long r = blockIdx.x;
  const int seq = tok_seq[r];
  if (seq < 0) {
    for (int m = 0; m < n_mix; ++m)
      for (int c = threadIdx.x; c < W; c += blockDim.x)
        st(out + ((long)m * R + r) * W + c, 0.f);
    return;
  }
  const int s0 = seg_start[seq];
  const bool first = r == s0;
  const float* prev = nullptr;
  float* srow = state + (long)seg_slot[seq] * W;
  if (!first) prev = x + (r - 1) * W;
  else if (!seg_fresh[seq]) prev = srow;
  const float* last = x + ((long)s0 + seg_len[seq] - 1) * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float cur = x[r * W + c];
    const float d = (prev != nullptr ? prev[c] : 0.f) - cur;
    for (int m = 0; m < n_mix; ++m)
      st(out + ((long)m * R + r) * W + c, cur + d * ld(mu + (long)m * W + c));
    if (first) srow[c] = last[c];  // after this thread's own read of srow[c]
  }
}

// 8 elements per thread and access: W % 8 == 0, 16-byte aligned rows.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_mix_vec_kernel(
    T* __restrict__ out, const float* __restrict__ x, const T* __restrict__ mu,
    float* __restrict__ state, const int* __restrict__ tok_seq,
    const int* __restrict__ seg_start, const int* __restrict__ seg_len,
    const int* __restrict__ seg_slot, const int* __restrict__ seg_fresh,
    int n_mix, int R, int W) {
  const long r = blockIdx.x;
  const int seq = tok_seq[r];
  if (seq < 0) {
    float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int m = 0; m < n_mix; ++m)
      for (int c = threadIdx.x * 8; c < W; c += blockDim.x * 8)
        st8(out + ((long)m * R + r) * W + c, z);
    return;
  }
  const int s0 = seg_start[seq];
  const bool first = r == s0;
  const float* prev = nullptr;
  float* srow = state + (long)seg_slot[seq] * W;
  if (!first) prev = x + (r - 1) * W;
  else if (!seg_fresh[seq]) prev = srow;
  const float* last = x + ((long)s0 + seg_len[seq] - 1) * W;
  for (int c = threadIdx.x * 8; c < W; c += blockDim.x * 8) {
    float cur[8], d[8];
    ld8(x + r * W + c, cur);
    if (prev != nullptr) {
      ld8(prev + c, d);
#pragma unroll
      for (int i = 0; i < 8; ++i) d[i] -= cur[i];
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) d[i] = -cur[i];
    }
    for (int m = 0; m < n_mix; ++m) {
      float u[8];
      ld8(mu + (long)m * W + c, u);
#pragma unroll
      for (int i = 0; i < 8; ++i) u[i] = cur[i] + d[i] * u[i];
      st8(out + ((long)m * R + r) * W + c, u);
    }
    if (first) {  // after this thread's own read of srow[c..c+8)
      float l8[8];
      ld8(last + c, l8);
      st8(srow + c, l8);
    }
  }
}

extern "C" void lig_token_shift_mix(void* out, const float* x, const void* mu,
                                    float* state, const int* tok_seq,
                                    const int* seg_start, const int* seg_len,
                                    const int* seg_slot, const int* seg_fresh,
                                    int n_mix, int R, int W, int is_f32,
                                    hipStream_t s) {
  if (R <= 0 || W <= 0) return;
  if (W % 8 == 0 && aligned16(out) && aligned16(x) && aligned16(mu) && aligned16(state)) {
    if (is_f32)
      hipLaunchKernelGGL(token_shift_mix_vec_kernel<float>, dim3(R), dim3(256), 0, s,
                         (float*)out, x, (const float*)mu, state, tok_seq, seg_start,
                         seg_len, seg_slot, seg_fresh, n_mix, R, W);
    else
      hipLaunchKernelGGL(token_shift_mix_vec_kernel<bf16s>, dim3(R), dim3(256), 0, s,
                         (bf16s*)out, x, (const bf16s*)mu, state, tok_seq, seg_start,
                         seg_len, seg_slot, seg_fresh, n_mix, R, W);
    return;
  }
  if (is_f32)
    hipLaunchKernelGGL(token_shift_mix_kernel<float>, dim3(R), dim3(256), 0, s,
                       (float*)out, x, (const float*)mu, state, tok_seq, seg_start,
                       seg_len, seg_slot, seg_fresh, n_mix, R, W);
  else
    hipLaunchKernelGGL(token_shift_mix_kernel<bf16s>, dim3(R), dim3(256), 0, s,
                       (bf16s*)out, x, (const bf16s*)mu, state, tok_seq, seg_start,
                       seg_len, seg_slot, seg_fresh, n_mix, R, W);
}
