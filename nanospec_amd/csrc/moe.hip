// A mixture of small gated feed-forward experts, and the per-layer token input of a decoder that has one.
//
// Router: z = W_r h + b in 32-bit; the ``top`` largest logits are chosen (the lower index wins a tie) and weighted by the
// soft-max over the chosen logits alone.
// Expert (``clipped GLU``): g = min(W_gate h, limit); u = clamp(W_up h, -limit, limit); y = W_down (g sigmoid(alpha g) (u + 1)).
// The experts' matrices are stacked: gate and up [experts][ff][W], down [experts][W][ff].
#include "common.h"

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 32

// One workgroup a token: every wave takes experts in turn, its lanes share the row; thread 0 then chooses.
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ h, int h_stride, const float* __restrict__ wr,
                                                        const float* __restrict__ br, int* __restrict__ sel, float* __restrict__ wt,
                                                        int W, int experts, int top) {
  __shared__ float z[MOE_MAX_EXPERTS];
  const int t = blockIdx.x, lane = threadIdx.x % NS_WAVE, wave = threadIdx.x / NS_WAVE, waves = blockDim.x / NS_WAVE;
  const T* x = h + (size_t)t * h_stride;
  for (int e = wave; e < experts; e += waves) {
    const float* w = wr + (size_t)e * W;
    float acc = 0.f;
    for (int c = lane; c < W; c += NS_WAVE) acc = fmaf(to_f(x[c]), w[c], acc);
    acc = wave_sum(acc);
    if (lane == 0) z[e] = acc + (br ? br[e] : 0.f);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int idx[MOE_MAX_TOP];
    float val[MOE_MAX_TOP];
    for (int k = 0; k < top; ++k) {
      int best = -1;
      float bv = -INFINITY;
      for (int e = 0; e < experts; ++e) {
        bool taken = false;
        for (int j = 0; j < k; ++j) taken |= idx[j] == e;
        if (!taken && (best < 0 || z[e] > bv)) best = e, bv = z[e];
      }
      idx[k] = best, val[k] = bv;
    }
    float sum = 0.f;
    const float largest = val[0];
    for (int k = 0; k < top; ++k) {
      val[k] = expf(val[k] - largest);
      sum += val[k];
    }
    for (int k = 0; k < top; ++k) {
      sel[(size_t)t * top + k] = idx[k];
      wt[(size_t)t * top + k] = val[k] / sum;
    }
  }
}

extern "C" int ns_moe_route(const void* h, int h_stride, const float* wr, const float* br, int* sel, float* wt, int n, int W, int experts,
                            int top, int dtype, hipStream_t stream) {
  if (n <= 0 || W <= 0 || experts <= 0 || experts > MOE_MAX_EXPERTS || top <= 0 || top > MOE_MAX_TOP || top > experts) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    moe_route_kernel<float><<<n, 256, 0, stream>>>((const float*)h, h_stride, wr, br, sel, wt, W, experts, top);
  else if (dtype == NS_DTYPE_BF16)
    moe_route_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)h, h_stride, wr, br, sel, wt, W, experts, top);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

__device__ __forceinline__ float clipped_glu(float g, float u, float limit, float alpha) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + 1.f);
}

// One workgroup a (token, chosen expert): the row in LDS, a wave an inner channel in turn (gate and up together), then a
// wave an output channel in turn.  out [tokens][top][W] in 32-bit, already times the router's weight.
template <typename T>
__global__ __launch_bounds__(256) void moe_expert_rows_kernel(const T* __restrict__ h, int h_stride, const T* __restrict__ wg,
                                                              const T* __restrict__ wu, const T* __restrict__ wd, const int* __restrict__ sel,
                                                              const float* __restrict__ wt, float* __restrict__ out, int W, int ff, int top,
                                                              float limit, float alpha) {
  extern __shared__ float moe_lds[];
  float* x = moe_lds;      // [W]
  float* act = x + W;      // [ff]
  const int t = blockIdx.x, k = blockIdx.y, lane = threadIdx.x % NS_WAVE, wave = threadIdx.x / NS_WAVE, waves = blockDim.x / NS_WAVE;
  const int e = sel[(size_t)t * top + k];
  const float share = wt[(size_t)t * top + k];
  for (int c = threadIdx.x; c < W; c += blockDim.x) x[c] = to_f(h[(size_t)t * h_stride + c]);
  __syncthreads();
  const T* g_rows = wg + (size_t)e * ff * W;
  const T* u_rows = wu + (size_t)e * ff * W;
  for (int f = wave; f < ff; f += waves) {
    const T* gr = g_rows + (size_t)f * W;
    const T* ur = u_rows + (size_t)f * W;
    float g = 0.f, u = 0.f;
    for (int c = lane; c < W; c += NS_WAVE) {
      g = fmaf(to_f(gr[c]), x[c], g);
      u = fmaf(to_f(ur[c]), x[c], u);
    }
    g = wave_sum(g), u = wave_sum(u);
    if (lane == 0) act[f] = round_to<T>(clipped_glu(round_to<T>(g), round_to<T>(u), limit, alpha));
  }
  __syncthreads();
  const T* d_rows = wd + (size_t)e * W * ff;
  for (int c = wave; c < W; c += waves) {
    const T* dr = d_rows + (size_t)c * ff;
    float y = 0.f;
    for (int f = lane; f < ff; f += NS_WAVE) y = fmaf(to_f(dr[f]), act[f], y);
    y = wave_sum(y);
    if (lane == 0) out[((size_t)t * top + k) * W + c] = share * y;
  }
}

extern "C" int ns_moe_expert_rows(const void* h, int h_stride, const void* wg, const void* wu, const void* wd, const int* sel, const float* wt,
                                  float* out, int n, int W, int ff, int top, float limit, float alpha, int dtype, hipStream_t stream) {
  if (n <= 0 || W <= 0 || ff <= 0 || top <= 0 || top > 65535) return NS_ERR_BAD_ARG;
  const size_t lds = (size_t)(W + ff) * sizeof(float);
  if (lds > 64 * 1024) return NS_ERR_UNSUPPORTED;
  dim3 grid(n, top);
  if (dtype == NS_DTYPE_F32)
    moe_expert_rows_kernel<float><<<grid, 256, lds, stream>>>((const float*)h, h_stride, (const float*)wg, (const float*)wu, (const float*)wd, sel,
                                                               wt, out, W, ff, top, limit, alpha);
  else if (dtype == NS_DTYPE_BF16)
    moe_expert_rows_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)h, h_stride, (const bf16_t*)wg, (const bf16_t*)wu, (const bf16_t*)wd,
                                                                sel, wt, out, W, ff, top, limit, alpha);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// out[t][f] = clipped_glu(gu[t][f], gu[t][ff + f]) for the result of a product with the stacked [gate; up] matrix
template <typename T>
__global__ void clipped_glu_kernel(T* __restrict__ out, const T* __restrict__ gu, int gu_stride, int ff, size_t count, float limit, float alpha) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / ff, f = i % ff;
    out[i] = from_f<T>(clipped_glu(to_f(gu[t * gu_stride + f]), to_f(gu[t * gu_stride + ff + f]), limit, alpha));
  }
}

extern "C" int ns_clipped_glu(void* out, const void* gu, int gu_stride, int n, int ff, float limit, float alpha, int dtype, hipStream_t stream) {
  if (n <= 0 || ff <= 0) return NS_ERR_BAD_ARG;
  const size_t count = (size_t)n * ff;
  size_t blocks = (count + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  if (dtype == NS_DTYPE_F32)
    clipped_glu_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)gu, gu_stride, ff, count, limit, alpha);
  else if (dtype == NS_DTYPE_BF16)
    clipped_glu_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, gu_stride, ff, count, limit, alpha);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// out[t][c] = (base ? base[t][c] : 0) + sum_k parts[t][k][c], in a fixed order
template <typename T>
__global__ void moe_combine_kernel(T* __restrict__ out, const T* __restrict__ base, const float* __restrict__ parts, int top, int W, size_t count) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / W, c = i % W;
    float acc = 0.f;
    for (int k = 0; k < top; ++k) acc += parts[(t * top + k) * W + c];
    out[i] = from_f<T>(acc + (base ? to_f(base[i]) : 0.f));
  }
}

extern "C" int ns_moe_combine(void* out, const void* base, const float* parts, int n, int top, int W, int dtype, hipStream_t stream) {
  if (n <= 0 || top <= 0 || W <= 0) return NS_ERR_BAD_ARG;
  const size_t count = (size_t)n * W;
  size_t blocks = (count + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  if (dtype == NS_DTYPE_F32)
    moe_combine_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)base, parts, top, W, count);
  else if (dtype == NS_DTYPE_BF16)
    moe_combine_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)base, parts, top, W, count);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// out = sa * (a + bias_a) + sb * (b + bias_b) in 32-bit: two mixers side by side, each with a weight (the biases: a mixer's
// last bias that it left to its caller; either may be null)
template <typename T>
__global__ void scaled_sum_kernel(T* __restrict__ out, const T* __restrict__ a, const T* __restrict__ b, const T* __restrict__ bias,
                                  const T* __restrict__ bias_b, float sa, float sb, int W, size_t count) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    const float av = to_f(a[i]) + (bias ? to_f(bias[i % W]) : 0.f);
    const float bv = to_f(b[i]) + (bias_b ? to_f(bias_b[i % W]) : 0.f);
    out[i] = from_f<T>(sa * av + sb * bv);
  }
}

extern "C" int ns_scaled_sum(void* out, const void* a, const void* b, const void* bias, const void* bias_b, float sa, float sb, int n, int W,
                             int dtype, hipStream_t stream) {
  if (n <= 0 || W <= 0) return NS_ERR_BAD_ARG;
  const size_t count = (size_t)n * W;
  size_t blocks = (count + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  if (dtype == NS_DTYPE_F32)
    scaled_sum_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)a, (const float*)b, (const float*)bias, (const float*)bias_b, sa, sb, W, count);
  else if (dtype == NS_DTYPE_BF16)
    scaled_sum_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)bias, (const bf16_t*)bias_b, sa, sb, W, count);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// The per-layer token input: y = W_proj (gelu_tanh(W_gate x) * e) with e = table[token] (this layer's ``dim`` columns of a
// row).  One workgroup a token: a wave a gate channel in turn, then a thread an output channel.
template <typename T>
__global__ __launch_bounds__(256) void token_side_kernel(T* __restrict__ out, const T* __restrict__ x, int x_stride, const int* __restrict__ ids,
                                                         const T* __restrict__ table, const T* __restrict__ wg, const T* __restrict__ wp, int W,
                                                         int dim) {
  extern __shared__ float side_lds[];  // [dim]
  const int t = blockIdx.x, lane = threadIdx.x % NS_WAVE, wave = threadIdx.x / NS_WAVE, waves = blockDim.x / NS_WAVE;
  const T* xr = x + (size_t)t * x_stride;
  const T* e = table + (size_t)ids[t] * dim;
  for (int j = wave; j < dim; j += waves) {
    const T* w = wg + (size_t)j * W;
    float acc = 0.f;
    for (int c = lane; c < W; c += NS_WAVE) acc = fmaf(to_f(w[c]), to_f(xr[c]), acc);
    acc = round_to<T>(wave_sum(acc));
    if (lane == 0) {
      const float gl = 0.5f * acc * (1.f + tanhf(0.7978845608028654f * (acc + 0.044715f * acc * acc * acc)));
      side_lds[j] = round_to<T>(round_to<T>(gl) * to_f(e[j]));
    }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const T* w = wp + (size_t)c * dim;
    float acc = 0.f;
    for (int j = 0; j < dim; ++j) acc = fmaf(to_f(w[j]), side_lds[j], acc);
    out[(size_t)t * W + c] = from_f<T>(acc);
  }
}

extern "C" int ns_token_side(void* out, const void* x, int x_stride, const int* ids, const void* table, const void* wg, const void* wp, int n,
                             int W, int dim, int dtype, hipStream_t stream) {
  if (n <= 0 || W <= 0 || dim <= 0 || dim > 8192) return NS_ERR_BAD_ARG;
  const size_t lds = (size_t)dim * sizeof(float);
  if (dtype == NS_DTYPE_F32)
    token_side_kernel<float><<<n, 256, lds, stream>>>((float*)out, (const float*)x, x_stride, ids, (const float*)table, (const float*)wg,
                                                       (const float*)wp, W, dim);
  else if (dtype == NS_DTYPE_BF16)
    token_side_kernel<bf16_t><<<n, 256, lds, stream>>>((bf16_t*)out, (const bf16_t*)x, x_stride, ids, (const bf16_t*)table, (const bf16_t*)wg,
                                                        (const bf16_t*)wp, W, dim);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
