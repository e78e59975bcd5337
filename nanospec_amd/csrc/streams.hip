// A residual stream that is kept in 32-bit whatever the model computes in, and that may be several parallel streams
// (hyper-connections): x [tokens][S][W], float.  A sublayer reads one mix of the streams through an RMS norm and
// writes its output back into all of them while the streams are mixed among themselves:
//   read:   u = sum_s a[s] x_s;            h = w * u / sqrt(mean(u^2) + eps)      (h in the model's precision; without a
//                                                                                   weight h = u: the sublayer reads the stream itself)
//   write:  x_t <- sum_s M[s][t] x_s + c[t] y     for all t at once, from the old streams
// S = 1 with a = M = 1 is the plain pre-norm residual x <- x + c y with its sum in 32-bit.
// Two options on either side.  A norm's stored weight may be the factor minus one: the factor is then ``w_offset`` + w with
// w_offset = 1, formed in 32-bit (0 leaves the weight as it is).  A sublayer's output may pass a bias and an RMS norm of
// its own on its way into the streams (a block with norms on both sides of a sublayer):
//   y' = (y + bias) / sqrt(mean((y + bias)^2) + eps_y) * (yw_offset + yw),   then the write with y' in place of y.
#include "common.h"

// what happens to a sublayer's output before it is written; every pointer may be null
struct StreamPost {
  const void* bias;  // [W] in the type of y
  const void* yw;    // [W] in the type of y: the weight of the norm behind the sublayer
  float y_eps, yw_offset;
};

#define NS_MAX_STREAMS 16

// out[i][s][:] = table[ids[i]][:] * scale for every copy s
template <typename T>
__global__ void embed_streams_kernel(float* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids, int hidden,
                                     int copies, float scale) {
  const int row = blockIdx.x;
  const T* src = table + (size_t)ids[row] * hidden;
  float* dst = out + (size_t)row * copies * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = to_f(src[i]) * scale;
    for (int s = 0; s < copies; ++s) dst[(size_t)s * hidden + i] = v;
  }
}

extern "C" int ns_embed_streams(float* out, const void* table, const int* ids, int n_tokens, int hidden, int copies, float scale,
                                int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || hidden <= 0 || copies <= 0 || copies > NS_MAX_STREAMS) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    embed_streams_kernel<float><<<n_tokens, 256, 0, stream>>>(out, (const float*)table, ids, hidden, copies, scale);
  else if (dtype == NS_DTYPE_BF16)
    embed_streams_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(out, (const bf16_t*)table, ids, hidden, copies, scale);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// The same with a second table added, whose row is chosen by the token and the token before it in its sequence:
//   row = (prev * mul_prev + token * mul_cur) mod buckets;   a sequence's first token (position 0) takes row ``buckets``.
// The token before a step's first token of a request is part of the request's state: ``last_token`` [slots] holds the last
// token every request has brought so far.  The workgroup of a request's first row of this step reads it and then leaves
// the request's last token of this step there; nobody else touches that slot's word.
template <typename T>
__global__ void embed_pair_streams_kernel(float* __restrict__ out, const T* __restrict__ table, const T* __restrict__ pair_table,
                                          const int* __restrict__ ids, const int* __restrict__ positions, const int* __restrict__ token_req,
                                          const int* __restrict__ qo_indptr, const int* __restrict__ state_slots, int* __restrict__ last_token,
                                          int hidden, int copies, float scale, int buckets, int mul_prev, int mul_cur) {
  __shared__ int pair_row;
  const int row = blockIdx.x;
  const int tok = ids[row];
  if (threadIdx.x == 0) {
    const int b = token_req[row], first = qo_indptr[b], pos = positions[row];
    int prev = 0;
    if (row == first) {
      int* word = last_token + state_slots[b];
      prev = *word;
      const int last = qo_indptr[b + 1] - 1;
      if (last >= first) *word = ids[last];
    } else {
      prev = ids[row - 1];
    }
    long long v = ((long long)prev * mul_prev + (long long)tok * mul_cur) % buckets;
    if (v < 0) v += buckets;
    pair_row = pos == 0 ? buckets : (int)v;
  }
  __syncthreads();
  const T* src = table + (size_t)tok * hidden;
  const T* src2 = pair_table + (size_t)pair_row * hidden;
  float* dst = out + (size_t)row * copies * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = to_f(src[i]) * scale + to_f(src2[i]);
    for (int s = 0; s < copies; ++s) dst[(size_t)s * hidden + i] = v;
  }
}

extern "C" int ns_embed_pair_streams(float* out, const void* table, const void* pair_table, const int* ids, const int* positions,
                                     const int* token_req, const int* qo_indptr, const int* state_slots, int* last_token, int n_tokens,
                                     int hidden, int copies, float scale, int buckets, int mul_prev, int mul_cur, int dtype,
                                     hipStream_t stream) {
  if (n_tokens <= 0 || hidden <= 0 || copies <= 0 || copies > NS_MAX_STREAMS || buckets <= 0) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    embed_pair_streams_kernel<float><<<n_tokens, 256, 0, stream>>>(out, (const float*)table, (const float*)pair_table, ids, positions, token_req,
                                                                   qo_indptr, state_slots, last_token, hidden, copies, scale, buckets, mul_prev, mul_cur);
  else if (dtype == NS_DTYPE_BF16)
    embed_pair_streams_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(out, (const bf16_t*)table, (const bf16_t*)pair_table, ids, positions, token_req,
                                                                    qo_indptr, state_slots, last_token, hidden, copies, scale, buckets, mul_prev, mul_cur);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// One workgroup a row.  The mix u is formed twice (once for the sum of squares, once for the output) in the same order,
// so a row costs two reads of S*W floats from cache and no scratch.  ``sum_out`` (optional): the mix itself, float.
template <typename T>
__global__ void stream_read_norm_kernel(T* __restrict__ out, float* __restrict__ sum_out, const float* __restrict__ x,
                                        const float* __restrict__ coeff, const T* __restrict__ w, const int* __restrict__ rows, int S,
                                        int W, float eps, float w_offset) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  const float* xr = x + r * S * W;
  float a[NS_MAX_STREAMS];
  for (int s = 0; s < S; ++s) a[s] = coeff[s];
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u = fmaf(a[s], xr[(size_t)s * W + c], u);
    ss = fmaf(u, u, ss);
  }
  ss = block_sum(ss, scratch);
  const float rinv = w ? 1.f / sqrtf(ss / (float)W + eps) : 1.f;  // no weight: no norm, the mix itself is read
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u = fmaf(a[s], xr[(size_t)s * W + c], u);
    if (sum_out) sum_out[(size_t)i * W + c] = u;
    if (out) out[(size_t)i * W + c] = from_f<T>(w ? u * rinv * (w_offset + to_f(w[c])) : u);
  }
}

extern "C" int ns_stream_read_norm(void* out, float* sum_out, const float* x, const float* coeff, const void* w, const int* rows,
                                   int n, int S, int W, float eps, float w_offset, int dtype, hipStream_t stream) {
  if (n <= 0 || S <= 0 || S > NS_MAX_STREAMS || W <= 0) return NS_ERR_BAD_ARG;
  const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
  if (dtype == NS_DTYPE_F32)
    stream_read_norm_kernel<float><<<n, threads, 0, stream>>>((float*)out, sum_out, x, coeff, (const float*)w, rows, S, W, eps, w_offset);
  else if (dtype == NS_DTYPE_BF16)
    stream_read_norm_kernel<bf16_t><<<n, threads, 0, stream>>>((bf16_t*)out, sum_out, x, coeff, (const bf16_t*)w, rows, S, W, eps, w_offset);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// In place: a thread owns a column of a row, reads its S old values, then writes the S new ones.
template <typename T>
__global__ void stream_write_kernel(float* __restrict__ x, const float* __restrict__ mix, const float* __restrict__ gain,
                                    const T* __restrict__ y, int y_stride, int S, int W) {
  __shared__ float m_s[NS_MAX_STREAMS * NS_MAX_STREAMS + NS_MAX_STREAMS];
  for (int i = threadIdx.x; i < S * S + S; i += blockDim.x) m_s[i] = i < S * S ? mix[i] : gain[i - S * S];
  __syncthreads();
  const size_t r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  float* xr = x + r * S * W + c;
  float old[NS_MAX_STREAMS];
  for (int s = 0; s < S; ++s) old[s] = xr[(size_t)s * W];
  const float yv = to_f(y[r * y_stride + c]);
  for (int t = 0; t < S; ++t) {
    float v = 0.f;
    for (int s = 0; s < S; ++s) v = fmaf(m_s[s * S + t], old[s], v);
    xr[(size_t)t * W] = fmaf(m_s[S * S + t], yv, v);
  }
}

extern "C" int ns_stream_write(float* x, const float* mix, const float* gain, const void* y, int y_stride, int n, int S, int W,
                               int dtype, hipStream_t stream) {
  if (n <= 0 || S <= 0 || S > NS_MAX_STREAMS || W <= 0 || (W + 255) / 256 > 65535) return NS_ERR_BAD_ARG;
  dim3 grid(n, (W + 255) / 256);
  if (dtype == NS_DTYPE_F32)
    stream_write_kernel<float><<<grid, 256, 0, stream>>>(x, mix, gain, (const float*)y, y_stride, S, W);
  else if (dtype == NS_DTYPE_BF16)
    stream_write_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, mix, gain, (const bf16_t*)y, y_stride, S, W);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// The write with a bias and / or a norm of the sublayer's output before it: one workgroup a row, the row of y read twice.
template <typename T>
__global__ void stream_write_post_kernel(float* __restrict__ x, const float* __restrict__ mix, const float* __restrict__ gain,
                                         const T* __restrict__ y, int y_stride, int S, int W, StreamPost post) {
  __shared__ float m_s[NS_MAX_STREAMS * NS_MAX_STREAMS + NS_MAX_STREAMS];
  __shared__ float scratch[16];
  for (int i = threadIdx.x; i < S * S + S; i += blockDim.x) m_s[i] = i < S * S ? mix[i] : gain[i - S * S];
  const size_t r = blockIdx.x;
  const T* yr = y + r * y_stride;
  const T* bias = (const T*)post.bias;
  const T* yw = (const T*)post.yw;
  float rinv = 1.f;
  if (yw) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      const float v = to_f(yr[c]) + (bias ? to_f(bias[c]) : 0.f);
      ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    rinv = 1.f / sqrtf(ss / (float)W + post.y_eps);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float* xr = x + r * S * W + c;
    float old[NS_MAX_STREAMS];
    for (int s = 0; s < S; ++s) old[s] = xr[(size_t)s * W];
    float yv = to_f(yr[c]) + (bias ? to_f(bias[c]) : 0.f);
    if (yw) yv = yv * rinv * (post.yw_offset + to_f(yw[c]));
    for (int t = 0; t < S; ++t) {
      float v = 0.f;
      for (int s = 0; s < S; ++s) v = fmaf(m_s[s * S + t], old[s], v);
      xr[(size_t)t * W] = fmaf(m_s[S * S + t], yv, v);
    }
  }
}

extern "C" int ns_stream_write_post(float* x, const float* mix, const float* gain, const void* y, int y_stride, int n, int S, int W,
                                    const void* bias, const void* yw, float y_eps, float yw_offset, int dtype, hipStream_t stream) {
  if (n <= 0 || S <= 0 || S > NS_MAX_STREAMS || W <= 0) return NS_ERR_BAD_ARG;
  const StreamPost post{bias, yw, y_eps, yw_offset};
  const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
  if (dtype == NS_DTYPE_F32)
    stream_write_post_kernel<float><<<n, threads, 0, stream>>>(x, mix, gain, (const float*)y, y_stride, S, W, post);
  else if (dtype == NS_DTYPE_BF16)
    stream_write_post_kernel<bf16_t><<<n, threads, 0, stream>>>(x, mix, gain, (const bf16_t*)y, y_stride, S, W, post);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// The two in one pass with 16-byte accesses, for S <= 4 streams and rows of a multiple of four up to 8,192 columns: the
// write of one sublayer's output (``y`` given) followed by the read for the next sublayer (``coeff`` given), each
// optional.  A thread keeps its columns of the mix u in registers between the sum of squares and the output, so a row is
// read once.  ``store`` = 0 leaves x as it was (the last read of a step, whose written streams nobody reads again).
template <typename T, int S, int KMAX>
__global__ __launch_bounds__(256) void stream_step_kernel(float* __restrict__ x, const float* __restrict__ mix, const float* __restrict__ gain,
                                                          const T* __restrict__ y, int y_stride, const float* __restrict__ coeff,
                                                          const T* __restrict__ w, const int* __restrict__ rows, T* __restrict__ out,
                                                          float* __restrict__ sum_out, int W, float eps, int store, float w_offset,
                                                          StreamPost post) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  float* xr = x + r * S * W;
  const T* bias = (const T*)post.bias;
  const T* yw = (const T*)post.yw;
  float y_rinv = 1.f;
  if (y && yw) {  // the norm behind the sublayer wants the row's sum of squares first
    float ssy = 0.f;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int c = (threadIdx.x + k * 256) * 4;
      if (c < W) {
        const T* yp = y + r * y_stride + c;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float v = to_f(yp[e]) + (bias ? to_f(bias[c + e]) : 0.f);
          ssy = fmaf(v, v, ssy);
        }
      }
    }
    ssy = block_sum(ssy, scratch);
    y_rinv = 1.f / sqrtf(ssy / (float)W + post.y_eps);
  }
  float m[S][S], gn[S], a[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    gn[s] = y ? gain[s] : 0.f;
    a[s] = coeff ? coeff[s] : 0.f;
#pragma unroll
    for (int t = 0; t < S; ++t) m[s][t] = y ? mix[s * S + t] : (s == t ? 1.f : 0.f);
  }
  float4 u[KMAX];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int c = (threadIdx.x + k * 256) * 4;
    if (c < W) {
      float4 v[S];
#pragma unroll
      for (int s = 0; s < S; ++s) v[s] = *reinterpret_cast<const float4*>(xr + (size_t)s * W + c);
      if (y) {
        const T* yp = y + r * y_stride + c;
        float4 yv = {to_f(yp[0]), to_f(yp[1]), to_f(yp[2]), to_f(yp[3])};
        if (bias) yv.x += to_f(bias[c]), yv.y += to_f(bias[c + 1]), yv.z += to_f(bias[c + 2]), yv.w += to_f(bias[c + 3]);
        if (yw) {
          yv.x *= y_rinv * (post.yw_offset + to_f(yw[c])), yv.y *= y_rinv * (post.yw_offset + to_f(yw[c + 1]));
          yv.z *= y_rinv * (post.yw_offset + to_f(yw[c + 2])), yv.w *= y_rinv * (post.yw_offset + to_f(yw[c + 3]));
        }
        float4 nv[S];
#pragma unroll
        for (int t = 0; t < S; ++t) {
          float4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < S; ++s) {
            acc.x = fmaf(m[s][t], v[s].x, acc.x), acc.y = fmaf(m[s][t], v[s].y, acc.y);
            acc.z = fmaf(m[s][t], v[s].z, acc.z), acc.w = fmaf(m[s][t], v[s].w, acc.w);
          }
          nv[t] = {fmaf(gn[t], yv.x, acc.x), fmaf(gn[t], yv.y, acc.y), fmaf(gn[t], yv.z, acc.z), fmaf(gn[t], yv.w, acc.w)};
        }
#pragma unroll
        for (int t = 0; t < S; ++t) {
          v[t] = nv[t];
          if (store) *reinterpret_cast<float4*>(xr + (size_t)t * W + c) = nv[t];
        }
      }
      float4 mixv = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < S; ++s) {
        mixv.x = fmaf(a[s], v[s].x, mixv.x), mixv.y = fmaf(a[s], v[s].y, mixv.y);
        mixv.z = fmaf(a[s], v[s].z, mixv.z), mixv.w = fmaf(a[s], v[s].w, mixv.w);
      }
      u[k] = mixv;
      ss += mixv.x * mixv.x + mixv.y * mixv.y + mixv.z * mixv.z + mixv.w * mixv.w;
    }
  }
  if (!coeff) return;
  if (w) ss = block_sum(ss, scratch);
  const float rinv = w ? 1.f / sqrtf(ss / (float)W + eps) : 1.f;  // no weight: no norm, the mix itself is read
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int c = (threadIdx.x + k * 256) * 4;
    if (c < W) {
      if (sum_out) *reinterpret_cast<float4*>(sum_out + (size_t)i * W + c) = u[k];
      if (out && w) {
        T* op = out + (size_t)i * W + c;
        op[0] = from_f<T>(u[k].x * rinv * (w_offset + to_f(w[c]))), op[1] = from_f<T>(u[k].y * rinv * (w_offset + to_f(w[c + 1])));
        op[2] = from_f<T>(u[k].z * rinv * (w_offset + to_f(w[c + 2]))), op[3] = from_f<T>(u[k].w * rinv * (w_offset + to_f(w[c + 3])));
      } else if (out) {
        T* op = out + (size_t)i * W + c;
        op[0] = from_f<T>(u[k].x), op[1] = from_f<T>(u[k].y), op[2] = from_f<T>(u[k].z), op[3] = from_f<T>(u[k].w);
      }
    }
  }
}

template <typename T, int S>
static void stream_step_launch(float* x, const float* mix, const float* gain, const void* y, int y_stride, const float* coeff, const void* w,
                               const int* rows, void* out, float* sum_out, int n, int W, float eps, int store, float w_offset,
                               StreamPost post, hipStream_t stream) {
  if (W <= 2048)
    stream_step_kernel<T, S, 2><<<n, 256, 0, stream>>>(x, mix, gain, (const T*)y, y_stride, coeff, (const T*)w, rows, (T*)out, sum_out, W, eps, store, w_offset, post);
  else
    stream_step_kernel<T, S, 8><<<n, 256, 0, stream>>>(x, mix, gain, (const T*)y, y_stride, coeff, (const T*)w, rows, (T*)out, sum_out, W, eps, store, w_offset, post);
}

extern "C" int ns_stream_step(float* x, const float* mix, const float* gain, const void* y, int y_stride, const float* coeff, const void* w,
                              const int* rows, void* out, float* sum_out, int n, int S, int W, float eps, int store, float w_offset,
                              const void* bias, const void* yw, float y_eps, float yw_offset, int dtype, hipStream_t stream) {
  const StreamPost post{bias, yw, y_eps, yw_offset};
  if (n <= 0 || S <= 0 || S > 4 || W <= 0 || W > 8192 || W % 4 || (!y && !coeff)) return NS_ERR_BAD_ARG;
  if (y && (!mix || !gain)) return NS_ERR_BAD_ARG;
  if (y && rows && store) return NS_ERR_BAD_ARG;  // a write that is kept covers every row
  if (dtype != NS_DTYPE_F32 && dtype != NS_DTYPE_BF16) return NS_ERR_UNSUPPORTED;
#define NS_STEP(SS)                                                                                                                  \
  if (dtype == NS_DTYPE_F32) stream_step_launch<float, SS>(x, mix, gain, y, y_stride, coeff, w, rows, out, sum_out, n, W, eps, store, w_offset, post, stream); \
  else stream_step_launch<bf16_t, SS>(x, mix, gain, y, y_stride, coeff, w, rows, out, sum_out, n, W, eps, store, w_offset, post, stream)
  switch (S) {
    case 1: NS_STEP(1); break;
    case 2: NS_STEP(2); break;
    case 3: NS_STEP(3); break;
    default: NS_STEP(4); break;
  }
#undef NS_STEP
  return ns_launch_status();
}

// out = act(x), element by element; act 0: the tanh form of GELU, 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))); 1: SiLU
template <typename T>
__global__ void activation_kernel(T* __restrict__ out, const T* __restrict__ x, size_t count, int act) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    const float z = to_f(x[i]);
    float v;
    if (act == 0)
      v = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    else
      v = z / (1.f + expf(-z));
    out[i] = from_f<T>(v);
  }
}

__device__ __forceinline__ float act_of(float z, int act) {
  return act == 0 ? 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))) : z / (1.f + expf(-z));
}

// The same with 16-byte accesses, for counts that are a multiple of 16 bytes' worth and aligned pointers.
template <typename T>
__global__ void activation_vec_kernel(T* __restrict__ out, const T* __restrict__ x, size_t nvec, int act) {
  constexpr int V = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const vec_t* xv = reinterpret_cast<const vec_t*>(x);
  vec_t* ov = reinterpret_cast<vec_t*>(out);
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (size_t)gridDim.x * blockDim.x) {
    const vec_t a = xv[i];
    vec_t r;
#pragma unroll
    for (int e = 0; e < V; ++e) r[e] = from_f<T>(act_of(to_f(a[e]), act));
    ov[i] = r;
  }
}

extern "C" int ns_activation(void* out, const void* x, size_t count, int act, int dtype, hipStream_t stream) {
  if (count == 0 || act < 0 || act > 1) return NS_ERR_BAD_ARG;
  if (dtype != NS_DTYPE_F32 && dtype != NS_DTYPE_BF16) return NS_ERR_UNSUPPORTED;
  const size_t per = dtype == NS_DTYPE_F32 ? 4 : 8;
  if (count % per == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)x % 16) == 0) {
    const size_t nvec = count / per;
    size_t blocks = (nvec + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    if (dtype == NS_DTYPE_F32)
      activation_vec_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)x, nvec, act);
    else
      activation_vec_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, nvec, act);
    return ns_launch_status();
  }
  size_t blocks = (count + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  if (dtype == NS_DTYPE_F32)
    activation_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)x, count, act);
  else
    activation_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, count, act);
  return ns_launch_status();
}

// What a pass over a range of layers that runs several times adds to the streams in front of it:
//   x[r][s][:] += scale * table[ids[r]][:]  (the embedding's output again, if ``table``)  +  vec[:]  (if ``vec``)
// for every copy s, in 32-bit.  ``table`` and ``vec`` are in the model's storage type.
template <typename T>
__global__ void stream_add_rows_kernel(float* __restrict__ x, const T* __restrict__ table, const int* __restrict__ ids, const T* __restrict__ vec,
                                       int hidden, int copies, float scale) {
  const int row = blockIdx.x;
  const T* src = table ? table + (size_t)ids[row] * hidden : nullptr;
  float* dst = x + (size_t)row * copies * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    // (the two terms are added to the stream one after the other, as they are defined)
    const float e = src ? to_f(src[i]) * scale : 0.f, v = vec ? to_f(vec[i]) : 0.f;
    for (int s = 0; s < copies; ++s) {
      float cur = dst[(size_t)s * hidden + i];
      if (src) cur += e;
      if (vec) cur += v;
      dst[(size_t)s * hidden + i] = cur;
    }
  }
}

extern "C" int ns_stream_add_rows(float* x, const void* table, const int* ids, const void* vec, int n_tokens, int hidden, int copies, float scale,
                                  int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || hidden <= 0 || copies <= 0 || copies > NS_MAX_STREAMS || (table && !ids)) return NS_ERR_BAD_ARG;
  if (!table && !vec) return NS_OK;
  if (dtype == NS_DTYPE_F32)
    stream_add_rows_kernel<float><<<n_tokens, 256, 0, stream>>>(x, (const float*)table, ids, (const float*)vec, hidden, copies, scale);
  else if (dtype == NS_DTYPE_BF16)
    stream_add_rows_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(x, (const bf16_t*)table, ids, (const bf16_t*)vec, hidden, copies, scale);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
