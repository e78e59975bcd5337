// Attention through latents: a layer caches, per token, one normed latent c [C] and one rotated key part r [R] shared by
// all heads, instead of keys and values per head.  With per-head matrices Uk [D, C] (keys) and Uv [E, C] (values):
//   score_h(i, j) = (q_h(i) . Uk_h c(j) + qr_h(i) . r(j)) * scale  =  ((Uk_h^T q_h(i)) . c(j) + qr_h(i) . r(j)) * scale
//   out_h(i)      = Uv_h sum_j p_h(i, j) c(j)
// so the attention itself runs over ONE key/value head whose key is [c | r] (C + R channels) and whose value is c, with
// queries [Uk_h^T q_h | qr_h]; the kernels here are what surrounds it:
//   latent_prep      the row [dq | dkv | gate] of the first product -> normed query latent, [c | r] into the K page,
//                    c into the V page, sigmoid of the gate logits (32-bit); a layer without a query latent has no dq part
//   latent_q_absorb  q [H][D + R] -> [H][C + R]: the unrotated part through Uk_h^T, the rotated part turned by its position
//   latent_out       o [H][C] -> [H][E] through Uv_h, times the gate
//   headwise_mfma    the two per-head products on the matrix cores (bfloat16, sizes that are multiples of 32 and 16)
// Norms, angles, rotations, the sigmoid and every sum are 32-bit.  Rotation pairs channel i with i + R/2.
#include "common.h"
#include "rope.h"

// One workgroup a token.  row: [q_rank | C | R | H] of type T.
template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(
    const T* __restrict__ proj, int stride, const T* __restrict__ qn_w, const T* __restrict__ cn_w, const float* __restrict__ inv_freq,
    float factor, T* __restrict__ cq, float* __restrict__ gate, const int* __restrict__ positions, const int* __restrict__ token_req,
    const int* __restrict__ block_table, int table_stride, T* __restrict__ k_cache, T* __restrict__ v_cache, int q_rank, int C, int R,
    int H, int page_size, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * stride;
  const int pos = positions[t];
  const int page = block_table[(size_t)token_req[t] * table_stride + pos / page_size];
  const int slot = pos % page_size;
  float ss = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) ss = fmaf(to_f(row[i]), to_f(row[i]), ss);
  const float fq = q_rank > 0 ? 1.f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps) : 1.f;  // (no query latent: q_rank = 0)
  ss = 0.f;
  for (int i = threadIdx.x; i < C; i += blockDim.x) ss = fmaf(to_f(row[q_rank + i]), to_f(row[q_rank + i]), ss);
  const float fc = 1.f / sqrtf(block_sum(ss, scratch) / (float)C + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) cq[(size_t)t * q_rank + i] = from_f<T>(to_f(row[i]) * fq * to_f(qn_w[i]));
  const int hd = C + R;
  T* kdst = k_cache + ((size_t)page * page_size + slot) * hd;
  T* vdst = v_cache + (size_t)page * C * page_size + slot;
  for (int i = threadIdx.x; i < C; i += blockDim.x) {
    const T c = from_f<T>(to_f(row[q_rank + i]) * fc * to_f(cn_w[i]));
    kdst[i] = c;
    vdst[(size_t)i * page_size] = c;
  }
  const RopeForm form{R, 0, factor};
  for (int j = threadIdx.x; j < R / 2; j += blockDim.x) {
    float c, s, a, b;
    rope_cos_sin(form, pos, inv_freq[j], c, s);
    rope_turn(to_f(row[q_rank + C + j]), to_f(row[q_rank + C + j + R / 2]), c, s, a, b);
    kdst[C + j] = from_f<T>(a);
    kdst[C + j + R / 2] = from_f<T>(b);
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) gate[(size_t)t * H + h] = 1.f / (1.f + expf(-to_f(row[q_rank + C + R + h])));
}

extern "C" int ns_latent_prep(const void* proj, int stride, const void* qn_w, const void* cn_w, const float* inv_freq, float factor, void* cq,
                              float* gate, const int* positions, const int* token_req, const int* block_table, int table_stride,
                              void* k_cache, void* v_cache, int n_tokens, int q_rank, int C, int R, int H, int page_size, float eps,
                              int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || q_rank < 0 || (q_rank > 0 && (!cq || !qn_w)) || C <= 0 || R < 0 || R % 2 || H < 0 || (H > 0 && !gate) || page_size <= 0) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    latent_prep_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)proj, stride, (const float*)qn_w, (const float*)cn_w, inv_freq, factor,
        (float*)cq, gate, positions, token_req, block_table, table_stride, (float*)k_cache, (float*)v_cache, q_rank, C, R, H, page_size, eps);
  else if (dtype == NS_DTYPE_BF16)
    latent_prep_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const bf16_t*)proj, stride, (const bf16_t*)qn_w, (const bf16_t*)cn_w, inv_freq, factor,
        (bf16_t*)cq, gate, positions, token_req, block_table, table_stride, (bf16_t*)k_cache, (bf16_t*)v_cache, q_rank, C, R, H, page_size, eps);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

#define LAT_TOKENS 8  // tokens a workgroup takes through one head's matrix, which it then reads once for all of them

// grid (ceil(n / LAT_TOKENS), H).  uk: [H * D][C] (the checkpoint's layout, rows are key channels): thread c walks a column.
template <typename T>
__global__ __launch_bounds__(256) void latent_q_absorb_kernel(const T* __restrict__ q, int q_stride, const T* __restrict__ uk,
                                                              const float* __restrict__ inv_freq, float factor,
                                                              const int* __restrict__ positions, T* __restrict__ out, int n, int H, int D,
                                                              int R, int C, int absorb) {
  extern __shared__ float q_s[];  // [LAT_TOKENS][D]
  const int t0 = blockIdx.x * LAT_TOKENS, h = blockIdx.y;
  const int nt = min(LAT_TOKENS, n - t0);
  for (int i = threadIdx.x; i < LAT_TOKENS * D; i += blockDim.x) {
    const int tt = i / D, d = i % D;
    q_s[i] = tt < nt ? to_f(q[(size_t)(t0 + tt) * q_stride + (size_t)h * (D + R) + d]) : 0.f;
  }
  __syncthreads();
  const T* w = uk + (size_t)h * D * C;
  for (int c = threadIdx.x; c < (absorb ? C : 0); c += blockDim.x) {
    float acc[LAT_TOKENS] = {};
    for (int d = 0; d < D; ++d) {
      const float wv = to_f(w[(size_t)d * C + c]);
#pragma unroll
      for (int tt = 0; tt < LAT_TOKENS; ++tt) acc[tt] = fmaf(q_s[tt * D + d], wv, acc[tt]);
    }
#pragma unroll
    for (int tt = 0; tt < LAT_TOKENS; ++tt)
      if (tt < nt) out[((size_t)(t0 + tt) * H + h) * (C + R) + c] = from_f<T>(acc[tt]);
  }
  const RopeForm form{R, 0, factor};
  for (int i = threadIdx.x; i < nt * (R / 2); i += blockDim.x) {
    const int tt = i / (R / 2), j = i % (R / 2);
    const T* qr = q + (size_t)(t0 + tt) * q_stride + (size_t)h * (D + R) + D;
    float c, s, a, b;
    rope_cos_sin(form, positions[t0 + tt], inv_freq[j], c, s);
    rope_turn(to_f(qr[j]), to_f(qr[j + R / 2]), c, s, a, b);
    T* o = out + ((size_t)(t0 + tt) * H + h) * (C + R) + C;
    o[j] = from_f<T>(a);
    o[j + R / 2] = from_f<T>(b);
  }
}

extern "C" int ns_latent_q_absorb(const void* q, int q_stride, const void* uk, const float* inv_freq, float factor, const int* positions,
                                  void* out, int n, int H, int D, int R, int C, int absorb, int dtype, hipStream_t stream) {
  if (n <= 0 || H <= 0 || H > 65535 || D <= 0 || R < 0 || R % 2 || C <= 0 || (size_t)LAT_TOKENS * D * sizeof(float) > 64 * 1024) return NS_ERR_BAD_ARG;
  if (!absorb && !uk) uk = q;  // (not read)
  const dim3 grid((n + LAT_TOKENS - 1) / LAT_TOKENS, H);
  const size_t smem = (size_t)LAT_TOKENS * D * sizeof(float);
  const int threads = C >= 256 ? 256 : (C >= 128 ? 128 : 64);
  if (dtype == NS_DTYPE_F32)
    latent_q_absorb_kernel<float><<<grid, threads, smem, stream>>>((const float*)q, q_stride, (const float*)uk, inv_freq, factor, positions,
                                                                   (float*)out, n, H, D, R, C, absorb);
  else if (dtype == NS_DTYPE_BF16)
    latent_q_absorb_kernel<bf16_t><<<grid, threads, smem, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)uk, inv_freq, factor, positions,
                                                                    (bf16_t*)out, n, H, D, R, C, absorb);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// grid (ceil(n / LAT_TOKENS), H).  uv_t: [H][C][E], the checkpoint's [H * E][C] transposed per head at load time, so that
// thread e walks a column.  out[t][h][e] = gate[t][h] * sum_c o[t][h][c] uv_t[h][c][e].
template <typename T>
__global__ __launch_bounds__(256) void latent_out_kernel(const T* __restrict__ o, const T* __restrict__ uv_t, const float* __restrict__ gate,
                                                         T* __restrict__ out, int n, int H, int C, int E) {
  extern __shared__ float o_s[];  // [LAT_TOKENS][C]
  const int t0 = blockIdx.x * LAT_TOKENS, h = blockIdx.y;
  const int nt = min(LAT_TOKENS, n - t0);
  for (int i = threadIdx.x; i < LAT_TOKENS * C; i += blockDim.x) {
    const int tt = i / C, c = i % C;
    o_s[i] = tt < nt ? to_f(o[((size_t)(t0 + tt) * H + h) * C + c]) : 0.f;
  }
  __syncthreads();
  const T* w = uv_t + (size_t)h * C * E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    float acc[LAT_TOKENS] = {};
    for (int c = 0; c < C; ++c) {
      const float wv = to_f(w[(size_t)c * E + e]);
#pragma unroll
      for (int tt = 0; tt < LAT_TOKENS; ++tt) acc[tt] = fmaf(o_s[tt * C + c], wv, acc[tt]);
    }
#pragma unroll
    for (int tt = 0; tt < LAT_TOKENS; ++tt)
      if (tt < nt) out[((size_t)(t0 + tt) * H + h) * E + e] = from_f<T>(acc[tt] * (gate ? gate[(size_t)(t0 + tt) * H + h] : 1.f));
  }
}

extern "C" int ns_latent_out(const void* o, const void* uv_t, const float* gate, void* out, int n, int H, int C, int E, int dtype,
                             hipStream_t stream) {
  if (n <= 0 || H <= 0 || H > 65535 || C <= 0 || E <= 0 || (size_t)LAT_TOKENS * C * sizeof(float) > 64 * 1024) return NS_ERR_BAD_ARG;
  const dim3 grid((n + LAT_TOKENS - 1) / LAT_TOKENS, H);
  const size_t smem = (size_t)LAT_TOKENS * C * sizeof(float);
  const int threads = E >= 256 ? 256 : (E >= 128 ? 128 : 64);
  if (dtype == NS_DTYPE_F32)
    latent_out_kernel<float><<<grid, threads, smem, stream>>>((const float*)o, (const float*)uv_t, gate, (float*)out, n, H, C, E);
  else if (dtype == NS_DTYPE_BF16)
    latent_out_kernel<bf16_t><<<grid, threads, smem, stream>>>((const bf16_t*)o, (const bf16_t*)uv_t, gate, (bf16_t*)out, n, H, C, E);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// The two per-head products on the matrix cores (bfloat16): out[t][h][n] = gate[t][h] * sum_k x[t][h][k] w[h][n][k], with
// w [H][N][K] (every head's matrix as [out, in] rows), K a multiple of 32 and N of 16.  Kept transposed, D[n][token] =
// W[n][:] . X[token][:], so that both operands are 16-byte loads of consecutive k straight from memory and a lane ends up
// with four consecutive n of one token.  A wave takes 16 tokens of one head and NT tiles of 16 outputs; x is re-read per
// wave from the caches (16 tokens of one head are a few KB).
// ------------------------------------------------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 hw_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 hw_bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float hw_f32x4;

template <int NT>
__global__ __launch_bounds__(256) void headwise_mfma_kernel(const bf16_t* __restrict__ x, long x_row, int x_head, const bf16_t* __restrict__ w,
                                                            const float* __restrict__ gate, bf16_t* __restrict__ out, long out_row,
                                                            int out_head, int n_tokens, int H, int N, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int t0 = blockIdx.x * 16, h = blockIdx.y;
  const int n0 = (blockIdx.z * 4 + wave) * NT * 16;
  if (n0 >= N) return;
  const int token = t0 + c;
  const bool tok_ok = token < n_tokens;
  const bf16_t* xp = x + (size_t)(tok_ok ? token : 0) * x_row + (size_t)h * x_head + g * 8;
  const bf16_t* wp[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) wp[i] = w + ((size_t)h * N + min(n0 + i * 16 + c, N - 1)) * K + g * 8;
  hw_f32x4 acc[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) acc[i] = hw_f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    hw_bf16x8 b = *reinterpret_cast<const hw_bf16x8*>(xp + k0);
    if (!tok_ok) b = hw_bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    hw_bf16x8 a[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) a[i] = *reinterpret_cast<const hw_bf16x8*>(wp[i] + k0);
#pragma unroll
    for (int i = 0; i < NT; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b, acc[i], 0, 0, 0);
  }
  if (!tok_ok) return;
  const float gt = gate ? gate[(size_t)token * H + h] : 1.f;
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    const int n = n0 + i * 16 + g * 4;  // acc[i][j] is output n + j of this lane's token
    if (n < N) {
      const hw_bf16x4 r = {(bf16_t)(acc[i][0] * gt), (bf16_t)(acc[i][1] * gt), (bf16_t)(acc[i][2] * gt), (bf16_t)(acc[i][3] * gt)};
      *reinterpret_cast<hw_bf16x4*>(out + (size_t)token * out_row + (size_t)h * out_head + n) = r;
    }
  }
}

extern "C" int ns_headwise_bf16(const void* x, long x_row, int x_head, const void* w, const float* gate, void* out, long out_row, int out_head,
                                int n_tokens, int H, int N, int K, hipStream_t stream) {
  if (n_tokens <= 0 || H <= 0 || H > 65535 || N <= 0 || N % 16 || K <= 0 || K % 32 || (x_row & 7) || (x_head & 7) || (out_row & 3) || (out_head & 3) ||
      ((uintptr_t)x & 15) || ((uintptr_t)w & 15) || ((uintptr_t)out & 7))
    return NS_ERR_BAD_ARG;
  const int tiles = N / 16;
  if (tiles >= 16) {
    const dim3 grid((n_tokens + 15) / 16, H, (tiles + 15) / 16);
    headwise_mfma_kernel<4><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, gate, (bf16_t*)out, out_row, out_head,
                                                      n_tokens, H, N, K);
  } else {
    const dim3 grid((n_tokens + 15) / 16, H, (tiles + 3) / 4);
    headwise_mfma_kernel<1><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w, gate, (bf16_t*)out, out_row, out_head,
                                                      n_tokens, H, N, K);
  }
  return ns_launch_status();
}
