// Soft-max attention over the paged cache for any head size and either storage type, one query row
// and one head per workgroup.  It is the attention of the true 32-bit path.  Keys are walked in
// fixed chunks of 256 counted from key 0, so a row's result does not depend on how the tokens were
// cut into steps or on what else is in the batch.
//
// Query row i of request b stands at position p = kv_len[b] - q_len[b] + i and sees the keys
// max(0, p - window + 1) .. p  (window == 0: 0 .. p).          (reference: model/attention.py:22-43)
// Options that the reference's attention does not have, each off at 0: ``chunk`` (a query also sees no key before the
// start of its own chunk, floor(p / chunk) * chunk, chunks counted from position 0), ``cap`` (a score s, after the
// scale, becomes cap * tanh(s / cap)), ``sink`` (the soft-max's denominator holds one more term of score 0 that has no
// value; with ``sink_logit`` [heads] the term is exp(sink_logit[h]) instead, a learned number that is not scaled), values of another size ``vd`` than the keys' ``hd``, and ``slope_exp`` (a bias by distance: head h of H loses
// 2^(-slope_exp (h + 1) / H) * (p - key) from its score, after the cap).
// Query head h reads key/value head h / (heads / kv_heads).    (reference: model/attention.py:33)
// K pages: [page][kv head][token][hd];  V pages: [page][kv head][vd][token].
#include "common.h"
#include "rope.h"

#define AG_THREADS 256
#define AG_MAX_VD 1024  // the largest value size (a thread holds up to four channels of the output)

template <typename T>
__global__ __launch_bounds__(AG_THREADS) void attn_generic_kernel(
    T* __restrict__ out, const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ token_req, const int* __restrict__ positions,
    const int* __restrict__ block_table, int table_stride, int heads, int kv_heads, int hd, int vd, int page_size, float scale,
    int window, int chunk, float cap, int sink, const float* __restrict__ sink_logit, float slope_exp) {
  extern __shared__ float smem[];  // q_s[hd] | p_s[AG_THREADS] | scratch[16]
  float* q_s = smem;
  float* p_s = smem + hd;
  float* scratch = p_s + AG_THREADS;
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (heads / kv_heads);
  const int pos = positions[t];
  const int* table = block_table + (size_t)token_req[t] * table_stride;
  const T* qrow = q + (size_t)t * q_stride + h * hd;
  for (int d = tid; d < hd; d += AG_THREADS) q_s[d] = to_f(qrow[d]) * scale;
  __syncthreads();
  int lo = window > 0 ? max(0, pos - window + 1) : 0;
  if (chunk > 0) lo = max(lo, pos / chunk * chunk);
  const float inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  const float slope = slope_exp > 0.f ? exp2f(-slope_exp * (float)(h + 1) / (float)heads) : 0.f;
  float m = -INFINITY, l = 0.f;
  float acc[AG_MAX_VD / AG_THREADS] = {};  // channels tid, tid + 256, ... of the output
  for (int c0 = (lo / AG_THREADS) * AG_THREADS; c0 <= pos; c0 += AG_THREADS) {
    const int key = c0 + tid;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    if (valid) {
      const int page = table[key / page_size];
      const T* kr = k_cache + (((size_t)page * kv_heads + kvh) * page_size + key % page_size) * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(q_s[d], to_f(kr[d]), dot);
      s = cap > 0.f ? cap * tanhf(dot * inv_cap) : dot;
      s -= slope * (float)(pos - key);
    }
    const float m_new = fmaxf(m, block_max(s, scratch));
    const float p = valid ? expf(s - m_new) : 0.f;
    p_s[tid] = p;
    const float csum = block_sum(p, scratch);  // its barriers also publish p_s
    const float alpha = m == -INFINITY ? 0.f : expf(m - m_new);
    l = l * alpha + csum;
    m = m_new;
#pragma unroll
    for (int ci = 0; ci < AG_MAX_VD / AG_THREADS; ++ci) {
      const int ch = tid + ci * AG_THREADS;
      if (ch < vd) {
        float a = acc[ci] * alpha;
        const int hi = min(AG_THREADS, pos - c0 + 1);
        for (int j = max(0, lo - c0); j < hi; ++j) {
          const int kj = c0 + j;
          const int page = table[kj / page_size];
          const T* vp = v_cache + (((size_t)page * kv_heads + kvh) * vd + ch) * page_size + kj % page_size;
          a = fmaf(p_s[j], to_f(*vp), a);
        }
        acc[ci] = a;
      }
    }
    __syncthreads();
  }
  if (sink_logit)
    l += expf(sink_logit[h] - m);  // the learned term, in the units of the running maximum
  else if (sink)
    l += expf(-m);  // the term of score 0
#pragma unroll
  for (int ci = 0; ci < AG_MAX_VD / AG_THREADS; ++ci)
    if (tid + ci * AG_THREADS < vd) out[((size_t)t * heads + h) * vd + tid + ci * AG_THREADS] = from_f<T>(acc[ci] / l);
}

extern "C" int ns_attn_generic(void* out, const void* q, int q_stride, const void* k_cache, const void* v_cache,
                               const int* token_req, const int* positions, const int* block_table, int table_stride,
                               int n_tokens, int heads, int kv_heads, int hd, int vd, int page_size, float scale, int window,
                               int chunk, float cap, int sink, const float* sink_logit, float slope_exp, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || hd <= 0 || hd > 1024 || vd <= 0 || vd > AG_MAX_VD || page_size <= 0 ||
      window < 0 || chunk < 0 || cap < 0.f || slope_exp < 0.f)
    return NS_ERR_BAD_ARG;
  if (heads > 65535) return NS_ERR_BAD_ARG;
  dim3 grid(n_tokens, heads);
  const size_t smem = (size_t)(hd + AG_THREADS + 16) * sizeof(float);
  if (dtype == NS_DTYPE_F32)
    attn_generic_kernel<float><<<grid, AG_THREADS, smem, stream>>>((float*)out, (const float*)q, q_stride, (const float*)k_cache,
        (const float*)v_cache, token_req, positions, block_table, table_stride, heads, kv_heads, hd, vd, page_size, scale, window, chunk, cap, sink, sink_logit, slope_exp);
  else if (dtype == NS_DTYPE_BF16)
    attn_generic_kernel<bf16_t><<<grid, AG_THREADS, smem, stream>>>((bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache,
        (const bf16_t*)v_cache, token_req, positions, block_table, table_stride, heads, kv_heads, hd, vd, page_size, scale, window, chunk, cap, sink, sink_logit, slope_exp);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// What an attention layer without rotation does between its projections and its scores: the queries and keys of every
// head are divided by their root mean square over the head (``eps`` >= 0; a negative eps leaves them as they are), the
// queries in place; keys and values go into the pages of their positions.  A row of ``qkv`` is q [heads][hd], then, if
// the layer has keys and values of its own (``own_kv``), k [kv_heads][hd] and v [kv_heads][vd].
// ------------------------------------------------------------------------------------------------
// grid (tokens, Y): a wave takes one head's vector; the blocks after those copy the values, 1,024 a block.
template <typename T>
__global__ void unit_kv_write_kernel(T* __restrict__ qkv, int stride, const int* __restrict__ positions, const int* __restrict__ token_req,
                                     const int* __restrict__ block_table, int table_stride, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                     int heads, int kv_heads, int hd, int vd, int page_size, float eps, int own_kv, int vec_blocks) {
  const int t = blockIdx.x, lane = threadIdx.x & (NS_WAVE - 1), wave = threadIdx.x / NS_WAVE;
  T* row = qkv + (size_t)t * stride;
  const int pos = positions[t];
  const int page = own_kv ? block_table[(size_t)token_req[t] * table_stride + pos / page_size] : 0;
  const int slot = pos % page_size;
  if ((int)blockIdx.y < vec_blocks) {
    const int vec = blockIdx.y * 4 + wave;
    if (vec >= heads + (own_kv ? kv_heads : 0)) return;
    T* p = row + (size_t)vec * hd;
    float f = 1.f;
    if (eps >= 0.f) {
      float ss = 0.f;
      for (int d = lane; d < hd; d += NS_WAVE) ss = fmaf(to_f(p[d]), to_f(p[d]), ss);
      ss = wave_sum(ss);
      f = 1.f / sqrtf(ss / (float)hd + eps);
    }
    if (vec < heads) {
      if (eps >= 0.f)
        for (int d = lane; d < hd; d += NS_WAVE) p[d] = from_f<T>(to_f(p[d]) * f);
    } else {
      T* dst = k_cache + (((size_t)page * kv_heads + (vec - heads)) * page_size + slot) * hd;
      for (int d = lane; d < hd; d += NS_WAVE) dst[d] = from_f<T>(to_f(p[d]) * f);
    }
    return;
  }
  if (own_kv) {
    const T* v = row + (size_t)(heads + kv_heads) * hd;
    const int part = blockIdx.y - vec_blocks;
    for (int i = part * 1024 + threadIdx.x; i < min(kv_heads * vd, (part + 1) * 1024); i += blockDim.x)
      v_cache[(((size_t)page * kv_heads + i / vd) * vd + i % vd) * page_size + slot] = v[i];
  }
}

extern "C" int ns_unit_kv_write(void* qkv, int stride, const int* positions, const int* token_req, const int* block_table, int table_stride,
                                void* k_cache, void* v_cache, int n_tokens, int heads, int kv_heads, int hd, int vd, int page_size,
                                float eps, int own_kv, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || heads <= 0 || kv_heads <= 0 || hd <= 0 || vd <= 0 || page_size <= 0) return NS_ERR_BAD_ARG;
  const int vec_blocks = (heads + (own_kv ? kv_heads : 0) + 3) / 4, copy_blocks = own_kv ? (kv_heads * vd + 1023) / 1024 : 0;
  if (vec_blocks + copy_blocks > 65535) return NS_ERR_BAD_ARG;
  const dim3 grid(n_tokens, vec_blocks + copy_blocks);
  if (dtype == NS_DTYPE_F32)
    unit_kv_write_kernel<float><<<grid, 256, 0, stream>>>((float*)qkv, stride, positions, token_req, block_table, table_stride,
                                                               (float*)k_cache, (float*)v_cache, heads, kv_heads, hd, vd, page_size, eps, own_kv, vec_blocks);
  else if (dtype == NS_DTYPE_BF16)
    unit_kv_write_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)qkv, stride, positions, token_req, block_table, table_stride,
                                                                (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, hd, vd, page_size, eps, own_kv, vec_blocks);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// The same place in a layer whose projections carry biases, whose queries and keys pass an RMS norm over the WHOLE
// projection (all heads at once) with a weight per channel, and whose values may be mixed with the values that an earlier
// layer made for the same token:
//   q <- (q + bq) / sqrt(mean((q + bq)^2 over heads*hd) + eps) * qw         (in place)
//   k <- likewise over kv_heads*hd with kw                                   (into the K pages)
//   v <- v + bv;  v <- (1 - lambda) v + lambda v_other  if v_other is given   (into the V pages; also to v_keep if given)
// With ``form.rot`` > 0 the first ``rot`` channels of every head of q and k are then rotated by the token's position
// (``inv_freq`` [rot / 2]); a thread owns both channels of a pair.
// ``bias`` [heads*hd + kv_heads*(hd + vd)], ``qw``, ``kw`` and ``lambda`` (one value) may each be null.  One workgroup a token.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void whole_norm_kv_write_kernel(
    T* __restrict__ qkv, int stride, const T* __restrict__ bias, const T* __restrict__ qw, const T* __restrict__ kw,
    const T* __restrict__ lambda, const T* __restrict__ v_other, int v_other_stride, T* __restrict__ v_keep, int v_keep_stride,
    const int* __restrict__ positions, const int* __restrict__ token_req, const int* __restrict__ block_table, int table_stride,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int heads, int kv_heads, int hd, int vd, int page_size, float eps,
    const float* __restrict__ inv_freq, RopeForm form) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * stride;
  const int nq = heads * hd, nk = kv_heads * hd, nv = kv_heads * vd;
  const int pos = positions[t];
  const int page = block_table[(size_t)token_req[t] * table_stride + pos / page_size];
  const int slot = pos % page_size;
  float fq = 1.f, fk = 1.f;
  if (qw) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nq; i += blockDim.x) {
      const float v = to_f(row[i]) + (bias ? to_f(bias[i]) : 0.f);
      ss = fmaf(v, v, ss);
    }
    fq = 1.f / sqrtf(block_sum(ss, scratch) / (float)nq + eps);
  }
  if (kw) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nk; i += blockDim.x) {
      const float v = to_f(row[nq + i]) + (bias ? to_f(bias[nq + i]) : 0.f);
      ss = fmaf(v, v, ss);
    }
    fk = 1.f / sqrtf(block_sum(ss, scratch) / (float)nk + eps);
  }
  if (form.rot > 0) {
    // the rotated pairs of q and of k: item = (head among q heads then k heads, pair)
    const int half = form.rot / 2;
    for (int i = threadIdx.x; i < (heads + kv_heads) * half; i += blockDim.x) {
      const int h = i / half, j = i % half;
      const bool is_q = h < heads;
      int d1, d2;
      rope_pair_channels(form, j, d1, d2);
      const int at = h * hd;  // q heads and k heads follow each other in the row
      const T* w = is_q ? qw : kw;
      const int wat = is_q ? at : at - nq;
      const float f = is_q ? fq : fk;
      float a = to_f(row[at + d1]) + (bias ? to_f(bias[at + d1]) : 0.f), b = to_f(row[at + d2]) + (bias ? to_f(bias[at + d2]) : 0.f);
      if (w) a = a * f * to_f(w[wat + d1]), b = b * f * to_f(w[wat + d2]);
      float c, sn;
      rope_cos_sin(form, pos, inv_freq[j], c, sn);
      rope_turn(a, b, c, sn, a, b);
      if (is_q) {
        row[at + d1] = from_f<T>(a);
        row[at + d2] = from_f<T>(b);
      } else {
        T* kd = k_cache + (((size_t)page * kv_heads + (h - heads)) * page_size + slot) * hd;
        kd[d1] = from_f<T>(a);
        kd[d2] = from_f<T>(b);
      }
    }
  }
  for (int i = threadIdx.x; i < nq; i += blockDim.x) {
    if (i % hd < form.rot) continue;
    const float v = to_f(row[i]) + (bias ? to_f(bias[i]) : 0.f);
    row[i] = from_f<T>(qw ? v * fq * to_f(qw[i]) : v);
  }
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    if (i % hd < form.rot) continue;
    const float v = to_f(row[nq + i]) + (bias ? to_f(bias[nq + i]) : 0.f);
    k_cache[(((size_t)page * kv_heads + i / hd) * page_size + slot) * hd + i % hd] = from_f<T>(kw ? v * fk * to_f(kw[i]) : v);
  }
  const float lam = (lambda && v_other) ? to_f(lambda[0]) : 0.f;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    float v = to_f(row[nq + nk + i]) + (bias ? to_f(bias[nq + nk + i]) : 0.f);
    if (v_other) v = (1.f - lam) * v + lam * to_f(v_other[(size_t)t * v_other_stride + i]);
    const T vs = from_f<T>(v);
    if (v_keep) v_keep[(size_t)t * v_keep_stride + i] = vs;
    v_cache[(((size_t)page * kv_heads + i / vd) * vd + i % vd) * page_size + slot] = vs;
  }
}

extern "C" int ns_whole_norm_kv_write(void* qkv, int stride, const void* bias, const void* qw, const void* kw, const void* lambda,
                                      const void* v_other, int v_other_stride, void* v_keep, int v_keep_stride, const int* positions,
                                      const int* token_req, const int* block_table, int table_stride, void* k_cache, void* v_cache,
                                      int n_tokens, int heads, int kv_heads, int hd, int vd, int page_size, float eps, const float* inv_freq,
                                      int rot, int interleaved, float factor, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || heads <= 0 || kv_heads <= 0 || hd <= 0 || vd <= 0 || page_size <= 0) return NS_ERR_BAD_ARG;
  if (rot < 0 || rot > hd || rot % 2 || (rot > 0 && !inv_freq)) return NS_ERR_BAD_ARG;
  const RopeForm form{rot, interleaved, factor};
  if (dtype == NS_DTYPE_F32)
    whole_norm_kv_write_kernel<float><<<n_tokens, 256, 0, stream>>>((float*)qkv, stride, (const float*)bias, (const float*)qw, (const float*)kw,
        (const float*)lambda, (const float*)v_other, v_other_stride, (float*)v_keep, v_keep_stride, positions, token_req, block_table,
        table_stride, (float*)k_cache, (float*)v_cache, heads, kv_heads, hd, vd, page_size, eps, inv_freq, form);
  else if (dtype == NS_DTYPE_BF16)
    whole_norm_kv_write_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((bf16_t*)qkv, stride, (const bf16_t*)bias, (const bf16_t*)qw, (const bf16_t*)kw,
        (const bf16_t*)lambda, (const bf16_t*)v_other, v_other_stride, (bf16_t*)v_keep, v_keep_stride, positions, token_req, block_table,
        table_stride, (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, hd, vd, page_size, eps, inv_freq, form);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// Queries and keys with biases, an RMS norm per head whose weight [hd] all heads share, and a rotation of the head's first
// ``rot`` channels; optionally the key projection's raw output (bias added, no norm, no rotation) is stored as the values.
// A workgroup a token (few tokens: several, each with its share of the heads), a wave a head in turn.  A row of ``qkv`` is [q heads | k heads | v heads] (no v part if
// ``v_is_k``); q is normed and rotated in place, k and v go into the token's slot of their pages.  All of it in 32-bit.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_rope_kv_write_kernel(
    T* __restrict__ qkv, int stride, const T* __restrict__ bias, const T* __restrict__ qw, const T* __restrict__ kw,
    const int* __restrict__ positions, const int* __restrict__ token_req, const int* __restrict__ block_table, int table_stride,
    const float* __restrict__ inv_freq, T* __restrict__ k_cache, T* __restrict__ v_cache, int heads, int kv_heads, int hd, int vd,
    int page_size, float eps, RopeForm form, int v_is_k) {
  const int t = blockIdx.x, lane = threadIdx.x % NS_WAVE, wave = threadIdx.x / NS_WAVE, waves = blockDim.x / NS_WAVE;
  T* row = qkv + (size_t)t * stride;
  const int pos = positions[t];
  const int page = block_table[(size_t)token_req[t] * table_stride + pos / page_size];
  const int slot = pos % page_size;
  const int half = form.rot / 2;
  for (int h = blockIdx.y * waves + wave; h < heads + kv_heads; h += waves * gridDim.y) {
    const bool is_q = h < heads;
    const int at = h * hd;  // q heads and k heads follow each other in the row
    const T* w = is_q ? qw : kw;
    float ss = 0.f;
    for (int c = lane; c < hd; c += NS_WAVE) {
      const float v = to_f(row[at + c]) + (bias ? to_f(bias[at + c]) : 0.f);
      ss = fmaf(v, v, ss);
    }
    const float rinv = w ? 1.f / sqrtf(wave_sum(ss) / (float)hd + eps) : 1.f;
    T* kd = is_q ? nullptr : k_cache + (((size_t)page * kv_heads + (h - heads)) * page_size + slot) * hd;
    if (!is_q && v_is_k) {
      T* vdst = v_cache + (((size_t)page * kv_heads + (h - heads)) * vd) * page_size + slot;
      for (int c = lane; c < hd; c += NS_WAVE)
        vdst[(size_t)c * page_size] = from_f<T>(to_f(row[at + c]) + (bias ? to_f(bias[at + c]) : 0.f));
    }
    // the rotated pairs: a lane reads both channels of its pair and writes both
    for (int j = lane; j < half; j += NS_WAVE) {
      int d1, d2;
      rope_pair_channels(form, j, d1, d2);
      float a = (to_f(row[at + d1]) + (bias ? to_f(bias[at + d1]) : 0.f)) * rinv * (w ? to_f(w[d1]) : 1.f);
      float b = (to_f(row[at + d2]) + (bias ? to_f(bias[at + d2]) : 0.f)) * rinv * (w ? to_f(w[d2]) : 1.f);
      float c, s;
      rope_cos_sin(form, pos, inv_freq[j], c, s);
      rope_turn(a, b, c, s, a, b);
      if (is_q) {
        row[at + d1] = from_f<T>(a);
        row[at + d2] = from_f<T>(b);
      } else {
        kd[d1] = from_f<T>(a);
        kd[d2] = from_f<T>(b);
      }
    }
    for (int c = form.rot + lane; c < hd; c += NS_WAVE) {
      const float v = (to_f(row[at + c]) + (bias ? to_f(bias[at + c]) : 0.f)) * rinv * (w ? to_f(w[c]) : 1.f);
      if (is_q)
        row[at + c] = from_f<T>(v);
      else
        kd[c] = from_f<T>(v);
    }
  }
  if (!v_is_k && blockIdx.y == 0) {
    const int nq = heads * hd, nk = kv_heads * hd, nv = kv_heads * vd;
    for (int i = threadIdx.x; i < nv; i += blockDim.x) {
      const float v = to_f(row[nq + nk + i]) + (bias ? to_f(bias[nq + nk + i]) : 0.f);
      v_cache[(((size_t)page * kv_heads + i / vd) * vd + i % vd) * page_size + slot] = from_f<T>(v);
    }
  }
}

extern "C" int ns_head_norm_rope_kv_write(void* qkv, int stride, const void* bias, const void* qw, const void* kw, const int* positions,
                                          const int* token_req, const int* block_table, int table_stride, const float* inv_freq,
                                          void* k_cache, void* v_cache, int n_tokens, int heads, int kv_heads, int hd, int vd, int page_size,
                                          float eps, int rot, int interleaved, float factor, int v_is_k, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || heads <= 0 || kv_heads <= 0 || hd <= 0 || vd <= 0 || page_size <= 0 || rot < 0 || rot > hd || rot % 2) return NS_ERR_BAD_ARG;
  if (v_is_k && vd != hd) return NS_ERR_BAD_ARG;
  if (rot > 0 && !inv_freq) return NS_ERR_BAD_ARG;
  const RopeForm form{rot, interleaved, factor};
  // few tokens: a wave a head at once, over several workgroups a token
  const int shares = n_tokens >= 256 ? 1 : (heads + kv_heads + 3) / 4;
  if (n_tokens > 65535 * 32768 || shares > 65535) return NS_ERR_BAD_ARG;
  dim3 grid(n_tokens, shares);
  if (dtype == NS_DTYPE_F32)
    head_norm_rope_kv_write_kernel<float><<<grid, 256, 0, stream>>>((float*)qkv, stride, (const float*)bias, (const float*)qw, (const float*)kw,
        positions, token_req, block_table, table_stride, inv_freq, (float*)k_cache, (float*)v_cache, heads, kv_heads, hd, vd, page_size, eps, form, v_is_k);
  else if (dtype == NS_DTYPE_BF16)
    head_norm_rope_kv_write_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)qkv, stride, (const bf16_t*)bias, (const bf16_t*)qw, (const bf16_t*)kw,
        positions, token_req, block_table, table_stride, inv_freq, (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, hd, vd, page_size, eps, form, v_is_k);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
