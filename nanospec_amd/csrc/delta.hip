// The gated delta rule with one decay per head and key channel, and what surrounds it: the short causal convolution
// over time with its carried inputs, the unit vectors, decays and write strengths, the recurrence over a request's
// tokens with the state carried in its slot, and the gated RMS norm of the read-out.
//
// Per head, with S [D key channels][E value channels] (float, one per request and head):
//   S <- diag(g_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
// Column j of S only ever meets column j of v and o, so the columns of a head are independent chains: a thread owns 16
// key channels of one column in registers, the RG = D/16 threads of a column sit in neighbouring lanes and add their
// parts of the two dot products by lane exchange, and nothing waits at a barrier.  Everything here is 32-bit.
//
// A request's slot holds S [H][D][E] and behind it the last K - 1 inputs of the convolution [K - 1][C] (oldest first).
#include "common.h"

#define ND_MAX_TAPS 16
#define ND_ROWS 16  // key channels of a column that one thread owns

// ------------------------------------------------------------------------------------------------
// y[r][c] = silu(sum_j taps[c][j] * in(i - (K-1) + j)),  i the token's index among its request's tokens of this step;
// in(t) is this step's input for t >= 0 and the carried input K-1+t for t < 0.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void conv_silu_kernel(float* __restrict__ out, const T* __restrict__ x, int x_stride, const float* __restrict__ taps,
                                 const float* __restrict__ state, size_t slot_stride, size_t conv_off, const int* __restrict__ token_req,
                                 const int* __restrict__ qo_indptr, const int* __restrict__ state_slots, int C, int K) {
  const int r = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = token_req[r];
  const int i = r - qo_indptr[b];
  const float* carried = state + (size_t)state_slots[b] * slot_stride + conv_off;
  float y = 0.f;
  for (int j = 0; j < K; ++j) {
    const int t = i - (K - 1) + j;
    const float v = t >= 0 ? to_f(x[(size_t)(r - (K - 1) + j) * x_stride + c]) : carried[(size_t)(K - 1 + t) * C + c];
    y = fmaf(taps[(size_t)c * K + j], v, y);
  }
  out[(size_t)r * C + c] = y / (1.f + expf(-y));
}

// The same for four neighbouring channels a thread, with 16-byte accesses to taps, carried inputs and results, for the
// usual numbers of taps (so that the taps are registers) and channels that are a multiple of four.
template <typename T, int K>
__global__ void conv_silu_vec_kernel(float* __restrict__ out, const T* __restrict__ x, int x_stride, const float* __restrict__ taps,
                                     const float* __restrict__ state, size_t slot_stride, size_t conv_off, const int* __restrict__ token_req,
                                     const int* __restrict__ qo_indptr, const int* __restrict__ state_slots, int C) {
  typedef T vec_t __attribute__((ext_vector_type(4)));
  const int r = blockIdx.x, c = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
  if (c >= C) return;
  const int b = token_req[r];
  const int i = r - qo_indptr[b];
  const float* carried = state + (size_t)state_slots[b] * slot_stride + conv_off;
  float tp[4 * K];  // taps of channel c + e / K, tap e % K
#pragma unroll
  for (int e = 0; e < K; ++e) {
    const float4 t = reinterpret_cast<const float4*>(taps + (size_t)c * K)[e];
    tp[4 * e] = t.x, tp[4 * e + 1] = t.y, tp[4 * e + 2] = t.z, tp[4 * e + 3] = t.w;
  }
  float y[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < K; ++j) {
    const int t = i - (K - 1) + j;
    float v[4];
    if (t >= 0) {
      const vec_t xv = *reinterpret_cast<const vec_t*>(x + (size_t)(r - (K - 1) + j) * x_stride + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = to_f(xv[e]);
    } else {
      const float4 cv = *reinterpret_cast<const float4*>(carried + (size_t)(K - 1 + t) * C + c);
      v[0] = cv.x, v[1] = cv.y, v[2] = cv.z, v[3] = cv.w;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = fmaf(tp[e * K + j], v[e], y[e]);
  }
  float4 res;
  res.x = y[0] / (1.f + expf(-y[0])), res.y = y[1] / (1.f + expf(-y[1]));
  res.z = y[2] / (1.f + expf(-y[2])), res.w = y[3] / (1.f + expf(-y[3]));
  *reinterpret_cast<float4*>(out + (size_t)r * C + c) = res;
}

// After the convolution has read them: the carried inputs become the last K-1 inputs including this step's.
template <typename T>
__global__ void conv_carry_kernel(const T* __restrict__ x, int x_stride, float* __restrict__ state, size_t slot_stride, size_t conv_off,
                                  const int* __restrict__ qo_indptr, const int* __restrict__ state_slots, int C, int K) {
  const int b = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r0 = qo_indptr[b], L = qo_indptr[b + 1] - r0;
  if (L <= 0) return;
  float* carried = state + (size_t)state_slots[b] * slot_stride + conv_off;
  float old[ND_MAX_TAPS];
  for (int j = 0; j < K - 1; ++j) old[j] = carried[(size_t)j * C + c];
  for (int j = 0; j < K - 1; ++j) {
    const int t = L - (K - 1) + j;
    carried[(size_t)j * C + c] = t >= 0 ? to_f(x[(size_t)(r0 + t) * x_stride + c]) : old[K - 1 + t];
  }
}

extern "C" int ns_conv_silu_carry(float* out, const void* x, int x_stride, const float* taps, float* state, size_t slot_stride,
                                  size_t conv_off, const int* token_req, const int* qo_indptr, const int* state_slots, int n_tokens,
                                  int n_reqs, int C, int K, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || n_reqs <= 0 || n_reqs > 65535 || C <= 0 || K < 1 || K > ND_MAX_TAPS) return NS_ERR_BAD_ARG;
  if (dtype != NS_DTYPE_F32 && dtype != NS_DTYPE_BF16) return NS_ERR_UNSUPPORTED;
  const int bx = (C + 255) / 256;
  if (bx > 65535) return NS_ERR_BAD_ARG;
  const size_t esize = dtype == NS_DTYPE_F32 ? 4 : 2;
  const bool vec = C % 4 == 0 && x_stride % 4 == 0 && ((uintptr_t)x % (4 * esize)) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)taps % 16) == 0 &&
                   ((uintptr_t)state % 16) == 0 && slot_stride % 4 == 0 && conv_off % 4 == 0 && K >= 2 && K <= 4;
  if (vec) {
    dim3 grid(n_tokens, (C / 4 + 255) / 256);
#define ND_CONV(KK)                                                                                                                         \
  case KK:                                                                                                                                  \
    if (dtype == NS_DTYPE_F32)                                                                                                              \
      conv_silu_vec_kernel<float, KK><<<grid, 256, 0, stream>>>(out, (const float*)x, x_stride, taps, state, slot_stride, conv_off, token_req, \
                                                                qo_indptr, state_slots, C);                                                \
    else                                                                                                                                    \
      conv_silu_vec_kernel<bf16_t, KK><<<grid, 256, 0, stream>>>(out, (const bf16_t*)x, x_stride, taps, state, slot_stride, conv_off, token_req, \
                                                                 qo_indptr, state_slots, C);                                               \
    break
    switch (K) {
      ND_CONV(2);
      ND_CONV(3);
      default: ND_CONV(4);
    }
#undef ND_CONV
  } else {
    dim3 grid(n_tokens, bx);
    if (dtype == NS_DTYPE_F32)
      conv_silu_kernel<float><<<grid, 256, 0, stream>>>(out, (const float*)x, x_stride, taps, state, slot_stride, conv_off, token_req,
                                                         qo_indptr, state_slots, C, K);
    else
      conv_silu_kernel<bf16_t><<<grid, 256, 0, stream>>>(out, (const bf16_t*)x, x_stride, taps, state, slot_stride, conv_off, token_req,
                                                          qo_indptr, state_slots, C, K);
  }
  if (K > 1) {
    dim3 grid(bx, n_reqs);
    if (dtype == NS_DTYPE_F32)
      conv_carry_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, state, slot_stride, conv_off, qo_indptr, state_slots, C, K);
    else
      conv_carry_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, state, slot_stride, conv_off, qo_indptr, state_slots, C, K);
  }
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// Per token: q and k of every key/value head become unit vectors, x / sqrt(sum(x^2) + 1e-6), q times D^(-1/2), in
// place in qkv [n][2 G D + H E]; g = exp(-exp(A_log[h]) softplus(a + dt_bias)) [n][H D]; beta = sigmoid(b) [n][H].
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// grid (tokens, Y): the first ceil(2 G / 4) blocks of a token take one vector a wave; the others 1,024 decays each (and
// the first of them the write strengths), so that no wave walks through a chain of dependent loads.
template <typename T>
__global__ void delta_prep_kernel(float* __restrict__ qkv, int C, float* __restrict__ g, float* __restrict__ beta, const T* __restrict__ a,
                                  int a_stride, const T* __restrict__ bp, int b_stride, const float* __restrict__ dt_bias,
                                  const float* __restrict__ a_log, int H, int G, int D, int norm_blocks) {
  const int r = blockIdx.x, lane = threadIdx.x & (NS_WAVE - 1), wave = threadIdx.x / NS_WAVE;
  if ((int)blockIdx.y < norm_blocks) {
    const int vec = blockIdx.y * 4 + wave;  // q heads, then k heads
    if (vec >= 2 * G) return;
    float* p = qkv + (size_t)r * C + (size_t)vec * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += NS_WAVE) ss = fmaf(p[d], p[d], ss);
    ss = wave_sum(ss);
    const float f = (vec < G ? 1.f / sqrtf((float)D) : 1.f) / sqrtf(ss + 1e-6f);
    for (int d = lane; d < D; d += NS_WAVE) p[d] *= f;
    return;
  }
  const int part = blockIdx.y - norm_blocks;
  for (int i = part * 1024 + threadIdx.x; i < min(H * D, (part + 1) * 1024); i += blockDim.x) {
    const float z = to_f(a[(size_t)r * a_stride + i]) + dt_bias[i];
    g[(size_t)r * H * D + i] = expf(-expf(a_log[i / D]) * softplus_f(z));
  }
  if (part == 0)
    for (int h = threadIdx.x; h < H; h += blockDim.x) beta[(size_t)r * H + h] = 1.f / (1.f + expf(-to_f(bp[(size_t)r * b_stride + h])));
}

extern "C" int ns_delta_prep(float* qkv, int C, float* g, float* beta, const void* a, int a_stride, const void* bp, int b_stride,
                             const float* dt_bias, const float* a_log, int n_tokens, int H, int G, int D, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || C < 2 * G * D) return NS_ERR_BAD_ARG;
  const int norm_blocks = (2 * G + 3) / 4, decay_blocks = (H * D + 1023) / 1024;
  if (norm_blocks + decay_blocks > 65535) return NS_ERR_BAD_ARG;
  const dim3 grid(n_tokens, norm_blocks + decay_blocks);
  if (dtype == NS_DTYPE_F32)
    delta_prep_kernel<float><<<grid, 256, 0, stream>>>(qkv, C, g, beta, (const float*)a, a_stride, (const float*)bp, b_stride, dt_bias,
                                                        a_log, H, G, D, norm_blocks);
  else if (dtype == NS_DTYPE_BF16)
    delta_prep_kernel<bf16_t><<<grid, 256, 0, stream>>>(qkv, C, g, beta, (const bf16_t*)a, a_stride, (const bf16_t*)bp, b_stride,
                                                         dt_bias, a_log, H, G, D, norm_blocks);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// The recurrence.  grid (blocks of columns, heads, requests); a thread = (column jl of the block, row group rg), lane
// = jl * RG + rg, RG a power of two (at most 64) with 16 RG >= D.  Channels beyond D carry zeros.
//
// A token's step is a chain (decay, dot product, lane exchange, update, dot product, lane exchange) that cannot start
// before the token's operands are there, so the operands of the next ND_STAGE_FLOATS floats' worth of tokens are
// fetched by the whole workgroup at once (coalesced, all loads in flight together), parked in registers while the
// current stage's tokens are worked through from LDS, and then written to the other LDS buffer.  The arithmetic of a
// token is the same whatever the stage it falls into: results do not depend on how a prompt was cut.
// ------------------------------------------------------------------------------------------------
#define ND_PITCH (ND_ROWS + 4)                     // floats between two row groups' channels in LDS
#define ND_STAGE_FLOATS 6144                       // floats of one stage in LDS (two stages are held)
#define ND_STAGE_REGS (ND_STAGE_FLOATS / 1024)     // of which each of the 256 threads fetches this many groups of four

struct DeltaShape {
  int C, H, G, D, E, RG, Dl, cols, tok_stride, stage_tokens, vec4;
};

template <bool VEC, int RG, int ROWS>
__global__ __launch_bounds__(256) void delta_scan_kernel(float* __restrict__ o, const float* __restrict__ qkv,
                                                         const float* __restrict__ g, const float* __restrict__ beta,
                                                         float* __restrict__ state, size_t slot_stride, const int* __restrict__ qo_indptr,
                                                         const int* __restrict__ state_slots, DeltaShape p) {
  __shared__ __attribute__((aligned(16))) float stage[2][ND_STAGE_FLOATS];
  // (the request is the slowest index of the launch: workgroups are dealt to the eight XCDs in turn, and with the request
  // as the fastest index all workgroups of the one long request among eight would land on one XCD)
  const int b = blockIdx.z, h = blockIdx.y;
  const int r0 = qo_indptr[b], r1 = qo_indptr[b + 1];
  if (r1 <= r0) return;
  const int D = p.D, E = p.E;
  constexpr int PITCH = ROWS + 4;  // floats between two row groups' channels in LDS
  constexpr int DL = RG * PITCH, COLS = 256 / RG;
  const int jl = threadIdx.x / RG, rg = threadIdx.x % RG;
  const int j0 = blockIdx.x * COLS, j = j0 + jl;
  const bool col_ok = j < E;
  const int d0 = rg * ROWS;
  const int kh = h / (p.H / p.G);
  float* S = state + (size_t)state_slots[b] * slot_stride + (size_t)h * D * E;
  float s[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) s[i] = (col_ok && d0 + i < D) ? S[(size_t)(d0 + i) * E + j] : 0.f;

  // what element e of a stage that starts at row `first` is: token e / tok_stride, then q [Dl] | k [Dl] | g [Dl] | v [cols] | beta;
  // in q, k and g the 16 channels of a row group are followed by four unused floats (PITCH), so that the row groups'
  // 16-byte reads fall into different banks
  const float* q_src = qkv + (size_t)kh * D;
  const float* k_src = qkv + (size_t)p.G * D + (size_t)kh * D;
  const float* v_src = qkv + (size_t)2 * p.G * D + (size_t)h * E + j0;
  const float* g_src = g + (size_t)h * D;
  const int stage_elems = p.stage_tokens * p.tok_stride;
  // A thread fetches groups of four floats; every part of a token's record starts at a multiple of four.  Which group of
  // which token's record a thread's i-th load is does not change from stage to stage, so source, row pitch and what is
  // kept of it are worked out once; a stage's loads then differ only in the row, and are issued without a branch around
  // any of them (a group that holds nothing reads the start of its source and is dropped when it is parked), so that
  // all of a stage's loads are in flight together and nothing waits for one before the stage's tokens are done.
  const float* src_of[ND_STAGE_REGS];
  int pitch_of[ND_STAGE_REGS], token_of[ND_STAGE_REGS];
  unsigned keep = 0, is_beta = 0;  // four bits a group: which of its floats are kept; one bit a group: its first float is beta
  {
    int tt = threadIdx.x * 4 / p.tok_stride, off = threadIdx.x * 4 - tt * p.tok_stride;  // of element e, kept up as e grows by 1024
#pragma unroll
    for (int i = 0; i < ND_STAGE_REGS; ++i) {
      const int e = (threadIdx.x + i * 256) * 4;
      const bool used = e < stage_elems;
      const int part = off < DL ? 0 : (off < 2 * DL ? 1 : (off < 3 * DL ? 2 : 3));
      const int within = off - part * DL, chunk = within / PITCH, w = within - chunk * PITCH;
      const int d = w < ROWS ? chunk * ROWS + w : 0x3fffffff;  // (the unused floats keep nothing)
      const int c = off - 3 * DL;
      const int at = part < 3 ? d : c;
      const int lim = !used ? 0 : (part < 3 ? D : min(COLS, E - j0));
      const float* src = part == 0 ? q_src : (part == 1 ? k_src : (part == 2 ? g_src : v_src));
      const unsigned bits = VEC ? (at < lim ? 0xfu : 0u)
                                : ((at < lim ? 1u : 0u) | (at + 1 < lim ? 2u : 0u) | (at + 2 < lim ? 4u : 0u) | (at + 3 < lim ? 8u : 0u));
      src_of[i] = src + (bits ? at : 0);
      pitch_of[i] = part == 2 ? p.H * D : p.C;
      token_of[i] = tt;
      keep |= bits << (4 * i);
      is_beta |= (used && part >= 3 && c == COLS ? 1u : 0u) << i;
      off += 1024;
      while (off >= p.tok_stride) off -= p.tok_stride, ++tt;
    }
  }
  struct Stage {
    float4 v[ND_STAGE_REGS];
    float bt[ND_STAGE_REGS];
    unsigned live;  // one bit a group: its token is one of the request's
  };
  auto fetch = [&](Stage& st, int first) {
    st.live = 0;
#pragma unroll
    for (int i = 0; i < ND_STAGE_REGS; ++i) {
      const int r = min(first + token_of[i], r1 - 1);
      st.live |= (first + token_of[i] < r1 ? 1u : 0u) << i;
      const float* src = src_of[i] + (size_t)r * pitch_of[i];
      if constexpr (VEC) {
        st.v[i] = *reinterpret_cast<const float4*>(src);
      } else {
        const unsigned k = keep >> (4 * i);
        st.v[i] = float4{src[0], src[k & 2u ? 1 : 0], src[k & 4u ? 2 : 0], src[k & 8u ? 3 : 0]};
      }
      st.bt[i] = beta[(size_t)r * p.H + h];
    }
  };
  auto park = [&](const Stage& st, float* buf) {
#pragma unroll
    for (int i = 0; i < ND_STAGE_REGS; ++i) {
      const int e = (threadIdx.x + i * 256) * 4;
      const bool live = (st.live >> i) & 1u;
      const unsigned k = live ? keep >> (4 * i) : 0u;
      float4 val = {k & 1u ? st.v[i].x : 0.f, k & 2u ? st.v[i].y : 0.f, k & 4u ? st.v[i].z : 0.f, k & 8u ? st.v[i].w : 0.f};
      if (live && ((is_beta >> i) & 1u)) val.x = st.bt[i];
      if (e < stage_elems) *reinterpret_cast<float4*>(buf + e) = val;
    }
  };

  // where this thread's output of the next token goes (the first lane of a column's group writes it)
  const bool writes = rg == 0 && col_ok;
  const size_t out_stride = (size_t)p.H * E;
  float* op = o + (size_t)r0 * out_stride + (size_t)h * E + (col_ok ? j : 0);
  Stage regs;
  fetch(regs, r0);
  park(regs, stage[0]);
  __syncthreads();
  int cur = 0;
  for (int first = r0; first < r1; first += p.stage_tokens) {
    const bool more = first + p.stage_tokens < r1;
    if (more) fetch(regs, first + p.stage_tokens);
    const float* buf = stage[cur];
    const int n = min(p.stage_tokens, r1 - first);
    // Two sets of operand registers take turns: the next token's operands are read from LDS into one while the chain of
    // the current token runs on the other (written out twice, so that no set is ever copied into the other).
    struct Operands {
      float4 q[ROWS / 4], k[ROWS / 4], g[ROWS / 4];
      float v, b;
    };
    auto read_token = [&](Operands& t, int tt) {
      const float* tok = buf + tt * p.tok_stride;
#pragma unroll
      for (int i = 0; i < ROWS / 4; ++i) {
        t.q[i] = reinterpret_cast<const float4*>(tok + rg * PITCH)[i];
        t.k[i] = reinterpret_cast<const float4*>(tok + DL + rg * PITCH)[i];
        t.g[i] = reinterpret_cast<const float4*>(tok + 2 * DL + rg * PITCH)[i];
      }
      t.v = tok[3 * DL + jl], t.b = tok[3 * DL + COLS];
    };
    auto chain = [&](const Operands& t) {
      float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < ROWS / 4; ++i) {
        s[4 * i] *= t.g[i].x, s[4 * i + 1] *= t.g[i].y, s[4 * i + 2] *= t.g[i].z, s[4 * i + 3] *= t.g[i].w;
        part[0] = fmaf(t.k[i].x, s[4 * i], part[0]);
        part[1] = fmaf(t.k[i].y, s[4 * i + 1], part[1]);
        part[2] = fmaf(t.k[i].z, s[4 * i + 2], part[2]);
        part[3] = fmaf(t.k[i].w, s[4 * i + 3], part[3]);
      }
      const float dot = group_sum<RG>((part[0] + part[1]) + (part[2] + part[3]));
      const float u = t.b * (t.v - dot);
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < ROWS / 4; ++i) {
        s[4 * i] = fmaf(t.k[i].x, u, s[4 * i]);
        s[4 * i + 1] = fmaf(t.k[i].y, u, s[4 * i + 1]);
        s[4 * i + 2] = fmaf(t.k[i].z, u, s[4 * i + 2]);
        s[4 * i + 3] = fmaf(t.k[i].w, u, s[4 * i + 3]);
        acc[0] = fmaf(t.q[i].x, s[4 * i], acc[0]);
        acc[1] = fmaf(t.q[i].y, s[4 * i + 1], acc[1]);
        acc[2] = fmaf(t.q[i].z, s[4 * i + 2], acc[2]);
        acc[3] = fmaf(t.q[i].w, s[4 * i + 3], acc[3]);
      }
      const float out = group_sum<RG>((acc[0] + acc[1]) + (acc[2] + acc[3]));
      if (writes) *op = out;
      op += out_stride;
    };
    Operands ta, tb;
    read_token(ta, 0);
    for (int tt = 0; tt < n; tt += 2) {
      if (tt + 1 < n) read_token(tb, tt + 1);
      chain(ta);
      if (tt + 1 < n) {
        if (tt + 2 < n) read_token(ta, tt + 2);
        chain(tb);
      }
    }
    if (more) park(regs, stage[cur ^ 1]);
    __syncthreads();
    cur ^= 1;
  }
#pragma unroll
  for (int i = 0; i < ROWS; ++i)
    if (col_ok && d0 + i < D) S[(size_t)(d0 + i) * E + j] = s[i];
}

extern "C" int ns_delta_scan(float* o, const float* qkv, int C, const float* g, const float* beta, float* state, size_t slot_stride,
                             const int* qo_indptr, const int* state_slots, int n_reqs, int H, int G, int D, int E, hipStream_t stream) {
  if (n_reqs <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || D > ND_ROWS * NS_WAVE || E <= 0 || H > 65535) return NS_ERR_BAD_ARG;
  DeltaShape p;
  p.C = C, p.H = H, p.G = G, p.D = D, p.E = E;
  // A thread owns 8 key channels of a column where the key size allows it (more, shorter chains: a token's step is
  // latency, and a single request leaves most of the GPU idle anyway), 16 beyond 512 channels.
  const int rows = D <= 8 * NS_WAVE ? 8 : ND_ROWS;
  p.RG = 1;
  while (p.RG * rows < D) p.RG *= 2;
  p.Dl = p.RG * (rows + 4);
  p.cols = 256 / p.RG;
  p.tok_stride = 3 * p.Dl + ((p.cols + 1 + 3) / 4) * 4;
  p.stage_tokens = ND_STAGE_FLOATS / p.tok_stride;
  if (p.stage_tokens < 1) return NS_ERR_BAD_ARG;
  if (p.stage_tokens > 64) p.stage_tokens = 64;
  // 16-byte loads where every group of four that a thread fetches starts at a multiple of four floats
  p.vec4 = (D % 4 == 0 && E % 4 == 0 && C % 4 == 0 && ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)g % 16) == 0) ? 1 : 0;
  const int zb = (E + p.cols - 1) / p.cols;
  if (n_reqs > 65535) return NS_ERR_BAD_ARG;
  const dim3 grid(zb, H, n_reqs);
#define ND_LAUNCH2(R, W)                                                                                                               \
  if (p.vec4) delta_scan_kernel<true, R, W><<<grid, 256, 0, stream>>>(o, qkv, g, beta, state, slot_stride, qo_indptr, state_slots, p); \
  else delta_scan_kernel<false, R, W><<<grid, 256, 0, stream>>>(o, qkv, g, beta, state, slot_stride, qo_indptr, state_slots, p)
#define ND_LAUNCH(R)                    \
  case R:                               \
    if (rows == 8) { ND_LAUNCH2(R, 8); } \
    else { ND_LAUNCH2(R, ND_ROWS); }    \
    break
  switch (p.RG) {
    ND_LAUNCH(1);
    ND_LAUNCH(2);
    ND_LAUNCH(4);
    ND_LAUNCH(8);
    ND_LAUNCH(16);
    ND_LAUNCH(32);
    default: ND_LAUNCH(64);
  }
#undef ND_LAUNCH2
#undef ND_LAUNCH
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// out[r][h][:] = o / sqrt(mean(o^2) + eps) * w[:] * sigmoid(gate[r][h][:]),  o float, gate and out in the model's type.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void gated_rms_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ gate, int gate_stride,
                                 const float* __restrict__ w, int w_stride, const float* __restrict__ den, int H, int E, float eps, int silu) {
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  if (w) w += (size_t)h * w_stride;  // 0: all heads share one weight; no weight at all: the factor is 1
  const float* p = o + ((size_t)r * H + h) * E;
  const float dinv = den ? 1.f / den[(size_t)r * H + h] : 1.f;  // a head's read-out that comes undivided
  float ss = 0.f;
  for (int e = lane; e < E; e += NS_WAVE) {
    const float v = p[e] * dinv;
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float rinv = 1.f / sqrtf(ss / (float)E + eps);
  for (int e = lane; e < E; e += NS_WAVE) {
    const float z = to_f(gate[(size_t)r * gate_stride + (size_t)h * E + e]);
    // the gate: sigmoid(z), or with ``silu`` z sigmoid(z)
    out[((size_t)r * H + h) * E + e] = from_f<T>(p[e] * dinv * rinv * (w ? w[e] : 1.f) * (silu ? z : 1.f) / (1.f + expf(-z)));
  }
}

extern "C" int ns_gated_rms(void* out, const float* o, const void* gate, int gate_stride, const float* w, int w_stride, const float* den,
                            int n_tokens, int H, int E, float eps, int silu, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || H <= 0 || H > 65535 || E <= 0) return NS_ERR_BAD_ARG;
  dim3 grid(n_tokens, H);
  if (dtype == NS_DTYPE_F32)
    gated_rms_kernel<float><<<grid, NS_WAVE, 0, stream>>>((float*)out, o, (const float*)gate, gate_stride, w, w_stride, den, H, E, eps, silu);
  else if (dtype == NS_DTYPE_BF16)
    gated_rms_kernel<bf16_t><<<grid, NS_WAVE, 0, stream>>>((bf16_t*)out, o, (const bf16_t*)gate, gate_stride, w, w_stride, den, H, E, eps, silu);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
