// Retention: linear attention with one fixed decay per head, no soft-max and no denominator, token by token in 32-bit.
// Per head, S [D][E] (a new sequence starts with S = 0):
//     S_t = decay_h S_(t-1) + k_t v_t^T;   o_t = S_t^T q_t
// q and k are rotated by their position and k is multiplied by ``k_scale`` first.
//
//   retention_prep   a token's row [.. q .. k .. v ..] of the layer's first product (the model's precision) -> 32-bit rows
//                    [q rotated | k rotated and scaled | v]: angles, cosine, sine and the rotation in 32-bit
//   retention_scan   the recurrence over every request's tokens of the step, in order, from the state in its slot
//   gate_mul         y = x * sigmoid(g) or x * g sigmoid(g), the gate formed in 32-bit (the soft-max attention's output gate)
//
// The scan is laid out like the matrix memory's (memory.hip): a column of S never meets another column, so a wave owns 64 / TPC
// columns and the TPC lanes of a column hold 8 key channels each; their partial sums meet through the vector unit's lane
// permutations (``group_sum``).  A workgroup is four waves that share the staged operands: the next block of tokens is
// fetched into registers while the current block is worked through from LDS; four tokens are worked through together, and
// only S passes from token to token.  A token's arithmetic is the same whatever portion it arrives in.
// State slot of a request: S as [H][E][D] (a column's key channels contiguous).
#include "common.h"
#include "rope.h"

// One workgroup a token.
template <typename T>
__global__ __launch_bounds__(256) void retention_prep_kernel(const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off,
                                                             const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                                             float* __restrict__ out, int H, int D, int E, RopeForm form, float k_scale) {
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * stride;
  float* o = out + (size_t)t * H * (2 * D + E);
  const int pos = positions[t];
  const int half = form.rot / 2;
  // rotated pairs of q and k: item = (which, head, pair)
  for (int i = threadIdx.x; i < 2 * H * half; i += blockDim.x) {
    const int which = i / (H * half), h = (i / half) % H, j = i % half;
    int d1, d2;
    rope_pair_channels(form, j, d1, d2);
    const T* src = row + (which ? k_off : q_off) + (size_t)h * D;
    float c, s, a, b;
    rope_cos_sin(form, pos, inv_freq[j], c, s);
    rope_turn(to_f(src[d1]), to_f(src[d2]), c, s, a, b);
    const float m = which ? k_scale : 1.f;
    float* dst = o + (size_t)which * H * D + (size_t)h * D;
    dst[d1] = a * m;
    dst[d2] = b * m;
  }
  const int rest = D - form.rot;
  for (int i = threadIdx.x; i < 2 * H * rest; i += blockDim.x) {
    const int which = i / (H * rest), h = (i / rest) % H, d = form.rot + i % rest;
    o[(size_t)which * H * D + (size_t)h * D + d] = to_f(row[(which ? k_off : q_off) + (size_t)h * D + d]) * (which ? k_scale : 1.f);
  }
  for (int i = threadIdx.x; i < H * E; i += blockDim.x) o[(size_t)2 * H * D + i] = to_f(row[v_off + i]);
}

extern "C" int ns_retention_prep(const void* proj, int stride, int q_off, int k_off, int v_off, const int* positions, const float* inv_freq,
                                 float* out, int n_tokens, int H, int D, int E, int rot, int interleaved, float factor, float k_scale, int dtype,
                                 hipStream_t stream) {
  if (n_tokens <= 0 || H <= 0 || D <= 0 || E <= 0 || rot < 0 || rot > D || rot % 2 || (rot > 0 && !inv_freq)) return NS_ERR_BAD_ARG;
  const RopeForm form{rot, interleaved, factor};
  if (dtype == NS_DTYPE_F32)
    retention_prep_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)proj, stride, q_off, k_off, v_off, positions, inv_freq, out, H, D, E, form, k_scale);
  else if (dtype == NS_DTYPE_BF16)
    retention_prep_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const bf16_t*)proj, stride, q_off, k_off, v_off, positions, inv_freq, out, H, D, E, form, k_scale);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

#define RT_KPT 8  // key channels a lane holds of its column
#define RT_WAVES 4
#define RT_THREADS (RT_WAVES * NS_WAVE)

struct RetentionParams {
  const float* qkv;  // [tokens][H * (2 D + E)]: q | k | v
  const float* decay;  // [H]
  float* state;        // [slots][state_stride]
  long long state_stride;
  const int* qo_indptr;
  const int* state_slots;
  float* out;  // [tokens][H * E]
  int H, D, E;
  int vec_ok;  // 8 channels of q and k can be fetched with aligned vector loads
};

template <int TPC>
__global__ __launch_bounds__(RT_THREADS) void retention_scan_kernel(const RetentionParams p) {
  constexpr int DP = RT_KPT * TPC;                           // key channels of a column as the lanes hold them (D padded)
  constexpr int CPW = NS_WAVE / TPC;                         // columns a wave owns
  constexpr int CPG = CPW * RT_WAVES;                        // columns a workgroup owns
  constexpr int TB = TPC <= 16 ? 16 : (TPC == 32 ? 8 : 4);   // tokens a block
  constexpr int SLICES = TB * 2 * TPC;                       // 8-channel pieces of q and k in a block
  constexpr int PER = (SLICES + RT_THREADS - 1) / RT_THREADS;  // pieces a thread fetches
  constexpr int VALS = TB * CPG;                             // values of v in a block
  constexpr int VPER = (VALS + RT_THREADS - 1) / RT_THREADS;
  __shared__ __attribute__((aligned(16))) float qk_s[TB * 2 * DP];  // per token: q [DP], k [DP]
  __shared__ float v_s[VALS];

  const int tid = threadIdx.x, lane = tid % NS_WAVE, wave = tid / NS_WAVE, h = blockIdx.y, b = blockIdx.z;
  const int t0 = p.qo_indptr[b], t1 = p.qo_indptr[b + 1];
  if (t1 <= t0) return;
  const int H = p.H, D = p.D, E = p.E;
  const int row_w = H * (2 * D + E);
  const int s = lane % TPC, cw = wave * CPW + lane / TPC, col = blockIdx.x * CPG + cw, d0 = s * RT_KPT;
  const bool col_ok = col < E;
  float* st_S = p.state + (long long)p.state_slots[b] * p.state_stride + ((size_t)h * E + (col_ok ? col : 0)) * D;
  const float a = p.decay[h];

  float S[RT_KPT];
#pragma unroll
  for (int j = 0; j < RT_KPT; ++j) S[j] = (col_ok && d0 + j < D) ? st_S[d0 + j] : 0.f;

  float pre[PER][RT_KPT], vpre[VPER];
  auto fetch = [&](int t) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = tid + i * RT_THREADS;  // (token, q or k, piece)
      const int tk = idx / (2 * TPC), which = (idx / TPC) % 2, piece = idx % TPC;
      const bool live = idx < SLICES && t + tk < t1;
      const float* src = p.qkv + (size_t)(t + (live ? tk : 0)) * row_w + (size_t)which * H * D + (size_t)h * D + piece * RT_KPT;
      if (live && p.vec_ok && piece * RT_KPT + RT_KPT <= D) {
        const float4 x = *reinterpret_cast<const float4*>(src), y = *reinterpret_cast<const float4*>(src + 4);
        pre[i][0] = x.x, pre[i][1] = x.y, pre[i][2] = x.z, pre[i][3] = x.w, pre[i][4] = y.x, pre[i][5] = y.y, pre[i][6] = y.z, pre[i][7] = y.w;
      } else {
#pragma unroll
        for (int j = 0; j < RT_KPT; ++j) pre[i][j] = (live && piece * RT_KPT + j < D) ? src[j] : 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < VPER; ++i) {
      const int idx = tid + i * RT_THREADS, tk = idx / CPG, c = blockIdx.x * CPG + idx % CPG;
      vpre[i] = (idx < VALS && t + tk < t1 && c < E) ? p.qkv[(size_t)(t + tk) * row_w + (size_t)2 * H * D + (size_t)h * E + c] : 0.f;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = tid + i * RT_THREADS;
      if (idx < SLICES) {
        float4* dst = reinterpret_cast<float4*>(qk_s + (size_t)idx * RT_KPT);
        dst[0] = make_float4(pre[i][0], pre[i][1], pre[i][2], pre[i][3]);
        dst[1] = make_float4(pre[i][4], pre[i][5], pre[i][6], pre[i][7]);
      }
    }
#pragma unroll
    for (int i = 0; i < VPER; ++i) {
      const int idx = tid + i * RT_THREADS;
      if (idx < VALS) v_s[idx] = vpre[i];
    }
  };

  fetch(t0);
  stage();
  __syncthreads();
  constexpr int UN = 4;  // tokens worked through together: only S passes from token to token
  static_assert(TB % UN == 0, "a block of tokens is whole groups");
  for (int t = t0; t < t1; t += TB) {
    if (t + TB < t1) fetch(t + TB);
    const int nb = min(TB, t1 - t);
    for (int tk0 = 0; tk0 < nb; tk0 += UN) {
      float num[UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const bool on = tk0 + u < nb;
        const float au = on ? a : 1.f;  // (tokens beyond the block's end change nothing: their k and v are zero)
        const float vv = v_s[(tk0 + u) * CPG + cw];
        const float4* qp = reinterpret_cast<const float4*>(qk_s + (size_t)((tk0 + u) * 2) * DP + d0);
        const float4* kp = reinterpret_cast<const float4*>(qk_s + (size_t)((tk0 + u) * 2 + 1) * DP + d0);
        const float4 q0 = qp[0], q1 = qp[1], k0 = kp[0], k1 = kp[1];
        const float q[RT_KPT] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        const float k[RT_KPT] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
        float p0 = 0.f, p1 = 0.f;  // two partial sums: shorter chains
#pragma unroll
        for (int j = 0; j < RT_KPT; j += 2) {
          S[j] = fmaf(au, S[j], k[j] * vv);
          S[j + 1] = fmaf(au, S[j + 1], k[j + 1] * vv);
          p0 = fmaf(S[j], q[j], p0);
          p1 = fmaf(S[j + 1], q[j + 1], p1);
        }
        num[u] = p0 + p1;
      }
#pragma unroll
      for (int u = 0; u < UN; ++u) num[u] = group_sum<TPC>(num[u]);
      if (s == 0 && col_ok) {
#pragma unroll
        for (int u = 0; u < UN; ++u)
          if (tk0 + u < nb) p.out[(size_t)(t + tk0 + u) * H * E + (size_t)h * E + col] = num[u];
      }
    }
    __syncthreads();
    if (t + TB < t1) stage();
    __syncthreads();
  }
  if (col_ok) {
#pragma unroll
    for (int j = 0; j < RT_KPT; ++j)
      if (d0 + j < D) st_S[d0 + j] = S[j];
  }
}

extern "C" int ns_retention_scan(const float* qkv, const float* decay, float* state, long long state_stride, const int* qo_indptr,
                                 const int* state_slots, float* out, int n_reqs, int H, int D, int E, hipStream_t stream) {
  if (n_reqs <= 0 || n_reqs > 65535 || H <= 0 || H > 65535 || D <= 0 || E <= 0) return NS_ERR_BAD_ARG;
  int tpc = 1;
  while (tpc * RT_KPT < D) tpc *= 2;
  if (tpc > NS_WAVE) return NS_ERR_UNSUPPORTED;
  if (state_stride < (long long)H * E * D) return NS_ERR_BAD_ARG;
  RetentionParams p{qkv, decay, state, state_stride, qo_indptr, state_slots, out, H, D, E, 0};
  p.vec_ok = D % 8 == 0 && (H * (2 * D + E)) % 4 == 0 && ((uintptr_t)qkv % 16) == 0;
  const int cpg = RT_WAVES * NS_WAVE / tpc;
  dim3 grid((E + cpg - 1) / cpg, H, n_reqs);
  switch (tpc) {
    case 1: retention_scan_kernel<1><<<grid, RT_THREADS, 0, stream>>>(p); break;
    case 2: retention_scan_kernel<2><<<grid, RT_THREADS, 0, stream>>>(p); break;
    case 4: retention_scan_kernel<4><<<grid, RT_THREADS, 0, stream>>>(p); break;
    case 8: retention_scan_kernel<8><<<grid, RT_THREADS, 0, stream>>>(p); break;
    case 16: retention_scan_kernel<16><<<grid, RT_THREADS, 0, stream>>>(p); break;
    case 32: retention_scan_kernel<32><<<grid, RT_THREADS, 0, stream>>>(p); break;
    default: retention_scan_kernel<64><<<grid, RT_THREADS, 0, stream>>>(p); break;
  }
  return ns_launch_status();
}

// y[t][i] = x[t][i] * sigmoid(g[t][i])  (silu = 0)  or  x[t][i] * g[t][i] sigmoid(g[t][i])  (silu = 1); g may be a column slice
template <typename T>
__global__ void gate_mul_kernel(T* __restrict__ out, const T* __restrict__ x, const T* __restrict__ g, int g_stride, int width, size_t count, int silu) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const size_t t = i / width, c = i % width;
  const float z = to_f(g[t * g_stride + c]);
  const float gate = (silu ? z : 1.f) / (1.f + expf(-z));
  out[i] = from_f<T>(to_f(x[i]) * gate);
}

extern "C" int ns_gate_mul(void* out, const void* x, const void* g, int g_stride, int n, int width, int silu, int dtype, hipStream_t stream) {
  if (n <= 0 || width <= 0) return NS_ERR_BAD_ARG;
  const size_t count = (size_t)n * width, blocks = (count + 255) / 256;
  if (blocks > 0x7fffffff) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    gate_mul_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)x, (const float*)g, g_stride, width, count, silu);
  else if (dtype == NS_DTYPE_BF16)
    gate_mul_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, (const bf16_t*)g, g_stride, width, count, silu);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
