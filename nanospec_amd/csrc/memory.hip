// A matrix memory with exponential gates (the mLSTM recurrence), token by token in 32-bit.  Per head: a matrix S [D][E], a
// vector n [D] and a running maximum m (a new sequence starts with S = 0, n = 0, m = 0):
//   i = cap tanh((x_i + b_i) / cap)                        log of the input gate
//   f = logsigmoid(cap tanh((x_f + b_f) / cap))            log of the forget gate
//   m' = max(f + m, i);   a = exp(f + m - m');   b = exp(i - m')
//   S <- a S + b k v^T;   n <- a n + b k;   o = S^T q / (max(|n . q|, exp(-m')) + den_eps)
// q (times ``q_scale``), k [H][D], v [H][E] and the two gate inputs x_i, x_f [H] are columns of one row per token (the
// result of one stacked product), in the model's precision; everything from there on is 32-bit.
//
// A column of S never meets another column, so a wave owns 64 / TPC columns and the TPC lanes of a column hold 8 key
// channels each; their partial sums meet through the vector unit's lane permutations (``group_sum``).  n is one more column
// of S, the one whose value is 1 for every token: one more workgroup a head carries it, and what it writes per token is the
// denominator max(|n . q|, exp(-m')) + den_eps.  The kernel leaves S^T q and the denominators; whoever reads the read-out
// divides (``gated_rms`` does, as it reads a head).  A workgroup is four waves that share the staged operands: the next
// block of tokens is fetched into registers while the current block is worked through from LDS, and four tokens are
// worked through together: only m, S and n pass from token to token.
//
// What a request keeps between steps lies in its state slot: S as [H][E][D] (a column's key channels contiguous), then
// room for n per workgroup of a head, [H][B][D] (the last workgroup's is the one in use), then m per workgroup, [H][B],
// with B = ``ns_memory_blocks(D, E)`` the workgroups of a head: each reads and writes only its own copy of m, so none can
// read what another has already written for the next step.
#include "common.h"

#define MM_KPT 8  // key channels a lane holds of its column
#define MM_WAVES 4
#define MM_THREADS (MM_WAVES * NS_WAVE)

template <typename T> struct Vec8;
template <> struct Vec8<float> {
  static __device__ __forceinline__ void load(const float* p, float* out) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    out[0] = a.x, out[1] = a.y, out[2] = a.z, out[3] = a.w, out[4] = b.x, out[5] = b.y, out[6] = b.z, out[7] = b.w;
  }
};
template <> struct Vec8<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float* out) {
    typedef bf16_t v8 __attribute__((ext_vector_type(8)));
    const v8 a = *reinterpret_cast<const v8*>(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) out[j] = (float)a[j];
  }
};

__device__ __forceinline__ float mm_log_sigmoid(float z) {
  // log(1 / (1 + exp(-z))) without overflow on either side
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

struct MemoryParams {
  const void* proj;  // [tokens][stride]
  int stride, q_off, k_off, v_off, i_off, f_off;
  const float* gate_bias_i;  // [H]
  const float* gate_bias_f;  // [H]
  float* state;              // [slots][state_stride]
  long long state_stride;
  const int* qo_indptr;
  const int* state_slots;
  float* out;  // [tokens][H * E]: S^T q, not yet divided
  float* den;  // [tokens][H]: max(|n . q|, exp(-m)) + den_eps
  int H, D, E;
  float cap, q_scale, den_eps;
  int vec_ok;  // 8 channels of q and k can be fetched with one aligned vector load
};

template <typename T, int TPC>
__global__ __launch_bounds__(MM_THREADS) void memory_scan_kernel(const MemoryParams p) {
  constexpr int DP = MM_KPT * TPC;                           // key channels of a column as the lanes hold them (D padded)
  constexpr int CPW = NS_WAVE / TPC;                         // columns a wave owns
  constexpr int CPG = CPW * MM_WAVES;                        // columns a workgroup owns
  constexpr int TB = TPC <= 16 ? 16 : (TPC == 32 ? 8 : 4);   // tokens a block
  constexpr int SLICES = TB * 2 * TPC;                       // 8-channel pieces of q and k in a block
  constexpr int PER = (SLICES + MM_THREADS - 1) / MM_THREADS;  // pieces a thread fetches
  constexpr int VALS = TB * CPG;                             // values of v in a block
  constexpr int VPER = (VALS + MM_THREADS - 1) / MM_THREADS;
  __shared__ __attribute__((aligned(16))) float qk_s[TB * 2 * DP];  // per token: q [DP], k [DP]
  __shared__ float v_s[VALS];
  __shared__ float gate_s[TB * 2];

  const int tid = threadIdx.x, lane = tid % NS_WAVE, wave = tid / NS_WAVE, h = blockIdx.y, b = blockIdx.z;
  const int t0 = p.qo_indptr[b], t1 = p.qo_indptr[b + 1];
  if (t1 <= t0) return;
  const int H = p.H, D = p.D, E = p.E;
  const int s = lane % TPC, cw = wave * CPW + lane / TPC, col = blockIdx.x * CPG + cw, d0 = s * MM_KPT;
  // the last workgroup of a head carries n as one more column of S whose value is 1 for every token: its first column's
  // lanes hold n where the others hold a column of S, and what it writes is the denominator
  const bool nblock = blockIdx.x == gridDim.x - 1;
  const bool col_ok = !nblock && col < E, n_lane = nblock && cw == 0;
  const T* proj = (const T*)p.proj;
  float* st = p.state + (long long)p.state_slots[b] * p.state_stride;
  float* st_S = st + ((size_t)h * E + (col_ok ? col : 0)) * D;
  const int B = gridDim.x;
  float* st_n = st + (size_t)H * E * D + ((size_t)h * B + blockIdx.x) * D;
  float* st_m = st + (size_t)H * E * D + (size_t)H * B * D + (size_t)h * B + blockIdx.x;

  float S[MM_KPT];
#pragma unroll
  for (int j = 0; j < MM_KPT; ++j) {
    const bool ok = d0 + j < D;
    S[j] = (ok && col_ok) ? st_S[d0 + j] : ((ok && n_lane) ? st_n[d0 + j] : 0.f);
  }
  float m = *st_m;
  const float bias_i = p.gate_bias_i ? p.gate_bias_i[h] : 0.f, bias_f = p.gate_bias_f ? p.gate_bias_f[h] : 0.f;

  float pre[PER][MM_KPT], vpre[VPER], gpre = 0.f;

  // fetch the operands of tokens [t, t + TB) into registers
  auto fetch = [&](int t) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = tid + i * MM_THREADS;  // (token, q or k, piece)
      const int tk = idx / (2 * TPC), which = (idx / TPC) % 2, piece = idx % TPC;
      const bool live = idx < SLICES && t + tk < t1;
      const T* src = proj + (size_t)(t + (live ? tk : 0)) * p.stride + (which ? p.k_off : p.q_off) + (size_t)h * D + piece * MM_KPT;
      if (live && p.vec_ok && piece * MM_KPT + MM_KPT <= D) {
        Vec8<T>::load(src, pre[i]);
      } else {
#pragma unroll
        for (int j = 0; j < MM_KPT; ++j) pre[i][j] = (live && piece * MM_KPT + j < D) ? to_f(src[j]) : 0.f;
      }
      if (!which) {
#pragma unroll
        for (int j = 0; j < MM_KPT; ++j) pre[i][j] *= p.q_scale;
      }
    }
#pragma unroll
    for (int i = 0; i < VPER; ++i) {
      const int idx = tid + i * MM_THREADS, tk = idx / CPG, c = blockIdx.x * CPG + idx % CPG;
      if (nblock)
        vpre[i] = idx % CPG == 0 ? 1.f : 0.f;
      else
        vpre[i] = (idx < VALS && t + tk < t1 && c < E) ? to_f(proj[(size_t)(t + tk) * p.stride + p.v_off + (size_t)h * E + c]) : 0.f;
    }
    if (tid < 2 * TB) {
      const int tk = tid / 2, which = tid % 2;
      if (t + tk < t1) {
        const float x = to_f(proj[(size_t)(t + tk) * p.stride + (which ? p.f_off : p.i_off) + h]) + (which ? bias_f : bias_i);
        const float capped = p.cap * tanhf(x / p.cap);
        gpre = which ? mm_log_sigmoid(capped) : capped;
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = tid + i * MM_THREADS;
      if (idx < SLICES) {
        float4* dst = reinterpret_cast<float4*>(qk_s + (size_t)idx * MM_KPT);
        dst[0] = make_float4(pre[i][0], pre[i][1], pre[i][2], pre[i][3]);
        dst[1] = make_float4(pre[i][4], pre[i][5], pre[i][6], pre[i][7]);
      }
    }
#pragma unroll
    for (int i = 0; i < VPER; ++i) {
      const int idx = tid + i * MM_THREADS;
      if (idx < VALS) v_s[idx] = vpre[i];
    }
    if (tid < 2 * TB) gate_s[tid] = gpre;
  };

  fetch(t0);
  stage();
  __syncthreads();
  constexpr int UN = 4;  // tokens worked through together: only m, S and n pass from token to token, the rest overlaps
  static_assert(TB % UN == 0, "a block of tokens is whole groups");
  for (int t = t0; t < t1; t += TB) {
    if (t + TB < t1) fetch(t + TB);
    const int nb = min(TB, t1 - t);
    for (int tk0 = 0; tk0 < nb; tk0 += UN) {
      float a[UN], bv[UN], em[UN], num[UN];
      // the gates' chain: additions and maxima only; the exponentials hang off it
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const bool on = tk0 + u < nb;
        const float gi = gate_s[2 * (tk0 + u)], gf = gate_s[2 * (tk0 + u) + 1];
        const float mn = fmaxf(gf + m, gi);
        a[u] = on ? expf(gf + m - mn) : 1.f;
        const float bb = on ? expf(gi - mn) : 0.f;
        m = on ? mn : m;
        em[u] = nblock ? expf(-m) : 0.f;
        bv[u] = bb * v_s[(tk0 + u) * CPG + cw];
      }
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const float4* qp = reinterpret_cast<const float4*>(qk_s + (size_t)((tk0 + u) * 2) * DP + d0);
        const float4* kp = reinterpret_cast<const float4*>(qk_s + (size_t)((tk0 + u) * 2 + 1) * DP + d0);
        const float4 q0 = qp[0], q1 = qp[1], k0 = kp[0], k1 = kp[1];
        const float q[MM_KPT] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        const float k[MM_KPT] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
        float p0 = 0.f, p1 = 0.f;  // two partial sums: shorter chains
#pragma unroll
        for (int j = 0; j < MM_KPT; j += 2) {
          S[j] = fmaf(a[u], S[j], k[j] * bv[u]);
          S[j + 1] = fmaf(a[u], S[j + 1], k[j + 1] * bv[u]);
          p0 = fmaf(S[j], q[j], p0);
          p1 = fmaf(S[j + 1], q[j + 1], p1);
        }
        num[u] = p0 + p1;
      }
#pragma unroll
      for (int u = 0; u < UN; ++u) num[u] = group_sum<TPC>(num[u]);
      if (s == 0 && (col_ok || n_lane)) {
#pragma unroll
        for (int u = 0; u < UN; ++u)
          if (tk0 + u < nb) {
            if (n_lane)
              p.den[(size_t)(t + tk0 + u) * H + h] = fmaxf(fabsf(num[u]), em[u]) + p.den_eps;
            else
              p.out[(size_t)(t + tk0 + u) * H * E + (size_t)h * E + col] = num[u];
          }
      }
    }
    __syncthreads();
    if (t + TB < t1) stage();
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < MM_KPT; ++j) {
    if (d0 + j < D) {
      if (col_ok) st_S[d0 + j] = S[j];
      if (n_lane) st_n[d0 + j] = S[j];
    }
  }
  if (tid == 0) *st_m = m;
}

template <typename T>
static int memory_scan_launch(const MemoryParams& p, int n_reqs, hipStream_t stream) {
  int tpc = 1;
  while (tpc * MM_KPT < p.D) tpc *= 2;
  if (tpc > NS_WAVE) return NS_ERR_UNSUPPORTED;
  const int cpg = MM_WAVES * NS_WAVE / tpc;
  dim3 grid((p.E + cpg - 1) / cpg + 1, p.H, n_reqs);  // one more workgroup a head: the one that carries n
  switch (tpc) {
    case 1: memory_scan_kernel<T, 1><<<grid, MM_THREADS, 0, stream>>>(p); break;
    case 2: memory_scan_kernel<T, 2><<<grid, MM_THREADS, 0, stream>>>(p); break;
    case 4: memory_scan_kernel<T, 4><<<grid, MM_THREADS, 0, stream>>>(p); break;
    case 8: memory_scan_kernel<T, 8><<<grid, MM_THREADS, 0, stream>>>(p); break;
    case 16: memory_scan_kernel<T, 16><<<grid, MM_THREADS, 0, stream>>>(p); break;
    case 32: memory_scan_kernel<T, 32><<<grid, MM_THREADS, 0, stream>>>(p); break;
    default: memory_scan_kernel<T, 64><<<grid, MM_THREADS, 0, stream>>>(p); break;
  }
  return ns_launch_status();
}

// workgroups of one head: those that share its columns and the one that carries n (each keeps a copy of m, and room for n, in the state)
extern "C" int ns_memory_blocks(int D, int E) {
  int tpc = 1;
  while (tpc * MM_KPT < D) tpc *= 2;
  if (tpc > NS_WAVE) return -1;
  const int cpg = MM_WAVES * NS_WAVE / tpc;
  return (E + cpg - 1) / cpg + 1;
}

extern "C" int ns_memory_scan(const void* proj, int stride, int q_off, int k_off, int v_off, int i_off, int f_off, const float* gate_bias_i,
                              const float* gate_bias_f, float* state, long long state_stride, const int* qo_indptr, const int* state_slots,
                              float* out, float* den, int n_reqs, int H, int D, int E, float cap, float q_scale, float den_eps, int dtype, hipStream_t stream) {
  if (n_reqs <= 0 || n_reqs > 65535 || H <= 0 || H > 65535 || D <= 0 || E <= 0 || !(cap > 0.f)) return NS_ERR_BAD_ARG;
  const int blocks = ns_memory_blocks(D, E);
  if (blocks < 0) return NS_ERR_UNSUPPORTED;
  if (state_stride < (long long)H * E * D + (long long)H * blocks * (D + 1)) return NS_ERR_BAD_ARG;
  MemoryParams p{proj, stride, q_off, k_off, v_off, i_off, f_off, gate_bias_i, gate_bias_f, state, state_stride, qo_indptr, state_slots,
                 out, den, H, D, E, cap, q_scale, den_eps, 0};
  const size_t elem = dtype == NS_DTYPE_F32 ? 4 : 2;
  p.vec_ok = D % 8 == 0 && stride % 8 == 0 && q_off % 8 == 0 && k_off % 8 == 0 && ((uintptr_t)proj % (8 * elem)) == 0;
  if (dtype == NS_DTYPE_F32) return memory_scan_launch<float>(p, n_reqs, stream);
  if (dtype == NS_DTYPE_BF16) return memory_scan_launch<bf16_t>(p, n_reqs, stream);
  return NS_ERR_UNSUPPORTED;
}
