// A mixture of small gated feed-forward experts, and the per-layer token input of a decoder that has one.
//
// Router: z = W_r h + b in 32-bit; the ``top`` largest logits are chosen (the lower index wins a tie) and weighted by the
// soft-max over the chosen logits alone; or sigmoid scores with a correction on the choice and groups of experts (see
// ``moe_choose_kernel``).
// Expert (``clipped GLU``): g = min(W_gate h, limit); u = clamp(W_up h, -limit, limit); y = W_down (g sigmoid(alpha g) (u + shift));
// an infinite limit clips nothing, and with alpha = 1 and shift = 0 the expert is W_down (silu(W_gate h) * W_up h).
// The experts' matrices are stacked: gate and up [experts][ff][W], down [experts][W][ff].
#include "common.h"

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 32

// Two kernels.  Logits: a workgroup takes ROUTE_TOK tokens and four experts, a wave an expert: it reads the expert's row
// once (16 bytes a lane a load where the sizes allow) for all of its tokens.  Choice: a wave a token.
#define ROUTE_TOK 8
template <typename T>
__global__ __launch_bounds__(256) void moe_logits_kernel(const T* __restrict__ h, int h_stride, const float* __restrict__ wr,
                                                         const float* __restrict__ br, float* __restrict__ z, int n, int W, int experts, int vec) {
  const int t0 = blockIdx.x * ROUTE_TOK, lane = threadIdx.x % NS_WAVE, wave = threadIdx.x / NS_WAVE;
  const int e = blockIdx.y * (blockDim.x / NS_WAVE) + wave;
  if (e >= experts) return;
  const int nt = min(ROUTE_TOK, n - t0);
  const float* w = wr + (size_t)e * W;
  float acc[ROUTE_TOK];
#pragma unroll
  for (int i = 0; i < ROUTE_TOK; ++i) acc[i] = 0.f;
  if (vec) {
#pragma unroll 2
    for (int c = lane * 4; c < W; c += NS_WAVE * 4) {
      const float4 wc = *reinterpret_cast<const float4*>(w + c);
#pragma unroll
      for (int i = 0; i < ROUTE_TOK; ++i)
        if (i < nt) {
          const T* x = h + (size_t)(t0 + i) * h_stride + c;
          acc[i] = fmaf(to_f(x[0]), wc.x, acc[i]), acc[i] = fmaf(to_f(x[1]), wc.y, acc[i]);
          acc[i] = fmaf(to_f(x[2]), wc.z, acc[i]), acc[i] = fmaf(to_f(x[3]), wc.w, acc[i]);
        }
    }
  } else {
    for (int c = lane; c < W; c += NS_WAVE) {
      const float wc = w[c];
#pragma unroll
      for (int i = 0; i < ROUTE_TOK; ++i)
        if (i < nt) acc[i] = fmaf(to_f(h[(size_t)(t0 + i) * h_stride + c]), wc, acc[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < ROUTE_TOK; ++i) {
    const float v = wave_sum(acc[i]);
    if (lane == 0 && i < nt) z[(size_t)(t0 + i) * experts + e] = v + (br ? br[e] : 0.f);
  }
}

// The same logits for a step of few tokens (up to ROUTE_TOK): a workgroup an expert, its four waves a quarter of the row each
// (a wave alone walks a row of 2,048 columns in eight dependent rounds; four waves in two), their sums joined in LDS in a
// fixed order.  A token's logit does not depend on how many tokens the step holds.
template <typename T>
__global__ __launch_bounds__(256) void moe_logits_few_kernel(const T* __restrict__ h, int h_stride, const float* __restrict__ wr,
                                                             const float* __restrict__ br, float* __restrict__ z, int n, int W, int experts, int vec) {
  __shared__ float part[4][ROUTE_TOK];
  const int e = blockIdx.x, lane = threadIdx.x % NS_WAVE, wave = threadIdx.x / NS_WAVE;
  const float* w = wr + (size_t)e * W;
  float acc[ROUTE_TOK];
#pragma unroll
  for (int i = 0; i < ROUTE_TOK; ++i) acc[i] = 0.f;
  if (vec) {
    for (int c = threadIdx.x * 4; c < W; c += 256 * 4) {
      const float4 wc = *reinterpret_cast<const float4*>(w + c);
#pragma unroll
      for (int i = 0; i < ROUTE_TOK; ++i)
        if (i < n) {
          const T* x = h + (size_t)i * h_stride + c;
          acc[i] = fmaf(to_f(x[0]), wc.x, acc[i]), acc[i] = fmaf(to_f(x[1]), wc.y, acc[i]);
          acc[i] = fmaf(to_f(x[2]), wc.z, acc[i]), acc[i] = fmaf(to_f(x[3]), wc.w, acc[i]);
        }
    }
  } else {
    for (int c = threadIdx.x; c < W; c += 256) {
      const float wc = w[c];
#pragma unroll
      for (int i = 0; i < ROUTE_TOK; ++i)
        if (i < n) acc[i] = fmaf(to_f(h[(size_t)i * h_stride + c]), wc, acc[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < ROUTE_TOK; ++i) {
    const float v = wave_sum(acc[i]);
    if (lane == 0) part[wave][i] = v;
  }
  __syncthreads();
  if (threadIdx.x < n) {
    const int i = threadIdx.x;
    z[(size_t)i * experts + e] = ((part[0][i] + part[1][i]) + (part[2][i] + part[3][i])) + (br ? br[e] : 0.f);
  }
}

// A wave a token: the choice scores in LDS, every lane looks through its share for the largest one not yet taken, the lanes'
// candidates meet by lane exchange (the larger value wins, the lower index among equals; what is no number counts as
// minus infinity, so a row of anything still chooses ``top`` different experts).
// ``sigmoid`` = 0: the choice goes by the logits and the weights are the soft-max over the chosen logits.
// ``sigmoid`` = 1: scores s = sigmoid(z); the choice goes by s + correction[e] (``correction`` may be null) and the weights are
// the chosen experts' s, not renormalized.  ``groups`` > 1: the experts form that many equal groups of neighbours; a group's
// score is the sum of its two largest choice scores (of its one, if it has one), and only the ``keep`` best groups' experts
// can be chosen: the others never enter the comparison, whatever their scores' sign.
__device__ __forceinline__ void wave_best(float& bv, int& best) {
#pragma unroll
  for (int o = NS_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, NS_WAVE);
    const int oi = __shfl_xor(best, o, NS_WAVE);
    if (oi >= 0 && (best < 0 || ov > bv || (ov == bv && oi < best))) best = oi, bv = ov;
  }
}

__global__ __launch_bounds__(64) void moe_choose_kernel(const float* __restrict__ z, int* __restrict__ sel, float* __restrict__ wt, int n,
                                                        int experts, int top, int sigmoid, const float* __restrict__ correction, int groups,
                                                        int keep) {
  __shared__ float zs[MOE_MAX_EXPERTS];   // choice scores
  __shared__ float ws[MOE_MAX_EXPERTS];   // what the weights are made from: the logits, or the sigmoid scores
  __shared__ float gs[MOE_MAX_EXPERTS];   // group scores
  __shared__ unsigned char taken[MOE_MAX_EXPERTS];
  __shared__ unsigned char gkept[MOE_MAX_EXPERTS];
  const int t = blockIdx.x, lane = threadIdx.x;
  for (int e = lane; e < experts; e += NS_WAVE) {
    float v = z[(size_t)t * experts + e];
    if (sigmoid) {
      v = 1.f / (1.f + expf(-v));
      ws[e] = v;
      if (correction) v += correction[e];
    } else {
      ws[e] = v;
    }
    zs[e] = v == v ? v : -INFINITY;
    taken[e] = 0;
  }
  __syncthreads();
  if (groups > 1) {
    const int per = experts / groups;
    for (int g = lane; g < groups; g += NS_WAVE) {
      float a = -INFINITY, b = -INFINITY;  // the two largest of the group
      for (int e = g * per; e < (g + 1) * per; ++e) {
        const float v = zs[e];
        if (v > a) b = a, a = v;
        else if (v > b) b = v;
      }
      gs[g] = per > 1 ? a + b : a;
      gkept[g] = 0;
    }
    __syncthreads();
    for (int k = 0; k < keep; ++k) {
      int best = -1;
      float bv = -INFINITY;
      for (int g = lane; g < groups; g += NS_WAVE)
        if (!gkept[g] && (best < 0 || gs[g] > bv)) best = g, bv = gs[g];
      wave_best(bv, best);
      if (lane == 0) gkept[best] = 1;
      __syncthreads();
    }
    for (int e = lane; e < experts; e += NS_WAVE)
      if (!gkept[e / per]) taken[e] = 1;
    __syncthreads();
  }
  float largest = 0.f, sum = 0.f, mine = 0.f;  // lane k keeps the k-th chosen value
  int mine_idx = 0;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bv = -INFINITY;
    for (int e = lane; e < experts; e += NS_WAVE)
      if (!taken[e] && (best < 0 || zs[e] > bv)) best = e, bv = zs[e];
    wave_best(bv, best);
    if (lane == 0) taken[best] = 1;
    float w;
    if (sigmoid) {
      w = ws[best];
    } else {
      if (k == 0) largest = bv;
      w = expf(bv - largest);
    }
    sum += w;
    if (lane == k % NS_WAVE && k < NS_WAVE) mine = w, mine_idx = best;
    __syncthreads();
  }
  if (lane < top) {
    sel[(size_t)t * top + lane] = mine_idx;
    wt[(size_t)t * top + lane] = sigmoid ? mine : mine / sum;
  }
}

// ``z``: scratch, float32 [n][experts]
extern "C" int ns_moe_route(const void* h, int h_stride, const float* wr, const float* br, float* z, int* sel, float* wt, int n, int W, int experts,
                            int top, int sigmoid, const float* correction, int groups, int keep, int dtype, hipStream_t stream) {
  if (n <= 0 || W <= 0 || experts <= 0 || experts > MOE_MAX_EXPERTS || top <= 0 || top > MOE_MAX_TOP || top > experts) return NS_ERR_BAD_ARG;
  if (groups < 1 || experts % groups || keep < 1 || keep > groups || top > keep * (experts / groups)) return NS_ERR_BAD_ARG;
  dim3 grid((n + ROUTE_TOK - 1) / ROUTE_TOK, (experts + 3) / 4);
  if (grid.y > 65535) return NS_ERR_UNSUPPORTED;
  const size_t elem = dtype == NS_DTYPE_F32 ? 4 : 2;
  const int vec = W % 4 == 0 && h_stride % 4 == 0 && (uintptr_t)wr % 16 == 0 && (uintptr_t)h % (4 * elem) == 0;
  if (dtype != NS_DTYPE_F32 && dtype != NS_DTYPE_BF16) return NS_ERR_UNSUPPORTED;
  if (n <= ROUTE_TOK) {  // few tokens: a workgroup an expert
    if (dtype == NS_DTYPE_F32)
      moe_logits_few_kernel<float><<<experts, 256, 0, stream>>>((const float*)h, h_stride, wr, br, z, n, W, experts, vec);
    else
      moe_logits_few_kernel<bf16_t><<<experts, 256, 0, stream>>>((const bf16_t*)h, h_stride, wr, br, z, n, W, experts, vec);
  } else if (dtype == NS_DTYPE_F32)
    moe_logits_kernel<float><<<grid, 256, 0, stream>>>((const float*)h, h_stride, wr, br, z, n, W, experts, vec);
  else
    moe_logits_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)h, h_stride, wr, br, z, n, W, experts, vec);
  moe_choose_kernel<<<n, 64, 0, stream>>>(z, sel, wt, n, experts, top, sigmoid, correction, groups, keep);
  return ns_launch_status();
}

__device__ __forceinline__ float clipped_glu(float g, float u, float limit, float alpha, float shift) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + shift);
}

// ------------------------------------------------------------------------------------------------ few rows
// Steps of few rows stream the chosen experts' matrices, each exactly once per (token, expert) that chose it, cut into
// slices so that the launch fills the chip:
//   first:  grid (slices of inner channels, top, tokens): the token's row in LDS, a wave an inner channel in turn (its gate row
//           and its up row together, 16 bytes a lane a load); act [tokens][top][ff] in 32-bit, rounded as a store in the
//           model's precision would round it
//   second: grid (slices of output channels, top, tokens): the activations in LDS, a wave an output channel in turn;
//           out [tokens][top][W] in 32-bit, already times the router's weight
template <typename T> struct Row8;
template <> struct Row8<float> {
  static __device__ __forceinline__ void load(const float* p, float* out) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    out[0] = a.x, out[1] = a.y, out[2] = a.z, out[3] = a.w, out[4] = b.x, out[5] = b.y, out[6] = b.z, out[7] = b.w;
  }
};
template <> struct Row8<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float* out) {
    typedef bf16_t v8 __attribute__((ext_vector_type(8)));
    const v8 a = __builtin_nontemporal_load(reinterpret_cast<const v8*>(p));
#pragma unroll
    for (int j = 0; j < 8; ++j) out[j] = (float)a[j];
  }
};

// sum_c w[c] x[c] over a wave; ``vec``: K is a multiple of 8 and the row starts at a multiple of 8 elements of an aligned base
template <typename T>
__device__ __forceinline__ float row_dot(const T* __restrict__ w, const float* __restrict__ x, int K, int lane, bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int c = lane * 8; c < K; c += NS_WAVE * 8) {
      float v[8];
      Row8<T>::load(w + c, v);
      const float4 x0 = *reinterpret_cast<const float4*>(x + c), x1 = *reinterpret_cast<const float4*>(x + c + 4);
      acc = fmaf(v[0], x0.x, acc), acc = fmaf(v[1], x0.y, acc), acc = fmaf(v[2], x0.z, acc), acc = fmaf(v[3], x0.w, acc);
      acc = fmaf(v[4], x1.x, acc), acc = fmaf(v[5], x1.y, acc), acc = fmaf(v[6], x1.z, acc), acc = fmaf(v[7], x1.w, acc);
    }
  } else {
    for (int c = lane; c < K; c += NS_WAVE) acc = fmaf(to_f(w[c]), x[c], acc);
  }
  return wave_sum(acc);
}

template <typename T>
__global__ __launch_bounds__(256) void moe_rows_up_kernel(const T* __restrict__ h, int h_stride, const T* __restrict__ wg, const T* __restrict__ wu,
                                                          const int* __restrict__ sel, float* __restrict__ act, int W, int ff, int top, int per,
                                                          float limit, float alpha, float shift, int vec) {
  extern __shared__ __attribute__((aligned(16))) float moe_lds[];  // [W]
  const int t = blockIdx.z, k = blockIdx.y, lane = threadIdx.x % NS_WAVE, wave = threadIdx.x / NS_WAVE, waves = blockDim.x / NS_WAVE;
  const int e = sel[(size_t)t * top + k];
  for (int c = threadIdx.x; c < W; c += blockDim.x) moe_lds[c] = to_f(h[(size_t)t * h_stride + c]);
  __syncthreads();
  const int f0 = blockIdx.x * per, f1 = min(ff, f0 + per);
  for (int f = f0 + wave; f < f1; f += waves) {
    const size_t row = ((size_t)e * ff + f) * W;
    const float g = row_dot(wg + row, moe_lds, W, lane, vec), u = row_dot(wu + row, moe_lds, W, lane, vec);
    if (lane == 0) act[((size_t)t * top + k) * ff + f] = round_to<T>(clipped_glu(round_to<T>(g), round_to<T>(u), limit, alpha, shift));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_rows_down_kernel(const float* __restrict__ act, const T* __restrict__ wd, const int* __restrict__ sel,
                                                            const float* __restrict__ wt, float* __restrict__ out, int W, int ff, int top, int per,
                                                            int vec) {
  extern __shared__ __attribute__((aligned(16))) float moe_lds[];  // [ff]
  const int t = blockIdx.z, k = blockIdx.y, lane = threadIdx.x % NS_WAVE, wave = threadIdx.x / NS_WAVE, waves = blockDim.x / NS_WAVE;
  const int e = sel[(size_t)t * top + k];
  const float share = wt[(size_t)t * top + k];
  for (int f = threadIdx.x; f < ff; f += blockDim.x) moe_lds[f] = act[((size_t)t * top + k) * ff + f];
  __syncthreads();
  const int c0 = blockIdx.x * per, c1 = min(W, c0 + per);
  for (int c = c0 + wave; c < c1; c += waves) {
    const float y = row_dot(wd + ((size_t)e * W + c) * ff, moe_lds, ff, lane, vec);
    if (lane == 0) out[((size_t)t * top + k) * W + c] = share * y;
  }
}

// channels a workgroup takes so that the launch has about 2048 workgroups, a multiple of the four waves
static int moe_slice(int channels, int rows) {
  int per = (int)(((long long)channels * rows + 2047) / 2048);
  per = (per + 3) / 4 * 4;
  return per < 4 ? 4 : per;
}

extern "C" int ns_moe_expert_rows(const void* h, int h_stride, const void* wg, const void* wu, const void* wd, const int* sel, const float* wt,
                                  float* act, float* out, int n, int W, int ff, int top, float limit, float alpha, float shift, int dtype, hipStream_t stream) {
  if (n <= 0 || n > 65535 || W <= 0 || ff <= 0 || top <= 0 || top > 65535) return NS_ERR_BAD_ARG;
  if ((size_t)W * sizeof(float) > 64 * 1024 || (size_t)ff * sizeof(float) > 64 * 1024) return NS_ERR_UNSUPPORTED;
  const size_t elem = dtype == NS_DTYPE_F32 ? 4 : 2;
  const int vec_up = W % 8 == 0 && (uintptr_t)wg % (8 * elem) == 0 && (uintptr_t)wu % (8 * elem) == 0;
  const int vec_down = ff % 8 == 0 && (uintptr_t)wd % (8 * elem) == 0;
  const int per_f = moe_slice(ff, n * top), per_c = moe_slice(W, n * top);
  dim3 g1((ff + per_f - 1) / per_f, top, n), g2((W + per_c - 1) / per_c, top, n);
  if (dtype == NS_DTYPE_F32) {
    moe_rows_up_kernel<float><<<g1, 256, W * sizeof(float), stream>>>((const float*)h, h_stride, (const float*)wg, (const float*)wu, sel, act, W, ff,
                                                                       top, per_f, limit, alpha, shift, vec_up);
    moe_rows_down_kernel<float><<<g2, 256, ff * sizeof(float), stream>>>(act, (const float*)wd, sel, wt, out, W, ff, top, per_c, vec_down);
  } else if (dtype == NS_DTYPE_BF16) {
    moe_rows_up_kernel<bf16_t><<<g1, 256, W * sizeof(float), stream>>>((const bf16_t*)h, h_stride, (const bf16_t*)wg, (const bf16_t*)wu, sel, act, W,
                                                                        ff, top, per_f, limit, alpha, shift, vec_up);
    moe_rows_down_kernel<bf16_t><<<g2, 256, ff * sizeof(float), stream>>>(act, (const bf16_t*)wd, sel, wt, out, W, ff, top, per_c, vec_down);
  } else {
    return NS_ERR_UNSUPPORTED;
  }
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------ many rows
// Steps of many rows (bfloat16): the (token, chosen expert) pairs are sorted by expert on the device, and every expert's
// pairs are cut into tiles of 128 rows.  A workgroup takes one tile and 128 output channels and multiplies on the matrix
// cores (v_mfma_f32_16x16x32_bf16): its four waves own 64 x 64 each, operands come through LDS in pieces of 64 along K,
// the next piece is fetched into registers while the current one is multiplied.  The host never learns which experts were
// chosen: the launch has as many tiles as any choice can need (pairs / 128 + experts), and a tile without rows returns.
//   first:  rows gathered from h by the sorted pairs; gate and up matrices in the same pass; act [pairs sorted][ff] in bfloat16
//   second: act times the down matrix; out [tokens][top][W] in 32-bit, each row back at its pair and times its weight
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

#define MG_TM 128
#define MG_TN 128
#define MG_KC 64
#define MG_LD (MG_KC + 8)  // bfloat16 values between two rows of a staged tile (padded: neighbouring rows start in other banks)
#define MG_RI (MG_TM / 32)  // 16-row blocks of a wave's 64 x 64 (the four waves are 2 x 2)
#define MG_CJ (MG_TN / 32)
#define MG_FA (MG_TM / 32)  // pieces of 8 values that a thread fetches of a staged tile of MG_TM rows (256 threads, 8 pieces a row)
#define MG_FB (MG_TN / 32)

__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ sel, int pairs, int experts, int* __restrict__ perm,
                                                        int* __restrict__ tile_e, int* __restrict__ tile_r0, int* __restrict__ tile_rows,
                                                        int max_tiles) {
  __shared__ int cnt[MOE_MAX_EXPERTS], off[MOE_MAX_EXPERTS], cur[MOE_MAX_EXPERTS];
  for (int e = threadIdx.x; e < experts; e += blockDim.x) cnt[e] = 0, cur[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) atomicAdd(&cnt[sel[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < experts; ++e) {
      off[e] = at;
      for (int r = 0; r < cnt[e] && tiles < max_tiles; r += MG_TM, ++tiles)
        tile_e[tiles] = e, tile_r0[tiles] = at + r, tile_rows[tiles] = min(MG_TM, cnt[e] - r);
      at += cnt[e];
    }
    for (; tiles < max_tiles; ++tiles) tile_e[tiles] = -1, tile_r0[tiles] = 0, tile_rows[tiles] = 0;
  }
  __syncthreads();
  // (which pair of an expert gets which of its places depends on timing; a pair's result does not depend on its place)
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = sel[p];
    perm[off[e] + atomicAdd(&cur[e], 1)] = p;
  }
}

template <bool DUAL>
__global__ __launch_bounds__(256) void moe_group_kernel(const bf16_t* __restrict__ A, int a_stride, const bf16_t* __restrict__ B0,
                                                        const bf16_t* __restrict__ B1, const int* __restrict__ perm,
                                                        const int* __restrict__ tile_e, const int* __restrict__ tile_r0,
                                                        const int* __restrict__ tile_rows, bf16_t* __restrict__ act_out, float* __restrict__ out,
                                                        const float* __restrict__ wt, int N, int K, int top, float limit, float alpha, float shift) {
  __shared__ __attribute__((aligned(16))) bf16_t As[MG_TM * MG_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[(DUAL ? 2 : 1) * MG_TN * MG_LD];
  const int tile = blockIdx.y, e = tile_e[tile];
  if (e < 0) return;
  const int r0 = tile_r0[tile], rows = tile_rows[tile], n0 = blockIdx.x * MG_TN;
  const int tid = threadIdx.x, lane = tid % NS_WAVE, wave = tid / NS_WAVE, r = lane % 16, g = lane / 16;
  const int wm = wave / 2, wn = wave % 2;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // the pieces (8 values along K) of each staged tile that this thread fetches: rows tid / 8 + 32 i, piece tid % 8
  const int kp = (tid % 8) * 8;
  const bf16_t* arow[MG_FA];
  const bf16_t* brow0[MG_FB];
  const bf16_t* brow1[MG_FB];
#pragma unroll
  for (int i = 0; i < MG_FA; ++i) {
    const int row = tid / 8 + 32 * i;
    const int slot = r0 + row;
    arow[i] = row < rows ? A + (size_t)(DUAL ? perm[slot] / top : slot) * a_stride : nullptr;
  }
#pragma unroll
  for (int i = 0; i < MG_FB; ++i) {
    const int col = n0 + tid / 8 + 32 * i;
    brow0[i] = col < N ? B0 + ((size_t)e * N + col) * K : nullptr;
    brow1[i] = (DUAL && col < N) ? B1 + ((size_t)e * N + col) * K : nullptr;
  }
  bf16x8 pa[MG_FA], pb0[MG_FB], pb1[MG_FB];
  auto fetch = [&](int k0) {
    const bool ok = k0 + kp < K;
#pragma unroll
    for (int i = 0; i < MG_FA; ++i) pa[i] = (ok && arow[i]) ? *reinterpret_cast<const bf16x8*>(arow[i] + k0 + kp) : zero;
#pragma unroll
    for (int i = 0; i < MG_FB; ++i) {
      pb0[i] = (ok && brow0[i]) ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(brow0[i] + k0 + kp)) : zero;
      if (DUAL) pb1[i] = (ok && brow1[i]) ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(brow1[i] + k0 + kp)) : zero;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < MG_FA; ++i) *reinterpret_cast<bf16x8*>(As + (tid / 8 + 32 * i) * MG_LD + kp) = pa[i];
#pragma unroll
    for (int i = 0; i < MG_FB; ++i) {
      const int at = (tid / 8 + 32 * i) * MG_LD + kp;
      *reinterpret_cast<bf16x8*>(Bs + at) = pb0[i];
      if (DUAL) *reinterpret_cast<bf16x8*>(Bs + MG_TN * MG_LD + at) = pb1[i];
    }
  };

  f32x4 acc0[MG_RI][MG_CJ], acc1[DUAL ? MG_RI : 1][DUAL ? MG_CJ : 1];
#pragma unroll
  for (int i = 0; i < MG_RI; ++i)
#pragma unroll
    for (int j = 0; j < MG_CJ; ++j) {
      acc0[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (DUAL) acc1[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

  const int a_at = (MG_TM / 2 * wm + r) * MG_LD + 8 * g, b_at = (MG_TN / 2 * wn + r) * MG_LD + 8 * g;
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += MG_KC) {
    stage();
    __syncthreads();
    if (k0 + MG_KC < K) fetch(k0 + MG_KC);
#pragma unroll
    for (int ks = 0; ks < MG_KC; ks += 32) {
      bf16x8 af[MG_RI], bf0[MG_CJ], bf1[MG_CJ];
#pragma unroll
      for (int i = 0; i < MG_RI; ++i) af[i] = *reinterpret_cast<const bf16x8*>(As + a_at + 16 * i * MG_LD + ks);
#pragma unroll
      for (int j = 0; j < MG_CJ; ++j) {
        bf0[j] = *reinterpret_cast<const bf16x8*>(Bs + b_at + 16 * j * MG_LD + ks);
        if (DUAL) bf1[j] = *reinterpret_cast<const bf16x8*>(Bs + MG_TN * MG_LD + b_at + 16 * j * MG_LD + ks);
      }
#pragma unroll
      for (int i = 0; i < MG_RI; ++i)
#pragma unroll
        for (int j = 0; j < MG_CJ; ++j) {
          acc0[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bf0[j], acc0[i][j], 0, 0, 0);
          if (DUAL) acc1[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bf1[j], acc1[i][j], 0, 0, 0);
        }
    }
    __syncthreads();
  }
  // element q of a lane's sums is row 4 g + q of the 16 x 16 block, column r
#pragma unroll
  for (int i = 0; i < MG_RI; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int row = MG_TM / 2 * wm + 16 * i + 4 * g + q;
      if (row >= rows) continue;
      const int slot = r0 + row;
      const int pair = DUAL ? 0 : perm[slot];
      const float share = DUAL ? 0.f : wt[pair];
#pragma unroll
      for (int j = 0; j < MG_CJ; ++j) {
        const int col = n0 + MG_TN / 2 * wn + 16 * j + r;
        if (col >= N) continue;
        if (DUAL)
          act_out[(size_t)slot * N + col] = from_f<bf16_t>(clipped_glu(round_to<bf16_t>(acc0[i][j][q]), round_to<bf16_t>(acc1[i][j][q]), limit, alpha, shift));
        else
          out[(size_t)pair * N + col] = share * acc0[i][j][q];
      }
    }
}

// tiles that any choice of experts can need
extern "C" int ns_moe_group_tiles(int pairs, int experts) { return (pairs + MG_TM - 1) / MG_TM + experts; }

// ``ints``: scratch of pairs + 3 * ns_moe_group_tiles(pairs, experts) 32-bit words; ``act``: bfloat16 [pairs][ff]
extern "C" int ns_moe_expert_groups(const void* h, int h_stride, const void* wg, const void* wu, const void* wd, const int* sel, const float* wt,
                                    int* ints, void* act, float* out, int n, int W, int ff, int top, int experts, float limit, float alpha, float shift,
                                    hipStream_t stream) {
  if (n <= 0 || W <= 0 || ff <= 0 || top <= 0 || experts <= 0 || experts > MOE_MAX_EXPERTS) return NS_ERR_BAD_ARG;
  if (W % 8 || ff % 8 || h_stride % 8 || (uintptr_t)h % 16 || (uintptr_t)wg % 16 || (uintptr_t)wu % 16 || (uintptr_t)wd % 16 || (uintptr_t)act % 16)
    return NS_ERR_UNSUPPORTED;
  const long long pairs = (long long)n * top;
  if (pairs > (1 << 24)) return NS_ERR_UNSUPPORTED;
  const int tiles = ns_moe_group_tiles((int)pairs, experts);
  int* perm = ints;
  int* tile_e = ints + pairs;
  int* tile_r0 = tile_e + tiles;
  int* tile_rows = tile_r0 + tiles;
  moe_sort_kernel<<<1, 1024, 0, stream>>>(sel, (int)pairs, experts, perm, tile_e, tile_r0, tile_rows, tiles);
  if (tiles > 65535) return NS_ERR_UNSUPPORTED;
  dim3 g1((ff + MG_TN - 1) / MG_TN, tiles), g2((W + MG_TN - 1) / MG_TN, tiles);
  moe_group_kernel<true><<<g1, 256, 0, stream>>>((const bf16_t*)h, h_stride, (const bf16_t*)wg, (const bf16_t*)wu, perm, tile_e, tile_r0, tile_rows,
                                                  (bf16_t*)act, nullptr, nullptr, ff, W, top, limit, alpha, shift);
  moe_group_kernel<false><<<g2, 256, 0, stream>>>((const bf16_t*)act, ff, (const bf16_t*)wd, nullptr, perm, tile_e, tile_r0, tile_rows, nullptr, out,
                                                   wt, W, ff, top, limit, alpha, shift);
  return ns_launch_status();
}

// out[t][f] = clipped_glu(gu[t][f], gu[t][ff + f]) for the result of a product with the stacked [gate; up] matrix
template <typename T>
__global__ void clipped_glu_kernel(T* __restrict__ out, const T* __restrict__ gu, int gu_stride, int ff, size_t count, float limit, float alpha, float shift) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / ff, f = i % ff;
    out[i] = from_f<T>(clipped_glu(to_f(gu[t * gu_stride + f]), to_f(gu[t * gu_stride + ff + f]), limit, alpha, shift));
  }
}

extern "C" int ns_clipped_glu(void* out, const void* gu, int gu_stride, int n, int ff, float limit, float alpha, float shift, int dtype, hipStream_t stream) {
  if (n <= 0 || ff <= 0) return NS_ERR_BAD_ARG;
  const size_t count = (size_t)n * ff;
  size_t blocks = (count + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  if (dtype == NS_DTYPE_F32)
    clipped_glu_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)gu, gu_stride, ff, count, limit, alpha, shift);
  else if (dtype == NS_DTYPE_BF16)
    clipped_glu_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, gu_stride, ff, count, limit, alpha, shift);
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
// row).  The two products are the framework's; between them: out[t][j] = gelu_tanh(g[t][j]) * table[ids[t]][j].
template <typename T>
__global__ void gelu_gather_mul_kernel(T* __restrict__ out, const T* __restrict__ g, int g_stride, const int* __restrict__ ids,
                                       const T* __restrict__ table, int dim, size_t count) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / dim, j = i % dim;
    const float z = to_f(g[t * g_stride + j]);
    const float gl = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    out[i] = from_f<T>(round_to<T>(gl) * to_f(table[(size_t)ids[t] * dim + j]));
  }
}

extern "C" int ns_gelu_gather_mul(void* out, const void* g, int g_stride, const int* ids, const void* table, int n, int dim, int dtype,
                                  hipStream_t stream) {
  if (n <= 0 || dim <= 0) return NS_ERR_BAD_ARG;
  const size_t count = (size_t)n * dim;
  size_t blocks = (count + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  if (dtype == NS_DTYPE_F32)
    gelu_gather_mul_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)g, g_stride, ids, (const float*)table, dim, count);
  else if (dtype == NS_DTYPE_BF16)
    gelu_gather_mul_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)g, g_stride, ids, (const bf16_t*)table, dim, count);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
