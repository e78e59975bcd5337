// Soft-max attention over the paged bfloat16 cache on the matrix cores for heads that the kernels of attn_mfma.hip do not
// take: keys of any size that is a multiple of 16 up to 1,024 channels (NS_HEAD_DIM), values of ANOTHER size, a multiple
// of 16 up to 512 (NS_VALUE_DIM), and a bias by distance with one slope per head.  Compiled for one (key size, value
// size, page size).  It serves attention through latents (one key/value head of latent + rotated channels whose values
// are the latent alone, read by every query head) and attention whose values are narrower than its keys.
//
// The arithmetic is that of attn_mfma.hip, kept transposed so that a column (a query token and head) is always lane % 16:
//   S^T[key][col] = K[key][:] . Q[col][:]     A = K rows straight from the page, B = Q^T held in registers
//   O^T[ch][col] += V^T[ch][key] . P^T[key][col]   A = V^T as the pages hold it ([channel][token])
// One wave owns 16 columns: hp consecutive heads of a group times 16 / hp consecutive tokens; a tile of the batch's tile
// list is qt such sets of tokens, each a wave's.  Keys are walked in blocks of 32.  With heads this wide a block's keys
// and values do not fit the registers beside the sums, so they stream through them in pieces, each used as it arrives.
// With splits > 1 the keys of a tile are cut into ranges, each a wave's, joined by attn_wide_reduce_kernel.
//
// Query at position p sees keys max(0, p - window + 1) .. p.  slope_exp > 0: head h of H loses
// 2^(-slope_exp (h + 1) / H) * (p - key) from its score.  Scores, soft-max and sums are 32-bit.
#include "common.h"

#if !defined(NS_HEAD_DIM) || !defined(NS_VALUE_DIM) || !defined(NS_PAGE_SIZE)
#error "compile with -DNS_HEAD_DIM=<multiple of 16> -DNS_VALUE_DIM=<multiple of 16> -DNS_PAGE_SIZE=<power of two from 4>"
#endif
constexpr int HD = NS_HEAD_DIM;
constexpr int VD = NS_VALUE_DIM;
constexpr int PS = NS_PAGE_SIZE;
static_assert(PS >= 4 && (PS & (PS - 1)) == 0, "page size must be a power of two from 4");
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 1024, "key size must be a multiple of 16 up to 1024");
static_assert(VD % 16 == 0 && VD >= 16 && VD <= 512, "value size must be a multiple of 16 up to 512");
constexpr int DT = VD / 16;                   // 16-channel tiles of the output
constexpr bool WIDE = HD % 32 == 0;           // q.k with the k=32 instruction, else with k=16
constexpr int NQ = WIDE ? HD / 32 : HD / 16;  // q.k instructions per 16-key tile
constexpr int TILE_INTS = 8;
constexpr int VPIECE = DT < 16 ? DT : 16;       // channel tiles of the values that are asked for together

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

struct WideParams {
  bf16_t* out;       // [tokens, heads, VD]
  float* part_o;     // [n_tiles * (qt * 16 / hp) * heads, splits, VD]   (splits > 1)
  float* part_ml;    // [n_tiles * (qt * 16 / hp) * heads, splits, 2]
  const bf16_t* q;   // row t at q + t * q_stride, head h at + h * HD
  const bf16_t* k_cache;  // [page][kv head][token][HD]
  const bf16_t* v_cache;  // [page][kv head][VD][token]
  const int* tiles;  // [n_tiles][TILE_INTS]: request, first token of the tile, row of the request's first token, tokens, keys
  const int* block_table;
  int q_stride, table_stride, n_tiles, heads, kv_heads, hp, splits, window, qt;
  float scale_log2;  // softmax scale * log2(e)
  float slope_exp;   // see above; 0: none
  float inv_scale;   // 1 / softmax scale: the slope in the units of the unscaled scores
  const float* sink_logits;  // null, or [heads]: the soft-max's denominator holds one more term exp(sink_logits[head]), not scaled
};

__device__ __forceinline__ int wmax_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ int wmin_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
  return v;
}

// SHARE: the four waves of a workgroup are four heads of one key/value head over the same tokens and the same range of
// keys (the host asks for it only with hp = 1 and a group that is a multiple of four, and pages of 8 tokens or more), so
// each block of 32 keys is fetched once per workgroup, a quarter by each wave, and read from LDS by all four; the next
// block's pieces are on their way in registers while this one is used.  Without it every wave fetches its own.
constexpr int KROW = HD + 8;          // elements of a key's row in LDS (16 bytes of padding)
constexpr int VROW = 32 + 8;          // elements of a channel's row in LDS
constexpr int KPIECES = 32 * (HD / 8);  // 16-byte pieces of a block's keys
constexpr int VPIECES = VD * 4;         // ... and of its values (a channel's 32 keys are four pieces)
constexpr int KPT = (KPIECES + 255) / 256, VPT = (VPIECES + 255) / 256;  // pieces a thread fetches

template <bool SHARE>
__global__ __launch_bounds__(256) void attn_wide_kernel(WideParams a) {
  __shared__ __align__(16) bf16_t lk[SHARE ? 32 * KROW : 8];
  __shared__ __align__(16) bf16_t lv[SHARE ? VD * VROW : 8];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  const int G = a.heads / a.kv_heads;
  const int hblks = (G + a.hp - 1) / a.hp;
  const int ny = a.kv_heads * hblks;
  const long item = (long)blockIdx.x * 4 + wave;
  if (item >= (long)a.n_tiles * a.qt * a.splits * ny) return;
  const int y = (int)(item % ny);
  long rest = item / ny;
  const int split = (int)(rest % a.splits);
  rest /= a.splits;
  const int u = (int)(rest % a.qt);
  const int tile = a.n_tiles - 1 - (int)(rest / a.qt);  // the last tiles see the most keys, so they start first
  const int kvh = y / hblks, hblk = y % hblks;
  const int4 info = *reinterpret_cast<const int4*>(a.tiles + (size_t)tile * TILE_INTS);
  const int b = info.x, t0 = info.y, q0 = info.z, n = info.w;
  const int kv_len = a.tiles[(size_t)tile * TILE_INTS + 4];
  const int* table = a.block_table + (size_t)b * a.table_stride;
  constexpr int psh = __builtin_ctz(PS), pmask = PS - 1;

  const int tt = u * (16 / a.hp) + c / a.hp;  // this lane's column: token of the tile ...
  const int ti = t0 + tt;
  const int hin = hblk * a.hp + c % a.hp;     // ... and head of the group
  const int head = kvh * G + (hin < G ? hin : 0);
  const bool col_ok = ti < n && hin < G;
  const int pos = col_ok ? kv_len - n + ti : -1;
  const int lo = (col_ok && a.window > 0) ? max(0, pos - a.window + 1) : 0;
  const int whi = wmax_i(pos) + 1;                                    // keys [wlo, whi) are seen by some column
  const int wlo = wmin_i(col_ok ? lo : 0x7fffffff);
  const int full_hi = wmin_i(col_ok ? pos : 0x7fffffff);              // keys <= full_hi are seen by every column ...
  const int full_lo = wmax_i(lo);                                     // ... if they are >= full_lo
  const float slope = a.slope_exp > 0.f ? exp2f(-a.slope_exp * (float)(head + 1) / (float)a.heads) * a.inv_scale : 0.f;

  int kb0 = whi > 0 ? wlo / 32 : 0, kb1 = whi > 0 ? (whi + 31) / 32 : 0;
  if (a.splits > 1) {
    const int per = (kb1 - kb0 + a.splits - 1) / a.splits;
    kb0 = kb0 + split * per;
    kb1 = min(kb1, kb0 + per);
  }
  kb0 = __builtin_amdgcn_readfirstlane(kb0);
  kb1 = __builtin_amdgcn_readfirstlane(kb1);

  // Q^T fragments of this lane's column
  bf16x8 qw[WIDE ? NQ : 1];
  s16x4 qn[WIDE ? 1 : NQ];
  {
    const bf16_t* qrow = a.q + (size_t)(q0 + (col_ok ? ti : 0)) * a.q_stride + (size_t)head * HD;
    if (WIDE) {
#pragma unroll
      for (int i = 0; i < NQ; ++i) {
        qw[i] = *reinterpret_cast<const bf16x8*>(qrow + i * 32 + g * 8);
        if (!col_ok) qw[i] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    } else {
#pragma unroll
      for (int i = 0; i < NQ; ++i) {
        qn[i] = *reinterpret_cast<const s16x4*>(qrow + i * 16 + g * 4);
        if (!col_ok) qn[i] = s16x4{0, 0, 0, 0};
      }
    }
  }

  f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;
  const int qlo = wlo & ~3, qhi = (whi - 1) & ~3;  // first and last 4-key group that holds a seen key
  const size_t k_page = ((size_t)a.kv_heads * HD) << psh, v_page = ((size_t)a.kv_heads * VD) << psh;  // elements of a page
  const bf16_t* kbase = a.k_cache + (((size_t)kvh * HD) << psh) + (WIDE ? g * 8 : g * 4);
  const bf16_t* vbase = a.v_cache + (((size_t)kvh * VD + c) << psh);
  constexpr size_t v_step = (size_t)16 * PS;  // elements between channel tiles of a V page

  // the pages of a block's keys (as the K loads and as the V loads walk them), looked up one block ahead
  int pk[2], pv[2], kk[2], kv2[2];
  auto lookup = [&](int kb) {
    const int key_base = kb * 32;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      kk[t] = min(max(key_base + t * 16 + c, wlo), whi - 1);  // (a key outside [wlo, whi) is masked anyway)
      pk[t] = table[kk[t] >> psh];
      // slot 8 g + j of the second product holds key key_base + 4 g + j for j < 4 and key_base + 16 + 4 g + (j - 4) for j >= 4
      kv2[t] = min(max(key_base + t * 16 + g * 4, qlo), qhi);
      pv[t] = table[kv2[t] >> psh];
    }
  };
  if (!SHARE && kb0 < kb1) lookup(kb0);

  // SHARE: the pieces of a block that this thread fetches for the workgroup, held in registers until the block before is
  // done with.  A key outside the pages that hold [wlo, whi) is read from the nearest such page instead: it is masked anyway.
  bf16x8 rk[KPT], rv[VPT];
  constexpr int NP = PS >= 32 ? 1 : 32 / PS;  // pages that a block of 32 keys touches
  auto fetch = [&](int kb) {
    const int key_base = kb * 32, plo = wlo >> psh, phi = (whi - 1) >> psh;
    int pg[NP];
#pragma unroll
    for (int j = 0; j < NP; ++j) pg[j] = table[min(max((key_base >> psh) + j, plo), phi)];
    auto page_at = [&](int j) {
      int page = pg[0];
#pragma unroll
      for (int jj = 1; jj < NP; ++jj)
        if (j == jj) page = pg[jj];
      return page;
    };
#pragma unroll
    for (int r = 0; r < KPT; ++r) {
      const int p = threadIdx.x + r * 256;
      if (p < KPIECES) {
        const int row = p / (HD / 8), col = p % (HD / 8);
        const int page = page_at(PS >= 32 ? 0 : row >> psh), tok = (key_base + row) & pmask;
        rk[r] = *reinterpret_cast<const bf16x8*>(a.k_cache + (size_t)page * k_page + (((size_t)kvh * HD) << psh) + (size_t)tok * HD + col * 8);
      }
    }
#pragma unroll
    for (int r = 0; r < VPT; ++r) {
      const int p = threadIdx.x + r * 256;
      if (p < VPIECES) {
        const int ch = p >> 2, key0 = (p & 3) * 8;
        const int page = page_at(PS >= 32 ? 0 : key0 >> psh), tok = (key_base + key0) & pmask;
        rv[r] = *reinterpret_cast<const bf16x8*>(a.v_cache + (size_t)page * v_page + (((size_t)kvh * VD + ch) << psh) + tok);
      }
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int r = 0; r < KPT; ++r) {
      const int p = threadIdx.x + r * 256;
      if (p < KPIECES) *reinterpret_cast<bf16x8*>(&lk[(p / (HD / 8)) * KROW + (p % (HD / 8)) * 8]) = rk[r];
    }
#pragma unroll
    for (int r = 0; r < VPT; ++r) {
      const int p = threadIdx.x + r * 256;
      if (p < VPIECES) *reinterpret_cast<bf16x8*>(&lv[(p >> 2) * VROW + (p & 3) * 8]) = rv[r];
    }
  };
  if constexpr (SHARE) {
    if (kb0 < kb1) fetch(kb0);
  }

  for (int kb = kb0; kb < kb1; ++kb) {
    const int key_base = kb * 32;
    const bf16_t* krow[2];
    const bf16_t* vrow[2];
    if constexpr (SHARE) {
      __syncthreads();  // every wave is done with the block before
      stash();
      __syncthreads();
      if (kb + 1 < kb1) fetch(kb + 1);
    } else {
      krow[0] = kbase + (size_t)pk[0] * k_page + (size_t)(kk[0] & pmask) * HD;
      krow[1] = kbase + (size_t)pk[1] * k_page + (size_t)(kk[1] & pmask) * HD;
      vrow[0] = vbase + (size_t)pv[0] * v_page + (kv2[0] & pmask);
      vrow[1] = vbase + (size_t)pv[1] * v_page + (kv2[1] & pmask);
      if (kb + 1 < kb1) lookup(kb + 1);
    }
    // a block's operands, from LDS or straight from the pages
    auto k_wide = [&](int t, int i) {
      if constexpr (SHARE) return *reinterpret_cast<const bf16x8*>(&lk[(t * 16 + c) * KROW + i * 32 + g * 8]);
      else return *reinterpret_cast<const bf16x8*>(krow[t] + i * 32);
    };
    auto k_narrow = [&](int t, int i) {
      if constexpr (SHARE) return *reinterpret_cast<const s16x4*>(&lk[(t * 16 + c) * KROW + i * 16 + g * 4]);
      else return *reinterpret_cast<const s16x4*>(krow[t] + i * 16);
    };
    auto v_at = [&](int t, int dt) {
      if constexpr (SHARE) return *reinterpret_cast<const bf16x4*>(&lv[(dt * 16 + c) * VROW + t * 16 + g * 4]);
      else return *reinterpret_cast<const bf16x4*>(vrow[t] + dt * v_step);
    };

    // scores: s[t][j] is key key_base + 16 t + 4 g + j of column c; both 16-key tiles' rows are asked for before the first
    // product, so that a block costs one trip to memory for its keys
    f32x4 s[2];
    if (WIDE) {
      bf16x8 kf[2][NQ];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < NQ; ++i) kf[t][i] = k_wide(t, i);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NQ; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][i], qw[i], acc, 0, 0, 0);
        s[t] = acc;
      }
    } else {
      s16x4 kf[2][NQ];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < NQ; ++i) kf[t][i] = k_narrow(t, i);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NQ; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf[t][i], qn[i], acc, 0, 0, 0);
        s[t] = acc;
      }
    }
    // the first piece of the values is on its way while the soft-max runs
    bf16x4 vf[VPIECE][2];
#pragma unroll
    for (int d = 0; d < VPIECE; ++d) {
      vf[d][0] = v_at(0, d);
      vf[d][1] = v_at(1, d);
    }

    // soft-max weights of the block, and the rescaling of what has been summed so far
    if (slope > 0.f) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) s[t][j] -= slope * (float)(pos - (key_base + t * 16 + g * 4 + j));
    }
    const bool full = key_base + 31 <= full_hi && key_base >= full_lo;  // no masks needed (uniform over the wave)
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = key_base + t * 16 + g * 4 + j;
        if (!full && !(key >= lo && key <= pos)) s[t][j] = -INFINITY;
        mx = fmaxf(mx, s[t][j]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const bool moved = m_new != m;
    const float alpha = __builtin_amdgcn_exp2f((m - m_safe) * a.scale_log2);
    const float shift = -m_safe * a.scale_log2;
    m = m_new;
    float psum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[t][j], a.scale_log2, shift));
        psum += p;
        pf[t * 4 + j] = (bf16_t)p;
      }
    if (__any(moved)) {
      lsum *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j) o[dt][j] *= alpha;
    }
    lsum += psum;

    // O^T += V^T P^T, the values in pieces of VPIECE channel tiles
#pragma unroll
    for (int d0 = 0; d0 < DT; d0 += VPIECE) {
      bf16x4 nx[VPIECE][2];
      if (d0 + VPIECE < DT) {
#pragma unroll
        for (int d = 0; d < VPIECE; ++d)
          if (d0 + VPIECE + d < DT) {
            nx[d][0] = v_at(0, d0 + VPIECE + d);
            nx[d][1] = v_at(1, d0 + VPIECE + d);
          }
      }
#pragma unroll
      for (int d = 0; d < VPIECE; ++d)
        if (d0 + d < DT) {
          const bf16x4 l4 = vf[d][0], h4 = vf[d][1];
          const bf16x8 v8 = {l4[0], l4[1], l4[2], l4[3], h4[0], h4[1], h4[2], h4[3]};
          o[d0 + d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v8, pf, o[d0 + d], 0, 0, 0);
        }
      if (d0 + VPIECE < DT) {
#pragma unroll
        for (int d = 0; d < VPIECE; ++d) {
          vf[d][0] = nx[d][0];
          vf[d][1] = nx[d][1];
        }
      }
    }
  }

  lsum += __shfl_xor(lsum, 16, 64);
  lsum += __shfl_xor(lsum, 32, 64);
  if (!col_ok) return;
  // o[dt][j] is channel 16 dt + 4 g + j of column c
  if (a.splits == 1) {
    const size_t col = (size_t)(q0 + ti) * a.heads + head;
    if (a.sink_logits) lsum += exp2f(a.sink_logits[head] * 1.4426950408889634f - m * a.scale_log2);  // the sink's term, in the units of the column's maximum
    const float inv = 1.f / lsum;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      bf16x4 r = {(bf16_t)(o[dt][0] * inv), (bf16_t)(o[dt][1] * inv), (bf16_t)(o[dt][2] * inv), (bf16_t)(o[dt][3] * inv)};
      *reinterpret_cast<bf16x4*>(a.out + col * VD + dt * 16 + g * 4) = r;
    }
  } else {
    const size_t pcol = ((size_t)tile * (a.qt * 16 / a.hp) + tt) * a.heads + head;
    float* po = a.part_o + (pcol * a.splits + split) * VD;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4*>(po + dt * 16 + g * 4) = o[dt];
    if (g == 0) {
      a.part_ml[(pcol * a.splits + split) * 2] = m * a.scale_log2;  // in the exponent's units
      a.part_ml[(pcol * a.splits + split) * 2 + 1] = lsum;
    }
  }
}

// Joining the key ranges: out[col] = sum_s o_s 2^(m_s - m*) / sum_s l_s 2^(m_s - m*), m* = max_s m_s.  One wave per
// (tile, token of the tile, head); lane s first holds range s (at most 64 ranges), then the lanes split the channels and
// add the ranges in order.
__global__ __launch_bounds__(64) void attn_wide_reduce_kernel(bf16_t* __restrict__ out, const float* __restrict__ part_o,
                                                              const float* __restrict__ part_ml, const int* __restrict__ tiles,
                                                              int heads, int tile_tokens, int splits, const float* __restrict__ sink_logits) {
  const int tile = blockIdx.x, head = blockIdx.y, tt = blockIdx.z;
  const int lane = threadIdx.x;
  const size_t pcol = ((size_t)tile * tile_tokens + tt) * heads + head;
  const float* ml = part_ml + pcol * splits * 2;
  const int4 info = *reinterpret_cast<const int4*>(tiles + (size_t)tile * TILE_INTS);
  const int ti = info.y + tt;
  if (ti >= info.w) return;  // the tile holds fewer tokens
  float ms = -INFINITY, ls = 0.f;
  if (lane < splits) {
    ms = ml[lane * 2];
    ls = ml[lane * 2 + 1];
  }
  float mstar = ms;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mstar = fmaxf(mstar, __shfl_xor(mstar, o, 64));
  const float wgt = ms == -INFINITY ? 0.f : exp2f(ms - mstar);
  float l = ls * wgt;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o, 64);
  if (sink_logits) l += exp2f(sink_logits[head] * 1.4426950408889634f - mstar);  // the sink's term (the ranges' maxima are in the exponent's units)
  const float inv = 1.f / l;
  constexpr int PER = (VD + 63) / 64;
  const float* po = part_o + pcol * splits * VD;
  float acc[PER];
#pragma unroll
  for (int p = 0; p < PER; ++p) acc[p] = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 4) {  // four ranges' loads in flight at a time
    float v[4][PER];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int p = 0; p < PER; ++p) {
        const int d = lane + p * 64;
        v[i][p] = (s0 + i < splits && d < VD) ? po[(size_t)(s0 + i) * VD + d] : 0.f;
      }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float ws = __shfl(wgt, (s0 + i) & 63, 64);
#pragma unroll
      for (int p = 0; p < PER; ++p) acc[p] += v[i][p] * ws;
    }
  }
  const size_t col = (size_t)(info.z + ti) * heads + head;
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int d = lane + p * 64;
    if (d < VD) out[col * VD + d] = (bf16_t)(acc[p] * inv);
  }
}

extern "C" int ns_attn_wide_head_dim() { return HD; }
extern "C" int ns_attn_wide_value_dim() { return VD; }
extern "C" int ns_attn_wide_page_size() { return PS; }

// Workspace, when splits > 1: with T = qt * 16 / hp tokens in a tile, part_o holds n_tiles * T * heads * splits * VD floats
// and part_ml n_tiles * T * heads * splits * 2.
extern "C" int ns_attn_wide(void* out, void* part_o, void* part_ml, const void* q, int q_stride, const void* k_cache, const void* v_cache,
                            const int* tiles, const int* block_table, int table_stride, int n_tiles, int heads, int kv_heads, int page_size,
                            int hp, int splits, int window, float scale, int qt, float slope_exp, const float* sink_logits, hipStream_t stream) {
  if (n_tiles <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || page_size != PS || window < 0 || splits < 1 || splits > 64 ||
      (q_stride & 7) || ((uintptr_t)tiles & 15) || slope_exp < 0.f)
    return NS_ERR_BAD_ARG;
  if (hp != 1 && hp != 2 && hp != 4 && hp != 8 && hp != 16) return NS_ERR_BAD_ARG;
  if (qt < 1 || qt > 4 || !(scale > 0.f)) return NS_ERR_BAD_ARG;
  if (splits > 1 && (!part_o || !part_ml)) return NS_ERR_BAD_ARG;
  WideParams a;
  a.out = (bf16_t*)out; a.part_o = (float*)part_o; a.part_ml = (float*)part_ml;
  a.q = (const bf16_t*)q; a.k_cache = (const bf16_t*)k_cache; a.v_cache = (const bf16_t*)v_cache;
  a.tiles = tiles; a.block_table = block_table;
  a.q_stride = q_stride; a.table_stride = table_stride; a.n_tiles = n_tiles; a.heads = heads; a.kv_heads = kv_heads;
  a.hp = hp; a.splits = splits; a.window = window; a.qt = qt;
  a.scale_log2 = scale * 1.4426950408889634f;
  a.slope_exp = slope_exp; a.inv_scale = 1.f / scale; a.sink_logits = sink_logits;
  const int G = heads / kv_heads;
  const long items = (long)n_tiles * qt * splits * kv_heads * ((G + hp - 1) / hp);
  const long blocks = (items + 3) / 4;
  if (blocks > 0x7fffffffL || heads > 65535) return NS_ERR_BAD_ARG;
  // prompt portions of a group of a multiple of four heads: the four waves of a workgroup share each block of keys.
  // (Measured with 32 heads over one key/value head, 2,048 tokens, windows of 1,024: keys of 64 and values of 64 channels
  // 60 against 85 us; keys of 544 and values of 512 channels 780 against 460 us: with heads that wide a wave's sums,
  // its queries and the pieces in flight leave no room, and one workgroup a compute unit waits at every barrier.)
  constexpr bool SHARE_PAYS = HD + VD <= 512;
  if (SHARE_PAYS && hp == 1 && G % 4 == 0 && PS >= 8 && qt > 1)
    attn_wide_kernel<true><<<(unsigned)blocks, 256, 0, stream>>>(a);
  else
    attn_wide_kernel<false><<<(unsigned)blocks, 256, 0, stream>>>(a);
  const int st = ns_launch_status();
  if (st != NS_OK || splits == 1) return st;
  const int tile_tokens = qt * 16 / hp;
  attn_wide_reduce_kernel<<<dim3(n_tiles, heads, tile_tokens), 64, 0, stream>>>((bf16_t*)out, (const float*)part_o, (const float*)part_ml,
                                                                                tiles, heads, tile_tokens, splits, sink_logits);
  return ns_launch_status();
}
