// Mixture of experts: routing, grouping of (token, choice) pairs by expert, and the experts' products.
//
// A step's T tokens each choose `top` of E experts: P = T * top pairs, pair p = t * top + j.  The pairs are
// grouped by expert (`order[i]` is the pair at sorted place i, `offsets[e]` the first place of expert e) and cut
// into tiles of 64 places that never span two experts; a product's workgroup owns one tile and 64 output
// columns.  The grid is sized for the most tiles there can be, and workgroups past `num_tiles` (which only the
// device knows) leave at once.  Which place a pair gets depends on the order in which the counters were bumped,
// but no value does: a pair's row is computed alone, an FMA chain in k order per output element, and the
// weighted sum over a token's choices runs in the order of the choices.
#include "common.h"
#include "group_tile.h"

constexpr int MOE_TILE = 64;      // places per tile of the 32-bit products; the matrix-core products take 128

// ---------------------------------------------------------------------------------------------
// One wave per token: the `top` largest of E logits (the lowest id wins a tie), and the softmax over those.
// Lane l looks after experts l, l + 64, ...; a bit per expert of its own says which are taken (E <= 4096).
//
// `groups` > 1: the experts form that many equal groups of neighbours, a group's score is its largest logit, and
// only experts of the `keep` best groups (the lowest group among equals) can be chosen.  `all_scores` 1: the weights are
// the chosen experts' shares of the softmax over all E logits, which do not add up to one; 2: the sigmoid of each chosen
// expert's own logit, not renormalized; 3: the experts are chosen by sigmoid(logit) + correction[e] (a learned number per
// expert that steers the choice only) and a chosen expert's weight is weight_scale * sigmoid(logit), not renormalized.
struct Routing {
  int groups, keep, all_scores;
  const float* correction = nullptr;
  float weight_scale = 1.f;
  long long ld = 0;     // floats between two tokens' logits; 0: the number of experts (rows one behind the other)
};

__device__ __forceinline__ float choice_score(const Routing& how, const float* z, int e) {
  return how.all_scores == 3 ? 1.0f / (1.0f + expf(-z[e])) + (how.correction ? how.correction[e] : 0.f) : z[e];
}

__device__ __forceinline__ void route_token(const float* __restrict__ logits, int experts, int top, int t, int lane,
                                            int* __restrict__ ids, float* __restrict__ weights,
                                            Routing how = Routing{1, 1, 0}) {
  constexpr int NONE = 0x7fffffff;
  const float* z = logits + (long long)t * (how.ld ? how.ld : experts);
  unsigned long long taken = 0;
  if (how.groups > 1 && how.keep < how.groups) {
    // lane g keeps group g's score (at most 64 groups); the experts of the groups that lose count as taken
    const int size = experts / how.groups;
    float score = -INFINITY;
    if (lane < how.groups)
      for (int e = lane * size; e < (lane + 1) * size; ++e) score = fmaxf(score, choice_score(how, z, e));
    unsigned long long kept = 0;
    for (int j = 0; j < how.keep; ++j) {
      float best = (lane < how.groups && !((kept >> lane) & 1ull)) ? score : -INFINITY;
      int arg = (lane < how.groups && !((kept >> lane) & 1ull)) ? lane : NONE;
      for (int off = WAVE / 2; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off, WAVE);
        const int oa = __shfl_xor(arg, off, WAVE);
        if (oa != NONE && (arg == NONE || ob > best || (ob == best && oa < arg))) {
          best = ob;
          arg = oa;
        }
      }
      if (arg != NONE) kept |= 1ull << arg;
    }
    for (int e = lane, i = 0; e < experts; e += WAVE, ++i)
      if (!((kept >> (e / size)) & 1ull)) taken |= 1ull << i;
  }
  float whole_max = -INFINITY, whole_sum = 1.f;
  if (how.all_scores == 1) {
    for (int e = lane; e < experts; e += WAVE) whole_max = fmaxf(whole_max, z[e]);
    whole_max = wave_max(whole_max);
    float part = 0.f;
    for (int e = lane; e < experts; e += WAVE) part += expf(z[e] - whole_max);
    whole_sum = wave_sum(part);
  }
  float first = 0.f, sum = 0.f, mine = 0.f;      // lane j keeps the weight of choice j
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int arg = NONE;
    for (int e = lane, i = 0; e < experts; e += WAVE, ++i) {
      if ((taken >> i) & 1ull) continue;
      const float v = choice_score(how, z, e);
      if (arg == NONE || v > best) {   // ascending e: an equal later one does not replace
        best = v;
        arg = e;
      }
    }
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, WAVE);
      const int oa = __shfl_xor(arg, off, WAVE);
      if (oa != NONE && (arg == NONE || ob > best || (ob == best && oa < arg))) {
        best = ob;
        arg = oa;
      }
    }
    if ((arg & (WAVE - 1)) == lane) taken |= 1ull << (arg / WAVE);
    if (j == 0) first = best;
    const float p = how.all_scores == 3 ? how.weight_scale / (1.0f + expf(-z[arg]))
                    : how.all_scores == 2 ? 1.0f / (1.0f + expf(-best)) : how.all_scores ? expf(best - whole_max) : expf(best - first);
    sum += p;
    if (lane == j) mine = p;
    if (lane == 0) ids[(long long)t * top + j] = arg;
  }
  if (lane < top) weights[(long long)t * top + lane] = how.all_scores >= 2 ? mine : mine / (how.all_scores ? whole_sum : sum);
}

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int experts, int top,
                                                        int num_tokens, int* __restrict__ ids,
                                                        float* __restrict__ weights, Routing how) {
  const int t = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (t < num_tokens) route_token(logits, experts, top, t, threadIdx.x & (WAVE - 1), ids, weights, how);
}

// One workgroup: counts per expert, offsets, the pairs' places, and the list of tiles.
//   offsets [E + 1], order [P], tiles [max_tiles][2] = (expert, first place), num_tiles [1]
// With `logits`: the same workgroup routes the step's tokens first, a wave per token in turn (a step of few tokens:
// one launch instead of two).
__global__ __launch_bounds__(1024) void moe_group_kernel(const float* __restrict__ logits, int top, int num_tokens,
                                                         float* __restrict__ weights, int* __restrict__ ids, int pairs,
                                                         int experts, int tile_rows, int* __restrict__ offsets,
                                                         int* __restrict__ order, int* __restrict__ tiles,
                                                         int* __restrict__ num_tiles, Routing how) {
  extern __shared__ int shared[];      // counts [E], cursor [E]
  int* counts = shared;
  int* cursor = shared + experts;
  if (logits) {
    for (int t = threadIdx.x / WAVE; t < num_tokens; t += blockDim.x / WAVE)
      route_token(logits, experts, top, t, threadIdx.x & (WAVE - 1), ids, weights, how);
    __threadfence_block();
    __syncthreads();
  }
  for (int e = threadIdx.x; e < experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) atomicAdd(&counts[ids[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tile = 0;
    for (int e = 0; e < experts; ++e) {
      offsets[e] = at;
      cursor[e] = at;
      for (int first = 0; first < counts[e]; first += tile_rows) {
        tiles[2 * tile] = e;
        tiles[2 * tile + 1] = at + first;
        ++tile;
      }
      at += counts[e];
    }
    offsets[experts] = at;
    num_tiles[0] = tile;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) order[atomicAdd(&cursor[ids[p]], 1)] = p;
}

// ---------------------------------------------------------------------------------------------
// The experts' activation of a gate sum g and an up sum u.  A finite `limit`: g = min(g, limit),
// u = clamp(u, -limit, limit), y = g * sigmoid(alpha * g) * (u + 1).  An infinite one: y = g * sigmoid(alpha * g) * u,
// which with alpha 1 is silu(g) * u.
__device__ __forceinline__ float expert_act(float g, float u, float limit, float alpha) {
  if (limit < INFINITY) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit) + 1.0f;
  }
  return g * (1.0f / (1.0f + expf(-alpha * g))) * u;
}

// Gate and up products of a tile with the experts' activation (expert_act above).
// h: [T, width] (row of pair p is p / top); wg, wu: [E, ff, width]; act: [P places, ff].
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const T* __restrict__ h, long long ldh,
                                                          const T* __restrict__ wg, const T* __restrict__ wu,
                                                          const int* __restrict__ offsets,
                                                          const int* __restrict__ order, const int* __restrict__ tiles,
                                                          const int* __restrict__ num_tiles, int top, int width, int ff,
                                                          float limit, float alpha, const float* __restrict__ in_weights,
                                                          T* __restrict__ act) {
  if ((int)blockIdx.x >= num_tiles[0]) return;
  __shared__ float As[16][MOE_TILE + 4];
  __shared__ float Gs[16][MOE_TILE + 4];
  __shared__ float Us[16][MOE_TILE + 4];
  __shared__ int rows[MOE_TILE];
  const int e = tiles[2 * blockIdx.x], first = tiles[2 * blockIdx.x + 1];
  const int count = min(MOE_TILE, offsets[e + 1] - first);
  const int n0 = blockIdx.y * MOE_TILE;
  for (int i = threadIdx.x; i < MOE_TILE; i += 256) rows[i] = i < count ? order[first + i] / top : -1;
  __syncthreads();
  const T* g_w = wg + (long long)e * ff * width;
  const T* u_w = wu + (long long)e * ff * width;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float ga[4][4] = {}, ua[4][4] = {};
  for (int k0 = 0; k0 < width; k0 += 16) {
    for (int i = threadIdx.x; i < MOE_TILE * 16; i += 256) {
      const int r = i >> 4, kk = i & 15, k = k0 + kk, n = n0 + r;
      As[kk][r] = (rows[r] >= 0 && k < width) ? to_float<T>(h[(long long)rows[r] * ldh + k]) : 0.f;
      const bool in = n < ff && k < width;
      Gs[kk][r] = in ? to_float<T>(g_w[(long long)n * width + k]) : 0.f;
      Us[kk][r] = in ? to_float<T>(u_w[(long long)n * width + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], gv[4], uv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        gv[j] = Gs[kk][tx * 4 + j];
        uv[j] = Us[kk][tx * 4 + j];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          ga[i][j] = fmaf(av[i], gv[j], ga[i][j]);
          ua[i][j] = fmaf(av[i], uv[j], ua[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= count) continue;
    const float w = in_weights ? in_weights[order[first + r]] : 1.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= ff) continue;
      act[(long long)(first + r) * ff + n] = from_float<T>(expert_act(w * ga[i][j], w * ua[i][j], limit, alpha));
    }
  }
}

// Down product of a tile: pair_out[pair, :] = Wd_e act[place, :]  (32-bit out, one row per pair).
template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ act, const T* __restrict__ wd,
                                                       const int* __restrict__ offsets, const int* __restrict__ order,
                                                       const int* __restrict__ tiles, const int* __restrict__ num_tiles,
                                                       int width, int ff, float* __restrict__ pair_out) {
  if ((int)blockIdx.x >= num_tiles[0]) return;
  __shared__ float As[16][MOE_TILE + 4];
  __shared__ float Ws[16][MOE_TILE + 4];
  const int e = tiles[2 * blockIdx.x], first = tiles[2 * blockIdx.x + 1];
  const int count = min(MOE_TILE, offsets[e + 1] - first);
  const int n0 = blockIdx.y * MOE_TILE;
  const T* w = wd + (long long)e * width * ff;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < ff; k0 += 16) {
    for (int i = threadIdx.x; i < MOE_TILE * 16; i += 256) {
      const int r = i >> 4, kk = i & 15, k = k0 + kk, n = n0 + r;
      As[kk][r] = (r < count && k < ff) ? to_float<T>(act[(long long)(first + r) * ff + k]) : 0.f;
      Ws[kk][r] = (n < width && k < ff) ? to_float<T>(w[(long long)n * ff + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= count) continue;
    const long long pair = order[first + r];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < width) pair_out[pair * width + n] = acc[i][j];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The same two products on the matrix cores (bfloat16): tiles of 128 places, see group_tile.h.  A workgroup of the
// gate/up product owns 64 columns of an expert's width: each wave holds gate and up of the same 32 columns.
__global__ __launch_bounds__(256) void moe_gate_up_mma_kernel(const __bf16* __restrict__ h, long long ldh,
                                                              const __bf16* __restrict__ wg,
                                                              const __bf16* __restrict__ wu,
                                                              const int* __restrict__ offsets,
                                                              const int* __restrict__ order,
                                                              const int* __restrict__ tiles,
                                                              const int* __restrict__ num_tiles, int top, int width,
                                                              int ff, float limit, float alpha,
                                                              const float* __restrict__ in_weights,
                                                              __bf16* __restrict__ act) {
  if ((int)blockIdx.x >= num_tiles[0]) return;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  __shared__ int rows[GT_TILE];
  const int e = tiles[2 * blockIdx.x], first = tiles[2 * blockIdx.x + 1];
  const int count = min(GT_TILE, offsets[e + 1] - first);
  const int n0 = blockIdx.y * 64;
  for (int i = threadIdx.x; i < GT_TILE; i += 256) rows[i] = i < count ? order[first + i] / top : -1;
  __syncthreads();
  const __bf16* g_w = wg + (long long)e * ff * width;
  const __bf16* u_w = wu + (long long)e * ff * width;
  gt_f32x4 acc[4][4];
  group_tile_mma(
      [&](int r) -> const __bf16* { return rows[r] >= 0 ? h + (long long)rows[r] * ldh : nullptr; },
      [&](int r) -> const __bf16* {
        const int col = n0 + (r >> 6) * 32 + ((r >> 4) & 1) * 16 + (r & 15);
        if (col >= ff) return nullptr;
        return (((r >> 5) & 1) ? u_w : g_w) + (long long)col * width;
      },
      width, lds, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 15, lg = lane >> 4;
#pragma unroll
  for (int tm = 0; tm < 4; ++tm) {
    const int r = wm * 64 + tm * 16 + lr;
    if (r >= count) continue;
    const float w = in_weights ? in_weights[order[first + r]] : 1.f;
#pragma unroll
    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int col = n0 + wn * 32 + tn * 16 + lg * 4 + i;
        if (col >= ff) continue;
        act[(long long)(first + r) * ff + col] = (__bf16)expert_act(w * acc[tn][tm][i], w * acc[tn + 2][tm][i], limit, alpha);
      }
  }
}

__global__ __launch_bounds__(256) void moe_down_mma_kernel(const __bf16* __restrict__ act, const __bf16* __restrict__ wd,
                                                           const int* __restrict__ offsets,
                                                           const int* __restrict__ order,
                                                           const int* __restrict__ tiles,
                                                           const int* __restrict__ num_tiles, int width, int ff,
                                                           float* __restrict__ pair_out) {
  if ((int)blockIdx.x >= num_tiles[0]) return;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int e = tiles[2 * blockIdx.x], first = tiles[2 * blockIdx.x + 1];
  const int count = min(GT_TILE, offsets[e + 1] - first);
  const int n0 = blockIdx.y * GT_TILE;
  const __bf16* w = wd + (long long)e * width * ff;
  gt_f32x4 acc[4][4];
  group_tile_mma([&](int r) -> const __bf16* { return r < count ? act + (long long)(first + r) * ff : nullptr; },
                 [&](int r) -> const __bf16* { return n0 + r < width ? w + (long long)(n0 + r) * ff : nullptr; }, ff,
                 lds, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 15, lg = lane >> 4;
#pragma unroll
  for (int tm = 0; tm < 4; ++tm) {
    const int r = wm * 64 + tm * 16 + lr;
    if (r >= count) continue;
    float* dst = pair_out + (long long)order[first + r] * width;
#pragma unroll
    for (int tn = 0; tn < 4; ++tn)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int col = n0 + wn * 64 + tn * 16 + lg * 4 + i;
        if (col < width) dst[col] = acc[tn][tm][i];
      }
  }
}

// residual[t, :] (+)= sum_j weights[t, j] * pair_out[t * top + j, :], j ascending (weights null: every weight is 1).
__global__ void moe_combine_kernel(const float* __restrict__ pair_out, const float* __restrict__ weights, int top,
                                   int width, long long total, float* __restrict__ residual, int accumulate) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long t = idx / width;
  const int c = (int)(idx % width);
  float sum = 0.f;
  for (int j = 0; j < top; ++j) sum = fmaf(weights ? weights[t * top + j] : 1.f, pair_out[(t * top + j) * width + c], sum);
  residual[idx] = accumulate ? residual[idx] + sum : sum;
}

// ---------------------------------------------------------------------------------------------
extern "C" int vk_moe_max_tiles(int pairs, int experts, int tile_rows) {
  return (pairs + tile_rows - 1) / tile_rows + experts;
}

// Whether the products of these operands run on the matrix cores (tiles of 128 places) or as 32-bit FMAs (64).
static inline bool moe_on_matrix_cores(int dtype, int width, int ff, long long ldh) {
  return dtype == DT_BF16 && width % 8 == 0 && ff % 8 == 0 && ldh % 8 == 0;
}

extern "C" int vk_moe_tile_rows(int dtype, int width, int ff, long long ldh) {
  return moe_on_matrix_cores(dtype, width, ff, ldh) ? GT_TILE : MOE_TILE;
}

extern "C" int vk_moe_route_steered(const float* logits, int experts, int top, int num_tokens, int tile_rows, int groups,
                                    int keep, int all_scores, const float* correction, float weight_scale, long long ld,
                                    int* ids, float* weights, int* offsets, int* order, int* tiles, int* num_tiles,
                                    void* stream) {
  if (tile_rows != MOE_TILE && tile_rows != GT_TILE) return VK_BAD_ARGUMENT;
  if (groups < 1 || keep < 1 || keep > groups || experts % groups != 0) return VK_BAD_ARGUMENT;
  if (groups > WAVE) return VK_UNSUPPORTED_SIZE;
  if (keep < groups && (long long)keep * (experts / groups) < top) return VK_BAD_ARGUMENT;
  if (all_scores < 0 || all_scores > 3 || (correction && all_scores != 3)) return VK_BAD_ARGUMENT;
  if (ld != 0 && ld < experts) return VK_BAD_ARGUMENT;
  const Routing how{groups, keep, all_scores, correction, weight_scale, ld};
  if (num_tokens <= 0) return 0;
  if (experts < 1 || top < 1 || top > experts || top > WAVE) return VK_BAD_ARGUMENT;
  if (experts > 4096) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  const long long pairs = (long long)num_tokens * top;
  if (pairs > 0x7fffffff) return VK_UNSUPPORTED_SIZE;
  const bool together = num_tokens <= 16;     // a wave of the one workgroup for every token
  if (!together) {
    moe_route_kernel<<<(num_tokens + 3) / 4, 256, 0, s>>>(logits, experts, top, num_tokens, ids, weights, how);
    VK_LAUNCH_CHECK();
  }
  moe_group_kernel<<<1, 1024, (size_t)experts * 2 * sizeof(int), s>>>(together ? logits : nullptr, top, num_tokens,
                                                                       weights, ids, (int)pairs, experts, tile_rows,
                                                                       offsets, order, tiles, num_tiles, how);
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_moe_route_grouped(const float* logits, int experts, int top, int num_tokens, int tile_rows, int groups,
                                    int keep, int all_scores, int* ids, float* weights, int* offsets, int* order,
                                    int* tiles, int* num_tiles, void* stream) {
  if (all_scores > 2) return VK_BAD_ARGUMENT;
  return vk_moe_route_steered(logits, experts, top, num_tokens, tile_rows, groups, keep, all_scores, nullptr, 1.f, 0, ids,
                              weights, offsets, order, tiles, num_tiles, stream);
}

extern "C" int vk_moe_route(const float* logits, int experts, int top, int num_tokens, int tile_rows, int* ids,
                            float* weights, int* offsets, int* order, int* tiles, int* num_tiles, void* stream) {
  return vk_moe_route_grouped(logits, experts, top, num_tokens, tile_rows, 1, 1, 0, ids, weights, offsets, order, tiles,
                              num_tiles, stream);
}

// accumulate 0: the weighted sums are written to `residual` instead of added to it.  weigh_input: a pair's weight
// multiplies what its expert reads (w h, applied to the gate and up sums, which are linear in h) instead of what it
// returns.
extern "C" int vk_moe_experts_weighed(const void* h, long long ldh, const void* wg, const void* wu, const void* wd,
                                      int dtype, const int* offsets, const int* order, const int* tiles,
                                      const int* num_tiles, const float* weights, int num_tokens, int experts, int top,
                                      int width, int ff, float limit, float alpha, void* act, float* pair_out,
                                      float* residual, int accumulate, int weigh_input, void* stream) {
  if (num_tokens <= 0) return 0;
  const float* in_weights = weigh_input ? weights : nullptr;
  const float* out_weights = weigh_input ? nullptr : weights;
  if (experts < 1 || top < 1 || width < 1 || ff < 1) return VK_BAD_ARGUMENT;
  const int pairs = num_tokens * top;
  hipStream_t s = (hipStream_t)stream;
  if (moe_on_matrix_cores(dtype, width, ff, ldh)) {
    if (((uintptr_t)h | (uintptr_t)wg | (uintptr_t)wu | (uintptr_t)wd | (uintptr_t)act) & 15) return VK_BAD_ARGUMENT;
    const int wide_tiles = vk_moe_max_tiles(pairs, experts, GT_TILE);
    dim3 up(wide_tiles, (ff + 63) / 64), down(wide_tiles, (width + GT_TILE - 1) / GT_TILE);
    if (up.y > 65535 || down.y > 65535) return VK_UNSUPPORTED_SIZE;
    static bool sized = false;
    if (!sized) {
      hipError_t e1 = hipFuncSetAttribute((const void*)moe_gate_up_mma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, GT_LDS_BYTES);
      hipError_t e2 = hipFuncSetAttribute((const void*)moe_down_mma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, GT_LDS_BYTES);
      if (e1 != hipSuccess || e2 != hipSuccess) return (int)(e1 != hipSuccess ? e1 : e2);
      sized = true;
    }
    moe_gate_up_mma_kernel<<<up, 256, GT_LDS_BYTES, s>>>((const __bf16*)h, ldh, (const __bf16*)wg, (const __bf16*)wu,
                                                        offsets, order, tiles, num_tiles, top, width, ff, limit, alpha,
                                                        in_weights, (__bf16*)act);
    VK_LAUNCH_CHECK();
    moe_down_mma_kernel<<<down, 256, GT_LDS_BYTES, s>>>((const __bf16*)act, (const __bf16*)wd, offsets, order, tiles,
                                                        num_tiles, width, ff, pair_out);
    VK_LAUNCH_CHECK();
    const long long all = (long long)num_tokens * width;
    moe_combine_kernel<<<(unsigned)((all + 255) / 256), 256, 0, s>>>(pair_out, out_weights, top, width, all, residual, accumulate);
    VK_LAUNCH_CHECK();
    return 0;
  }
  const int max_tiles = vk_moe_max_tiles(pairs, experts, MOE_TILE);
  dim3 up_grid(max_tiles, (ff + MOE_TILE - 1) / MOE_TILE), down_grid(max_tiles, (width + MOE_TILE - 1) / MOE_TILE);
  if (up_grid.y > 65535 || down_grid.y > 65535) return VK_UNSUPPORTED_SIZE;
  if (dtype == DT_F32) {
    moe_gate_up_kernel<float><<<up_grid, 256, 0, s>>>((const float*)h, ldh, (const float*)wg, (const float*)wu,
                                                      offsets, order, tiles, num_tiles, top, width, ff, limit, alpha,
                                                      in_weights, (float*)act);
    VK_LAUNCH_CHECK();
    moe_down_kernel<float><<<down_grid, 256, 0, s>>>((const float*)act, (const float*)wd, offsets, order, tiles,
                                                     num_tiles, width, ff, pair_out);
  } else if (dtype == DT_BF16) {
    moe_gate_up_kernel<bf16_t><<<up_grid, 256, 0, s>>>((const bf16_t*)h, ldh, (const bf16_t*)wg, (const bf16_t*)wu,
                                                       offsets, order, tiles, num_tiles, top, width, ff, limit, alpha,
                                                       in_weights, (bf16_t*)act);
    VK_LAUNCH_CHECK();
    moe_down_kernel<bf16_t><<<down_grid, 256, 0, s>>>((const bf16_t*)act, (const bf16_t*)wd, offsets, order, tiles,
                                                      num_tiles, width, ff, pair_out);
  } else {
    return VK_BAD_ARGUMENT;
  }
  VK_LAUNCH_CHECK();
  const long long total = (long long)num_tokens * width;
  moe_combine_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(pair_out, out_weights, top, width, total, residual, accumulate);
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_moe_experts_into(const void* h, long long ldh, const void* wg, const void* wu, const void* wd, int dtype,
                                   const int* offsets, const int* order, const int* tiles, const int* num_tiles,
                                   const float* weights, int num_tokens, int experts, int top, int width, int ff,
                                   float limit, float alpha, void* act, float* pair_out, float* residual,
                                   int accumulate, void* stream) {
  return vk_moe_experts_weighed(h, ldh, wg, wu, wd, dtype, offsets, order, tiles, num_tiles, weights, num_tokens, experts,
                                top, width, ff, limit, alpha, act, pair_out, residual, accumulate, 0, stream);
}

extern "C" int vk_moe_experts(const void* h, long long ldh, const void* wg, const void* wu, const void* wd, int dtype,
                              const int* offsets, const int* order, const int* tiles, const int* num_tiles,
                              const float* weights, int num_tokens, int experts, int top, int width, int ff,
                              float limit, float alpha, void* act, float* pair_out, float* residual, void* stream) {
  return vk_moe_experts_into(h, ldh, wg, wu, wd, dtype, offsets, order, tiles, num_tiles, weights, num_tokens, experts,
                             top, width, ff, limit, alpha, act, pair_out, residual, 1, stream);
}
