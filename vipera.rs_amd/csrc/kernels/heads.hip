// Work on the heads of an attention layer before and behind the paged attention kernels, and small per-row steps of
// layers whose sublayers are normed behind instead of in front. All arithmetic is 32-bit.
#include "common.h"

namespace {
constexpr int HEAD_REGS = 4;   // a lane keeps up to four numbers of a head: heads of up to 256 numbers

// ---------------------------------------------------------------------------------------------
// head_prepare: the 32-bit sums of a [q | k | v] product become the rows that the rotation-free cache write and the
// attention kernels read, every head at one padded width W.
//   proj [T, ldp]: q (heads * maps * dim) | k (kv_heads * maps * dim) | v (kv_heads * vdim) from column 0 on
//   rotation   the first rot_dims numbers of a q or k head in the half-split layout: pair (i, i + rot_dims / 2) turns
//              by float(position) * inv_freq[i]; rot_dims 0: none
//   norm       0 none; 1 every q and k head divided by its root mean square (eps inside the root) and multiplied by a
//              weight of `dim` numbers shared by the heads (null: no weight); norm_first: before the rotation, else
//              behind it
//   maps       1, or m attention maps per head: a query head's m maps lie one behind the other in proj and become m
//              query heads, map j in columns [j dim, (j + 1) dim) of its padded head and zeros elsewhere; a key head's
//              m maps stay side by side as one key head of m dim numbers. Query (h, j) then meets exactly map j of its
//              key head, and all maps of a head read the same values.
//   qkv  [T, (heads * maps + 2 kv_heads) * W], W >= max(maps * dim, vdim)
//   k_cache [page, kv_head, slot, W], v_cache [page, kv_head, W, slot] (transposed), or null: the tokens' key and
//   value heads, as they stand in qkv, also go into their pages (page of position p = table[entry, p / block_size]; a
//   negative page id writes nothing), which saves the launch that would only copy them there
// One wave per (token, source head): heads * maps + kv_heads * maps + kv_heads of them a token.
template <typename TO>
__global__ __launch_bounds__(256) void head_prepare_kernel(
    const float* __restrict__ proj, long long ldp, const float* __restrict__ q_weight, const float* __restrict__ k_weight,
    int norm, int norm_first, float eps, const int* __restrict__ positions, const float* __restrict__ inv_freq,
    int rot_dims, int heads, int kv_heads, int maps, int dim, int vdim, int W, long long units, TO* __restrict__ qkv,
    TO* __restrict__ k_cache, TO* __restrict__ v_cache, const int* __restrict__ entry_of_token,
    const int* __restrict__ block_table, int table_width, int block_size) {
  const int lane = threadIdx.x & (WAVE - 1);
  const long long unit = (long long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (unit >= units) return;
  const int qk_units = (heads + kv_heads) * maps, all = qk_units + kv_heads;
  const long long t = unit / all;
  const int u = (int)(unit % all);
  const float* src = proj + t * ldp;
  TO* row = qkv + t * (long long)(heads * maps + 2 * kv_heads) * W;
  int page = -1, slot = 0;
  if (k_cache != nullptr && u >= heads * maps) {
    const int pos = positions[t];
    page = block_table[(size_t)entry_of_token[t] * table_width + pos / block_size];
    slot = pos % block_size;
  }
  if (u >= qk_units) {                                   // a value head: copied, padded with zeros
    const int g = u - qk_units;
    const float* x = src + (long long)qk_units * dim + (long long)g * vdim;
    TO* dst = row + (long long)(heads * maps + kv_heads + g) * W;
    TO* paged = page >= 0 ? v_cache + (((size_t)page * kv_heads + g) * W) * block_size + slot : nullptr;
    for (int d = lane; d < W; d += WAVE) {
      const TO v = from_float<TO>(d < vdim ? x[d] : 0.f);
      dst[d] = v;
      if (paged) paged[(size_t)d * block_size] = v;
    }
    return;
  }
  const bool is_q = u < heads * maps;
  const float* x = src + (long long)u * dim;             // q maps and k maps lie one behind the other
  const float* weight = is_q ? q_weight : k_weight;
  const int half = rot_dims / 2;
  float y[HEAD_REGS];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < HEAD_REGS; ++i) {
    const int d = lane + WAVE * i;
    y[i] = d < dim ? x[d] : 0.f;
    ss = fmaf(y[i], y[i], ss);
  }
  float inv = 1.f;
  if (norm && norm_first) {
    inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < HEAD_REGS; ++i) {
      const int d = lane + WAVE * i;
      if (d < dim) y[i] = weight ? y[i] * inv * weight[d] : y[i] * inv;
    }
  }
  if (rot_dims > 0) {
    const float pos = (float)positions[t];
    float partner[HEAD_REGS];
#pragma unroll
    for (int i = 0; i < HEAD_REGS; ++i) {                // the partner's number, normed as this lane's own is
      const int d = lane + WAVE * i;
      const int other = d < half ? d + half : d - half;
      float v = 0.f;
      if (d < rot_dims) {
        v = x[other];
        if (norm && norm_first) v = weight ? v * inv * weight[other] : v * inv;
      }
      partner[i] = v;
    }
    ss = 0.f;
#pragma unroll
    for (int i = 0; i < HEAD_REGS; ++i) {
      const int d = lane + WAVE * i;
      if (d < rot_dims) {
        float sn, cs;
        sincosf(pos * inv_freq[d < half ? d : d - half], &sn, &cs);
        y[i] = d < half ? y[i] * cs - partner[i] * sn : y[i] * cs + partner[i] * sn;
      }
      ss = fmaf(y[i], y[i], ss);
    }
  }
  if (norm && !norm_first) {
    inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < HEAD_REGS; ++i) {
      const int d = lane + WAVE * i;
      if (d < dim) y[i] = weight ? y[i] * inv * weight[d] : y[i] * inv;
    }
  }
  if (is_q) {
    TO* dst = row + (long long)u * W;
    const int at = (u % maps) * dim;
    for (int d = lane; d < W; d += WAVE)
      if (d < at || d >= at + dim) dst[d] = from_float<TO>(0.f);
#pragma unroll
    for (int i = 0; i < HEAD_REGS; ++i) {
      const int d = lane + WAVE * i;
      if (d < dim) dst[at + d] = from_float<TO>(y[i]);
    }
  } else {
    const int ku = u - heads * maps, g = ku / maps, j = ku % maps;
    TO* dst = row + (long long)(heads * maps + g) * W;
    TO* paged = page >= 0 ? k_cache + (((size_t)page * kv_heads + g) * block_size + slot) * W : nullptr;
#pragma unroll
    for (int i = 0; i < HEAD_REGS; ++i) {
      const int d = lane + WAVE * i;
      if (d < dim) {
        const TO v = from_float<TO>(y[i]);
        dst[j * dim + d] = v;
        if (paged) paged[j * dim + d] = v;
      }
    }
    if (j == maps - 1)
      for (int d = maps * dim + lane; d < W; d += WAVE) {
        dst[d] = from_float<TO>(0.f);
        if (paged) paged[d] = from_float<TO>(0.f);
      }
  }
}

// ---------------------------------------------------------------------------------------------
// head_finish: the attention kernels' output, heads padded to W, becomes the output product's input.
//   attn [T, heads * maps * W]
//   maps 2: o = a_1 - lambda a_2 with the two maps of a head (differential attention); maps 1: o = a
//   unit_norm: o / sqrt(mean(o^2) + eps) over the head's vdim numbers
//   times `factor`
//   gate [T, ldg] 32-bit, null: none; gate_per_head: one number per head (column h), else one per number (column
//   h vdim + d); the gate is act(g) with act as in the activation kernel (2 silu, 4 sigmoid)
//   out [T, heads * vdim]
// One wave per (token, head).
__device__ __forceinline__ float gate_act(float z, int act) {
  switch (act) {
    case 2: return z / (1.0f + expf(-z));
    case 4: return 1.0f / (1.0f + expf(-z));
    default: return z;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void head_finish_kernel(const T* __restrict__ attn, int maps, float lambda, int unit_norm,
                                                          float eps, float factor, const float* __restrict__ gate,
                                                          long long ldg, int gate_per_head, int act, int heads, int vdim,
                                                          int W, long long units, T* __restrict__ out) {
  const int lane = threadIdx.x & (WAVE - 1);
  const long long unit = (long long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (unit >= units) return;
  const long long t = unit / heads;
  const int h = (int)(unit % heads);
  const T* a = attn + (t * heads + h) * (long long)maps * W;
  float o[HEAD_REGS];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < HEAD_REGS; ++i) {
    const int d = lane + WAVE * i;
    float v = 0.f;
    if (d < vdim) {
      v = to_float<T>(a[d]);
      if (maps == 2) v -= lambda * to_float<T>(a[W + d]);
    }
    o[i] = v;
    ss = fmaf(v, v, ss);
  }
  float mult = factor;
  if (unit_norm) mult *= 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
  if (gate && gate_per_head) mult *= gate_act(gate[t * ldg + h], act);
#pragma unroll
  for (int i = 0; i < HEAD_REGS; ++i) {
    const int d = lane + WAVE * i;
    if (d >= vdim) continue;
    float v = o[i] * mult;
    if (gate && !gate_per_head) v *= gate_act(gate[t * ldg + (long long)h * vdim + d], act);
    out[(t * heads + h) * (long long)vdim + d] = from_float<T>(v);
  }
}

// ---------------------------------------------------------------------------------------------
// rotate_scale: heads of 32-bit numbers rotated in place by their token's position (half-split layout over the first
// rot_dims numbers of a head) and multiplied by `factor`.  x [T, ld], `heads` heads of `dim` numbers from column 0 on.
__global__ void rotate_scale_kernel(float* __restrict__ x, long long ld, const int* __restrict__ positions,
                                    const float* __restrict__ inv_freq, int rot_dims, int heads, int dim, float factor,
                                    long long total) {
  // a thread owns one pair (or, past the rotated numbers, one number)
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int half = rot_dims / 2, per_head = dim - half;
  const long long t = idx / ((long long)heads * per_head);
  const int rest = (int)(idx % ((long long)heads * per_head)), h = rest / per_head, i = rest % per_head;
  float* head = x + t * ld + (long long)h * dim;
  if (i < half) {
    float sn, cs;
    sincosf((float)positions[t] * inv_freq[i], &sn, &cs);
    const float u = head[i], v = head[i + half];
    head[i] = (u * cs - v * sn) * factor;
    head[i + half] = (v * cs + u * sn) * factor;
  } else {
    head[i + half] *= factor;
  }
}

// ---------------------------------------------------------------------------------------------
// row_gate_add: out[r, :] (+)= act(g[r]) * y[r, :], one learned number per row (a sublayer's output gated per token).
__global__ void row_gate_add_kernel(const float* __restrict__ y, const float* __restrict__ g, long long ldg, int act,
                                    float* __restrict__ out, int width, long long total, int accumulate) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const float v = gate_act(g[(idx / width) * ldg], act) * y[idx];
  out[idx] = accumulate ? out[idx] + v : v;
}
}  // namespace

extern "C" int vk_head_prepare(const float* proj, long long ldp, const float* q_weight, const float* k_weight, int norm,
                               int norm_first, float eps, const int* positions, const float* inv_freq, int rot_dims,
                               int num_tokens, int heads, int kv_heads, int maps, int dim, int vdim, int W, void* qkv,
                               int dtype, void* k_cache, void* v_cache, const int* entry_of_token, const int* block_table,
                               int table_width, int block_size, void* stream) {
  if (num_tokens <= 0) return 0;
  if (k_cache && (!v_cache || !entry_of_token || !block_table || !positions || table_width <= 0 || block_size <= 0))
    return VK_BAD_ARGUMENT;
  if (heads < 1 || kv_heads < 1 || maps < 1 || dim < 1 || vdim < 1 || W < maps * dim || W < vdim) return VK_BAD_ARGUMENT;
  if (dim > HEAD_REGS * WAVE) return VK_UNSUPPORTED_SIZE;
  if (rot_dims < 0 || rot_dims > dim || (rot_dims & 1) || (rot_dims > 0 && (!positions || !inv_freq))) return VK_BAD_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  const long long units = (long long)num_tokens * ((heads + kv_heads) * maps + kv_heads);
  const long long blocks = (units + 3) / 4;
  if (blocks > 0x7fffffffLL) return VK_UNSUPPORTED_SIZE;
  if (dtype == DT_F32)
    head_prepare_kernel<float><<<(unsigned)blocks, 256, 0, s>>>(proj, ldp, q_weight, k_weight, norm, norm_first, eps, positions,
                                                                inv_freq, rot_dims, heads, kv_heads, maps, dim, vdim, W, units,
                                                                (float*)qkv, (float*)k_cache, (float*)v_cache, entry_of_token,
                                                                block_table, table_width, block_size);
  else if (dtype == DT_BF16)
    head_prepare_kernel<bf16_t><<<(unsigned)blocks, 256, 0, s>>>(proj, ldp, q_weight, k_weight, norm, norm_first, eps, positions,
                                                                 inv_freq, rot_dims, heads, kv_heads, maps, dim, vdim, W, units,
                                                                 (bf16_t*)qkv, (bf16_t*)k_cache, (bf16_t*)v_cache,
                                                                 entry_of_token, block_table, table_width, block_size);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_head_finish(const void* attn, int dtype, int maps, float lambda, int unit_norm, float eps, float factor,
                              const float* gate, long long ldg, int gate_per_head, int act, int num_tokens, int heads,
                              int vdim, int W, void* out, void* stream) {
  if (num_tokens <= 0) return 0;
  if (heads < 1 || vdim < 1 || W < vdim || maps < 1 || maps > 2 || (act != 0 && act != 2 && act != 4)) return VK_BAD_ARGUMENT;
  if (vdim > HEAD_REGS * WAVE) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  const long long units = (long long)num_tokens * heads;
  const long long blocks = (units + 3) / 4;
  if (blocks > 0x7fffffffLL) return VK_UNSUPPORTED_SIZE;
  if (dtype == DT_F32)
    head_finish_kernel<float><<<(unsigned)blocks, 256, 0, s>>>((const float*)attn, maps, lambda, unit_norm, eps, factor, gate,
                                                               ldg, gate_per_head, act, heads, vdim, W, units, (float*)out);
  else if (dtype == DT_BF16)
    head_finish_kernel<bf16_t><<<(unsigned)blocks, 256, 0, s>>>((const bf16_t*)attn, maps, lambda, unit_norm, eps, factor,
                                                                gate, ldg, gate_per_head, act, heads, vdim, W, units,
                                                                (bf16_t*)out);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_rotate_scale(float* x, long long ld, const int* positions, const float* inv_freq, int rot_dims,
                               int num_tokens, int heads, int dim, float factor, void* stream) {
  if (num_tokens <= 0) return 0;
  if (heads < 1 || dim < 1 || rot_dims < 0 || rot_dims > dim || (rot_dims & 1)) return VK_BAD_ARGUMENT;
  if (rot_dims > 0 && (!positions || !inv_freq)) return VK_BAD_ARGUMENT;
  const long long total = (long long)num_tokens * heads * (dim - rot_dims / 2);
  const long long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return VK_UNSUPPORTED_SIZE;
  rotate_scale_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(x, ld, positions, inv_freq, rot_dims, heads, dim,
                                                                         factor, total);
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_row_gate_add(const float* y, const float* g, long long ldg, int act, float* out, int num_rows, int width,
                               int accumulate, void* stream) {
  if (num_rows <= 0) return 0;
  if (width < 1 || (act != 0 && act != 2 && act != 4)) return VK_BAD_ARGUMENT;
  const long long total = (long long)num_rows * width;
  const long long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return VK_UNSUPPORTED_SIZE;
  row_gate_add_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(y, g, ldg, act, out, width, total, accumulate);
  VK_LAUNCH_CHECK();
  return 0;
}
