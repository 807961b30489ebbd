// Recurrent mixers: linear-attention layers that carry a matrix of state per head from token to token.
//
// Everything that enters a recurrence is 32-bit: the state, decays, gates, unit norms.  A request's state is one
// row of a `[slots + 1, floats]` tensor; an entry that starts at position 0 treats its row as zeros, so a slot
// that is used again needs no clearing.  The tokens of a step lie flat, entry after entry; `entry_start[e]` is
// the first token of entry e, `entry_first_pos[e]` its position in the request, `slots[e]` the state row.
//
// The recurrence kernels keep a head's state matrix in registers, a column of it spread over four lanes, and walk an
// entry's tokens in order; a sum over the key channels has one fixed order, whatever else is in the launch.
#include "common.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// ---------------------------------------------------------------------------------------------
// Short causal convolution over time per channel, then silu; q and k heads made unit vectors; gates.
//   proj  [T, ldp] 32-bit: channels [q: kh*dim | k: kh*dim | v: heads*vdim] first, later columns are the caller's
//   conv  [C, taps] 32-bit, the last column is the current token's
//   state row: `(taps - 1) * C` floats from `conv_offset` on, the inputs of the last taps - 1 tokens, oldest first
//   ba    columns `b_col + h` and `a_col + h` of proj hold the projections for beta and the decay's step
// Outputs (32-bit): qkv [T, ldq >= C] (q unit * dim^-1/2, k unit, v), beta [T, heads], decay [T, heads] (a_col < 0:
// the decay is the caller's business, see channel_decay_kernel).
// Grid (tokens, segments): a segment is one q or k head (its unit norm needs the whole head) or up to 1,024 value
// channels.  No load sits behind a branch: where an input comes from (the step, the state, nowhere) picks an
// address, and the value is masked.
constexpr int PREP_SPAN = 1024;

__device__ __forceinline__ float conv_input(const float* __restrict__ proj, long long ldp, const float* __restrict__ old,
                                            int C, int taps, int t, int offset, bool fresh, int back, int c) {
  const bool in_step = back <= offset, in_state = !in_step && !fresh;
  const float* from = in_step ? proj + (long long)(t - back) * ldp + c
                              : in_state ? old + (long long)(taps - 1 - (back - offset)) * C + c : proj + (long long)t * ldp + c;
  const float x = *from;
  return (in_step || in_state) ? x : 0.f;
}

__global__ __launch_bounds__(256) void delta_prepare_kernel(
    const float* __restrict__ proj, long long ldp, const float* __restrict__ conv, int taps,
    const float* __restrict__ state, long long state_stride, long long conv_offset, const int* __restrict__ entry_of,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first, const int* __restrict__ slots,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, int kv_heads, int dim, int heads, int vdim,
    int b_col, int a_col, float unit_eps, float* __restrict__ qkv, long long ldq, float* __restrict__ beta,
    float* __restrict__ decay) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, seg = blockIdx.y;
  const int e = entry_of[t];
  const int offset = t - entry_start[e];
  const bool fresh = entry_first[e] == 0;
  const int unit_heads = 2 * kv_heads;
  const int C = unit_heads * dim + heads * vdim;
  const float* old = state + (long long)slots[e] * state_stride + conv_offset;
  float* out = qkv + (long long)t * ldq;
  const bool unit = seg < unit_heads;
  const int first = unit ? seg * dim : unit_heads * dim + (seg - unit_heads) * PREP_SPAN;
  const int last = unit ? first + dim : min(C, first + PREP_SPAN);
  float kept[PREP_SPAN / 256];      // a segment is at most 1,024 channels: four to a thread
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < PREP_SPAN / 256; ++i) {
    const int c = first + threadIdx.x + i * 256;
    float y = 0.f;
    if (c < last) {
      float sum = 0.f;
      for (int j = 0; j < taps; ++j)
        sum = fmaf(conv[(long long)c * taps + j], conv_input(proj, ldp, old, C, taps, t, offset, fresh, taps - 1 - j, c), sum);
      y = silu_f(sum);
    }
    kept[i] = y;
    ss += y * y;
  }
  float scale = 1.f;
  if (unit) {       // the same for all threads of the workgroup
    ss = block_sum(ss, scratch);
    scale = 1.0f / sqrtf(ss + unit_eps);
    if (seg < kv_heads) scale *= 1.0f / sqrtf((float)dim);
  }
#pragma unroll
  for (int i = 0; i < PREP_SPAN / 256; ++i) {
    const int c = first + threadIdx.x + i * 256;
    if (c < last) out[c] = kept[i] * scale;
  }
  if (seg == 0)
    for (int h = threadIdx.x; h < heads; h += blockDim.x) {
      const float* p = proj + (long long)t * ldp;
      beta[(long long)t * heads + h] = sigmoid_f(p[b_col + h]);
      if (a_col >= 0) decay[(long long)t * heads + h] = expf(-expf(a_log[h]) * softplus_f(p[a_col + h] + dt_bias[h]));
    }
}

// The convolution's inputs of an entry's last taps - 1 tokens become the state.  Grid (entries, ceil(C / 256)), a
// thread per channel; runs after delta_prepare has read the old rows.
__global__ __launch_bounds__(256) void conv_state_kernel(const float* __restrict__ proj, long long ldp, int taps, int C,
                                                         float* __restrict__ state, long long state_stride,
                                                         long long conv_offset, const int* __restrict__ entry_start,
                                                         const int* __restrict__ entry_first,
                                                         const int* __restrict__ slots) {
  const int e = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int start = entry_start[e], count = entry_start[e + 1] - start;
  const bool fresh = entry_first[e] == 0;
  float* rows = state + (long long)slots[e] * state_stride + conv_offset;
  const int keep = taps - 1;
  for (int j = 0; j < keep; ++j) {           // ascending: row j + count is read before it is written
    const int from = j + count;              // index into [old rows (keep) | the entry's tokens (count)]
    const bool in_step = from >= keep;
    const float* source = in_step ? proj + (long long)(start + from - keep) * ldp + c : rows + (long long)from * C + c;
    const float x = *source;
    rows[(long long)j * C + c] = (in_step || !fresh) ? x : 0.f;
  }
}

// ---------------------------------------------------------------------------------------------
// The two recurrences share their shape.  A workgroup of four waves owns 16 value channels of one (entry, head), a
// wave four of them; the sixteen lanes of a row of the wave share one value channel and each keeps R of its key
// channels in registers (16 R >= dim; rows past dim stay zero).  A sum over the key channels is R terms in a lane, in
// ascending order, then four exchanges inside the 16-lane row (DPP, no LDS).  The entry's tokens are walked in
// blocks of 16: a block's k, q (or r, k, decay), values and gates are fetched into registers while the block before
// is worked on, and passed on through LDS, so that a token's step waits for no memory.
//
// This form runs the steps of single tokens (BLOCK 1: few registers, many waves a SIMD); prompts' portions run on
// the scan kernels further down, a wave to a value channel.
//
// The state of a head lies in memory as [value channel, padded to 16][key channel, padded to 16 R]: a lane's R
// numbers are contiguous, a row's sixteen lanes hold one value channel's run, and a workgroup reads and writes one
// contiguous run.  Both forms read it; nobody else does.
constexpr int REC_BLOCK = 16;    // tokens per LDS block; 1 for steps of single tokens (few registers, many waves a SIMD)
constexpr int REC_COLS = 16;     // value channels per workgroup

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false);
  return v + __int_as_float(moved);
}

// Lane l of a row of 16 gets the value of lane l - N of its row, or `edge` where the row has no such lane.
template <int N>
__device__ __forceinline__ float row_shifted(float v, float edge) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(edge), __float_as_int(v), 0x110 + N, 0xF, 0xF, false));
}

// The sum over the 16 lanes of a row, in every lane: neighbours, pairs of neighbours, the halves of eight, the eights.
__device__ __forceinline__ float row_sum16(float v) {
  v = dpp_add<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  v = dpp_add<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  v = dpp_add<0x141>(v);    // row_half_mirror: the other quad of the eight
  v = dpp_add<0x140>(v);    // row_mirror: the other eight
  return v;
}

// Gated delta rule.  Per head, with S [dim, vdim]:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.
// Grid (entries, heads, ceil(vdim / 16)).  An LDS row of a token: [q: 16R | k: 16R | (CH: g: 16R) | v: 16 | beta, decay].
// CH: one decay per head and key channel, which scales that row of S; it lies in the token's qkv row from column
// g_col on, [heads, dim].  `ldq` is the row stride of qkv.
template <int R, int BLOCK, bool CH>
__global__ __launch_bounds__(256) void delta_rule_kernel(
    const float* __restrict__ qkv, long long ldq, int g_col, const float* __restrict__ beta,
    const float* __restrict__ decay, float* __restrict__ state, long long state_stride,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first, const int* __restrict__ slots,
    int kv_heads, int dim, int heads, int vdim, float* __restrict__ out) {
  constexpr int DP = 16 * R, VOFF = (CH ? 3 : 2) * DP, ROW = VOFF + REC_COLS + 2, COUNT = BLOCK * ROW;
  constexpr int LOADS = (COUNT + 255) / 256;
  __shared__ float rows[COUNT];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = lane & 15, d0 = grp * R;
  const int v0 = blockIdx.z * REC_COLS, mine_col = wave * 4 + (lane >> 4), v = v0 + mine_col;
  const bool live = v < vdim;
  const int kh = h / (heads / kv_heads);
  const int start = entry_start[e], end = entry_start[e + 1];
  float* mine = state + (long long)slots[e] * state_stride + (((long long)h * gridDim.z * REC_COLS + v) * 16 + grp) * R;
  const bool fresh = entry_first[e] == 0;
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = fresh ? 0.f : mine[i];
  // what this thread fetches of a block: element x of the block is token x / ROW, column x % ROW
  float held[LOADS];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int x = tid + i * 256, j = x / ROW, col = x % ROW, t = t0 + j;
      // one load per element and no branch around it (a load inside a branch would be waited for there, and a
      // block's loads would arrive one after the other): the address is chosen by selects, a clamped one where
      // the element does not exist, and the value is masked afterwards
      const bool is_q = col < DP, is_k = !is_q && col < 2 * DP, is_g = CH && !is_q && !is_k && col < VOFF;
      const bool is_v = col >= VOFF && col < VOFF + REC_COLS;
      const bool is_b = col == VOFF + REC_COLS;
      const int d = is_q ? col : is_k ? col - DP : col - 2 * DP, c = col - VOFF;
      const bool ok = x < COUNT && t < end && (is_q || is_k || is_g ? d < dim : is_v ? v0 + c < vdim : (is_b || !CH));
      const long long tt = ok ? t : start;
      const float* base = (is_q || is_k || is_g || is_v) ? qkv + tt * ldq : ((is_b || CH) ? beta : decay) + tt * heads + h;
      const int within = is_q ? kh * dim + d : is_k ? (kv_heads + kh) * dim + d : is_g ? g_col + h * dim + d
                         : is_v ? 2 * kv_heads * dim + h * vdim + v0 + c : 0;
      const float loaded = base[ok ? within : 0];
      const float value = ok ? loaded : 0.f;
      held[i] = value;
    }
  };
  fetch(start);
  for (int t0 = start; t0 < end; t0 += BLOCK) {
    __syncthreads();     // the block before has been read
#pragma unroll
    for (int i = 0; i < LOADS; ++i)
      if (tid + i * 256 < COUNT) rows[tid + i * 256] = held[i];
    __syncthreads();
    if (t0 + BLOCK < end) fetch(t0 + BLOCK);
    const int count = min(BLOCK, end - t0);
    // a token's numbers are read from LDS while the token before it is worked on
    float kk[R], qq[R], gg[CH ? R : 1], b, g, val;
    auto read = [&](int j) {
      const float* row = rows + j * ROW;
      b = row[VOFF + REC_COLS], g = row[VOFF + REC_COLS + 1], val = row[VOFF + mine_col];
#pragma unroll
      for (int i = 0; i < R; ++i) {
        kk[i] = row[DP + d0 + i];
        qq[i] = row[d0 + i];
        if (CH) gg[i] = row[2 * DP + d0 + i];
      }
    };
    read(0);
    for (int j = 0; j < count; ++j) {
      float k_now[R], q_now[R], g_rows[CH ? R : 1];
      const float b_now = b, g_now = g, val_now = val;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        k_now[i] = kk[i];
        q_now[i] = qq[i];
        if (CH) g_rows[i] = gg[i];
      }
      if (j + 1 < count) read(j + 1);
      float dot[2] = {0.f, 0.f};     // two chains, even and odd rows, added at the end: a fixed order
#pragma unroll
      for (int i = 0; i < R; ++i) {
        S[i] *= CH ? g_rows[i] : g_now;
        dot[i & 1] = fmaf(S[i], k_now[i], dot[i & 1]);
      }
      const float u = b_now * (val_now - row_sum16(dot[0] + dot[1]));
      float o[2] = {0.f, 0.f};
#pragma unroll
      for (int i = 0; i < R; ++i) {
        S[i] = fmaf(k_now[i], u, S[i]);
        o[i & 1] = fmaf(S[i], q_now[i], o[i & 1]);
      }
      const float sum = row_sum16(o[0] + o[1]);
      if (live && grp == 0) out[((long long)(t0 + j) * heads + h) * vdim + v] = sum;
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) mine[i] = S[i];
}

// RWKV-style time mixing.  Per head, with S [dim, dim]:  o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T,
// w = exp(-exp(wraw + w0)) per key channel.  r, k, v, wraw are 32-bit [T, heads * dim] with row strides of their own.
// Grid (entries, heads, ceil(dim / 16)).  An LDS row of a token: [r: 16R | k: 16R | w: 16R | v: 16].
template <int R, int BLOCK>
__global__ __launch_bounds__(256) void wkv_rule_kernel(
    const float* __restrict__ r, long long ldr, const float* __restrict__ k, long long ldk, const float* __restrict__ v,
    long long ldv, const float* __restrict__ wraw, long long ldw, const float* __restrict__ w0,
    const float* __restrict__ bonus, float* __restrict__ state, long long state_stride,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first, const int* __restrict__ slots, int dim,
    int heads, int decayed, float* __restrict__ out) {
  constexpr int DP = 16 * R, ROW = 3 * DP + REC_COLS, COUNT = BLOCK * ROW, LOADS = (COUNT + 255) / 256;
  __shared__ float rows[COUNT];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = lane & 15, d0 = grp * R;
  const int v0 = blockIdx.z * REC_COLS, mine_col = wave * 4 + (lane >> 4), col_v = v0 + mine_col;
  const bool live = col_v < dim;
  const int start = entry_start[e], end = entry_start[e + 1];
  float* mine = state + (long long)slots[e] * state_stride + (((long long)h * gridDim.z * REC_COLS + col_v) * 16 + grp) * R;
  const bool fresh = entry_first[e] == 0;
  float S[R], U[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    S[i] = fresh ? 0.f : mine[i];
    U[i] = d0 + i < dim ? bonus[h * dim + d0 + i] : 0.f;
  }
  float held[LOADS];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int x = tid + i * 256, j = x / ROW, col = x % ROW, t = t0 + j;
      // branch-free, as in the delta rule's kernel: selected addresses, one load each, masked values
      const bool is_r = col < DP, is_k = !is_r && col < 2 * DP, is_w = !is_r && !is_k && col < 3 * DP;
      const int d = is_r ? col : is_k ? col - DP : col - 2 * DP, c = col - 3 * DP;
      const bool ok = x < COUNT && t < end && (is_r || is_k || is_w ? d < dim : v0 + c < dim);
      const long long tt = ok ? t : start;
      const float* base = is_r ? r + tt * ldr : is_k ? k + tt * ldk : is_w ? wraw + tt * ldw : v + tt * ldv;
      const int within = ok ? h * dim + ((is_r || is_k || is_w) ? d : v0 + c) : 0;
      const float loaded = base[within];
      const float shift = w0[(ok && is_w) ? h * dim + d : 0];
      const float value = !ok ? 0.f : (is_w && !decayed) ? expf(-expf(loaded + shift)) : loaded;
      held[i] = value;
    }
  };
  fetch(start);
  for (int t0 = start; t0 < end; t0 += BLOCK) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < LOADS; ++i)
      if (tid + i * 256 < COUNT) rows[tid + i * 256] = held[i];
    __syncthreads();
    if (t0 + BLOCK < end) fetch(t0 + BLOCK);
    const int count = min(BLOCK, end - t0);
    float rr[R], kk[R], ww[R], val;
    auto read = [&](int j) {
      const float* row = rows + j * ROW;
      val = row[3 * DP + mine_col];
#pragma unroll
      for (int i = 0; i < R; ++i) {
        rr[i] = row[d0 + i];
        kk[i] = row[DP + d0 + i];
        ww[i] = row[2 * DP + d0 + i];
      }
    };
    read(0);
    for (int j = 0; j < count; ++j) {
      float r_now[R], k_now[R], w_now[R];
      const float val_now = val;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        r_now[i] = rr[i];
        k_now[i] = kk[i];
        w_now[i] = ww[i];
      }
      if (j + 1 < count) read(j + 1);
      float o[2] = {0.f, 0.f};
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const float kv = k_now[i] * val_now;
        o[i & 1] = fmaf(fmaf(U[i], kv, S[i]), r_now[i], o[i & 1]);
        S[i] = fmaf(w_now[i], S[i], kv);
      }
      const float sum = row_sum16(o[0] + o[1]);
      if (live && grp == 0) out[((long long)(t0 + j) * heads + h) * dim + col_v] = sum;
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) mine[i] = S[i];
}

// ---------------------------------------------------------------------------------------------
// The same recurrences for prompts' portions: a wave owns ONE value channel and its 64 lanes the key channels, Q of
// them each (64 Q >= the state's padded key width), so that one prompt of a few thousand tokens is heads x value
// channels waves, two or more to a SIMD, each with a short step per token: Q terms a lane, four DPP exchanges inside
// the rows, and the four rows' sums read by every lane.  A workgroup is eight waves (eight value channels) that share a
// block's k, q (r, k, decay) in LDS.  What a thread fetches of a block is worked out once, before the first block.
constexpr int SCAN_COLS = 8;
constexpr int SCAN_THREADS = SCAN_COLS * 64;

__device__ __forceinline__ float wave_total(float v) {
  v = row_sum16(v);
  const int bits = __float_as_int(v);
  return __int_as_float(__builtin_amdgcn_readlane(bits, 0)) + __int_as_float(__builtin_amdgcn_readlane(bits, 16)) +
         (__int_as_float(__builtin_amdgcn_readlane(bits, 32)) + __int_as_float(__builtin_amdgcn_readlane(bits, 48)));
}

// A block's fetch plan: element x = tid + i * SCAN_THREADS of the block is token x / ROW, column x % ROW; `plan[i]` is
// token * 2^24 + the column's offset inside the token's row of the source, or -1 for an element that is always zero.
template <int Q, bool CH>
__global__ __launch_bounds__(SCAN_THREADS) void delta_scan_kernel(
    const float* __restrict__ qkv, long long ldq, int g_col, const float* __restrict__ beta,
    const float* __restrict__ decay, float* __restrict__ state, long long state_stride,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first, const int* __restrict__ slots,
    int kv_heads, int dim, int heads, int vdim, int key_pad, int value_pad, float* __restrict__ out) {
  constexpr int DP = 64 * Q, VOFF = (CH ? 3 : 2) * DP, ROW = VOFF + SCAN_COLS, COUNT = REC_BLOCK * ROW;
  constexpr int LOADS = (COUNT + SCAN_THREADS - 1) / SCAN_THREADS;
  __shared__ float rows[COUNT];
  __shared__ float gates[REC_BLOCK][2];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int d0 = lane * Q;
  const int v0 = blockIdx.z * SCAN_COLS, v = v0 + wave;
  const bool live = v < vdim;
  const int kh = h / (heads / kv_heads);
  const int start = entry_start[e], end = entry_start[e + 1];
  if (start >= end) return;      // the whole workgroup
  float* mine = state + (long long)slots[e] * state_stride + ((long long)h * value_pad + v) * key_pad + d0;
  const bool fresh = entry_first[e] == 0, kept = v < value_pad;
  float S[Q];
#pragma unroll
  for (int i = 0; i < Q; ++i) S[i] = (!fresh && kept && d0 + i < key_pad) ? mine[i] : 0.f;
  int plan[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int x = tid + i * SCAN_THREADS, j = x / ROW, col = x % ROW;
    int within = -1;
    if (x < COUNT) {
      if (col < DP) { if (col < dim) within = kh * dim + col; }
      else if (col < 2 * DP) { if (col - DP < dim) within = (kv_heads + kh) * dim + col - DP; }
      else if (CH && col < VOFF) { if (col - 2 * DP < dim) within = g_col + h * dim + col - 2 * DP; }
      else if (v0 + col - VOFF < vdim) within = 2 * kv_heads * dim + h * vdim + v0 + col - VOFF;
    }
    plan[i] = within < 0 ? -1 : (j << 24) | within;
  }
  // A fetch only issues loads, every thread the same number of them and none inside a branch, from addresses that
  // exist whatever the block holds (the entry's last token stands in for tokens past its end, which are never worked
  // on; column 0 for numbers that are always zero).  A loaded number is first used when it is stored into LDS, a block
  // later, so that nothing waits for memory before the block in between has been worked on.
  float held[LOADS], held_gate;
  const float* gate_src = ((tid & 1) && !CH ? decay : beta) + h;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int t = min(t0 + (plan[i] >> 24 & 127), end - 1);
      held[i] = qkv[(long long)t * ldq + (plan[i] < 0 ? 0 : plan[i] & 0xFFFFFF)];
    }
    held_gate = gate_src[(long long)min(t0 + ((tid >> 1) & (REC_BLOCK - 1)), end - 1) * heads];
  };
  fetch(start);
  for (int t0 = start; t0 < end; t0 += REC_BLOCK) {
    __syncthreads();     // the block before has been read
#pragma unroll
    for (int i = 0; i < LOADS; ++i)
      if (tid + i * SCAN_THREADS < COUNT) rows[tid + i * SCAN_THREADS] = plan[i] < 0 ? 0.f : held[i];
    if (tid < 2 * REC_BLOCK) gates[tid >> 1][tid & 1] = held_gate;
    __syncthreads();
    fetch(min(t0 + REC_BLOCK, end - 1));
    const int count = min(REC_BLOCK, end - t0);
    float outs = 0.f;      // lane j of every row: its row's part of token j's read-out, which nothing waits for
    for (int j = 0; j < count; ++j) {
      const float* row = rows + j * ROW;
      const float b = gates[j][0], g = gates[j][1], val = row[VOFF + wave];
      float kk[Q], qq[Q];
#pragma unroll
      for (int i = 0; i < Q; ++i) {
        kk[i] = row[DP + d0 + i];
        qq[i] = row[d0 + i];
      }
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < Q; ++i) {
        S[i] *= CH ? row[2 * DP + d0 + i] : g;
        dot = fmaf(S[i], kk[i], dot);
      }
      const float u = b * (val - wave_total(dot));
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < Q; ++i) {
        S[i] = fmaf(kk[i], u, S[i]);
        o = fmaf(S[i], qq[i], o);
      }
      o = row_sum16(o);
      outs = (lane & (REC_BLOCK - 1)) == j ? o : outs;
    }
    outs += __shfl_xor(outs, 16, 64);     // (row 0 + row 1) + (row 2 + row 3), in every row
    outs += __shfl_xor(outs, 32, 64);
    if (live && lane < count) out[((long long)(t0 + lane) * heads + h) * vdim + v] = outs;
  }
  if (kept) {
#pragma unroll
    for (int i = 0; i < Q; ++i)
      if (d0 + i < key_pad) mine[i] = S[i];
  }
}

// An LDS row of a token: [r: 64Q | k: 64Q | w: 64Q | v: 8]; sources differ by column, so the plan keeps which.
template <int Q>
__global__ __launch_bounds__(SCAN_THREADS) void wkv_scan_kernel(
    const float* __restrict__ r, long long ldr, const float* __restrict__ k, long long ldk, const float* __restrict__ v,
    long long ldv, const float* __restrict__ wraw, long long ldw, const float* __restrict__ w0,
    const float* __restrict__ bonus, float* __restrict__ state, long long state_stride,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first, const int* __restrict__ slots, int dim,
    int heads, int key_pad, int value_pad, int decayed, float* __restrict__ out) {
  constexpr int DP = 64 * Q, ROW = 3 * DP + SCAN_COLS, COUNT = REC_BLOCK * ROW, LOADS = (COUNT + SCAN_THREADS - 1) / SCAN_THREADS;
  __shared__ float rows[COUNT];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int d0 = lane * Q;
  const int v0 = blockIdx.z * SCAN_COLS, col_v = v0 + wave;
  const bool live = col_v < dim;
  const int start = entry_start[e], end = entry_start[e + 1];
  if (start >= end) return;      // the whole workgroup
  float* mine = state + (long long)slots[e] * state_stride + ((long long)h * value_pad + col_v) * key_pad + d0;
  const bool fresh = entry_first[e] == 0, kept = col_v < value_pad;
  float S[Q], U[Q];
#pragma unroll
  for (int i = 0; i < Q; ++i) {
    S[i] = (!fresh && kept && d0 + i < key_pad) ? mine[i] : 0.f;
    U[i] = d0 + i < dim ? bonus[h * dim + d0 + i] : 0.f;
  }
  // kind * 2^28 + token * 2^21 + offset inside the head's dim (kinds: 0 r, 1 k, 2 decay, 3 value), or -1
  int plan[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int x = tid + i * SCAN_THREADS, j = x / ROW, col = x % ROW;
    const int kind = col < DP ? 0 : col < 2 * DP ? 1 : col < 3 * DP ? 2 : 3;
    const int d = kind < 3 ? col - kind * DP : v0 + col - 3 * DP;
    plan[i] = (x < COUNT && d < dim) ? (kind << 28) | (j << 21) | d : -1;
  }
  // A fetch only issues loads, the same number in every thread and none inside a branch, from addresses that exist
  // whatever the block holds; a loaded number is first used when it is stored into LDS, a block later.
  float held[LOADS];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int kind = plan[i] >> 28 & 3, d = plan[i] < 0 ? 0 : plan[i] & 0x1FFFFF;
      const long long t = min(t0 + (plan[i] >> 21 & 127), end - 1);
      const float* base = kind == 0 ? r + t * ldr : kind == 1 ? k + t * ldk : kind == 2 ? wraw + t * ldw : v + t * ldv;
      held[i] = base[h * dim + d];
    }
  };
  fetch(start);
  for (int t0 = start; t0 < end; t0 += REC_BLOCK) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      float value = held[i];
      if (!decayed) {      // the same for every thread: the caller has not turned wraw into the decay yet
        const float shift = w0[h * dim + (plan[i] < 0 ? 0 : plan[i] & 0x1FFFFF)];
        value = (plan[i] >> 28 & 3) == 2 ? expf(-expf(value + shift)) : value;
      }
      if (tid + i * SCAN_THREADS < COUNT) rows[tid + i * SCAN_THREADS] = plan[i] < 0 ? 0.f : value;
    }
    __syncthreads();
    fetch(min(t0 + REC_BLOCK, end - 1));
    const int count = min(REC_BLOCK, end - t0);
    float outs = 0.f;      // lane j of every row: its row's part of token j's read-out, which nothing waits for
    for (int j = 0; j < count; ++j) {
      const float* row = rows + j * ROW;
      const float val = row[3 * DP + wave];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < Q; ++i) {
        const float kv = row[DP + d0 + i] * val;
        o = fmaf(fmaf(U[i], kv, S[i]), row[d0 + i], o);
        S[i] = fmaf(row[2 * DP + d0 + i], S[i], kv);
      }
      o = row_sum16(o);
      outs = (lane & (REC_BLOCK - 1)) == j ? o : outs;
    }
    outs += __shfl_xor(outs, 16, 64);     // (row 0 + row 1) + (row 2 + row 3), in every row
    outs += __shfl_xor(outs, 32, 64);
    if (live && lane < count) out[((long long)(t0 + lane) * heads + h) * dim + col_v] = outs;
  }
  if (kept) {
#pragma unroll
    for (int i = 0; i < Q; ++i)
      if (d0 + i < key_pad) mine[i] = S[i];
  }
}

// ---------------------------------------------------------------------------------------------
// Token shift: mix_s[t] = h[t] + (h[t-1] - h[t]) * mu_s for `mixes` vectors mu; h[t-1] of an entry's first token
// is the state's saved row (zeros at position 0).  out [mixes, T, width] in the run's dtype.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(const T* __restrict__ h, int width, const float* __restrict__ mu,
                                                          int mixes, const float* __restrict__ state,
                                                          long long state_stride, long long prev_offset,
                                                          const int* __restrict__ entry_of,
                                                          const int* __restrict__ entry_start,
                                                          const int* __restrict__ entry_first,
                                                          const int* __restrict__ slots, int num_tokens,
                                                          T* __restrict__ out) {
  const int t = blockIdx.x;
  const int e = entry_of[t];
  const bool first = t == entry_start[e];
  const bool fresh = entry_first[e] == 0;
  const float* saved = state + (long long)slots[e] * state_stride + prev_offset;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    const float cur = to_float<T>(h[(long long)t * width + c]);
    // one load from a selected address, masked: no load behind a branch
    const float before = first ? saved[c] : to_float<T>(h[(long long)(t - 1) * width + c]);
    const float prev = (first && fresh) ? 0.f : before;
    const float diff = prev - cur;
    for (int s = 0; s < mixes; ++s)
      out[((long long)s * num_tokens + t) * width + c] = from_float<T>(fmaf(diff, mu[(long long)s * width + c], cur));
  }
}

// An entry's last h becomes the state's saved row; one workgroup per entry, after token_shift has read the old one.
template <typename T>
__global__ __launch_bounds__(256) void save_last_kernel(const T* __restrict__ h, int width, float* __restrict__ state,
                                                        long long state_stride, long long prev_offset,
                                                        const int* __restrict__ entry_start,
                                                        const int* __restrict__ slots) {
  const int e = blockIdx.x;
  const int last = entry_start[e + 1] - 1;
  float* saved = state + (long long)slots[e] * state_stride + prev_offset;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x)
    saved[c] = to_float<T>(h[(long long)last * width + c]);
}

// ---------------------------------------------------------------------------------------------
// Read-out of a recurrent head: o / rms(o) (per head, over its `vdim` channels) * weight * gate.
// weight: [vdim] shared by the heads, or [heads * vdim]; gate: a column range of a [T, ldg] buffer of type TG,
// as it is (`gate_silu` 0), through silu (1) or through the sigmoid (2).  One wave per (token, head).
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ weight,
                                                             int weight_per_head, const TG* __restrict__ gate,
                                                             long long ldg, int gate_silu, float eps, int heads,
                                                             int vdim, int num_tokens, TO* __restrict__ out) {
  const int lane = threadIdx.x & (WAVE - 1);
  const long long unit = (long long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (unit >= (long long)num_tokens * heads) return;
  const int t = (int)(unit / heads), h = (int)(unit % heads);
  const float* src = o + unit * vdim;
  float ss = 0.f;
  for (int c = lane; c < vdim; c += WAVE) ss += src[c] * src[c];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
  for (int c = lane; c < vdim; c += WAVE) {
    float g = to_float<TG>(gate[(long long)t * ldg + h * vdim + c]);
    if (gate_silu == 1) g = silu_f(g);
    else if (gate_silu == 2) g = sigmoid_f(g);
    const float w = weight[(weight_per_head ? h * vdim : 0) + c];
    out[unit * vdim + c] = from_float<TO>(src[c] * inv * w * g);
  }
}

// ---------------------------------------------------------------------------------------------
// Matrix memory with exponential gates (mLSTM).  Per head, with S [dim, vdim], n [dim] and a running maximum m of the
// gates' logarithms (all zero at position 0):
//   li = cap tanh(i_raw / cap),  lf = logsigmoid(cap tanh(f_raw / cap))
//   m' = max(lf + m, li);  a = exp(lf + m - m'),  b = exp(li - m')
//   S <- a S + b k v^T;  n <- a n + b k;  o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)
// All operands are columns of one 32-bit buffer `proj [T, ldp]`: q (heads * dim) from q_col on, k from k_col, v
// (heads * vdim) from v_col, the raw gates at i_col + h and f_col + h; q is multiplied by `q_scale` as it is read.
// State row of a request: the heads' matrices in the recurrences' common layout, then n and m once per tile of eight
// value channels ([heads][tiles][key_pad] and [heads][tiles]): every workgroup carries n and m itself, so it reads and
// writes copies of its own and no workgroup waits for another.
struct MemoryColumns {
  int q, k, v, i, f;
};

__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float log_gate(float raw, float cap, bool forget) {
  const float z = cap * tanhf(raw / cap);
  return forget ? log_sigmoid_f(z) : z;
}

// Steps of single tokens: the delta rule's shape (a workgroup owns 16 value channels of one (entry, head), the sixteen
// lanes of a row keep R key channels each of S and of n).  Grid (entries, heads, ceil(vdim / 16)).
template <int R>
__global__ __launch_bounds__(256) void memory_rule_kernel(
    const float* __restrict__ proj, long long ldp, MemoryColumns col, float q_scale, float cap,
    float* __restrict__ state, long long state_stride, long long n_offset, long long m_offset,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first, const int* __restrict__ slots, int dim,
    int heads, int vdim, float* __restrict__ out) {
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = lane & 15, d0 = grp * R, key_pad = 16 * R;
  const int v0 = blockIdx.z * REC_COLS, v = v0 + wave * 4 + (lane >> 4);
  const bool live = v < vdim;
  const int tiles = 2 * gridDim.z;       // tiles of eight value channels: this workgroup owns 2 z and 2 z + 1
  const int start = entry_start[e], end = entry_start[e + 1];
  float* row = state + (long long)slots[e] * state_stride;
  float* mine = row + (((long long)h * gridDim.z * REC_COLS + v) * 16 + grp) * R;
  float* my_n = row + n_offset + ((long long)h * tiles + 2 * blockIdx.z) * key_pad + d0;
  float* my_m = row + m_offset + (long long)h * tiles + 2 * blockIdx.z;
  const bool fresh = entry_first[e] == 0;
  float S[R], N[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const float s_old = mine[i], n_old = my_n[i];
    S[i] = fresh ? 0.f : s_old;
    N[i] = fresh ? 0.f : n_old;
  }
  const float m_old = my_m[0];
  float m = fresh ? 0.f : m_old;
  for (int t = start; t < end; ++t) {
    const float* p = proj + (long long)t * ldp;
    const float li = log_gate(p[col.i + h], cap, false), lf = log_gate(p[col.f + h], cap, true);
    const float val_loaded = p[col.v + h * vdim + (live ? v : 0)];
    const float val = live ? val_loaded : 0.f;
    float kk[R], qq[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const bool in = d0 + i < dim;
      const float k_loaded = p[col.k + h * dim + (in ? d0 + i : 0)], q_loaded = p[col.q + h * dim + (in ? d0 + i : 0)];
      kk[i] = in ? k_loaded : 0.f;
      qq[i] = in ? q_loaded * q_scale : 0.f;
    }
    const float m_new = fmaxf(lf + m, li);
    const float a = expf(lf + m - m_new), b = expf(li - m_new);
    m = m_new;
    float num[2] = {0.f, 0.f}, den[2] = {0.f, 0.f};     // two chains each, even and odd rows: a fixed order
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const float bk = b * kk[i];
      S[i] = fmaf(bk, val, a * S[i]);
      N[i] = fmaf(a, N[i], bk);
      num[i & 1] = fmaf(S[i], qq[i], num[i & 1]);
      den[i & 1] = fmaf(N[i], qq[i], den[i & 1]);
    }
    const float top = row_sum16(num[0] + num[1]), under = row_sum16(den[0] + den[1]);
    if (live && grp == 0) out[((long long)t * heads + h) * vdim + v] = top / (fmaxf(fabsf(under), expf(-m)) + 1e-6f);
  }
#pragma unroll
  for (int i = 0; i < R; ++i) mine[i] = S[i];
  if (wave == 0 && lane < 16) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      my_n[i] = N[i];
      my_n[key_pad + i] = N[i];
    }
    if (lane == 0) my_m[0] = my_m[1] = m;
  }
}

// The gates' logarithms of a step's tokens, in place: proj[t, i_col + h] <- li, proj[t, f_col + h] <- lf.  A prompt's
// recurrence reads them a block of tokens at a time and takes no tanh or logarithm itself.
__global__ __launch_bounds__(256) void memory_gates_kernel(float* __restrict__ proj, long long ldp, int i_col, int f_col,
                                                           int heads, float cap, long long count) {
  const long long x = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (x >= count) return;
  float* p = proj + x / heads * ldp + x % heads;
  p[i_col] = log_gate(p[i_col], cap, false);
  p[f_col] = log_gate(p[f_col], cap, true);
}

// Prompts' portions: the scan shape (a wave owns one value channel and its 64 lanes the key channels, eight waves to a
// workgroup, tokens through LDS in blocks of 16 fetched a block ahead).  Every wave carries n and m itself, but n . q
// is the same number in all eight waves: each works it out for two of the block's tokens and leaves it in LDS.  Nothing
// of a token's read-out goes back into the state, so S^T q is summed inside each row of sixteen lanes as the tokens
// pass (lane j of a row keeps token j's) and across the four rows once per block.
// An LDS row of a token: [q: 64Q | k: 64Q | v: 8]; the two gates' logarithms lie beside.  Grid (entries, heads, tiles).
// The gates' columns of `proj` hold the logarithms li and lf already (memory_gates_kernel).
template <int Q>
__global__ __launch_bounds__(SCAN_THREADS) void memory_scan_kernel(
    const float* __restrict__ proj, long long ldp, MemoryColumns col, float q_scale,
    float* __restrict__ state, long long state_stride, long long n_offset, long long m_offset,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first, const int* __restrict__ slots, int dim,
    int heads, int vdim, int key_pad, int value_pad, float* __restrict__ out) {
  constexpr int DP = 64 * Q, ROW = 2 * DP + SCAN_COLS, COUNT = REC_BLOCK * ROW, LOADS = (COUNT + SCAN_THREADS - 1) / SCAN_THREADS;
  constexpr int PER_WAVE = REC_BLOCK / SCAN_COLS;     // tokens of a block whose n . q a wave works out
  static_assert(PER_WAVE * SCAN_COLS == REC_BLOCK && REC_BLOCK == 16, "a block's tokens are a row of lanes, dealt to the waves");
  __shared__ float rows[COUNT];
  __shared__ float gates[REC_BLOCK][2];
  __shared__ float dens[REC_BLOCK];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int d0 = lane * Q;
  const int v0 = blockIdx.z * SCAN_COLS, v = v0 + wave;
  const bool live = v < vdim;
  const int start = entry_start[e], end = entry_start[e + 1];
  if (start >= end) return;      // the whole workgroup
  float* row0 = state + (long long)slots[e] * state_stride;
  float* mine = row0 + ((long long)h * value_pad + v) * key_pad + d0;
  float* my_n = row0 + n_offset + ((long long)h * gridDim.z + blockIdx.z) * key_pad + d0;
  float* my_m = row0 + m_offset + (long long)h * gridDim.z + blockIdx.z;
  const bool fresh = entry_first[e] == 0;
  float S[Q], N[Q];
#pragma unroll
  for (int i = 0; i < Q; ++i) {
    const bool in = d0 + i < key_pad;
    const float s_old = mine[in ? i : -d0], n_old = my_n[in ? i : -d0];     // a clamped address where the lane has no row
    S[i] = (!fresh && in) ? s_old : 0.f;
    N[i] = (!fresh && in) ? n_old : 0.f;
  }
  const float m_old = my_m[0];
  float m = fresh ? 0.f : m_old;
  // a block's fetch plan: token * 2^24 + the column inside the token's row of proj, or -1 for what is always zero
  int plan[LOADS];
  unsigned is_q = 0;     // bit i: element i of this thread is a query's number
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int x = tid + i * SCAN_THREADS, j = x / ROW, c = x % ROW;
    int within = -1;
    if (x < COUNT) {
      if (c < DP) { if (c < dim) within = col.q + h * dim + c; }
      else if (c < 2 * DP) { if (c - DP < dim) within = col.k + h * dim + c - DP; }
      else if (v0 + c - 2 * DP < vdim) within = col.v + h * vdim + v0 + c - 2 * DP;
    }
    plan[i] = within < 0 ? -1 : (j << 24) | within;
    is_q |= (unsigned)(c < DP) << i;
  }
  // A fetch only issues loads, every thread the same number of them and none inside a branch, from addresses that
  // exist whatever the block holds (the entry's last token stands in for tokens past its end, column 0 for numbers that
  // are always zero); what a loaded number becomes is decided when it is stored into LDS, a block later, so that
  // nothing waits for memory before the block in between has been worked on.
  float held[LOADS], held_gate;
  const int gate_col = ((tid & 1) ? col.f : col.i) + h;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int t = min(t0 + (plan[i] >> 24 & 127), end - 1);
      held[i] = proj[(long long)t * ldp + (plan[i] < 0 ? 0 : plan[i] & 0xFFFFFF)];
    }
    held_gate = proj[(long long)min(t0 + ((tid >> 1) & (REC_BLOCK - 1)), end - 1) * ldp + gate_col];
  };
  fetch(start);
  for (int t0 = start; t0 < end; t0 += REC_BLOCK) {
    // the block before has been read: every wave has passed the barrier at its end
#pragma unroll
    for (int i = 0; i < LOADS; ++i)
      if (tid + i * SCAN_THREADS < COUNT)
        rows[tid + i * SCAN_THREADS] = plan[i] < 0 ? 0.f : (is_q >> i & 1) ? held[i] * q_scale : held[i];
    if (tid < 2 * REC_BLOCK) gates[tid >> 1][tid & 1] = held_gate;
    __syncthreads();
    fetch(min(t0 + REC_BLOCK, end - 1));
    const int count = min(REC_BLOCK, end - t0);
    // The block's running maxima in closed form, so that no exponential waits for the token before it: with F_j the sum
    // of the forget gates' logarithms up to token j of the block and m0 the maximum the block starts from,
    // m_j = F_j + max(m0, max over l <= j of (li_l - F_l)).  Lane l of every row of sixteen works out token l & 15: two
    // scans along the row (sum, then maximum), its maximum and its neighbour's before it, and from those its three
    // exponentials; the token loop fetches them by lane.  Which sequence of maxima is used does not change the result
    // beyond rounding, as long as S, n and the floor of the denominator use the same one; the sequence here is one fixed
    // function of the block's gates and m0.
    float keep_j, take_j, floor_j, m_j;
    {
      const int jj = lane & (REC_BLOCK - 1);
      const float li_j = gates[jj][0], lf_j = gates[jj][1];
      float F = lf_j;
      F += row_shifted<1>(F, 0.f);
      F += row_shifted<2>(F, 0.f);
      F += row_shifted<4>(F, 0.f);
      F += row_shifted<8>(F, 0.f);
      float p = li_j - F;
      p = fmaxf(p, row_shifted<1>(p, -INFINITY));
      p = fmaxf(p, row_shifted<2>(p, -INFINITY));
      p = fmaxf(p, row_shifted<4>(p, -INFINITY));
      p = fmaxf(p, row_shifted<8>(p, -INFINITY));
      m_j = F + fmaxf(m, p);
      const float m_before = row_shifted<1>(m_j, m);      // the first token's: what the block starts from
      keep_j = expf(lf_j + m_before - m_j), take_j = expf(li_j - m_j), floor_j = expf(-m_j);
    }
    m = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(m_j), count - 1));
    float tops = 0.f;      // lane j of every row: its row's part of token j's S^T q
    auto token = [&](int j) {
      const float* row = rows + j * ROW;
      const float val = row[2 * DP + wave];
      const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(keep_j), j));
      const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(take_j), j));
      float num = 0.f, qq[Q];
#pragma unroll
      for (int i = 0; i < Q; ++i) {
        const float bk = b * row[DP + d0 + i];
        qq[i] = row[d0 + i];
        S[i] = fmaf(bk, val, a * S[i]);
        N[i] = fmaf(a, N[i], bk);
        num = fmaf(S[i], qq[i], num);
      }
      if (wave == j / PER_WAVE) {       // the whole wave or none of it
        float den = 0.f;
#pragma unroll
        for (int i = 0; i < Q; ++i) den = fmaf(N[i], qq[i], den);
        den = wave_total(den);
        if (lane == 0) dens[j] = den;
      }
      num = row_sum16(num);
      tops = (lane & (REC_BLOCK - 1)) == j ? num : tops;
    };
    if (count == REC_BLOCK) {      // a whole block: every lane index and LDS offset is a constant
#pragma unroll
      for (int j = 0; j < REC_BLOCK; ++j) token(j);
    } else {
      for (int j = 0; j < count; ++j) token(j);
    }
    // the four rows' parts: (row 0 + row 1) + (row 2 + row 3) in every row, whichever it is
    tops += __shfl_xor(tops, 16, 64);
    tops += __shfl_xor(tops, 32, 64);
    __syncthreads();     // every token's n . q is in LDS, and the block has been read
    if (live && lane < count)     // lane j < 16 also holds token j's floor; the division waits for the block's end
      out[((long long)(t0 + lane) * heads + h) * vdim + v] = tops / (fmaxf(fabsf(dens[lane]), floor_j) + 1e-6f);
  }
#pragma unroll
  for (int i = 0; i < Q; ++i)
    if (d0 + i < key_pad) {
      mine[i] = S[i];
      if (wave == 0) my_n[i] = N[i];
    }
  if (tid == 0) my_m[0] = m;
}

// x[t, c] = exp(-exp(x[t, c] + w0[c])) in place: time mixing's decay, for a step whose recurrence reads it many times.
__global__ void decay_kernel(float* __restrict__ x, const float* __restrict__ w0, int width, long long count) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) x[i] = expf(-expf(x[i] + w0[i % width]));
}

// out = tanh(x), elementwise, 32-bit in, TO out.
template <typename TO>
__global__ void tanh_kernel(const float* __restrict__ x, TO* __restrict__ out, long long count) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) out[i] = from_float<TO>(tanhf(x[i]));
}

// ---------------------------------------------------------------------------------------------

extern "C" int vk_delta_prepare_strided(const float* proj, long long ldp, const float* conv, int taps, float* state,
                                        long long state_stride, long long conv_offset, const int* entry_of,
                                        const int* entry_start, const int* entry_first, const int* slots,
                                        const float* a_log, const float* dt_bias, int kv_heads, int dim, int heads,
                                        int vdim, int b_col, int a_col, float unit_eps, float* qkv, long long ldq,
                                        float* beta, float* decay, int num_tokens, int num_entries, void* stream) {
  if (num_tokens <= 0) return 0;
  if (taps < 1 || kv_heads < 1 || heads < 1 || dim < 1 || vdim < 1 || heads % kv_heads) return VK_BAD_ARGUMENT;
  const long long C = 2LL * kv_heads * dim + (long long)heads * vdim;
  if (dim > PREP_SPAN || C > 0x7fffffff) return VK_UNSUPPORTED_SIZE;
  if (ldq < C || (a_col >= 0 && (!decay || !a_log || !dt_bias))) return VK_BAD_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  const long long segments = 2LL * kv_heads + ((long long)heads * vdim + PREP_SPAN - 1) / PREP_SPAN;
  if (segments > 65535) return VK_UNSUPPORTED_SIZE;
  delta_prepare_kernel<<<dim3(num_tokens, (unsigned)segments), 256, 0, s>>>(
      proj, ldp, conv, taps, state, state_stride, conv_offset, entry_of, entry_start, entry_first, slots, a_log, dt_bias,
      kv_heads, dim, heads, vdim, b_col, a_col, unit_eps, qkv, ldq, beta, decay);
  VK_LAUNCH_CHECK();
  if (taps > 1) {
    conv_state_kernel<<<dim3(num_entries, (unsigned)((C + 255) / 256)), 256, 0, s>>>(
        proj, ldp, taps, (int)C, state, state_stride, conv_offset, entry_start, entry_first, slots);
    VK_LAUNCH_CHECK();
  }
  return 0;
}

extern "C" int vk_delta_prepare(const float* proj, long long ldp, const float* conv, int taps, float* state,
                                long long state_stride, long long conv_offset, const int* entry_of,
                                const int* entry_start, const int* entry_first, const int* slots, const float* a_log,
                                const float* dt_bias, int kv_heads, int dim, int heads, int vdim, int b_col, int a_col,
                                float unit_eps, float* qkv, float* beta, float* decay, int num_tokens, int num_entries,
                                void* stream) {
  if (a_col < 0) return VK_BAD_ARGUMENT;
  return vk_delta_prepare_strided(proj, ldp, conv, taps, state, state_stride, conv_offset, entry_of, entry_start,
                                  entry_first, slots, a_log, dt_bias, kv_heads, dim, heads, vdim, b_col, a_col, unit_eps,
                                  qkv, 2LL * kv_heads * dim + (long long)heads * vdim, beta, decay, num_tokens,
                                  num_entries, stream);
}

// out[t, h * dim + d] = exp(-exp(a_log[h]) * softplus(raw[t, h * dim + d] + dt_bias[h * dim + d])): the delta rule's
// decay per head and key channel.  `raw` and `out` are 32-bit with row strides of their own.
__global__ void channel_decay_kernel(const float* __restrict__ raw, long long ldr, const float* __restrict__ a_log,
                                     const float* __restrict__ dt_bias, int dim, int width, long long total,
                                     float* __restrict__ out, long long ldo) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long t = idx / width;
  const int c = (int)(idx % width);
  out[t * ldo + c] = expf(-expf(a_log[c / dim]) * softplus_f(raw[t * ldr + c] + dt_bias[c]));
}

extern "C" int vk_channel_decay(const float* raw, long long ldr, const float* a_log, const float* dt_bias, int heads,
                                int dim, int num_tokens, float* out, long long ldo, void* stream) {
  if (num_tokens <= 0) return 0;
  if (heads < 1 || dim < 1) return VK_BAD_ARGUMENT;
  const int width = heads * dim;
  const long long total = (long long)num_tokens * width;
  channel_decay_kernel<<<(unsigned)((total + 255) / 256), 256, 0, (hipStream_t)stream>>>(raw, ldr, a_log, dt_bias, dim,
                                                                                        width, total, out, ldo);
  VK_LAUNCH_CHECK();
  return 0;
}

// Key channels a lane of the single-token form keeps: the state's key width is padded to 16 times this.
static inline int rows_of(int dim) { return dim <= 16 ? 1 : dim <= 32 ? 2 : dim <= 64 ? 4 : dim <= 128 ? 8 : 16; }

// Floats of one head's state as the recurrence kernels lay it out: [value channels padded to 16][key channels padded].
extern "C" long long vk_recurrent_head_floats(int dim, int vdim) {
  return (long long)((vdim + REC_COLS - 1) / REC_COLS) * REC_COLS * 16 * rows_of(dim);
}

// `g_col` >= 0: one decay per head and key channel, in columns g_col.. of the qkv rows ([heads, dim]; `decay` is not
// read); below 0: one decay per head, `decay` [T, heads].  `ldq` is the row stride of qkv.
extern "C" int vk_delta_rule_strided(const float* qkv, long long ldq, int g_col, const float* beta, const float* decay,
                                     float* state, long long state_stride, const int* entry_start,
                                     const int* entry_first, const int* slots, int kv_heads, int dim, int heads, int vdim,
                                     float* out, int num_entries, int short_entries, void* stream) {
  if (num_entries <= 0) return 0;
  if (kv_heads < 1 || heads < 1 || dim < 1 || vdim < 1 || heads % kv_heads) return VK_BAD_ARGUMENT;
  if (dim > 256 || heads > 65535) return VK_UNSUPPORTED_SIZE;
  const long long C = 2LL * kv_heads * dim + (long long)heads * vdim;
  if (ldq < C || (g_col < 0 && !decay) || (g_col >= 0 && g_col + (long long)heads * dim > ldq)) return VK_BAD_ARGUMENT;
  if (ldq >= (1 << 24)) return VK_UNSUPPORTED_SIZE;      // the prompt form keeps a column in 24 bits
  dim3 grid(num_entries, heads, (vdim + REC_COLS - 1) / REC_COLS);
  hipStream_t s = (hipStream_t)stream;
  const int key_pad = 16 * rows_of(dim), value_pad = (vdim + REC_COLS - 1) / REC_COLS * REC_COLS;
  const bool ch = g_col >= 0;
  if (!short_entries) {
    dim3 scan_grid(num_entries, heads, value_pad / SCAN_COLS);
#define VK_DELTA_SCAN(Q, CH)                                                                                         \
  delta_scan_kernel<Q, CH><<<scan_grid, SCAN_THREADS, 0, s>>>(qkv, ldq, g_col, beta, decay, state, state_stride,       \
                                                              entry_start, entry_first, slots, kv_heads, dim, heads,  \
                                                              vdim, key_pad, value_pad, out)
    if (key_pad <= 64) { if (ch) VK_DELTA_SCAN(1, true); else VK_DELTA_SCAN(1, false); }
    else if (key_pad <= 128) { if (ch) VK_DELTA_SCAN(2, true); else VK_DELTA_SCAN(2, false); }
    else { if (ch) VK_DELTA_SCAN(4, true); else VK_DELTA_SCAN(4, false); }
#undef VK_DELTA_SCAN
    VK_LAUNCH_CHECK();
    return 0;
  }
#define VK_DELTA(R)                                                                                                     \
  do {                                                                                                                  \
    if (ch)                                                                                                             \
      delta_rule_kernel<R, 1, true><<<grid, 256, 0, s>>>(qkv, ldq, g_col, beta, decay, state, state_stride, entry_start, \
                                                         entry_first, slots, kv_heads, dim, heads, vdim, out);          \
    else                                                                                                                \
      delta_rule_kernel<R, 1, false><<<grid, 256, 0, s>>>(qkv, ldq, g_col, beta, decay, state, state_stride,            \
                                                          entry_start, entry_first, slots, kv_heads, dim, heads, vdim,  \
                                                          out);                                                         \
  } while (0)
  if (dim <= 16) { VK_DELTA(1); }
  else if (dim <= 32) { VK_DELTA(2); }
  else if (dim <= 64) { VK_DELTA(4); }
  else if (dim <= 128) { VK_DELTA(8); }
  else { VK_DELTA(16); }
#undef VK_DELTA
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_delta_rule(const float* qkv, const float* beta, const float* decay, float* state,
                             long long state_stride, const int* entry_start, const int* entry_first, const int* slots,
                             int kv_heads, int dim, int heads, int vdim, float* out, int num_entries, int short_entries,
                             void* stream) {
  return vk_delta_rule_strided(qkv, 2LL * kv_heads * dim + (long long)heads * vdim, -1, beta, decay, state, state_stride,
                               entry_start, entry_first, slots, kv_heads, dim, heads, vdim, out, num_entries,
                               short_entries, stream);
}

// Floats of one request's matrix-memory state: the heads' matrices, then n and m per tile of eight value channels.
extern "C" long long vk_memory_state_floats(int heads, int dim, int vdim) {
  const long long tiles = (vdim + REC_COLS - 1) / REC_COLS * (REC_COLS / SCAN_COLS);
  return (long long)heads * (vk_recurrent_head_floats(dim, vdim) + tiles * 16 * rows_of(dim) + tiles);
}

// `proj` holds `num_tokens` rows.  Unless `short_entries` says that every entry is a single token, the gates' columns
// of `proj` are overwritten with their logarithms.
extern "C" int vk_memory_rule(float* proj, long long ldp, int num_tokens, int q_col, int k_col, int v_col, int i_col,
                              int f_col, float q_scale, float cap, float* state, long long state_stride,
                              const int* entry_start, const int* entry_first, const int* slots, int dim, int heads,
                              int vdim, float* out, int num_entries, int short_entries, void* stream) {
  if (num_entries <= 0 || num_tokens <= 0) return 0;
  if (heads < 1 || dim < 1 || vdim < 1 || !(cap > 0.f)) return VK_BAD_ARGUMENT;
  if (dim > 256 || heads > 65535 || ldp >= (1 << 24)) return VK_UNSUPPORTED_SIZE;
  if (min(min(q_col, k_col), min(v_col, min(i_col, f_col))) < 0) return VK_BAD_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  const int key_pad = 16 * rows_of(dim), value_pad = (vdim + REC_COLS - 1) / REC_COLS * REC_COLS;
  const long long tiles = value_pad / SCAN_COLS;
  const long long n_offset = (long long)heads * vk_recurrent_head_floats(dim, vdim);
  const long long m_offset = n_offset + (long long)heads * tiles * key_pad;
  const MemoryColumns col{q_col, k_col, v_col, i_col, f_col};
  if (!short_entries) {
    const long long gates = (long long)num_tokens * heads;
    memory_gates_kernel<<<(unsigned)((gates + 255) / 256), 256, 0, s>>>(proj, ldp, i_col, f_col, heads, cap, gates);
    dim3 scan_grid(num_entries, heads, (unsigned)tiles);
#define VK_MEMORY_SCAN(Q)                                                                                            \
  memory_scan_kernel<Q><<<scan_grid, SCAN_THREADS, 0, s>>>(proj, ldp, col, q_scale, state, state_stride, n_offset,     \
                                                           m_offset, entry_start, entry_first, slots, dim, heads, vdim, \
                                                           key_pad, value_pad, out)
    if (key_pad <= 64) VK_MEMORY_SCAN(1);
    else if (key_pad <= 128) VK_MEMORY_SCAN(2);
    else VK_MEMORY_SCAN(4);
#undef VK_MEMORY_SCAN
    VK_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid(num_entries, heads, value_pad / REC_COLS);
#define VK_MEMORY(R)                                                                                                  \
  memory_rule_kernel<R><<<grid, 256, 0, s>>>(proj, ldp, col, q_scale, cap, state, state_stride, n_offset, m_offset,   \
                                             entry_start, entry_first, slots, dim, heads, vdim, out)
  if (dim <= 16) { VK_MEMORY(1); }
  else if (dim <= 32) { VK_MEMORY(2); }
  else if (dim <= 64) { VK_MEMORY(4); }
  else if (dim <= 128) { VK_MEMORY(8); }
  else { VK_MEMORY(16); }
#undef VK_MEMORY
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_wkv_rule(const float* r, long long ldr, const float* k, long long ldk, const float* v, long long ldv,
                           const float* wraw, long long ldw, const float* w0, const float* bonus, float* state,
                           long long state_stride, const int* entry_start, const int* entry_first, const int* slots,
                           int dim, int heads, float* out, int num_entries, int short_entries, int decayed,
                           void* stream) {
  if (num_entries <= 0) return 0;
  if (heads < 1 || dim < 1) return VK_BAD_ARGUMENT;
  if (dim > 256 || heads > 65535) return VK_UNSUPPORTED_SIZE;
  dim3 grid(num_entries, heads, (dim + REC_COLS - 1) / REC_COLS);
  hipStream_t s = (hipStream_t)stream;
  const int key_pad = 16 * rows_of(dim), value_pad = (dim + REC_COLS - 1) / REC_COLS * REC_COLS;
  if (!short_entries) {
    dim3 scan_grid(num_entries, heads, value_pad / SCAN_COLS);
#define VK_WKV_SCAN(Q)                                                                                               \
  wkv_scan_kernel<Q><<<scan_grid, SCAN_THREADS, 0, s>>>(r, ldr, k, ldk, v, ldv, wraw, ldw, w0, bonus, state,          \
                                                        state_stride, entry_start, entry_first, slots, dim, heads,    \
                                                        key_pad, value_pad, decayed, out)
    if (key_pad <= 64) VK_WKV_SCAN(1);
    else if (key_pad <= 128) VK_WKV_SCAN(2);
    else VK_WKV_SCAN(4);
#undef VK_WKV_SCAN
    VK_LAUNCH_CHECK();
    return 0;
  }
#define VK_WKV(R)                                                                                                     \
  wkv_rule_kernel<R, 1><<<grid, 256, 0, s>>>(r, ldr, k, ldk, v, ldv, wraw, ldw, w0, bonus, state, state_stride,       \
                                             entry_start, entry_first, slots, dim, heads, decayed, out)
  if (dim <= 16) { VK_WKV(1); }
  else if (dim <= 32) { VK_WKV(2); }
  else if (dim <= 64) { VK_WKV(4); }
  else if (dim <= 128) { VK_WKV(8); }
  else { VK_WKV(16); }
#undef VK_WKV
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_token_shift(const void* h, int dtype, int width, const float* mu, int mixes, float* state,
                              long long state_stride, long long prev_offset, const int* entry_of,
                              const int* entry_start, const int* entry_first, const int* slots, int num_tokens,
                              int num_entries, void* out, void* stream) {
  if (num_tokens <= 0) return 0;
  if (width < 1 || mixes < 1) return VK_BAD_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  // a step of few tokens spreads a row over several workgroups; a prompt's many tokens fill the GPU by themselves
  const unsigned spans = num_tokens >= 512 ? 1u : (unsigned)min(64, (width + 255) / 256);
  const dim3 tokens_grid(num_tokens, spans), entries_grid(num_entries, spans);
  if (dtype == DT_F32) {
    token_shift_kernel<float><<<tokens_grid, 256, 0, s>>>((const float*)h, width, mu, mixes, state, state_stride,
                                                         prev_offset, entry_of, entry_start, entry_first, slots,
                                                         num_tokens, (float*)out);
    VK_LAUNCH_CHECK();
    save_last_kernel<float><<<entries_grid, 256, 0, s>>>((const float*)h, width, state, state_stride, prev_offset,
                                                        entry_start, slots);
  } else if (dtype == DT_BF16) {
    token_shift_kernel<bf16_t><<<tokens_grid, 256, 0, s>>>((const bf16_t*)h, width, mu, mixes, state, state_stride,
                                                          prev_offset, entry_of, entry_start, entry_first, slots,
                                                          num_tokens, (bf16_t*)out);
    VK_LAUNCH_CHECK();
    save_last_kernel<bf16_t><<<entries_grid, 256, 0, s>>>((const bf16_t*)h, width, state, state_stride, prev_offset,
                                                         entry_start, slots);
  } else {
    return VK_BAD_ARGUMENT;
  }
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_head_norm_gate(const float* o, const float* weight, int weight_per_head, const void* gate,
                                 int gate_dtype, long long ldg, int gate_silu, float eps, int heads, int vdim,
                                 int num_tokens, void* out, int out_dtype, void* stream) {
  if (num_tokens <= 0) return 0;
  if (heads < 1 || vdim < 1) return VK_BAD_ARGUMENT;
  const long long units = (long long)num_tokens * heads;
  const unsigned blocks = (unsigned)((units + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
#define VK_HNG(TG, TO)                                                                                         \
  head_norm_gate_kernel<TG, TO><<<blocks, 256, 0, s>>>(o, weight, weight_per_head, (const TG*)gate, ldg,      \
                                                       gate_silu, eps, heads, vdim, num_tokens, (TO*)out)
  if (gate_dtype == DT_F32 && out_dtype == DT_F32) VK_HNG(float, float);
  else if (gate_dtype == DT_F32 && out_dtype == DT_BF16) VK_HNG(float, bf16_t);
  else if (gate_dtype == DT_BF16 && out_dtype == DT_BF16) VK_HNG(bf16_t, bf16_t);
  else if (gate_dtype == DT_BF16 && out_dtype == DT_F32) VK_HNG(bf16_t, float);
  else return VK_BAD_ARGUMENT;
#undef VK_HNG
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_decay(float* x, const float* w0, int width, long long count, void* stream) {
  if (count <= 0) return 0;
  if (width < 1) return VK_BAD_ARGUMENT;
  decay_kernel<<<(unsigned)((count + 255) / 256), 256, 0, (hipStream_t)stream>>>(x, w0, width, count);
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_tanh(const float* x, void* out, int out_dtype, long long count, void* stream) {
  if (count <= 0) return 0;
  const unsigned blocks = (unsigned)((count + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == DT_F32) tanh_kernel<float><<<blocks, 256, 0, s>>>(x, (float*)out, count);
  else if (out_dtype == DT_BF16) tanh_kernel<bf16_t><<<blocks, 256, 0, s>>>(x, (bf16_t*)out, count);
  else return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}
