// Gated delta rule: a recurrent mixer whose state is one matrix S [D, Dv] per head and request.
//
//   S <- diag(g_t) S            (g_t one number per head, or one per key channel = row of S)
//   u_t = beta_t (v_t - S^T k_t)
//   S <- S + k_t u_t^T
//   o_t = S^T q_t               (the read-out sees the token's own write)
//
// Three kernels: (1) the short causal convolution over time of the q | k | v channels with silu,
// and the scaling of every query and key head to a unit vector; (2) the recurrence itself;
// (3) the per-head RMS norm of the read-out times a gate. State, decays, step sizes, unit norms and
// the read-out are float32 in every mode. A request's state lives in its slot: S transposed,
// [heads, Dv, D], and the last taps - 1 inputs of every convolved channel.
#include "common.h"
#include <math.h>

#define DELTA_MAX_TAPS 16

__device__ __forceinline__ float load_code(const void* p, int code, size_t i) {
  return code == QRT_F32 ? ((const float*)p)[i] : (float)((const bf16_t*)p)[i];
}

// ------------------------------------------------- convolution, silu, unit vectors
// Channels are the columns [0, C) of x (row stride x_stride), cut into heads: `nseg` segments, each
// `heads` heads of `width` channels, with `mode` 0 (convolved and activated only), 1 (then scaled
// to a unit vector per head) or 2 (unit vector times width^(-1/2)). One wave per (token, head).
// Token i of its span reads the inputs i-K+1 .. i; those before the span come from the slot's
// tail [C, K-1] (oldest first), which holds zeros at the start of a sequence.
struct ConvArgs {
  const void* x; long x_stride;
  const float* taps;        // [C, K], the last column multiplies the current token
  const float* tail;        // [slots, C, K-1]
  const int* cu_q; const int* seq_of_token; const int* state_slots;
  float* out;               // [T, C] float32
  int num_tokens, channels, num_taps, nseg;
  int seg_first[4], seg_heads[4], seg_width[4], seg_mode[4];
  int total_heads;
  float unit_eps;
  // every span is one token (a decode step): the wave that reads a channel's tail also moves it on,
  // and no second kernel runs
  int fuse_tail;
};

template <typename T>
__global__ __launch_bounds__(256) void conv_unit_kernel(ConvArgs a) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long)a.num_tokens * a.total_heads) return;
  const int t = (int)(item / a.total_heads);
  int h = (int)(item - (long)t * a.total_heads);
  int seg = 0;
  while (seg + 1 < a.nseg && h >= a.seg_heads[seg]) { h -= a.seg_heads[seg]; ++seg; }
  const int width = a.seg_width[seg], mode = a.seg_mode[seg];
  const int c0 = a.seg_first[seg] + h * width;
  const int s = a.seq_of_token[t];
  const int i = t - a.cu_q[s];            // place within the span
  const int K = a.num_taps;
  float* tail = (float*)a.tail + (size_t)a.state_slots[s] * a.channels * (K - 1);
  const T* x = (const T*)a.x;
  float ss = 0.f;
  float y[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    y[r] = 0.f;
    const int c = c0 + lane + 64 * r;
    if (lane + 64 * r < width) {
      float acc = 0.f;
      for (int j = 0; j < K; ++j) {
        const int back = K - 1 - j;        // this tap reads the token `back` places earlier
        const float in = back <= i ? to_f32<T>(x[(size_t)(t - back) * a.x_stride + c])
                                   : tail[(size_t)c * (K - 1) + (i + j)];
        acc = fmaf(a.taps[(size_t)c * K + j], in, acc);
        if (a.fuse_tail && j >= 1) tail[(size_t)c * (K - 1) + (j - 1)] = in;  // i is 0: the inputs were tail[0..K-2], x
      }
      y[r] = acc / (1.0f + expf(-acc));
      ss += y[r] * y[r];
    }
  }
  float mul = 1.f;
  if (mode) {
    ss = wave_sum(ss);
    mul = 1.0f / sqrtf(ss + a.unit_eps);
    if (mode == 2) mul *= 1.0f / sqrtf((float)width);
  }
#pragma unroll
  for (int r = 0; r < 8; ++r)
    if (lane + 64 * r < width) a.out[(size_t)t * a.channels + c0 + lane + 64 * r] = y[r] * mul;
}

// The same for steps of many tokens, K <= 4 taps and heads of at most 128 channels: a wave takes
// eight consecutive tokens of one head, loads the 8 + K - 1 rows of inputs they read once (a
// window in registers; the taps once), and computes the eight outputs from it. A token near the
// start of its span reads the slot's tail instead of the rows before it, which belong to another
// sequence of the batch.
#define CONV_TILE 8
template <typename T, int K>
__global__ __launch_bounds__(256) void conv_unit_tile_kernel(ConvArgs a) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int tiles = (a.num_tokens + CONV_TILE - 1) / CONV_TILE;
  if (item >= (long)tiles * a.total_heads) return;
  const int tile = (int)(item / a.total_heads);
  int h = (int)(item - (long)tile * a.total_heads);
  int seg = 0;
  while (seg + 1 < a.nseg && h >= a.seg_heads[seg]) { h -= a.seg_heads[seg]; ++seg; }
  const int width = a.seg_width[seg], mode = a.seg_mode[seg];
  const int c0 = a.seg_first[seg] + h * width;
  const int t0 = tile * CONV_TILE, nt = min(CONV_TILE, a.num_tokens - t0);
  const T* x = (const T*)a.x;
  float w[2][K], xw[2][CONV_TILE + K - 1], y[2][CONV_TILE];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const bool on = lane + 64 * r < width;
    const int c = c0 + (on ? lane + 64 * r : 0);
#pragma unroll
    for (int j = 0; j < K; ++j) w[r][j] = a.taps[(size_t)c * K + j];
#pragma unroll
    for (int j = 0; j < CONV_TILE + K - 1; ++j) {
      const int row = t0 - (K - 1) + j;
      const int at = min(max(row, 0), a.num_tokens - 1);
      const float v = to_f32<T>(x[(size_t)at * a.x_stride + c]);
      xw[r][j] = (on && row >= 0 && row < a.num_tokens) ? v : 0.f;
    }
  }
  float ss[CONV_TILE];
#pragma unroll
  for (int tt = 0; tt < CONV_TILE; ++tt) {
    ss[tt] = 0.f;
    const int t = min(t0 + tt, a.num_tokens - 1);
    const int s = a.seq_of_token[t];
    const int i = t - a.cu_q[s];
    const float* tail = a.tail + (size_t)a.state_slots[s] * a.channels * (K - 1);
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < K; ++j) {
        float in = xw[r][tt + j];
        if (K - 1 - j > i) in = (lane + 64 * r < width) ? tail[(size_t)(c0 + lane + 64 * r) * (K - 1) + (i + j)] : 0.f;
        acc = fmaf(w[r][j], in, acc);
      }
      y[r][tt] = acc / (1.0f + __expf(-acc));
      ss[tt] += y[r][tt] * y[r][tt];
    }
  }
  if (mode) {
#pragma unroll
    for (int tt = 0; tt < CONV_TILE; ++tt) {
      const float total = wave_sum(ss[tt]);
      ss[tt] = 1.0f / sqrtf(total + a.unit_eps);
      if (mode == 2) ss[tt] *= 1.0f / sqrtf((float)width);
    }
  }
#pragma unroll
  for (int tt = 0; tt < CONV_TILE; ++tt) {
    if (tt < nt) {
#pragma unroll
      for (int r = 0; r < 2; ++r)
        if (lane + 64 * r < width)
          a.out[(size_t)(t0 + tt) * a.channels + c0 + lane + 64 * r] = mode ? y[r][tt] * ss[tt] : y[r][tt];
    }
  }
}

template <typename T>
static void conv_launch(const ConvArgs& a, bool tiled, hipStream_t stream) {
  if (tiled) {
    const long items = (long)((a.num_tokens + CONV_TILE - 1) / CONV_TILE) * a.total_heads;
    dim3 grid((unsigned)((items + 3) / 4)), block(256);
    switch (a.num_taps) {
      case 1: conv_unit_tile_kernel<T, 1><<<grid, block, 0, stream>>>(a); break;
      case 2: conv_unit_tile_kernel<T, 2><<<grid, block, 0, stream>>>(a); break;
      case 3: conv_unit_tile_kernel<T, 3><<<grid, block, 0, stream>>>(a); break;
      default: conv_unit_tile_kernel<T, 4><<<grid, block, 0, stream>>>(a); break;
    }
  } else {
    const long items = (long)a.num_tokens * a.total_heads;
    dim3 grid((unsigned)((items + 3) / 4)), block(256);
    conv_unit_kernel<T><<<grid, block, 0, stream>>>(a);
  }
}

// After the convolution has read them: the tail of every (sequence, channel) becomes the last
// K-1 inputs, those of the step where it brought enough tokens, older ones from the old tail.
template <typename T>
__global__ void conv_tail_kernel(const T* __restrict__ x, long x_stride, float* __restrict__ tail_all,
                                 const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                                 int channels, int K) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = cu_q[s], n = cu_q[s + 1] - first;
  float* tail = tail_all + ((size_t)state_slots[s] * channels + c) * (K - 1);
  float keep[DELTA_MAX_TAPS];
  for (int r = 0; r < K - 1; ++r) {
    const int idx = n - (K - 1) + r;     // place within the span, negative: before it
    keep[r] = idx >= 0 ? to_f32<T>(x[(size_t)(first + idx) * x_stride + c]) : tail[r + n];
  }
  for (int r = 0; r < K - 1; ++r) tail[r] = keep[r];
}

extern "C" int qrt_delta_conv(const ConvArgs* args, int dtype, int num_seqs, int num_slots, int max_span,
                              hipStream_t stream) {
  ConvArgs a = *args;
  a.fuse_tail = max_span == 1 && a.num_tokens == num_seqs;
  QRT_CHECK(a.num_tokens >= 0 && a.channels > 0 && a.nseg >= 1 && a.nseg <= 4, "delta_conv: bad sizes");
  QRT_CHECK(a.num_taps >= 1 && a.num_taps <= DELTA_MAX_TAPS, "delta_conv: %d taps (1 to %d)", a.num_taps, DELTA_MAX_TAPS);
  QRT_CHECK(a.x_stride >= a.channels && num_seqs >= 0 && num_slots > 0, "delta_conv: row stride %ld under %d channels", a.x_stride, a.channels);
  int covered = 0;
  a.total_heads = 0;
  for (int g = 0; g < a.nseg; ++g) {
    QRT_CHECK(a.seg_first[g] == covered && a.seg_heads[g] > 0 && a.seg_width[g] > 0 && a.seg_width[g] <= 512,
              "delta_conv: segment %d does not follow the one before, or its heads are wider than 512", g);
    covered += a.seg_heads[g] * a.seg_width[g];
    a.total_heads += a.seg_heads[g];
  }
  QRT_CHECK(covered == a.channels, "delta_conv: segments cover %d of %d channels", covered, a.channels);
  if (a.num_tokens == 0) return 0;
  bool tiled = a.num_tokens >= 64 && a.num_taps <= 4 && !a.fuse_tail;
  for (int g = 0; g < a.nseg; ++g) tiled = tiled && a.seg_width[g] <= 128;
  dim3 tgrid((a.channels + 255) / 256, num_seqs);
  if (dtype == QRT_F32) {
    conv_launch<float>(a, tiled, stream);
    if (a.num_taps > 1 && !a.fuse_tail)
      conv_tail_kernel<float><<<tgrid, 256, 0, stream>>>((const float*)a.x, a.x_stride, (float*)a.tail, a.cu_q,
                                                        a.state_slots, a.channels, a.num_taps);
  } else if (dtype == QRT_BF16) {
    conv_launch<bf16_t>(a, tiled, stream);
    if (a.num_taps > 1 && !a.fuse_tail)
      conv_tail_kernel<bf16_t><<<tgrid, 256, 0, stream>>>((const bf16_t*)a.x, a.x_stride, (float*)a.tail, a.cu_q,
                                                         a.state_slots, a.channels, a.num_taps);
  } else return qrt_fail("delta_conv: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("delta_conv");
  return 0;
}

// ------------------------------------------------------------------ the recurrence
// A block of 256 threads owns 16 (or 32) value channels (columns of S) of one head of one sequence
// and walks the span's tokens in order. A column is shared by L = 16 (or 8) neighbouring lanes:
// lane l holds the rows 4l .. 4l+3, 4L + 4l .. 4L + 4l+3, ... (four neighbours at a time: one
// 16-byte access to memory or LDS) in registers, so the two sums over rows that a token
// needs, S^T k and S^T q, are sums inside a row of lanes (four or three DPP steps each, no LDS),
// and they run side by side: the read-out is taken from the decayed state, before the write, and
// completed by (k . q) u, which is the write's share of it.
// Tokens are staged through LDS 16 at a time, in two buffers: while the block walks one tile its
// threads hold the next tile's keys, queries, decay logits, values and step-size logits in
// registers, asked for before the walk began, and put them into the other buffer afterwards;
// so the walk never waits for memory. Decays exp(-exp(A) softplus(a + bias)) and step sizes
// sigmoid(b) are formed on the way into LDS, in float32, and k . q per token after it.
struct RuleArgs {
  const float* qkv;         // [T, C] float32: q heads | k heads | v heads, as delta_conv leaves them
  int channels, q_first, k_first, v_first;
  const void* b; long b_stride; int b_code;    // [T, heads] step-size logits
  const void* a; long a_stride; int a_code;    // [T, heads] or [T, heads * D] decay logits
  const float* a_log;       // [heads]
  const float* dt_bias;     // [heads] or [heads * D]
  float* state;             // [slots, heads, Dv, D]
  float* out;               // [T, heads, Dv] float32
  const int* cu_q; const int* state_slots;
  int heads, kv_heads, dim, vdim, per_channel;
};

// exp(-rate * softplus(logit)), float32 with the hardware's exponential and logarithm: the
// softplus is good to 1e-7 absolute, which is what the decay's exponent needs
__device__ __forceinline__ float decay_of(float logit, float rate) {
  const float sp = logit > 15.f ? logit : __logf(1.0f + __expf(logit));
  return __expf(-rate * sp);
}

// L lanes share a column (16 or 8); RULE_TOKENS tokens a tile (fewer for the widest heads, whose
// two buffers would not fit 64 KB otherwise).
template <int L>
__device__ __forceinline__ float lanes_sum(float x) {
  int v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true));  // row_half_mirror
  if (L == 16) {
    v = __builtin_bit_cast(int, x);
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true));  // row_mirror
  }
  return x;
}

template <int G, bool PER_CHANNEL, int RULE_TOKENS, int L>
__global__ __launch_bounds__(256) void delta_rule_kernel(RuleArgs a) {
  constexpr int COLS = 256 / L;         // columns of S a block owns
  constexpr int RR = 4 * G;             // rows a lane holds: G groups of four neighbours
  constexpr int DP = 4 * L * G;         // rows staged, the head's D padded with zero rows
  constexpr int PER = (DP * RULE_TOKENS + 255) / 256;   // staged elements a thread fetches per tile and array
  constexpr int PERV = (RULE_TOKENS * COLS + 255) / 256;
  constexpr int TILE = RULE_TOKENS * DP * (PER_CHANNEL ? 3 : 2) + (PER_CHANNEL ? 0 : RULE_TOKENS) + 2 * RULE_TOKENS * COLS +
                       2 * RULE_TOKENS;
  static_assert(TILE % 4 == 0 && RULE_TOKENS <= 256 / L, "tile shape");
  extern __shared__ __align__(16) float lds[];
  const int tid = threadIdx.x, l = tid & (L - 1), col = tid / L;
  const int head = blockIdx.y, s = blockIdx.z;
  const int kvh = head / (a.heads / a.kv_heads);
  const int c = blockIdx.x * COLS + col;
  const bool live = c < a.vdim;
  const int t0 = a.cu_q[s], t1 = a.cu_q[s + 1];
  const int D = a.dim;
  float* st = a.state + (((size_t)a.state_slots[s] * a.heads + head) * a.vdim + (live ? c : 0)) * D;
  const bool wide = D % 4 == 0;
  float S[RR];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int row = 4 * L * g + 4 * l;
    if (live && wide && row < D) {
      const f32x4_t v = *(const f32x4_t*)(st + row);
#pragma unroll
      for (int e = 0; e < 4; ++e) S[4 * g + e] = v[e];
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) S[4 * g + e] = (live && row + e < D) ? st[row + e] : 0.f;
    }
  }
  const float rate = __expf(a.a_log[head]);
  // what a thread fetches for a tile: element tid + 256 j of [token][row] for k, q (and the decay
  // logits), its share of the values, and (the first threads) a token's step-size and per-head decay logit
  float fk[PER], fq[PER], fa[PER], fv[PERV], fb, fg;
  auto fetch = [&](int base) {
    const int n = min(RULE_TOKENS, t1 - base);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = tid + 256 * j, tok = idx / DP, row = idx - tok * DP;
      const bool in = tok < n && row < D;
      const size_t at = (size_t)(base + (in ? tok : 0)) * a.channels + kvh * D + (in ? row : 0);
      fk[j] = a.qkv[at + a.k_first];
      fq[j] = a.qkv[at + a.q_first];
      if (PER_CHANNEL) {
        const size_t ai = (size_t)(base + (in ? tok : 0)) * a.a_stride + head * D + (in ? row : 0);
        fa[j] = (a.a_code == QRT_F32 ? ((const float*)a.a)[ai] : (float)((const bf16_t*)a.a)[ai]) +
                a.dt_bias[head * D + (in ? row : 0)];
      }
      if (!in) fk[j] = fq[j] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < PERV; ++j) {
      const int idx = tid + 256 * j, tok = idx / COLS, cc = blockIdx.x * COLS + (idx - tok * COLS);
      const bool in = tok < n && cc < a.vdim;
      fv[j] = a.qkv[(size_t)(base + (in ? tok : 0)) * a.channels + a.v_first + head * a.vdim + (in ? cc : 0)];
      if (!in) fv[j] = 0.f;
    }
    fb = fg = 0.f;
    if (tid < n) {
      fb = load_code(a.b, a.b_code, (size_t)(base + tid) * a.b_stride + head);
      if (!PER_CHANNEL) fg = load_code(a.a, a.a_code, (size_t)(base + tid) * a.a_stride + head) + a.dt_bias[head];
    }
  };
  auto put = [&](float* buf, int base) {
    const int n = min(RULE_TOKENS, t1 - base);
    float* ks = buf;
    float* qs = ks + RULE_TOKENS * DP;
    float* gs = qs + RULE_TOKENS * DP;
    float* vs = gs + (PER_CHANNEL ? RULE_TOKENS * DP : RULE_TOKENS);
    float* bs = vs + RULE_TOKENS * COLS;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = tid + 256 * j, tok = idx / DP, row = idx - tok * DP;
      if (idx < RULE_TOKENS * DP) {
        ks[idx] = fk[j];
        qs[idx] = fq[j];
        if (PER_CHANNEL) gs[idx] = (tok < n && row < D) ? decay_of(fa[j], rate) : 1.f;
      }
    }
#pragma unroll
    for (int j = 0; j < PERV; ++j)
      if (tid + 256 * j < RULE_TOKENS * COLS) vs[tid + 256 * j] = fv[j];
    if (tid < RULE_TOKENS) {
      bs[tid] = tid < n ? 1.0f / (1.0f + __expf(-fb)) : 0.f;
      if (!PER_CHANNEL) gs[tid] = tid < n ? decay_of(fg, rate) : 1.f;
    }
  };
  if (t0 < t1) {
    fetch(t0);
    put(lds, t0);
  }
  int which = 0;
  for (int base = t0; base < t1; base += RULE_TOKENS, which ^= 1) {
    const int n = min(RULE_TOKENS, t1 - base);
    float* buf = lds + which * TILE;
    const float* ks = buf;
    const float* qs = ks + RULE_TOKENS * DP;
    const float* gs = qs + RULE_TOKENS * DP;
    const float* vs = gs + (PER_CHANNEL ? RULE_TOKENS * DP : RULE_TOKENS);
    const float* bs = vs + RULE_TOKENS * COLS;
    float* kqs = buf + TILE - RULE_TOKENS;
    // The read-outs of the tile wait in LDS and leave after the walk, a row of columns at a time:
    // a store to memory inside the walk would have every token wait for the memory system.
    float* os = buf + TILE - RULE_TOKENS - RULE_TOKENS * COLS;
    const bool more = base + RULE_TOKENS < t1;
    if (more) fetch(base + RULE_TOKENS);  // on its way while this tile is walked
    __syncthreads();                      // this tile is in LDS
    {  // k . q of every token of the tile: the lanes of group `col` take token `col`
      float p = 0.f;
      const int mine = col < RULE_TOKENS ? col : 0;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const f32x4_t kv = *(const f32x4_t*)(ks + mine * DP + 4 * L * g + 4 * l);
        const f32x4_t qv = *(const f32x4_t*)(qs + mine * DP + 4 * L * g + 4 * l);
#pragma unroll
        for (int e = 0; e < 4; ++e) p = fmaf(kv[e], qv[e], p);
      }
      p = lanes_sum<L>(p);
      if (l == 0 && col < RULE_TOKENS) kqs[col] = p;
    }
    __syncthreads();
    // One token: decay, the two sums over rows, the write, the read-out (returned).
    auto step = [&](int tok) -> float {
      float pk[4] = {0.f, 0.f, 0.f, 0.f}, pq[4] = {0.f, 0.f, 0.f, 0.f};
      f32x4_t kr[G];
      const float gh = PER_CHANNEL ? 1.f : gs[tok];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        kr[g] = *(const f32x4_t*)(ks + tok * DP + 4 * L * g + 4 * l);
        const f32x4_t qv = *(const f32x4_t*)(qs + tok * DP + 4 * L * g + 4 * l);
        f32x4_t gv = {gh, gh, gh, gh};
        if (PER_CHANNEL) gv = *(const f32x4_t*)(gs + tok * DP + 4 * L * g + 4 * l);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = 4 * g + e;
          S[r] *= gv[e];
          pk[e] = fmaf(S[r], kr[g][e], pk[e]);
          pq[e] = fmaf(S[r], qv[e], pq[e]);
        }
      }
      const float sk = lanes_sum<L>((pk[0] + pk[1]) + (pk[2] + pk[3]));
      const float sq = lanes_sum<L>((pq[0] + pq[1]) + (pq[2] + pq[3]));
      const float u = bs[tok] * (vs[tok * COLS + col] - sk);
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) S[4 * g + e] = fmaf(kr[g][e], u, S[4 * g + e]);
      return fmaf(kqs[tok], u, sq);
    };
    if (n == RULE_TOKENS) {
      // A full tile: no branch and no store between the tokens, so that the LDS reads of the tokens
      // to come are asked for while one is worked on; the read-outs wait in registers.
      float keep[RULE_TOKENS];
#pragma unroll
      for (int tok = 0; tok < RULE_TOKENS; ++tok) keep[tok] = step(tok);
      if (l == 0) {
#pragma unroll
        for (int tok = 0; tok < RULE_TOKENS; ++tok) os[tok * COLS + col] = keep[tok];
      }
    } else {
      for (int tok = 0; tok < n; ++tok) {
        const float o = step(tok);
        if (l == 0) os[tok * COLS + col] = o;
      }
    }
    __syncthreads();
    for (int idx = tid; idx < n * COLS; idx += 256) {
      const int tok = idx / COLS, cc = blockIdx.x * COLS + (idx - tok * COLS);
      if (cc < a.vdim) a.out[((size_t)(base + tok) * a.heads + head) * a.vdim + cc] = os[idx];
    }
    if (more) put(lds + (which ^ 1) * TILE, base + RULE_TOKENS);  // nobody reads that buffer now
  }
  if (live) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int row = 4 * L * g + 4 * l;
      if (wide && row < D) {
        f32x4_t v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = S[4 * g + e];
        *(f32x4_t*)(st + row) = v;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (row + e < D) st[row + e] = S[4 * g + e];
      }
    }
  }
}

// lanes a column: -1 lets the launch choose
static int g_rule_lanes = -1;
extern "C" void qrt_delta_rule_lanes(int lanes) { g_rule_lanes = lanes; }

extern "C" int qrt_delta_rule(const RuleArgs* args, int num_tokens, int num_seqs, int max_span, hipStream_t stream) {
  RuleArgs a = *args;
  QRT_CHECK(a.heads > 0 && a.kv_heads > 0 && a.heads % a.kv_heads == 0, "delta_rule: %d heads on %d key heads", a.heads, a.kv_heads);
  QRT_CHECK(a.dim >= 1 && a.dim <= 512 && a.vdim >= 1, "delta_rule: key size %d (1 to 512), value size %d", a.dim, a.vdim);
  QRT_CHECK(num_tokens >= 0 && num_seqs >= 0 && num_seqs <= 65535 && a.heads <= 65535, "delta_rule: bad counts");
  QRT_CHECK((uintptr_t)a.state % 16 == 0, "delta_rule: the state is not aligned to 16 bytes");
  if (num_tokens == 0 || num_seqs == 0) return 0;
  // Eight lanes a column shorten the sums across lanes and halve the blocks; sixteen keep a block's
  // chain of tokens shorter, which is what a launch of few blocks waits for. Measured at 32 heads of
  // 128 x 128: one 2,048-token prompt 478 us with sixteen lanes against 645 with eight; eight
  // sequences of 256 tokens 216 against 187; 64 single tokens 57 against 53. Eight from four blocks
  // a compute unit on, and never where a lane would hold more than 16 rows.
  int L = g_rule_lanes;
  if (L != 8 && L != 16) L = ((long)num_seqs * a.heads * ((a.vdim + 31) / 32) >= 1024 && a.dim <= 128) ? 8 : 16;
  if (a.dim > 128) L = 16;
  const int G = (a.dim + 4 * L - 1) / (4 * L), DP = 4 * L * G, cols = 256 / L;
  // Spans of a few tokens (decoding) take tiles of four: a quarter of the LDS, so that four times as
  // many blocks fit a compute unit, and what such a launch waits for is the states' trip from memory.
  const bool few = max_span > 0 && max_span <= 4;
  const int tokens = (few || DP > 256) ? 4 : DP <= 128 ? 16 : 8;
  dim3 grid((a.vdim + cols - 1) / cols, a.heads, num_seqs), block(256);
  const size_t tile = (size_t)tokens * DP * (a.per_channel ? 3 : 2) + (a.per_channel ? 0 : tokens) + 2 * tokens * cols + 2 * tokens;
  const size_t smem = sizeof(float) * 2 * tile;
  QRT_CHECK(smem <= 64 * 1024, "delta_rule: %zu bytes of LDS", smem);
#define GO(GG, TT, LL)                                                                          \
  do {                                                                                          \
    if (a.per_channel) delta_rule_kernel<GG, true, TT, LL><<<grid, block, smem, stream>>>(a);   \
    else delta_rule_kernel<GG, false, TT, LL><<<grid, block, smem, stream>>>(a);                \
  } while (0)
  QRT_CHECK(G <= 8, "delta_rule: %d groups of rows a lane", G);
  if (L == 16 && G > 4) {  // heads of more than 256 rows: four-token tiles whatever the step
    switch (G) {
      case 5: GO(5, 4, 16); break;
      case 6: GO(6, 4, 16); break;
      case 7: GO(7, 4, 16); break;
      default: GO(8, 4, 16); break;
    }
  } else if (few && L == 16) {
    switch (G) {
      case 1: GO(1, 4, 16); break;
      case 2: GO(2, 4, 16); break;
      case 3: GO(3, 4, 16); break;
      default: GO(4, 4, 16); break;
    }
  } else if (few) {
    switch (G) {
      case 1: GO(1, 4, 8); break;
      case 2: GO(2, 4, 8); break;
      case 3: GO(3, 4, 8); break;
      default: GO(4, 4, 8); break;
    }
  } else if (L == 16) {
    switch (G) {
      case 1: GO(1, 16, 16); break;
      case 2: GO(2, 16, 16); break;
      case 3: GO(3, 8, 16); break;
      default: GO(4, 8, 16); break;
    }
  } else {
    switch (G) {
      case 1: GO(1, 16, 8); break;
      case 2: GO(2, 16, 8); break;
      case 3: GO(3, 16, 8); break;
      default: GO(4, 16, 8); break;
    }
  }
#undef GO
  QRT_LAUNCH_CHECK("delta_rule");
  return 0;
}

// ------------------------------------------------------- read-out: norm and gate
// out[t, h, :] = o[t, h, :] / sqrt(mean(o^2) + eps) * weight * act(gate[t, h, :]),
// act = silu (kind 0) or sigmoid (kind 1); one wave per (token, head).
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void delta_out_kernel(const float* __restrict__ o, const float* __restrict__ weight,
                                                        const TG* __restrict__ gate, long gate_stride, TO* __restrict__ out,
                                                        long items, int heads, int vdim, float eps, int kind) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const long t = item / heads;
  const int h = (int)(item - t * heads);
  const float* row = o + (size_t)item * vdim;
  float ss = 0.f;
  for (int c = lane; c < vdim; c += 64) ss += row[c] * row[c];
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
  for (int c = lane; c < vdim; c += 64) {
    const float z = to_f32<TG>(gate[(size_t)t * gate_stride + (size_t)h * vdim + c]);
    const float sg = 1.0f / (1.0f + expf(-z));
    out[(size_t)item * vdim + c] = from_f32<TO>(row[c] * inv * weight[c] * (kind == 0 ? z * sg : sg));
  }
}

extern "C" int qrt_delta_out(const float* o, const float* weight, const void* gate, long gate_stride, int gate_dtype,
                             void* out, int out_dtype, int num_tokens, int heads, int vdim, float eps, int kind,
                             hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && heads > 0 && vdim > 0 && gate_stride >= (long)heads * vdim, "delta_out: bad sizes");
  QRT_CHECK(kind == 0 || kind == 1, "delta_out: unknown gate %d", kind);
  if (num_tokens == 0) return 0;
  const long items = (long)num_tokens * heads;
  dim3 grid((unsigned)((items + 3) / 4)), block(256);
#define GO(TG, TO) delta_out_kernel<TG, TO><<<grid, block, 0, stream>>>(o, weight, (const TG*)gate, gate_stride, (TO*)out, \
                                                                        items, heads, vdim, eps, kind)
  if (gate_dtype == QRT_F32 && out_dtype == QRT_F32) GO(float, float);
  else if (gate_dtype == QRT_BF16 && out_dtype == QRT_BF16) GO(bf16_t, bf16_t);
  else if (gate_dtype == QRT_F32 && out_dtype == QRT_BF16) GO(float, bf16_t);
  else return qrt_fail("delta_out: unknown dtypes %d %d", gate_dtype, out_dtype);
#undef GO
  QRT_LAUNCH_CHECK("delta_out");
  return 0;
}
