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
  const float* tail = a.tail + (size_t)a.state_slots[s] * a.channels * (K - 1);
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

extern "C" int qrt_delta_conv(const ConvArgs* args, int dtype, int num_seqs, int num_slots, hipStream_t stream) {
  ConvArgs a = *args;
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
  const long items = (long)a.num_tokens * a.total_heads;
  dim3 grid((unsigned)((items + 3) / 4)), block(256);
  dim3 tgrid((a.channels + 255) / 256, num_seqs);
  if (dtype == QRT_F32) {
    conv_unit_kernel<float><<<grid, block, 0, stream>>>(a);
    if (a.num_taps > 1)
      conv_tail_kernel<float><<<tgrid, 256, 0, stream>>>((const float*)a.x, a.x_stride, (float*)a.tail, a.cu_q,
                                                        a.state_slots, a.channels, a.num_taps);
  } else if (dtype == QRT_BF16) {
    conv_unit_kernel<bf16_t><<<grid, block, 0, stream>>>(a);
    if (a.num_taps > 1)
      conv_tail_kernel<bf16_t><<<tgrid, 256, 0, stream>>>((const bf16_t*)a.x, a.x_stride, (float*)a.tail, a.cu_q,
                                                         a.state_slots, a.channels, a.num_taps);
  } else return qrt_fail("delta_conv: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("delta_conv");
  return 0;
}

// ------------------------------------------------------------------ the recurrence
// A block of 256 threads owns 16 value channels (columns of S) of one head of one sequence and
// walks the span's tokens in order. A column is shared by 16 neighbouring lanes: lane l holds
// the rows l, l + 16, ... (R of them) in registers, so the two sums over rows that a token
// needs, S^T k and S^T q, are sums inside a row of 16 lanes (four DPP steps each, no LDS), and
// they run side by side: the read-out is taken from the decayed state, before the write, and
// completed by (k . q) u, which is the write's share of it.
// Tokens are staged through LDS 16 at a time: keys, queries, per-row decays, values, step
// sizes, and k . q; decays exp(-exp(A) softplus(a + bias)) and step sizes sigmoid(b) are formed
// there, in float32, from the projections' outputs.
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

__device__ __forceinline__ float row16_sum(float x) {
  // all 16 lanes of a DPP row get the row's sum: two swaps inside quads, then the mirrors
  int v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true));  // row_half_mirror
  v = __builtin_bit_cast(int, x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true));  // row_mirror
  return x;
}

__device__ __forceinline__ float decay_of(float logit, float rate) {
  const float sp = logit > 20.f ? logit : log1pf(expf(logit));
  return expf(-rate * sp);
}

#define RULE_TOKENS 16
template <int R, bool PER_CHANNEL>
__global__ __launch_bounds__(256) void delta_rule_kernel(RuleArgs a) {
  constexpr int DP = 16 * R;  // rows held, the head's D padded with zero rows
  extern __shared__ float lds[];
  float* ks = lds;                                   // [16][DP]
  float* qs = ks + RULE_TOKENS * DP;                 // [16][DP]
  float* gs = qs + RULE_TOKENS * DP;                 // [16][DP] (per channel) or [16]
  float* vs = gs + (PER_CHANNEL ? RULE_TOKENS * DP : RULE_TOKENS);  // [16][16]
  float* bs = vs + RULE_TOKENS * 16;                 // [16]
  float* kqs = bs + RULE_TOKENS;                     // [16]
  const int tid = threadIdx.x, l = tid & 15, col = tid >> 4;
  const int head = blockIdx.y, s = blockIdx.z;
  const int kvh = head / (a.heads / a.kv_heads);
  const int c = blockIdx.x * 16 + col;
  const bool live = c < a.vdim;
  const int t0 = a.cu_q[s], t1 = a.cu_q[s + 1];
  const int D = a.dim;
  float* st = a.state + (((size_t)a.state_slots[s] * a.heads + head) * a.vdim + (live ? c : 0)) * D;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = (live && l + 16 * r < D) ? st[l + 16 * r] : 0.f;
  const float rate = expf(a.a_log[head]);
  for (int base = t0; base < t1; base += RULE_TOKENS) {
    const int n = min(RULE_TOKENS, t1 - base);
    __syncthreads();  // the tile before has been used
    for (int idx = tid; idx < n * DP; idx += 256) {
      const int tok = idx / DP, row = idx - tok * DP;
      const size_t at = (size_t)(base + tok) * a.channels;
      const bool in = row < D;
      ks[idx] = in ? a.qkv[at + a.k_first + kvh * D + row] : 0.f;
      qs[idx] = in ? a.qkv[at + a.q_first + kvh * D + row] : 0.f;
      if (PER_CHANNEL)
        gs[idx] = in ? decay_of(load_code(a.a, a.a_code, (size_t)(base + tok) * a.a_stride + head * D + row) +
                                a.dt_bias[head * D + row], rate) : 1.f;
    }
    {
      const int tok = tid >> 4, cc = blockIdx.x * 16 + (tid & 15);
      vs[tid] = (tok < n && cc < a.vdim) ? a.qkv[(size_t)(base + tok) * a.channels + a.v_first + head * a.vdim + cc] : 0.f;
    }
    if (tid < n) {
      const float z = load_code(a.b, a.b_code, (size_t)(base + tid) * a.b_stride + head);
      bs[tid] = 1.0f / (1.0f + expf(-z));
      if (!PER_CHANNEL)
        gs[tid] = decay_of(load_code(a.a, a.a_code, (size_t)(base + tid) * a.a_stride + head) + a.dt_bias[head], rate);
    }
    __syncthreads();
    {  // k . q of every token of the tile: the 16 lanes of group `col` take token `col`
      float p = 0.f;
      if (col < n) {
#pragma unroll
        for (int r = 0; r < R; ++r) p = fmaf(ks[col * DP + l + 16 * r], qs[col * DP + l + 16 * r], p);
      }
      p = row16_sum(p);
      if (l == 0) kqs[col] = p;
    }
    __syncthreads();
    for (int tok = 0; tok < n; ++tok) {
      const float* k = ks + tok * DP + l;
      const float* q = qs + tok * DP + l;
      float pk0 = 0.f, pk1 = 0.f, pq0 = 0.f, pq1 = 0.f;
      float kr[R];
      const float gh = PER_CHANNEL ? 1.f : gs[tok];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        kr[r] = k[16 * r];
        const float g = PER_CHANNEL ? gs[tok * DP + l + 16 * r] : gh;
        S[r] *= g;
        if (r & 1) { pk1 = fmaf(S[r], kr[r], pk1); pq1 = fmaf(S[r], q[16 * r], pq1); }
        else { pk0 = fmaf(S[r], kr[r], pk0); pq0 = fmaf(S[r], q[16 * r], pq0); }
      }
      const float sk = row16_sum(pk0 + pk1);
      const float sq = row16_sum(pq0 + pq1);
      const float u = bs[tok] * (vs[tok * 16 + col] - sk);
#pragma unroll
      for (int r = 0; r < R; ++r) S[r] = fmaf(kr[r], u, S[r]);
      if (l == 0 && live) a.out[((size_t)(base + tok) * a.heads + head) * a.vdim + c] = fmaf(kqs[tok], u, sq);
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (l + 16 * r < D) st[l + 16 * r] = S[r];
  }
}

extern "C" int qrt_delta_rule(const RuleArgs* args, int num_tokens, int num_seqs, hipStream_t stream) {
  RuleArgs a = *args;
  QRT_CHECK(a.heads > 0 && a.kv_heads > 0 && a.heads % a.kv_heads == 0, "delta_rule: %d heads on %d key heads", a.heads, a.kv_heads);
  QRT_CHECK(a.dim >= 1 && a.dim <= 256 && a.vdim >= 1, "delta_rule: key size %d (1 to 256), value size %d", a.dim, a.vdim);
  QRT_CHECK(num_tokens >= 0 && num_seqs >= 0 && num_seqs <= 65535 && a.heads <= 65535, "delta_rule: bad counts");
  if (num_tokens == 0 || num_seqs == 0) return 0;
  const int R = a.dim <= 16 ? 1 : a.dim <= 32 ? 2 : a.dim <= 64 ? 4 : a.dim <= 128 ? 8 : 16;
  const int DP = 16 * R;
  dim3 grid((a.vdim + 15) / 16, a.heads, num_seqs), block(256);
  const size_t smem = sizeof(float) * ((size_t)RULE_TOKENS * DP * (a.per_channel ? 3 : 2) + (a.per_channel ? 0 : RULE_TOKENS) +
                                       RULE_TOKENS * 16 + 2 * RULE_TOKENS);
#define GO(RR)                                                                          \
  do {                                                                                  \
    if (a.per_channel) delta_rule_kernel<RR, true><<<grid, block, smem, stream>>>(a);   \
    else delta_rule_kernel<RR, false><<<grid, block, smem, stream>>>(a);                \
  } while (0)
  switch (R) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    case 4: GO(4); break;
    case 8: GO(8); break;
    default: GO(16); break;
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
