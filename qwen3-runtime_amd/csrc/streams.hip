// The step between two sub-layers when the residual is kept in several streams
// (hyper-connections), and layer norm: one pass over a token's streams that
//   1. applies the update the sub-layer before left pending,
//        new[t] = sum_s mix[s, t] * old[s] + out[t] * y          (y: the sub-layer's output),
//      and writes the streams back,
//   2. reads them for the sub-layer to come, u = sum_t read[t] * new[t],
//   3. normalises u: (u - mean) / sqrt(var + eps) * w + b (var the mean of the squared
//      deviations), or, without b, u / sqrt(mean(u^2) + eps) * w.
// With one stream, mix and out absent and read absent this is residual add + layer norm. All
// arithmetic is float32; a row's sums are taken in a fixed order, whatever else is in the batch.
// One block of 256 threads per token; a thread owns the columns tid, tid + 256, ... and keeps
// their u in registers between the passes (KEEP of them: rows up to 256 * KEEP wide).
#include "common.h"
#include <math.h>

#define MAX_STREAMS 8

struct MixNormArgs {
  const float* x_in;   // [T, s_in, H]; s_in is 1 (every stream starts as this one) or `streams`
  float* x_out;        // [T, streams, H], may be x_in; null: the streams are not written back
  const void* y;       // [planes, T, H] or null: nothing pending
  const float* mix;    // [streams, streams], indexed [from, to]; null: the identity
  const float* out_w;  // [streams]; null: ones
  const float* read;   // [streams]; null: stream 0 alone
  const float* weight; // [H]
  const float* bias;   // [H] or null: RMS norm
  const int* rows;     // [R] or null: every token
  void* out;           // [R, H]
  int num_out, hidden, streams, s_in, planes, y_dtype, out_dtype;
  long plane_stride;
  float eps;
};

template <int KEEP>
__global__ __launch_bounds__(256) void mix_norm_kernel(MixNormArgs a) {
  __shared__ float red[32];
  __shared__ float cmix[MAX_STREAMS * MAX_STREAMS], cout[MAX_STREAMS], cread[MAX_STREAMS];
  const int S = a.streams, H = a.hidden;
  const int b = blockIdx.x;
  const int r = a.rows ? a.rows[b] : b;
  if (threadIdx.x < MAX_STREAMS * MAX_STREAMS) {
    const int s = threadIdx.x / MAX_STREAMS, t = threadIdx.x % MAX_STREAMS;
    float m = s == t ? 1.f : 0.f;
    if (a.mix && s < S && t < S) m = a.mix[s * S + t];
    cmix[threadIdx.x] = m;
    if (s == 0) {
      cout[t] = (a.out_w && t < S) ? a.out_w[t] : 1.f;
      cread[t] = a.read ? (t < S ? a.read[t] : 0.f) : (t == 0 ? 1.f : 0.f);
    }
  }
  __syncthreads();
  const float* xin = a.x_in + (size_t)r * a.s_in * H;
  float* xout = a.x_out ? a.x_out + (size_t)r * S * H : nullptr;
  float u[KEEP];
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int c = threadIdx.x + 256 * j;
    u[j] = 0.f;
    if (c < H) {
      float old[MAX_STREAMS];
#pragma unroll
      for (int s = 0; s < MAX_STREAMS; ++s) old[s] = s < S ? xin[(size_t)(a.s_in == 1 ? 0 : s) * H + c] : 0.f;
      float y = 0.f;
      if (a.y) {
        for (int p = 0; p < a.planes; ++p) {
          const size_t at = (size_t)p * a.plane_stride + (size_t)r * H + c;
          y += a.y_dtype == QRT_F32 ? ((const float*)a.y)[at] : (float)((const bf16_t*)a.y)[at];
        }
      }
      float acc = 0.f;
#pragma unroll
      for (int t = 0; t < MAX_STREAMS; ++t) {
        if (t < S) {
          float v;
          if (a.y) {
            v = 0.f;
#pragma unroll
            for (int s = 0; s < MAX_STREAMS; ++s)
              if (s < S) v = fmaf(cmix[s * MAX_STREAMS + t], old[s], v);
            v = fmaf(cout[t], y, v);
            if (xout) xout[(size_t)t * H + c] = v;
          } else {
            v = old[t];
            if (xout && (a.s_in != S || xout != xin)) xout[(size_t)t * H + c] = v;
          }
          acc = fmaf(cread[t], v, acc);
        }
      }
      u[j] = acc;
      sum += acc;
    }
  }
  float mean = 0.f;
  if (a.bias) mean = block_sum(sum, red) / (float)H;
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int c = threadIdx.x + 256 * j;
    if (c < H) {
      const float d = u[j] - mean;
      ss += d * d;
    }
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)H + a.eps);
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int c = threadIdx.x + 256 * j;
    if (c < H) {
      float v = (u[j] - mean) * inv * a.weight[c];
      if (a.bias) v += a.bias[c];
      const size_t at = (size_t)b * H + c;
      if (a.out_dtype == QRT_F32) ((float*)a.out)[at] = v;
      else ((bf16_t*)a.out)[at] = (bf16_t)v;
    }
  }
}

extern "C" int qrt_mix_norm(const MixNormArgs* args, hipStream_t stream) {
  MixNormArgs a = *args;
  QRT_CHECK(a.num_out >= 0 && a.hidden > 0, "mix_norm: bad sizes R=%d H=%d", a.num_out, a.hidden);
  QRT_CHECK(a.streams >= 1 && a.streams <= MAX_STREAMS, "mix_norm: %d streams (1 to %d)", a.streams, MAX_STREAMS);
  QRT_CHECK(a.s_in == 1 || a.s_in == a.streams, "mix_norm: %d streams come in, %d go on", a.s_in, a.streams);
  QRT_CHECK(a.x_in && a.weight && a.out, "mix_norm: a null tensor");
  QRT_CHECK(!a.y || (a.planes >= 1 && (a.y_dtype == QRT_F32 || a.y_dtype == QRT_BF16)), "mix_norm: bad pending output");
  QRT_CHECK(a.y || (!a.mix && !a.out_w), "mix_norm: mixing coefficients without an output to add");
  QRT_CHECK(a.out_dtype == QRT_F32 || a.out_dtype == QRT_BF16, "mix_norm: unknown output dtype %d", a.out_dtype);
  QRT_CHECK(a.hidden <= 256 * 32, "mix_norm: rows of %d elements (at most %d)", a.hidden, 256 * 32);
  QRT_CHECK(!(a.x_out && a.rows), "mix_norm: rows picked out are not written back");
  if (a.num_out == 0) return 0;
  dim3 grid(a.num_out), block(256);
  const int keep = (a.hidden + 255) / 256;
  if (keep <= 1) mix_norm_kernel<1><<<grid, block, 0, stream>>>(a);
  else if (keep <= 2) mix_norm_kernel<2><<<grid, block, 0, stream>>>(a);
  else if (keep <= 4) mix_norm_kernel<4><<<grid, block, 0, stream>>>(a);
  else if (keep <= 8) mix_norm_kernel<8><<<grid, block, 0, stream>>>(a);
  else if (keep <= 16) mix_norm_kernel<16><<<grid, block, 0, stream>>>(a);
  else mix_norm_kernel<32><<<grid, block, 0, stream>>>(a);
  QRT_LAUNCH_CHECK("mix_norm");
  return 0;
}
