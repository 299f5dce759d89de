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
// One block per token; a thread owns VEC neighbouring columns at tid, tid + BT, ... (VEC = 4
// where rows allow 16-byte accesses) and keeps them in registers between the passes (KEEP
// vectors: rows up to 8,192 wide).
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

// PL: the number of planes of the pending output where it is known when compiling (0: nothing
// pending; 4 and 8: float32 planes, as the products cut along K leave them), -1: any number, in a
// loop. With PL >= 0 every load of the row (streams, planes, norm weights, coefficients) stands
// in one stretch of code ahead of the first use, so a token costs one round of memory latency;
// steps of few tokens run blocks of 1,024 threads (BT) so that a thread owns one vector of the row.
template <int KEEP, int VEC, int BT, int PL>
__global__ __launch_bounds__(BT) void mix_norm_kernel(MixNormArgs a) {
  typedef float fvec_t __attribute__((ext_vector_type(VEC)));
  typedef bf16_t bvec_t __attribute__((ext_vector_type(VEC)));
  __shared__ float red[32];
  __shared__ float cmix[MAX_STREAMS * MAX_STREAMS], cout[MAX_STREAMS], cread[MAX_STREAMS];
  const int S = a.streams, H = a.hidden;
  const int b = blockIdx.x;
  const int r = a.rows ? a.rows[b] : b;
  // the coefficients: asked for now, put into LDS after the row's loads have been asked for
  float my_mix = 0.f, my_out = 1.f, my_read = 0.f;
  if (threadIdx.x < MAX_STREAMS * MAX_STREAMS) {
    const int s = threadIdx.x / MAX_STREAMS, t = threadIdx.x % MAX_STREAMS;
    my_mix = s == t ? 1.f : 0.f;
    if (a.mix && s < S && t < S) my_mix = a.mix[s * S + t];
    if (s == 0) {
      my_out = (a.out_w && t < S) ? a.out_w[t] : 1.f;
      my_read = a.read ? (t < S ? a.read[t] : 0.f) : (t == 0 ? 1.f : 0.f);
    }
  }
  const float* xin = a.x_in + (size_t)r * a.s_in * H;
  float* xout = a.x_out ? a.x_out + (size_t)r * S * H : nullptr;
  const bool copy_through = xout && (a.s_in != S || xout != xin);  // nothing pending, but streams to write
  const bool y_f32 = a.y_dtype == QRT_F32;

  fvec_t old[KEEP][MAX_STREAMS], y[KEEP], w[KEEP], bias[KEEP];
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int c = min((int)(threadIdx.x + BT * j) * VEC, H - VEC);  // beyond the row: its last vector, dropped below
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s)
      if (s < S) old[j][s] = *(const fvec_t*)(xin + (size_t)(a.s_in == 1 ? 0 : s) * H + c);
    w[j] = *(const fvec_t*)(a.weight + c);
    if (a.bias) bias[j] = *(const fvec_t*)(a.bias + c);
#pragma unroll
    for (int e = 0; e < VEC; ++e) y[j][e] = 0.f;
    if (PL == 1) {
      const size_t at = (size_t)r * H + c;
      if (y_f32) {
        y[j] = *(const fvec_t*)((const float*)a.y + at);
      } else {
        const bvec_t v = *(const bvec_t*)((const bf16_t*)a.y + at);
#pragma unroll
        for (int e = 0; e < VEC; ++e) y[j][e] = (float)v[e];
      }
    } else if (PL > 1) {  // float32 planes, added in order
      fvec_t part[PL > 1 ? PL : 1];
#pragma unroll
      for (int p = 0; p < PL; ++p) part[p] = *(const fvec_t*)((const float*)a.y + (size_t)p * a.plane_stride + (size_t)r * H + c);
#pragma unroll
      for (int p = 0; p < PL; ++p) y[j] += part[p];
    } else if (PL < 0) {
      for (int p = 0; p < a.planes; ++p) {
        const size_t at = (size_t)p * a.plane_stride + (size_t)r * H + c;
        if (y_f32) {
          y[j] += *(const fvec_t*)((const float*)a.y + at);
        } else {
          const bvec_t v = *(const bvec_t*)((const bf16_t*)a.y + at);
#pragma unroll
          for (int e = 0; e < VEC; ++e) y[j][e] += (float)v[e];
        }
      }
    }
  }
  if (threadIdx.x < MAX_STREAMS * MAX_STREAMS) {
    cmix[threadIdx.x] = my_mix;
    if (threadIdx.x < MAX_STREAMS) {
      cout[threadIdx.x] = my_out;
      cread[threadIdx.x] = my_read;
    }
  }
  __syncthreads();

  fvec_t u[KEEP];
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int c = (threadIdx.x + BT * j) * VEC;
#pragma unroll
    for (int e = 0; e < VEC; ++e) u[j][e] = 0.f;
    if (c < H) {
      fvec_t acc;
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
#pragma unroll
      for (int t = 0; t < MAX_STREAMS; ++t) {
        if (t < S) {
          fvec_t v;
          if (PL != 0) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] = 0.f;
#pragma unroll
            for (int s = 0; s < MAX_STREAMS; ++s)
              if (s < S) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) v[e] = fmaf(cmix[s * MAX_STREAMS + t], old[j][s][e], v[e]);
              }
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] = fmaf(cout[t], y[j][e], v[e]);
            if (xout) *(fvec_t*)(xout + (size_t)t * H + c) = v;
          } else {
            v = old[j][t];
            if (copy_through) *(fvec_t*)(xout + (size_t)t * H + c) = v;
          }
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[e] = fmaf(cread[t], v[e], acc[e]);
        }
      }
      u[j] = acc;
#pragma unroll
      for (int e = 0; e < VEC; ++e) sum += acc[e];
    }
  }
  float mean = 0.f;
  if (a.bias) mean = block_sum(sum, red) / (float)H;
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int c = (threadIdx.x + BT * j) * VEC;
    if (c < H) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float d = u[j][e] - mean;
        ss += d * d;
      }
    }
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)H + a.eps);
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int c = (threadIdx.x + BT * j) * VEC;
    if (c < H) {
      fvec_t v;
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] = (u[j][e] - mean) * inv * w[j][e];
      if (a.bias) v += bias[j];
      const size_t at = (size_t)b * H + c;
      if (a.out_dtype == QRT_F32) {
        *(fvec_t*)((float*)a.out + at) = v;
      } else {
        bvec_t o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = (bf16_t)v[e];
        *(bvec_t*)((bf16_t*)a.out + at) = o;
      }
    }
  }
}

template <int VEC, int BT, int PL>
static void mix_norm_keep(const MixNormArgs& a, hipStream_t stream) {
  dim3 grid(a.num_out), block(BT);
  const int keep = (a.hidden + BT * VEC - 1) / (BT * VEC);  // vectors a thread keeps: at most 8 (see the launch)
  // what a thread holds must fit its registers (128 of them in a block of 1,024 threads): two vectors
  // there, and with eight planes known when compiling only one
  constexpr bool SMALL = BT == 1024 && VEC == 4;
  if (keep <= 1) mix_norm_kernel<1, VEC, BT, PL><<<grid, block, 0, stream>>>(a);
  else if (keep <= 2 && SMALL && PL == 8) mix_norm_kernel<2, VEC, BT, (SMALL && PL == 8 ? -1 : PL)><<<grid, block, 0, stream>>>(a);
  else if (keep <= 2) mix_norm_kernel<2, VEC, BT, (SMALL && PL == 8 ? -1 : PL)><<<grid, block, 0, stream>>>(a);
  else if (keep <= 4 && !SMALL) mix_norm_kernel<(SMALL ? 2 : 4), VEC, BT, (SMALL ? -1 : PL)><<<grid, block, 0, stream>>>(a);
  else if (VEC == 1) mix_norm_kernel<(VEC == 1 ? 8 : 2), VEC, BT, (VEC == 1 ? PL : -1)><<<grid, block, 0, stream>>>(a);
}

template <int VEC, int BT>
static void mix_norm_planes(const MixNormArgs& a, hipStream_t stream) {
  const bool f32 = a.y_dtype == QRT_F32;
  if (!a.y) mix_norm_keep<VEC, BT, 0>(a, stream);
  else if (a.planes == 1) mix_norm_keep<VEC, BT, 1>(a, stream);
  else if (VEC == 4 && f32 && a.planes == 4) mix_norm_keep<VEC, BT, (VEC == 4 ? 4 : -1)>(a, stream);
  else if (VEC == 4 && f32 && a.planes == 8) mix_norm_keep<VEC, BT, (VEC == 4 ? 8 : -1)>(a, stream);
  else mix_norm_keep<VEC, BT, -1>(a, stream);
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
  // four columns a thread where every row and pointer allows 16-byte accesses
  auto lined_up = [](const void* p, size_t n) { return ((uintptr_t)p % n) == 0; };
  const bool wide = a.hidden % 4 == 0 && lined_up(a.x_in, 16) && lined_up(a.x_out, 16) && lined_up(a.weight, 16) &&
                    lined_up(a.bias, 16) && lined_up(a.out, 16) && lined_up(a.y, 16) && a.plane_stride % 4 == 0;
  // few tokens: the launch is one round of memory latency, taken by as many threads as the row has vectors
  // (blocks of 256 threads keep up to four vectors a thread, which is rows of 4,096; wider rows
  // and rows without 16-byte accesses take 1,024 threads as well)
  if (wide && a.num_out > 512 && a.hidden <= 4096) mix_norm_planes<4, 256>(a, stream);
  else if (wide) mix_norm_planes<4, 1024>(a, stream);
  else mix_norm_planes<1, 1024>(a, stream);
  QRT_LAUNCH_CHECK("mix_norm");
  return 0;
}
