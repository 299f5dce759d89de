// Bias and rotation of a fused q | k | v product where it lies.
//
// Every column gets its bias (if any). Then, in each of the first `rot_heads` heads of `head_dim`
// columns (the query heads followed by the key heads), the first 2 * pairs columns turn:
// columns 2i and 2i + 1 are one pair (the interleaved layout), at position p by the angle
// p * freq[i]; (u, v) -> (u cos - v sin, v cos + u sin). The rest of a head passes. Angles, sines
// and cosines are float32.
#include "common.h"
#include <math.h>

template <typename T>
__global__ __launch_bounds__(256) void bias_rotate_pairs_kernel(T* __restrict__ x, long stride, int width,
                                                                const float* __restrict__ bias,
                                                                const int* __restrict__ positions,
                                                                const float* __restrict__ freq, int rot_heads,
                                                                int head_dim, int pairs) {
  const int t = blockIdx.x;
  T* row = x + (size_t)t * stride;
  const float pos = freq ? (float)positions[t] : 0.f;
  const int rot_end = freq ? rot_heads * head_dim : 0;
  // a thread owns columns 2j and 2j + 1; head sizes are even, so a pair never spans two heads.
  // With few tokens the columns are spread over blocks too (blockIdx.y), one pair a thread.
  for (int j = blockIdx.y * 256 + threadIdx.x; 2 * j < width; j += 256 * gridDim.y) {
    const int c = 2 * j;
    const bool two = c + 1 < width;
    float u = to_f32<T>(row[c]), v = two ? to_f32<T>(row[c + 1]) : 0.f;
    if (bias) {
      u += bias[c];
      if (two) v += bias[c + 1];
    }
    if (c < rot_end) {
      const int i = (c % head_dim) >> 1;
      if (i < pairs) {
        float sn, cs;
        sincos_angle(pos * freq[i], &sn, &cs);
        const float a = u * cs - v * sn, b = v * cs + u * sn;
        u = a;
        v = b;
      }
    }
    row[c] = from_f32<T>(u);
    if (two) row[c + 1] = from_f32<T>(v);
  }
}

extern "C" int qrt_bias_rotate_pairs(void* x, long stride, int width, int dtype, const float* bias, const int* positions,
                                     const float* freq, int rot_heads, int head_dim, int pairs, int num_tokens,
                                     hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && width > 0 && stride >= width, "bias_rotate_pairs: bad sizes");
  if (freq) {
    QRT_CHECK(positions && head_dim > 0 && head_dim % 2 == 0 && pairs >= 0 && 2 * pairs <= head_dim &&
              rot_heads >= 0 && (long)rot_heads * head_dim <= width,
              "bias_rotate_pairs: %d pairs in heads of %d, %d heads in %d columns", pairs, head_dim, rot_heads, width);
  }
  if (num_tokens == 0 || (!bias && !freq)) return 0;
  const int chunks = num_tokens >= 512 ? 1 : min((width + 511) / 512, 64);
  const dim3 grid(num_tokens, chunks);
  if (dtype == QRT_F32)
    bias_rotate_pairs_kernel<float><<<grid, 256, 0, stream>>>((float*)x, stride, width, bias, positions, freq, rot_heads, head_dim, pairs);
  else if (dtype == QRT_BF16)
    bias_rotate_pairs_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)x, stride, width, bias, positions, freq, rot_heads, head_dim, pairs);
  else return qrt_fail("bias_rotate_pairs: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("bias_rotate_pairs");
  return 0;
}
