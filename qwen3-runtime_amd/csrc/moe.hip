// Routed mixture of SwiGLU experts: the router, and the experts' products for
// (token, chosen expert) pairs taken one by one.
//
// Router: logits z[e] = x . W_r[e] + b[e] in float32 (the router's matrix is held in float32
// in every mode), the `top` largest per token (ties: the lower index), softmax over those.
// Experts: pair p = (token t, its j-th expert e) computes act[p] = silu(G_e x) * (U_e x) with
// gate_up [E, 2I, H] (gate rows, then up rows), then out[t] = sum_j w[t, j] * D_e act[p] with
// down [E, H, I], float32 out. Every output element is one wave's sum over its row in a fixed
// order: it depends on neither the batch nor the other pairs. This form streams an expert's
// matrices once per pair and suits steps of few tokens (decoding).
#include "common.h"
#include <math.h>

// sum over lanes of x[c] * w[c], c < n: 16-byte loads of w where the row allows them
template <typename T>
__device__ __forceinline__ float lane_dot(const T* __restrict__ w, const float* __restrict__ xs, int n, int lane, bool wide) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  float acc = 0.f;
  if (wide) {
    for (int c = lane * VEC; c < n; c += 64 * VEC) {
      const vec_t v = *(const vec_t*)(w + c);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc = fmaf(xs[c + e], to_f32<T>(v[e]), acc);
    }
  } else {
    for (int c = lane; c < n; c += 64) acc = fmaf(xs[c], to_f32<T>(w[c]), acc);
  }
  return acc;
}

// ------------------------------------------------------------------- router
#define MAX_EXPERTS 1024
template <typename T>
__global__ __launch_bounds__(256) void route_top_kernel(const T* __restrict__ x, const float* __restrict__ router,
                                                        const float* __restrict__ bias, int* __restrict__ index,
                                                        float* __restrict__ weight, int hidden, int experts, int top) {
  extern __shared__ float smem[];
  float* xs = smem;               // [hidden]
  float* logit = smem + hidden;   // [experts]
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = threadIdx.x; c < hidden; c += 256) xs[c] = to_f32<T>(x[(size_t)t * hidden + c]);
  __syncthreads();
  const bool wide = hidden % 4 == 0;
  for (int e = wave; e < experts; e += 4) {
    const float z = wave_sum(lane_dot<float>(router + (size_t)e * hidden, xs, hidden, lane, wide));
    if (lane == 0) logit[e] = z + (bias ? bias[e] : 0.f);
  }
  __syncthreads();
  if (wave != 0) return;
  // `top` rounds of "largest that is left", ties to the lower index
  float chosen = 0.f, first = 0.f, denom = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < experts; e += 64) {
      const float z = logit[e];
      if (z > best) { best = z; at = e; }  // ascending e: the first of equals stays
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oa = __shfl_xor(at, o, 64);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (j == 0) first = best;
    const float p = expf(best - first);
    denom += p;
    if (lane == j) chosen = p;
    if (lane == 0) {
      index[(size_t)t * top + j] = at;
      logit[at] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane < top) weight[(size_t)t * top + lane] = chosen / denom;
}

extern "C" int qrt_route_top(const void* x, int x_dtype, const float* router, const float* bias, int* index,
                             float* weight, int num_tokens, int hidden, int experts, int top, hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && hidden > 0, "route_top: bad sizes T=%d H=%d", num_tokens, hidden);
  QRT_CHECK(experts >= 1 && experts <= MAX_EXPERTS && top >= 1 && top <= experts && top <= 64,
            "route_top: %d of %d experts (at most %d experts, 64 chosen)", top, experts, MAX_EXPERTS);
  const size_t smem = (size_t)(hidden + experts) * sizeof(float);
  QRT_CHECK(smem <= 64 * 1024, "route_top: rows of %d elements do not fit", hidden);
  if (num_tokens == 0) return 0;
  dim3 grid(num_tokens), block(256);
  if (x_dtype == QRT_F32)
    route_top_kernel<float><<<grid, block, smem, stream>>>((const float*)x, router, bias, index, weight, hidden, experts, top);
  else if (x_dtype == QRT_BF16)
    route_top_kernel<bf16_t><<<grid, block, smem, stream>>>((const bf16_t*)x, router, bias, index, weight, hidden, experts, top);
  else return qrt_fail("route_top: unknown dtype %d", x_dtype);
  QRT_LAUNCH_CHECK("route_top");
  return 0;
}

// ------------------------------------------- experts, pair by pair (few tokens)
#define ROWS_PER_WAVE 4
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const T* __restrict__ x, const T* __restrict__ gate_up,
                                                          const int* __restrict__ index, T* __restrict__ act,
                                                          int hidden, int inter, int top) {
  extern __shared__ float xs[];  // [hidden]
  const int p = blockIdx.x, t = p / top;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e = index[p];
  for (int c = threadIdx.x; c < hidden; c += 256) xs[c] = to_f32<T>(x[(size_t)t * hidden + c]);
  __syncthreads();
  const bool wide = hidden % (16 / sizeof(T)) == 0;
  const T* w = gate_up + (size_t)e * 2 * inter * hidden;
  const int i0 = (blockIdx.y * 4 + wave) * ROWS_PER_WAVE;
#pragma unroll
  for (int r = 0; r < ROWS_PER_WAVE; ++r) {
    const int i = i0 + r;
    if (i >= inter) break;
    const float g = wave_sum(lane_dot<T>(w + (size_t)i * hidden, xs, hidden, lane, wide));
    const float u = wave_sum(lane_dot<T>(w + (size_t)(inter + i) * hidden, xs, hidden, lane, wide));
    if (lane == 0) act[(size_t)p * inter + i] = from_f32<T>(g / (1.0f + expf(-g)) * u);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ act, const T* __restrict__ down,
                                                       const int* __restrict__ index, const float* __restrict__ weight,
                                                       float* __restrict__ out, int hidden, int inter, int top) {
  extern __shared__ float as[];  // [top, inter]
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = threadIdx.x; c < top * inter; c += 256) as[c] = to_f32<T>(act[(size_t)t * top * inter + c]);
  __syncthreads();
  const bool wide = inter % (16 / sizeof(T)) == 0;
  const int n0 = (blockIdx.y * 4 + wave) * ROWS_PER_WAVE;
#pragma unroll
  for (int r = 0; r < ROWS_PER_WAVE; ++r) {
    const int n = n0 + r;
    if (n >= hidden) break;
    float sum = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = index[(size_t)t * top + j];
      const float d = wave_sum(lane_dot<T>(down + ((size_t)e * hidden + n) * inter, as + (size_t)j * inter, inter, lane, wide));
      sum = fmaf(weight[(size_t)t * top + j], d, sum);
    }
    if (lane == 0) out[(size_t)t * hidden + n] = sum;
  }
}

extern "C" int qrt_moe_pairs(const void* x, const void* gate_up, const void* down, const int* index,
                             const float* weight, void* act, float* out, int dtype, int num_tokens, int hidden,
                             int inter, int experts, int top, hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && hidden > 0 && inter > 0 && experts > 0 && top > 0, "moe: bad sizes");
  QRT_CHECK((size_t)hidden * 4 <= 64 * 1024 && (size_t)top * inter * 4 <= 64 * 1024,
            "moe: a token's row (%d) or its experts' inner rows (%d x %d) do not fit", hidden, top, inter);
  QRT_CHECK(dtype == QRT_F32 || dtype == QRT_BF16, "moe: unknown dtype %d", dtype);
  if (num_tokens == 0) return 0;
  const int per_block = 4 * ROWS_PER_WAVE;
  dim3 g1(num_tokens * top, (inter + per_block - 1) / per_block), g2(num_tokens, (hidden + per_block - 1) / per_block);
  QRT_CHECK(g1.y <= 65535 && g2.y <= 65535, "moe: rows too wide for one launch");
  if (dtype == QRT_F32) {
    moe_gate_up_kernel<float><<<g1, 256, hidden * 4, stream>>>((const float*)x, (const float*)gate_up, index, (float*)act, hidden, inter, top);
    moe_down_kernel<float><<<g2, 256, top * inter * 4, stream>>>((const float*)act, (const float*)down, index, weight, out, hidden, inter, top);
  } else {
    moe_gate_up_kernel<bf16_t><<<g1, 256, hidden * 4, stream>>>((const bf16_t*)x, (const bf16_t*)gate_up, index, (bf16_t*)act, hidden, inter, top);
    moe_down_kernel<bf16_t><<<g2, 256, top * inter * 4, stream>>>((const bf16_t*)act, (const bf16_t*)down, index, weight, out, hidden, inter, top);
  }
  QRT_LAUNCH_CHECK("moe_pairs");
  return 0;
}

// ------------------------------------------------ sigmoid gate on a matrix
// out[t, c] *= sigmoid(gate[t, c]), gate rows `gate_stride` elements apart
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ out, const T* __restrict__ gate, long gate_stride, int width) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float g = to_f32<T>(gate[(size_t)t * gate_stride + c]);
    out[(size_t)t * width + c] = from_f32<T>(to_f32<T>(out[(size_t)t * width + c]) / (1.0f + expf(-g)));
  }
}

extern "C" int qrt_sigmoid_gate(void* out, const void* gate, long gate_stride, int dtype, int num_tokens, int width,
                                hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && width > 0 && gate_stride >= width, "sigmoid_gate: bad sizes");
  if (num_tokens == 0) return 0;
  if (dtype == QRT_F32) sigmoid_gate_kernel<float><<<num_tokens, 256, 0, stream>>>((float*)out, (const float*)gate, gate_stride, width);
  else if (dtype == QRT_BF16) sigmoid_gate_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gate, gate_stride, width);
  else return qrt_fail("sigmoid_gate: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("sigmoid_gate");
  return 0;
}
