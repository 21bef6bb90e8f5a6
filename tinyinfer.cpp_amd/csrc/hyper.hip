// libti_hyper: the layer norm (mean and variance, a gain, no bias) and the kernels of a residual kept in several streams
// (hyper-connections): what a sublayer reads is a weighted sum of the streams behind a norm, and its output goes back into
// every stream beside a learned mixing of the old ones.  All arithmetic is 32-bit; a norm's rows are rounded once to T.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

#define HY_THREADS 256
#define HY_MAX_STREAMS 16

// out[r, :] = (u - mean(u)) / sqrt(mean((u - mean(u))^2) + eps) * w with u = sum_s coef[s] x_s[row, :] (coef null: u = x_0),
// row = rows ? rows[r] : r.  A workgroup per row; u waits in LDS between the two passes (the variance is taken from the
// deviations themselves, not from a difference of means), so out may be x itself.
template <typename T>
__global__ void __launch_bounds__(HY_THREADS)
mixed_layernorm_kernel(const float* __restrict__ x, long stream_stride, int S, const float* __restrict__ coef,
                       const int* __restrict__ rows, const float* __restrict__ w, T* __restrict__ out, int H, float eps) {
  extern __shared__ float s_u[];
  __shared__ float red[HY_THREADS / TI_WAVE];
  const int r = blockIdx.x;
  const size_t row = (size_t)(rows ? rows[r] : r) * H;
  float sum = 0.f;
  for (int c = threadIdx.x; c < H; c += HY_THREADS) {
    float u = x[row + c];
    if (coef) {
      u *= coef[0];
      for (int s = 1; s < S; ++s) u = fmaf(coef[s], x[(size_t)s * stream_stride + row + c], u);
    }
    s_u[c] = u;
    sum += u;
  }
  const float mean = block_sum<HY_THREADS>(sum, red) / (float)H;
  float sq = 0.f;
  for (int c = threadIdx.x; c < H; c += HY_THREADS) {
    const float d = s_u[c] - mean;
    sq = fmaf(d, d, sq);
  }
  const float inv = 1.0f / sqrtf(block_sum<HY_THREADS>(sq, red) / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += HY_THREADS) st<T>(out + (size_t)r * H + c, (s_u[c] - mean) * inv * w[c]);
}

extern "C" int ti_mixed_layernorm(int out_dtype, const float* x, long stream_stride, int S, const float* coef, const int* rows,
                                  const float* w, void* out, int n_rows, int H, float eps, hipStream_t stream) {
  TI_REQUIRE(n_rows >= 0 && H > 0 && H <= 16384 && x && w && out, "layernorm: bad sizes rows=%d H=%d (a row of up to 16384)", n_rows, H);
  TI_REQUIRE(!coef || (S >= 1 && S <= HY_MAX_STREAMS), "layernorm: %d streams are not served (1 to %d)", S, HY_MAX_STREAMS);
  if (n_rows == 0) return 0;
  const size_t lds = (size_t)H * 4;
  if (out_dtype == TI_F32)
    mixed_layernorm_kernel<float><<<n_rows, HY_THREADS, lds, stream>>>(x, stream_stride, S, coef, rows, w, (float*)out, H, eps);
  else if (out_dtype == TI_BF16)
    mixed_layernorm_kernel<bf16_t><<<n_rows, HY_THREADS, lds, stream>>>(x, stream_stride, S, coef, rows, w, (bf16_t*)out, H, eps);
  else
    TI_REQUIRE(false, "layernorm: unknown dtype %d", out_dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// u = sum_s coef[s] x_s, for a norm that has no form of its own for several streams
__global__ void hyper_combine_kernel(const float* __restrict__ x, long stream_stride, int S, const float* __restrict__ coef,
                                     float* __restrict__ u, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    float v = coef ? x[i] * coef[0] : x[i];
    for (int s = 1; s < S; ++s) v = coef ? fmaf(coef[s], x[(size_t)s * stream_stride + i], v) : v + x[(size_t)s * stream_stride + i];
    u[i] = v;
  }
}

// coef null: the plain sum of the streams
extern "C" int ti_hyper_combine(const float* x, long stream_stride, int S, const float* coef, float* u, long n, hipStream_t stream) {
  TI_REQUIRE(n >= 0 && S >= 1 && S <= HY_MAX_STREAMS && x && u, "hyper_combine: bad sizes n=%ld streams=%d", n, S);
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  hyper_combine_kernel<<<blocks, 256, 0, stream>>>(x, stream_stride, S, coef, u, n);
  TI_LAUNCH_CHECK();
  return 0;
}

// every stream a copy of x
__global__ void hyper_spread_kernel(const float* __restrict__ x, float* __restrict__ streams, long stream_stride, int S, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const float v = x[i];
    for (int s = 0; s < S; ++s) streams[(size_t)s * stream_stride + i] = v;
  }
}

extern "C" int ti_hyper_spread(const float* x, float* streams, long stream_stride, int S, long n, hipStream_t stream) {
  TI_REQUIRE(n >= 0 && S >= 1 && S <= HY_MAX_STREAMS && x && streams, "hyper_spread: bad sizes n=%ld streams=%d", n, S);
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  hyper_spread_kernel<<<blocks, 256, 0, stream>>>(x, streams, stream_stride, S, n);
  TI_LAUNCH_CHECK();
  return 0;
}

// x_t <- sum_s mix[s, t] x_s + back[t] y for every t at once from the old streams (mix [S, S] indexed [from, to]); the sum
// over s ascending, then the sublayer's share
// y2 (null: none): the sublayer's output is f1 y + f2 y2, two branches that were left apart
__global__ void hyper_write_kernel(float* __restrict__ streams, long stream_stride, int S, const float* __restrict__ mix,
                                   const float* __restrict__ back, const float* __restrict__ y, const float* __restrict__ y2, float f1,
                                   float f2, long n) {
  __shared__ float s_mix[HY_MAX_STREAMS * HY_MAX_STREAMS], s_back[HY_MAX_STREAMS];
  for (int i = threadIdx.x; i < S * S; i += blockDim.x) s_mix[i] = mix[i];
  for (int i = threadIdx.x; i < S; i += blockDim.x) s_back[i] = back[i];
  __syncthreads();
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    float old[HY_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < HY_MAX_STREAMS; ++s)
      if (s < S) old[s] = streams[(size_t)s * stream_stride + i];
    const float v = y2 ? fmaf(f2, y2[i], f1 * y[i]) : y[i];
    for (int t = 0; t < S; ++t) {
      float acc = s_mix[t] * old[0];
#pragma unroll
      for (int s = 1; s < HY_MAX_STREAMS; ++s)
        if (s < S) acc = fmaf(s_mix[s * S + t], old[s], acc);
      streams[(size_t)t * stream_stride + i] = fmaf(s_back[t], v, acc);
    }
  }
}

extern "C" int ti_hyper_write(float* streams, long stream_stride, int S, const float* mix, const float* back, const float* y,
                              const float* y2, float f1, float f2, long n, hipStream_t stream) {
  TI_REQUIRE(n >= 0 && S >= 1 && S <= HY_MAX_STREAMS && streams && mix && back && y, "hyper_write: bad sizes n=%ld streams=%d", n, S);
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  hyper_write_kernel<<<blocks, 256, 0, stream>>>(streams, stream_stride, S, mix, back, y, y2, f1, f2, n);
  TI_LAUNCH_CHECK();
  return 0;
}

// A sublayer's write and the next sublayer's read in one pass over the streams, a workgroup per row: the streams get
// sum_s mix[s, t] x_s + back[t] y (y as above), and out[r, :] = layernorm(sum_t coef[t] x_t') * w of the new streams, in T.
// Same arithmetic, in the same order, as hyper_write followed by mixed_layernorm.
template <typename T>
__global__ void __launch_bounds__(HY_THREADS)
hyper_write_read_kernel(float* __restrict__ streams, long stream_stride, int S, const float* __restrict__ mix,
                        const float* __restrict__ back, const float* __restrict__ y, const float* __restrict__ y2, float f1, float f2,
                        const float* __restrict__ coef, const float* __restrict__ w, T* __restrict__ out, int H, float eps) {
  extern __shared__ float s_u[];
  __shared__ float red[HY_THREADS / TI_WAVE];
  __shared__ float s_mix[HY_MAX_STREAMS * HY_MAX_STREAMS], s_back[HY_MAX_STREAMS], s_coef[HY_MAX_STREAMS];
  for (int i = threadIdx.x; i < S * S; i += HY_THREADS) s_mix[i] = mix[i];
  for (int i = threadIdx.x; i < S; i += HY_THREADS) {
    s_back[i] = back[i];
    s_coef[i] = coef[i];
  }
  __syncthreads();
  const size_t row = (size_t)blockIdx.x * H;
  float sum = 0.f;
  for (int c = threadIdx.x; c < H; c += HY_THREADS) {
    float old[HY_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < HY_MAX_STREAMS; ++s)
      if (s < S) old[s] = streams[(size_t)s * stream_stride + row + c];
    const float v = y2 ? fmaf(f2, y2[row + c], f1 * y[row + c]) : y[row + c];
    float u = 0.f;
    for (int t = 0; t < S; ++t) {
      float acc = s_mix[t] * old[0];
#pragma unroll
      for (int s = 1; s < HY_MAX_STREAMS; ++s)
        if (s < S) acc = fmaf(s_mix[s * S + t], old[s], acc);
      const float x = fmaf(s_back[t], v, acc);
      streams[(size_t)t * stream_stride + row + c] = x;
      u = t == 0 ? x * s_coef[0] : fmaf(s_coef[t], x, u);
    }
    s_u[c] = u;
    sum += u;
  }
  const float mean = block_sum<HY_THREADS>(sum, red) / (float)H;
  float sq = 0.f;
  for (int c = threadIdx.x; c < H; c += HY_THREADS) {
    const float d = s_u[c] - mean;
    sq = fmaf(d, d, sq);
  }
  const float inv = 1.0f / sqrtf(block_sum<HY_THREADS>(sq, red) / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += HY_THREADS) st<T>(out + row + c, (s_u[c] - mean) * inv * w[c]);
}

extern "C" int ti_hyper_write_read(int out_dtype, float* streams, long stream_stride, int S, const float* mix, const float* back,
                                   const float* y, const float* y2, float f1, float f2, const float* coef, const float* w, void* out,
                                   int M, int H, float eps, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && H > 0 && H <= 16384 && S >= 1 && S <= HY_MAX_STREAMS && streams && mix && back && y && coef && w && out,
             "hyper_write_read: bad sizes M=%d H=%d streams=%d", M, H, S);
  if (M == 0) return 0;
  const size_t lds = (size_t)H * 4;
  if (out_dtype == TI_F32)
    hyper_write_read_kernel<float><<<M, HY_THREADS, lds, stream>>>(streams, stream_stride, S, mix, back, y, y2, f1, f2, coef, w, (float*)out, H, eps);
  else if (out_dtype == TI_BF16)
    hyper_write_read_kernel<bf16_t><<<M, HY_THREADS, lds, stream>>>(streams, stream_stride, S, mix, back, y, y2, f1, f2, coef, w, (bf16_t*)out, H, eps);
  else
    TI_REQUIRE(false, "hyper_write_read: unknown dtype %d", out_dtype);
  TI_LAUNCH_CHECK();
  return 0;
}
