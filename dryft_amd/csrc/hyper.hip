// Several copies of a float32 residual stream (hyper-connections): one launch mixes the copies, lets the last
// sublayer's output enter them, writes them back, and forms the weighted sum that the next sublayer reads,
// normed. Per row and column c, with n copies x_1..x_n and the output y of the sublayer before:
//
//   x'_t = sum_s mix[s][t] x_s + write[t] y          (all copies from the old ones; skipped when there is no y)
//   u    = sum_t read[t] x'_t                          (read == null: the plain sum)
//   h    = u / sqrt(mean_c(u^2) + eps) * weight        (or u itself, float32, when not normed)
//
// x is the copies [n, rows, width] in float32, or a single [rows, width] in the activation dtype that every
// copy equals (the embedding's output when the stream starts). y is a tensor in the activation dtype or float32
// partial sums over K of the product that made it, added up here in order. Statistics are float.
#include "common.h"

#define HYPER_MAX 8

template <typename T, int N>
__global__ __launch_bounds__(1024) void hyper_norm_kernel(const void* __restrict__ x_in, int x_is_copies,
                                                         const void* __restrict__ delta, int delta_kind, int n_partials,
                                                         int64_t partial_stride, const float* __restrict__ mix,
                                                         const float* __restrict__ write_w,
                                                         const float* __restrict__ read_w,
                                                         const float* __restrict__ weight, float* __restrict__ x_out,
                                                         void* __restrict__ y_out, int normed, int rows, int width,
                                                         float eps) {
  extern __shared__ float u_row[];          // [width]
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int64_t plane = (int64_t)rows * width;
  float m[N][N], wr[N], rd[N];
#pragma unroll
  for (int s = 0; s < N; ++s) {
    wr[s] = delta_kind ? write_w[s] : 0.f;
    rd[s] = read_w ? read_w[s] : 1.f;
#pragma unroll
    for (int t = 0; t < N; ++t) m[s][t] = delta_kind ? mix[s * N + t] : (s == t ? 1.f : 0.f);
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const int64_t at = row * width + c;
    float x[N];
    if (x_is_copies) {
#pragma unroll
      for (int s = 0; s < N; ++s) x[s] = ((const float*)x_in)[s * plane + at];
    } else {
      const float v = load_as_float((const T*)x_in + at);
#pragma unroll
      for (int s = 0; s < N; ++s) x[s] = v;
    }
    float y = 0.f;
    if (delta_kind == 1) {
      y = load_as_float((const T*)delta + at);
    } else if (delta_kind == 2) {
      for (int p = 0; p < n_partials; ++p) y += ((const float*)delta)[p * partial_stride + at];
      y = rounded_as<T>(y);                 // what the product would have stored in the activation dtype
    }
    float u = 0.f;
    float nx[N];
#pragma unroll
    for (int t = 0; t < N; ++t) {
      float a = 0.f;
      if (delta_kind) {
#pragma unroll
        for (int s = 0; s < N; ++s) a += m[s][t] * x[s];
        a += wr[t] * y;
      } else {
        a = x[t];
      }
      nx[t] = a;
      u += rd[t] * a;
    }
    if (x_out) {
#pragma unroll
      for (int t = 0; t < N; ++t) x_out[t * plane + at] = nx[t];
    }
    u_row[c] = u;
    ss += u * u;
  }
  if (!y_out) return;
  if (!normed) {
    for (int c = threadIdx.x; c < width; c += blockDim.x) ((float*)y_out)[row * width + c] = u_row[c];
    return;
  }
  ss = block_sum(ss, scratch);
  const float r = 1.f / sqrtf(ss / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    store_from_float((T*)y_out + row * width + c, u_row[c] * r * weight[c]);
}

template <typename T>
static int launch_hyper(int n, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const void* x, int x_is_copies,
                        const void* delta, int delta_kind, int n_partials, int64_t partial_stride, const float* mix,
                        const float* write_w, const float* read_w, const float* weight, float* x_out, void* y,
                        int normed, int rows, int width, float eps) {
#define HYPER_CASE(N)                                                                                              \
  case N:                                                                                                          \
    hipLaunchKernelGGL((hyper_norm_kernel<T, N>), grid, block, lds, stream, x, x_is_copies, delta, delta_kind,     \
                       n_partials, partial_stride, mix, write_w, read_w, weight, x_out, y, normed, rows, width, eps); \
    break;
  switch (n) {
    HYPER_CASE(1) HYPER_CASE(2) HYPER_CASE(3) HYPER_CASE(4) HYPER_CASE(5) HYPER_CASE(6) HYPER_CASE(7) HYPER_CASE(8)
    default: return -1;
  }
#undef HYPER_CASE
  return DRYFT_LAUNCH_CHECK();
}

DRYFT_API int dryft_hyper_max_streams() { return HYPER_MAX; }

DRYFT_API int dryft_hyper_norm(const void* x, int x_is_copies, int n, const void* delta, int delta_kind, int n_partials,
                               int64_t partial_stride, const float* mix, const float* write_w, const float* read_w,
                               const float* weight, float* x_out, void* y, int normed, int rows, int width, float eps,
                               int is_f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (n < 1 || n > HYPER_MAX || width <= 0 || width > 16384) return -1;
  if (delta_kind && (mix == nullptr || write_w == nullptr)) return -1;
  if (y && normed && weight == nullptr) return -1;
  // few rows: more threads a row, so that a row's loads are all in flight at once
  dim3 grid(rows), block(rows <= 128 && width >= 1024 ? 1024 : 256);
  const size_t lds = (size_t)width * sizeof(float);
  if (is_f32)
    return launch_hyper<float>(n, grid, block, lds, stream, x, x_is_copies, delta, delta_kind, n_partials,
                               partial_stride, mix, write_w, read_w, weight, x_out, y, normed, rows, width, eps);
  return launch_hyper<bf16_t>(n, grid, block, lds, stream, x, x_is_copies, delta, delta_kind, n_partials,
                              partial_stride, mix, write_w, read_w, weight, x_out, y, normed, rows, width, eps);
}
