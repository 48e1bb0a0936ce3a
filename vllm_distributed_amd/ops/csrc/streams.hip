// Residual streams (hyper-connections): instead of one residual row per token a model keeps `n` fp32 rows
// xs[s][t][:] and every sub-layer
//     reads   u = sum_s w_in[s] * xs[s]                       (then a norm feeds the sub-layer),
//     writes  xs[t] <- sum_s mix[s][t] * xs[s] + w_out[t] * y  (all streams from the old ones).
// n = 1 with w_in = mix = w_out = 1 is the ordinary pre-norm residual, kept in fp32.
// The norm here is RMS normalisation with ONE gain for the whole row (a device scalar).
//
//   vda_stream_embed     xs[s] = weight[ids] * scale for every stream
//   vda_stream_step      optional write (y given) followed by an optional read + norm (h given): the write of one
//                        sub-layer and the read of the next run as one pass over the rows, one workgroup per token
#include "common.h"

#define STREAMS_MAX 8

template <typename T>
__global__ __launch_bounds__(256) void stream_embed_kernel(float* __restrict__ xs, const int* __restrict__ ids,
                                                           const T* __restrict__ weight, float scale, int W,
                                                           int n, long stride) {
  const long t = blockIdx.x;
  const T* row = weight + (long)ids[t] * W;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = (float)row[c] * scale;
    for (int s = 0; s < n; ++s) xs[s * stride + t * W + c] = v;
  }
}

VDA_EXPORT int vda_stream_embed(float* xs, const int* ids, const void* weight, float scale, int T, int W, int n,
                                long stride, int dtype, hipStream_t st) {
  if (T <= 0) return 0;
  if (n < 1 || n > STREAMS_MAX) return -1;
#define L(TT) hipLaunchKernelGGL((stream_embed_kernel<TT>), dim3(T), dim3(256), 0, st, xs, ids, (const TT*)weight, \
                                 scale, W, n, stride)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
  VDA_CHECK_LAUNCH();
  return 0;
}

// dynamic LDS: W floats (the read-out row u) when h is given
template <typename TY, typename TH>
__global__ __launch_bounds__(256) void stream_step_kernel(
    float* __restrict__ xs, const TY* __restrict__ y, long y_stride, const float* __restrict__ mix,
    const float* __restrict__ w_out, TH* __restrict__ h, const float* __restrict__ w_in,
    const float* __restrict__ gain, float eps, int W, int n, long stride) {
  extern __shared__ float u_row[];
  __shared__ float red[16];
  __shared__ float c_mix[STREAMS_MAX * STREAMS_MAX], c_out[STREAMS_MAX], c_in[STREAMS_MAX];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  if (tid < n * n && y) c_mix[tid] = mix[tid];
  if (tid < n) {
    if (y) c_out[tid] = w_out[tid];
    if (h) c_in[tid] = w_in[tid];
  }
  __syncthreads();
  float ss = 0.f;
  for (int c = tid; c < W; c += 256) {
    float x[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s) x[s] = s < n ? xs[s * stride + t * W + c] : 0.f;
    if (y) {
      const float yv = (float)y[t * y_stride + c];
      float nx[STREAMS_MAX];
#pragma unroll
      for (int d = 0; d < STREAMS_MAX; ++d) {
        if (d < n) {
          float a = 0.f;
#pragma unroll
          for (int s = 0; s < STREAMS_MAX; ++s)
            if (s < n) a += c_mix[s * n + d] * x[s];
          nx[d] = a + c_out[d] * yv;
        } else {
          nx[d] = 0.f;
        }
      }
#pragma unroll
      for (int d = 0; d < STREAMS_MAX; ++d) {
        x[d] = nx[d];
        if (d < n) xs[d * stride + t * W + c] = nx[d];
      }
    }
    if (h) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < STREAMS_MAX; ++s)
        if (s < n) u += c_in[s] * x[s];
      u_row[c] = u;
      ss += u * u;
    }
  }
  if (!h) return;
  ss = block_sum(ss, red);
  const float r = gain[0] / sqrtf(ss / (float)W + eps);
  for (int c = tid; c < W; c += 256) h[t * W + c] = (TH)(u_row[c] * r);
}

VDA_EXPORT int vda_stream_step(float* xs, const void* y, long y_stride, const float* mix, const float* w_out, void* h,
                               const float* w_in, const float* gain, float eps, int T, int W, int n, long stride,
                               int y_dtype, int h_dtype, hipStream_t st) {
  if (T <= 0) return 0;
  if (n < 1 || n > STREAMS_MAX) return -1;
  if (!y && !h) return 0;
  const size_t lds = h ? (size_t)W * 4 : 0;
  if (lds > 60 * 1024) return -2;
#define L(TY, TH) hipLaunchKernelGGL((stream_step_kernel<TY, TH>), dim3(T), dim3(256), lds, st, xs, (const TY*)y, \
                                     y_stride, mix, w_out, (TH*)h, w_in, gain, eps, W, n, stride)
  // y and h share the model's activation type when both are given
  const int dt = y ? y_dtype : h_dtype;
  if (y && h && y_dtype != h_dtype) return -3;
  if (dt == VDA_BF16) L(bf16_t, bf16_t);
  else if (dt == VDA_F16) L(f16_t, f16_t);
  else if (dt == VDA_F32) L(float, float);
  else return -3;
#undef L
  VDA_CHECK_LAUNCH();
  return 0;
}
