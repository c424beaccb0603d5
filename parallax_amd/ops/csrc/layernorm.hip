// Layer norm (weight and bias, biased variance) over an fp32 residual stream,
// fused with the scaled residual update that precedes it:
//
//     resid <- resid + mult * scale[i] * y[i]        (skipped when y == null)
//     out   <- (resid - mean) / sqrt(var + eps) * w + b   (skipped when w == null)
//
// One 256-thread block per row. The residual stays fp32 in HBM whatever the
// activation type is; mean and variance are two separate passes (the variance
// is the mean of squared deviations, not E[x^2] - mean^2).
#include "seq_common.h"

template <typename TY, typename TP>
__global__ __launch_bounds__(256) void add_layernorm_kernel(
    float* __restrict__ resid, const TY* __restrict__ y, int64_t y_stride,
    const TP* __restrict__ scale, float mult, const TP* __restrict__ w,
    const TP* __restrict__ b, float eps, TP* __restrict__ out, int W) {
  __shared__ float scratch[8];
  const int64_t row = blockIdx.x;
  float* x = resid + row * W;
  float sum = 0.f;
  if (y != nullptr) {
    const TY* yr = y + row * y_stride;
    for (int i = threadIdx.x; i < W; i += 256) {
      float v = x[i] + mult * (ldf(scale + i) * ldf(yr + i));
      x[i] = v;
      sum += v;
    }
  } else {
    for (int i = threadIdx.x; i < W; i += 256) sum += x[i];
  }
  if (w == nullptr) return;
  const float mean = block256_sum(sum, scratch) / (float)W;
  float sq = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float d = x[i] - mean;
    sq += d * d;
  }
  const float var = block256_sum(sq, scratch) / (float)W;
  const float rstd = 1.0f / sqrtf(var + eps);
  TP* o = out + row * W;
  for (int i = threadIdx.x; i < W; i += 256) {
    stf(o + i, (x[i] - mean) * rstd * ldf(w + i) + ldf(b + i));
  }
}

template <typename TY, typename TP>
static void launch_t(float* resid, const void* y, int64_t y_stride,
                     const void* scale, float mult, const void* w,
                     const void* b, float eps, void* out, int rows, int W,
                     hipStream_t stream) {
  if (rows == 0) return;
  hipLaunchKernelGGL((add_layernorm_kernel<TY, TP>), dim3(rows), dim3(256), 0,
                     stream, resid, (const TY*)y, y_stride, (const TP*)scale,
                     mult, (const TP*)w, (const TP*)b, eps, (TP*)out, W);
}

// y_kind / p_kind: 0 = bf16, 1 = float
extern "C" void launch_add_layernorm(float* resid, const void* y,
                                     int64_t y_stride, int y_kind,
                                     const void* scale, float mult,
                                     const void* w, const void* b, float eps,
                                     void* out, int p_kind, int rows, int W,
                                     hipStream_t stream) {
  if (p_kind == 0) {
    if (y_kind == 0)
      launch_t<bf16_t, bf16_t>(resid, y, y_stride, scale, mult, w, b, eps, out,
                               rows, W, stream);
    else
      launch_t<float, bf16_t>(resid, y, y_stride, scale, mult, w, b, eps, out,
                              rows, W, stream);
  } else {
    if (y_kind == 0)
      launch_t<bf16_t, float>(resid, y, y_stride, scale, mult, w, b, eps, out,
                              rows, W, stream);
    else
      launch_t<float, float>(resid, y, y_stride, scale, mult, w, b, eps, out,
                             rows, W, stream);
  }
}
