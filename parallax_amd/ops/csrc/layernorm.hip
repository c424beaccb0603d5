// Layer norm (weight and bias, biased variance) over an fp32 residual stream,
// fused with the scaled residual update that precedes it:
//
//     resid <- resid + mult * scale[i] * y[i]        (skipped when y == null)
//     out   <- (resid - mean) / sqrt(var + eps) * w + b   (skipped when w == null)
//
// One 256-thread block per row. The residual stays fp32 in HBM whatever the
// activation type is; mean and variance are two separate passes (the variance
// is the mean of squared deviations, not E[x^2] - mean^2) over values held in
// registers (rows up to 4096 wide) or re-read from the just-written row.
#include "seq_common.h"

// REG: the row fits 256 threads x LN_NV registers and is read from HBM once.
#define LN_NV 16

template <typename TY, typename TP, bool REG>
__global__ __launch_bounds__(256) void add_layernorm_kernel(
    float* __restrict__ resid, const TY* __restrict__ y, int64_t y_stride,
    const TP* __restrict__ scale, float mult, const TP* __restrict__ w,
    const TP* __restrict__ b, float eps, TP* __restrict__ out, int W) {
  __shared__ float scratch[8];
  const int64_t row = blockIdx.x;
  float* x = resid + row * W;
  const TY* yr = y ? y + row * y_stride : nullptr;
  float v[REG ? LN_NV : 1];
  float sum = 0.f;
  if (REG) {
    // all loads first, unconditionally (index clamped), so they are in
    // flight together instead of one dependent wait per element
    float yv[LN_NV], sv[LN_NV];
#pragma unroll
    for (int k = 0; k < LN_NV; ++k) {
      const int i = threadIdx.x + k * 256;
      const int ic = i < W ? i : 0;
      v[k] = x[ic];
      yv[k] = yr ? ldf(yr + ic) : 0.f;
      sv[k] = yr ? ldf(scale + ic) : 0.f;
    }
#pragma unroll
    for (int k = 0; k < LN_NV; ++k) {
      const int i = threadIdx.x + k * 256;
      float t = 0.f;
      if (i < W) {
        t = v[k];
        if (yr) {
          t += mult * (sv[k] * yv[k]);
          x[i] = t;
        }
      }
      v[k] = t;
      sum += t;
    }
  } else if (yr) {
    for (int i = threadIdx.x; i < W; i += 256) {
      const float t = x[i] + mult * (ldf(scale + i) * ldf(yr + i));
      x[i] = t;
      sum += t;
    }
  } else {
    for (int i = threadIdx.x; i < W; i += 256) sum += x[i];
  }
  if (w == nullptr) return;
  const float mean = block256_sum(sum, scratch) / (float)W;
  float sq = 0.f;
  if (REG) {
#pragma unroll
    for (int k = 0; k < LN_NV; ++k) {
      const float d = (threadIdx.x + k * 256 < W) ? v[k] - mean : 0.f;
      sq += d * d;
    }
  } else {
    for (int i = threadIdx.x; i < W; i += 256) {
      const float d = x[i] - mean;
      sq += d * d;
    }
  }
  const float var = block256_sum(sq, scratch) / (float)W;
  const float rstd = 1.0f / sqrtf(var + eps);
  TP* o = out + row * W;
  if (REG) {
    float wv[LN_NV], bv[LN_NV];
#pragma unroll
    for (int k = 0; k < LN_NV; ++k) {
      const int i = threadIdx.x + k * 256;
      const int ic = i < W ? i : 0;
      wv[k] = ldf(w + ic);
      bv[k] = ldf(b + ic);
    }
#pragma unroll
    for (int k = 0; k < LN_NV; ++k) {
      const int i = threadIdx.x + k * 256;
      if (i < W) stf(o + i, (v[k] - mean) * rstd * wv[k] + bv[k]);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += 256)
      stf(o + i, (x[i] - mean) * rstd * ldf(w + i) + ldf(b + i));
  }
}

template <typename TY, typename TP>
static void launch_t(float* resid, const void* y, int64_t y_stride,
                     const void* scale, float mult, const void* w,
                     const void* b, float eps, void* out, int rows, int W,
                     hipStream_t stream) {
  if (rows == 0) return;
  if (W <= 256 * LN_NV)
    hipLaunchKernelGGL((add_layernorm_kernel<TY, TP, true>), dim3(rows),
                       dim3(256), 0, stream, resid, (const TY*)y, y_stride,
                       (const TP*)scale, mult, (const TP*)w, (const TP*)b, eps,
                       (TP*)out, W);
  else
    hipLaunchKernelGGL((add_layernorm_kernel<TY, TP, false>), dim3(rows),
                       dim3(256), 0, stream, resid, (const TY*)y, y_stride,
                       (const TP*)scale, mult, (const TP*)w, (const TP*)b, eps,
                       (TP*)out, W);
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
