// Residual step of a stack that norms every branch before AND after it, with
// an optional weighted average over the outputs of all earlier layers, in one
// pass over the row (one 256-thread block per token):
//
//     x <- x + table[index[t]]                      (add_table given)
//     x <- x + y / rms(y) * (offset + wb)           (y given)
//     hist[n - 1] <- x                              (hist given)
//     x <- sum_j dwa[j] * hist[j],  j < n           (dwa given)
//     out <- x / rms(x) * (offset + wn)             (wn given)
//
// rms(v) = sqrt(mean(v^2) + eps). x, hist and every sum are fp32 whatever the
// activation type; y, the weights, the table and out have the activation type.
// The row stays in registers up to width 4096 (REG); wider rows go through x
// in memory (each thread re-reads only what it wrote itself).
//
// Also here: the xIELU activation, elementwise.
#include "seq_common.h"

#define SN_NV 16

template <typename TY, typename TP, bool REG>
__global__ __launch_bounds__(256) void sandwich_rmsnorm_kernel(
    float* __restrict__ x, const TY* __restrict__ y, int64_t y_stride,
    const TP* __restrict__ wb, float* __restrict__ hist, int64_t hist_stride,
    int n_hist, const float* __restrict__ dwa, const TP* __restrict__ wn,
    float eps, float offset, TP* __restrict__ out,
    const TP* __restrict__ add_table, const int* __restrict__ add_index, int W) {
  __shared__ float scratch[8];
  const int64_t row = blockIdx.x;
  float* xr = x + row * W;
  float v[REG ? SN_NV : 1];
  const int iters = REG ? SN_NV : (W + 255) / 256;
#define SN_LOOP                                                     \
  _Pragma("unroll") for (int k = 0, i = threadIdx.x; k < iters; ++k, i += 256) \
      if (i < W)
#define SN_CUR (REG ? v[REG ? k : 0] : xr[i])

  const TP* trow = add_table ? add_table + (int64_t)add_index[row] * W : nullptr;
  if (REG || trow) {
    SN_LOOP {
      float t = xr[i];
      if (trow) t += ldf(trow + i);
      if (REG) v[REG ? k : 0] = t; else xr[i] = t;
    }
  }
  if (y) {
    const TY* yr = y + row * y_stride;
    float ss = 0.f;
    SN_LOOP {
      const float t = ldf(yr + i);
      ss += t * t;
    }
    const float rinv = 1.0f / sqrtf(block256_sum(ss, scratch) / (float)W + eps);
    SN_LOOP {
      const float t = SN_CUR + ldf(yr + i) * rinv * (offset + ldf(wb + i));
      if (REG) v[REG ? k : 0] = t; else xr[i] = t;
    }
  }
  if (hist) {
    float* hr = hist + (int64_t)(n_hist - 1) * hist_stride + row * W;
    SN_LOOP hr[i] = SN_CUR;
  }
  if (dwa) {
    SN_LOOP {
      float acc = 0.f;
      for (int j = 0; j < n_hist - 1; ++j)
        acc = fmaf(dwa[j], hist[(int64_t)j * hist_stride + row * W + i], acc);
      acc = fmaf(dwa[n_hist - 1], SN_CUR, acc);
      if (REG) v[REG ? k : 0] = acc; else xr[i] = acc;
    }
  }
  if (REG && (trow || y || dwa)) {
    SN_LOOP xr[i] = v[REG ? k : 0];
  }
  if (wn == nullptr) return;
  float ss = 0.f;
  SN_LOOP {
    const float t = SN_CUR;
    ss += t * t;
  }
  const float rinv = 1.0f / sqrtf(block256_sum(ss, scratch) / (float)W + eps);
  TP* o = out + row * W;
  SN_LOOP stf(o + i, SN_CUR * rinv * (offset + ldf(wn + i)));
#undef SN_LOOP
#undef SN_CUR
}

// ---- rows whose width is a multiple of 4 and at most 4096: 16-byte accesses -----
template <typename T>
DEVINL void sn_load4(const T* p, float* v);
template <>
DEVINL void sn_load4<float>(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
template <>
DEVINL void sn_load4<bf16_t>(const bf16_t* p, float* v) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  v[0] = bf16_bits_to_f32((uint16_t)(raw.x & 0xffff));
  v[1] = bf16_bits_to_f32((uint16_t)(raw.x >> 16));
  v[2] = bf16_bits_to_f32((uint16_t)(raw.y & 0xffff));
  v[3] = bf16_bits_to_f32((uint16_t)(raw.y >> 16));
}
template <typename T>
DEVINL void sn_store4(T* p, const float* v);
template <>
DEVINL void sn_store4<float>(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
template <>
DEVINL void sn_store4<bf16_t>(bf16_t* p, const float* v) {
  uint2 raw;
  raw.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
  raw.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
  *reinterpret_cast<uint2*>(p) = raw;
}

#define SN_NC 4  // 4-element pieces per thread

// Same steps as above. The history loop runs over the earlier layers on the
// outside and over the thread's pieces on the inside, so that the loads of
// one history row are in flight together.
template <typename TY, typename TP>
__global__ __launch_bounds__(256) void sandwich_rmsnorm_vec4_kernel(
    float* __restrict__ x, const TY* __restrict__ y, int64_t y_stride,
    const TP* __restrict__ wb, float* __restrict__ hist, int64_t hist_stride,
    int n_hist, const float* __restrict__ dwa, const TP* __restrict__ wn,
    float eps, float offset, TP* __restrict__ out,
    const TP* __restrict__ add_table, const int* __restrict__ add_index, int W) {
  __shared__ float scratch[8];
  const int64_t row = blockIdx.x;
  float* xr = x + row * W;
  float v[SN_NC][4];
  bool on[SN_NC];
  int at[SN_NC];
#pragma unroll
  for (int c = 0; c < SN_NC; ++c) {
    at[c] = (threadIdx.x + 256 * c) * 4;
    on[c] = at[c] < W;
    if (on[c]) sn_load4<float>(xr + at[c], v[c]);
    else v[c][0] = v[c][1] = v[c][2] = v[c][3] = 0.f;
  }
  if (add_table) {
    const TP* trow = add_table + (int64_t)add_index[row] * W;
#pragma unroll
    for (int c = 0; c < SN_NC; ++c)
      if (on[c]) {
        float t[4];
        sn_load4<TP>(trow + at[c], t);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[c][i] += t[i];
      }
  }
  if (y) {
    const TY* yr = y + row * y_stride;
    float yv[SN_NC][4];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < SN_NC; ++c) {
      if (on[c]) sn_load4<TY>(yr + at[c], yv[c]);
      else yv[c][0] = yv[c][1] = yv[c][2] = yv[c][3] = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) ss += yv[c][i] * yv[c][i];
    }
    const float rinv = 1.0f / sqrtf(block256_sum(ss, scratch) / (float)W + eps);
#pragma unroll
    for (int c = 0; c < SN_NC; ++c)
      if (on[c]) {
        float w4[4];
        sn_load4<TP>(wb + at[c], w4);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[c][i] += yv[c][i] * rinv * (offset + w4[i]);
      }
  }
  if (hist) {
    float* hr = hist + (int64_t)(n_hist - 1) * hist_stride + row * W;
#pragma unroll
    for (int c = 0; c < SN_NC; ++c)
      if (on[c]) sn_store4<float>(hr + at[c], v[c]);
  }
  if (dwa) {
    float acc[SN_NC][4];
#pragma unroll
    for (int c = 0; c < SN_NC; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[c][i] = 0.f;
#pragma unroll 4
    for (int j = 0; j < n_hist - 1; ++j) {
      const float wj = dwa[j];
      const float* hj = hist + (int64_t)j * hist_stride + row * W;
#pragma unroll
      for (int c = 0; c < SN_NC; ++c)
        if (on[c]) {
          float t[4];
          sn_load4<float>(hj + at[c], t);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[c][i] = fmaf(wj, t[i], acc[c][i]);
        }
    }
    const float wl = dwa[n_hist - 1];
#pragma unroll
    for (int c = 0; c < SN_NC; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) v[c][i] = fmaf(wl, v[c][i], acc[c][i]);
  }
  if (add_table || y || dwa) {
#pragma unroll
    for (int c = 0; c < SN_NC; ++c)
      if (on[c]) sn_store4<float>(xr + at[c], v[c]);
  }
  if (wn == nullptr) return;
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < SN_NC; ++c)
#pragma unroll
    for (int i = 0; i < 4; ++i) ss += v[c][i] * v[c][i];
  const float rinv = 1.0f / sqrtf(block256_sum(ss, scratch) / (float)W + eps);
  TP* o = out + row * W;
#pragma unroll
  for (int c = 0; c < SN_NC; ++c)
    if (on[c]) {
      float w4[4], r[4];
      sn_load4<TP>(wn + at[c], w4);
#pragma unroll
      for (int i = 0; i < 4; ++i) r[i] = v[c][i] * rinv * (offset + w4[i]);
      sn_store4<TP>(o + at[c], r);
    }
}

template <typename TY, typename TP>
static void launch_sn_t(float* x, const void* y, int64_t y_stride,
                        const void* wb, float* hist, int64_t hist_stride,
                        int n_hist, const float* dwa, const void* wn, float eps,
                        float offset, void* out, const void* add_table,
                        const int* add_index, int rows, int W,
                        hipStream_t stream) {
  if (rows == 0) return;
  if (W % 4 == 0 && W <= 256 * 4 * SN_NC && y_stride % 4 == 0 &&
      reinterpret_cast<uintptr_t>(y) % 16 == 0)
    hipLaunchKernelGGL((sandwich_rmsnorm_vec4_kernel<TY, TP>), dim3(rows),
                       dim3(256), 0, stream, x, (const TY*)y, y_stride,
                       (const TP*)wb, hist, hist_stride, n_hist, dwa,
                       (const TP*)wn, eps, offset, (TP*)out,
                       (const TP*)add_table, add_index, W);
  else if (W <= 256 * SN_NV)
    hipLaunchKernelGGL((sandwich_rmsnorm_kernel<TY, TP, true>), dim3(rows),
                       dim3(256), 0, stream, x, (const TY*)y, y_stride,
                       (const TP*)wb, hist, hist_stride, n_hist, dwa,
                       (const TP*)wn, eps, offset, (TP*)out,
                       (const TP*)add_table, add_index, W);
  else
    hipLaunchKernelGGL((sandwich_rmsnorm_kernel<TY, TP, false>), dim3(rows),
                       dim3(256), 0, stream, x, (const TY*)y, y_stride,
                       (const TP*)wb, hist, hist_stride, n_hist, dwa,
                       (const TP*)wn, eps, offset, (TP*)out,
                       (const TP*)add_table, add_index, W);
}

// y_kind / p_kind: 0 = bf16, 1 = float
extern "C" void launch_sandwich_rmsnorm(
    float* x, const void* y, int64_t y_stride, int y_kind, const void* wb,
    float* hist, int64_t hist_stride, int n_hist, const float* dwa,
    const void* wn, float eps, float offset, void* out, const void* add_table,
    const int* add_index, int p_kind, int rows, int W, hipStream_t stream) {
#define SN_ARGS                                                              \
  x, y, y_stride, wb, hist, hist_stride, n_hist, dwa, wn, eps, offset, out,  \
      add_table, add_index, rows, W, stream
  if (p_kind == 0) {
    if (y_kind == 0) launch_sn_t<bf16_t, bf16_t>(SN_ARGS);
    else launch_sn_t<float, bf16_t>(SN_ARGS);
  } else {
    if (y_kind == 0) launch_sn_t<bf16_t, float>(SN_ARGS);
    else launch_sn_t<float, float>(SN_ARGS);
  }
#undef SN_ARGS
}

// z > 0: a_pos z^2 + z / 2;  z <= 0: (1/2 + a_neg)(exp(z) - 1 - z) + z / 2
DEVINL float xielu_f(float z, float a_pos, float a_neg) {
  return z > 0.f ? fmaf(a_pos * z, z, 0.5f * z)
                 : fmaf(0.5f + a_neg, expm1f(z) - z, 0.5f * z);
}

template <typename T>
__global__ __launch_bounds__(256) void xielu_kernel(T* __restrict__ out,
                                                    const T* __restrict__ x,
                                                    int64_t n, float a_pos,
                                                    float a_neg) {
  const int64_t stride = (int64_t)gridDim.x * 256 * 8;
  for (int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8; i0 < n;
       i0 += stride) {
    if (i0 + 8 <= n) {
      float v[8];
      if (sizeof(T) == 2) {
        const bf16x8 raw = load_bf16x8(x + i0);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = xielu_f(bf16x8_get(raw, i), a_pos, a_neg);
        store_bf16x8(out + i0, v);
      } else {
        const float4 a = *reinterpret_cast<const float4*>(x + i0);
        const float4 b = *reinterpret_cast<const float4*>(x + i0 + 4);
        float4 ra, rb;
        ra.x = xielu_f(a.x, a_pos, a_neg); ra.y = xielu_f(a.y, a_pos, a_neg);
        ra.z = xielu_f(a.z, a_pos, a_neg); ra.w = xielu_f(a.w, a_pos, a_neg);
        rb.x = xielu_f(b.x, a_pos, a_neg); rb.y = xielu_f(b.y, a_pos, a_neg);
        rb.z = xielu_f(b.z, a_pos, a_neg); rb.w = xielu_f(b.w, a_pos, a_neg);
        *reinterpret_cast<float4*>(out + i0) = ra;
        *reinterpret_cast<float4*>(out + i0 + 4) = rb;
      }
    } else {
      for (int64_t i = i0; i < n; ++i) stf(out + i, xielu_f(ldf(x + i), a_pos, a_neg));
    }
  }
}

extern "C" void launch_xielu(void* out, const void* x, int64_t n, float a_pos,
                             float a_neg, int kind, hipStream_t stream) {
  if (n == 0) return;
  const int64_t want = (n + 256 * 8 - 1) / (256 * 8);
  const int blocks = (int)(want < 4096 ? want : 4096);
  if (kind == 0)
    hipLaunchKernelGGL((xielu_kernel<bf16_t>), dim3(blocks), dim3(256), 0,
                       stream, (bf16_t*)out, (const bf16_t*)x, n, a_pos, a_neg);
  else
    hipLaunchKernelGGL((xielu_kernel<float>), dim3(blocks), dim3(256), 0,
                       stream, (float*)out, (const float*)x, n, a_pos, a_neg);
}
