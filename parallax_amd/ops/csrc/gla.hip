// Gated linear attention: per head a [dk, dv] fp32 state with a decay per key
// channel,
//
//     S_t = diag(alpha_t) S_(t-1) + k_t v_t^T ,   o_t = S_t^T q_t ,
//     alpha = sigmoid(z + z_bias)^(1/tau)   (computed as exp(logsigmoid / tau)).
//
// The recurrence runs token by token inside the kernel, so a prompt cut into
// portions, or decoded one token at a time, goes through the very same
// operations in the same order. Parallelism comes from the state's columns:
// o_t[j] only needs column j of S, so a thread owns (part of) one column in
// registers for the whole portion. G lanes share a column when dk > 16 (each
// holds 16 rows; their partial dot products meet through wave shuffles).
// q, k, the decay and v of 16 tokens at a time are staged in LDS by the whole
// block, which also turns z into alpha once per (token, channel) and not once
// per column.
//
// The state lives in fp32 slots [slot, H, dk, dv]; a sequence whose first
// token of this launch sits at position 0 starts from zeros instead of the
// slot's old content. A decode step is the same kernel with one token per
// sequence.
#include "seq_common.h"

#define GLA_TC_MAX 16  // tokens staged per pass (fewer when dk is large)
#define GLA_ROWS 16  // state rows per lane

template <typename T>
__global__ __launch_bounds__(256) void gla_recurrence_kernel(
    float* __restrict__ o, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, const T* __restrict__ z, int64_t q_stride,
    int64_t k_stride, int64_t v_stride, int64_t z_stride,
    const T* __restrict__ z_bias, float* __restrict__ state,
    const int64_t* __restrict__ slots, const int* __restrict__ cu,
    const int* __restrict__ positions, int H, int dk, int dv, int G, int TC,
    float inv_tau, float q_scale) {
  extern __shared__ float lds[];
  const int b = blockIdx.z, h = blockIdx.y;
  const int C = 64 / G;  // columns per wave
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane / C;
  const int jb = wave * C + lane % C;  // column within the block
  const int j = blockIdx.x * 4 * C + jb;
  const bool jvalid = j < dv;
  const int t0 = cu ? cu[b] : b;
  const int t1 = cu ? cu[b + 1] : b + 1;
  if (t0 >= t1) return;
  const int dkp = G * GLA_ROWS;  // padded rows (pad: q = k = alpha = 0)
  float* sq = lds;
  float* sk = sq + TC * dkp;
  float* sa = sk + TC * dkp;
  float* sv = sa + TC * dkp;  // [TC][4 * C]

  const int64_t slot = slots[b];
  float* S = state + ((slot * H + h) * (int64_t)dk) * dv;
  const bool fresh = positions[t0] == 0;
  float s[GLA_ROWS];
#pragma unroll
  for (int r = 0; r < GLA_ROWS; ++r) {
    const int i = g * GLA_ROWS + r;
    s[r] = (!fresh && jvalid && i < dk) ? S[(int64_t)i * dv + j] : 0.f;
  }

  for (int tc = t0; tc < t1; tc += TC) {
    const int n = min(TC, t1 - tc);
    __syncthreads();
    for (int idx = threadIdx.x; idx < n * dkp; idx += 256) {
      const int tt = idx / dkp, i = idx % dkp;
      float qf = 0.f, kf = 0.f, af = 0.f;
      if (i < dk) {
        const int64_t tok = tc + tt;
        const int c = h * dk + i;
        qf = ldf(q + tok * q_stride + c) * q_scale;
        kf = ldf(k + tok * k_stride + c);
        const float zf = ldf(z + tok * z_stride + c) + ldf(z_bias + c);
        const float logsig = fminf(zf, 0.f) - log1pf(expf(-fabsf(zf)));
        af = expf(logsig * inv_tau);
      }
      sq[idx] = qf;
      sk[idx] = kf;
      sa[idx] = af;
    }
    for (int idx = threadIdx.x; idx < n * 4 * C; idx += 256) {
      const int tt = idx / (4 * C), jj = idx % (4 * C);
      const int col = blockIdx.x * 4 * C + jj;
      sv[idx] = col < dv
                    ? ldf(v + (int64_t)(tc + tt) * v_stride + h * dv + col)
                    : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float vj = sv[tt * 4 * C + jb];
      const float* aq = sq + tt * dkp + g * GLA_ROWS;
      const float* ak = sk + tt * dkp + g * GLA_ROWS;
      const float* aa = sa + tt * dkp + g * GLA_ROWS;
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < GLA_ROWS; ++r) {
        s[r] = aa[r] * s[r] + ak[r] * vj;
        acc = fmaf(s[r], aq[r], acc);
      }
      for (int off = C; off < 64; off <<= 1) acc += __shfl_xor(acc, off, 64);
      if (g == 0 && jvalid) o[((int64_t)(tc + tt) * H + h) * dv + j] = acc;
    }
  }
  if (jvalid) {
#pragma unroll
    for (int r = 0; r < GLA_ROWS; ++r) {
      const int i = g * GLA_ROWS + r;
      if (i < dk) S[(int64_t)i * dv + j] = s[r];
    }
  }
}

// out[t, h*dv + j] = o[t,h,j] / rms(o[t,h,:]) * w[j] * silu(gate[t, h*dv + j])
// one wave per (token, head)
template <typename T>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(
    T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ gate,
    int64_t gate_stride, const T* __restrict__ w, float eps, int rows, int H,
    int dv) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = row / H;
  const int h = row % H;
  const float* x = o + row * dv;
  float sq = 0.f;
  for (int i = lane; i < dv; i += 64) sq += x[i] * x[i];
  sq = wave_reduce_sum(sq);
  const float rinv = 1.0f / sqrtf(sq / (float)dv + eps);
  const T* gr = gate + t * gate_stride + h * dv;
  T* dst = out + row * dv;
  for (int i = lane; i < dv; i += 64) {
    const float gv = ldf(gr + i);
    const float sg = gv / (1.0f + expf(-gv));
    stf(dst + i, x[i] * rinv * ldf(w + i) * sg);
  }
}

template <typename T>
static void launch_gla_t(float* o, const void* q, const void* k, const void* v,
                         const void* z, int64_t q_stride, int64_t k_stride,
                         int64_t v_stride, int64_t z_stride, const void* z_bias,
                         float* state, const int64_t* slots, const int* cu,
                         const int* positions, int B, int H, int dk, int dv,
                         float inv_tau, float q_scale, hipStream_t stream) {
  int G = 1;
  while (G * GLA_ROWS < dk) G <<= 1;  // host checked dk <= 64 * GLA_ROWS
  const int C = 64 / G;
  const dim3 grid((dv + 4 * C - 1) / (4 * C), H, B);
  const size_t per_token = sizeof(float) * (size_t)(3 * G * GLA_ROWS + 4 * C);
  int TC = (int)((48 << 10) / per_token);
  TC = TC < 1 ? 1 : (TC > GLA_TC_MAX ? GLA_TC_MAX : TC);
  const size_t shm = per_token * TC;
  hipLaunchKernelGGL((gla_recurrence_kernel<T>), grid, dim3(256), shm, stream,
                     o, (const T*)q, (const T*)k, (const T*)v, (const T*)z,
                     q_stride, k_stride, v_stride, z_stride, (const T*)z_bias,
                     state, slots, cu, positions, H, dk, dv, G, TC,
                     inv_tau, q_scale);
}

extern "C" void launch_gla_recurrence(
    float* o, const void* q, const void* k, const void* v, const void* z,
    int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t z_stride,
    const void* z_bias, float* state, const int64_t* slots, const int* cu,
    const int* positions, int B, int H, int dk, int dv, float inv_tau,
    float q_scale, int kind, hipStream_t stream) {
  if (B == 0) return;
  if (kind == 0)
    launch_gla_t<bf16_t>(o, q, k, v, z, q_stride, k_stride, v_stride, z_stride,
                         z_bias, state, slots, cu, positions, B, H, dk, dv,
                         inv_tau, q_scale, stream);
  else
    launch_gla_t<float>(o, q, k, v, z, q_stride, k_stride, v_stride, z_stride,
                        z_bias, state, slots, cu, positions, B, H, dk, dv,
                        inv_tau, q_scale, stream);
}

extern "C" void launch_gated_rmsnorm(void* out, const float* o, const void* gate,
                                     int64_t gate_stride, const void* w,
                                     float eps, int rows, int H, int dv,
                                     int kind, hipStream_t stream) {
  if (rows == 0) return;
  const dim3 grid((rows + 3) / 4);
  if (kind == 0)
    hipLaunchKernelGGL((gated_rmsnorm_kernel<bf16_t>), grid, dim3(256), 0,
                       stream, (bf16_t*)out, o, (const bf16_t*)gate, gate_stride,
                       (const bf16_t*)w, eps, rows, H, dv);
  else
    hipLaunchKernelGGL((gated_rmsnorm_kernel<float>), grid, dim3(256), 0, stream,
                       (float*)out, o, (const float*)gate, gate_stride,
                       (const float*)w, eps, rows, H, dv);
}
