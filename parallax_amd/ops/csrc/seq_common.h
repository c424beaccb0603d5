// Shared helpers of the sequence-mixer kernels (layer norm with fp32 residual,
// sliding-window latent attention, gated linear attention). Every kernel is
// templated on the activation type: bf16 (stored as uint16_t bits) or float.
// What a design wants in 32-bit (scores, softmax, norms, decays, recurrent
// state, the residual sum) is fp32 in both instantiations.
#pragma once

#include "common.h"

typedef uint16_t bf16_t;

template <typename T>
DEVINL float ldf(const T* p);
template <>
DEVINL float ldf<float>(const float* p) {
  return *p;
}
template <>
DEVINL float ldf<bf16_t>(const bf16_t* p) {
  return bf16_bits_to_f32(*p);
}

template <typename T>
DEVINL void stf(T* p, float v);
template <>
DEVINL void stf<float>(float* p, float v) {
  *p = v;
}
template <>
DEVINL void stf<bf16_t>(bf16_t* p, float v) {
  *p = f32_to_bf16_bits(v);
}

// sum over a 256-thread block; every thread gets the result. `scratch` holds
// at least 8 floats and may be reused right after the call returns.
DEVINL float block256_sum(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  v = wave_reduce_sum(v);
  __syncthreads();  // scratch may still be read from a previous call
  if (lane == 0) scratch[wid] = v;
  __syncthreads();
  const int nw = (blockDim.x + 63) >> 6;
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += scratch[i];
  return r;
}
