// Sliding-window attention over a compressed latent cache.
//
// A cache entry is one row per token: [rank latent c | rot_w rotated key part],
// shared by every head. Queries arrive already absorbed into the latent space
// (q_lat = W_uk^T q_unrotated, fp32) plus their rotated part (fp32), so a score
// is   (q_lat . c + q_rot . k_rot) * scale   and the result is the softmax-
// weighted sum of the latent rows, which the caller expands through W_uv.
// Scores, softmax and the accumulation are fp32; only the cache rows have the
// activation type.
//
//   latent_kv_store : RMS norm of the latent + rotation of the key part +
//                     scatter into the paged cache, one kernel per layer.
//   rope_rows       : rotation of the queries' rotated part into an fp32 buffer.
//   latent_window_attention : one wave per (token, head), 64 keys per pass,
//                     online softmax. A token sees keys j with
//                     0 <= pos - j < window. Serves prompt portions and single
//                     decoded tokens alike (a decode row is a portion of one).
//
// Angles are computed in fp32 from a per-layer frequency vector: pair
// (i, i + rot_dims/2), a = pos * freq[i], cos and sin scaled by `mult`.
#include "seq_common.h"

template <typename T>
__global__ __launch_bounds__(128) void latent_kv_store_kernel(
    const T* __restrict__ dkv, int64_t dkv_stride, const T* __restrict__ norm_w,
    float eps, const float* __restrict__ freq, float mult, int rot_dims,
    const int* __restrict__ positions, const int64_t* __restrict__ slots,
    T* __restrict__ cache, int rank, int rot_w) {
  __shared__ float scratch[4];
  const int64_t t = blockIdx.x;
  const int64_t slot = slots[t];
  if (slot < 0) return;  // pad row of a captured graph
  const T* x = dkv + t * dkv_stride;
  T* dst = cache + slot * (int64_t)(rank + rot_w);
  float sq = 0.f;
  for (int i = threadIdx.x; i < rank; i += 128) {
    float v = ldf(x + i);
    sq += v * v;
  }
  sq = wave_reduce_sum(sq);
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = sq;
  __syncthreads();
  const float ms = (scratch[0] + scratch[1]) / (float)rank;
  const float rinv = 1.0f / sqrtf(ms + eps);
  for (int i = threadIdx.x; i < rank; i += 128) {
    stf(dst + i, ldf(x + i) * rinv * ldf(norm_w + i));
  }
  const int half = rot_dims >> 1;
  const float p = (float)positions[t];
  const T* kx = x + rank;
  T* kd = dst + rank;
  for (int i = threadIdx.x; i < half; i += 128) {
    float s, c;
    sincosf(p * freq[i], &s, &c);
    s *= mult;
    c *= mult;
    const float u = ldf(kx + i), v = ldf(kx + i + half);
    stf(kd + i, u * c - v * s);
    stf(kd + i + half, v * c + u * s);
  }
  for (int i = rot_dims + threadIdx.x; i < rot_w; i += 128) {
    stf(kd + i, ldf(kx + i));
  }
}

// q: [T, H, *] with the part to rotate at column `col0` of each head row
// (head stride `head_stride`, token stride `tok_stride`, in elements).
template <typename T>
__global__ __launch_bounds__(256) void rope_rows_kernel(
    float* __restrict__ out, const T* __restrict__ q, int64_t tok_stride,
    int64_t head_stride, int col0, const float* __restrict__ freq, float mult,
    int rot_dims, const int* __restrict__ positions, int H, int rot_w) {
  extern __shared__ float cs[];  // [rot_dims/2] cos, [rot_dims/2] sin
  const int64_t t = blockIdx.x;
  const int half = rot_dims >> 1;
  const float p = (float)positions[t];
  for (int i = threadIdx.x; i < half; i += 256) {
    float s, c;
    sincosf(p * freq[i], &s, &c);
    cs[i] = c * mult;
    cs[half + i] = s * mult;
  }
  __syncthreads();
  const int per_head = half + (rot_w - rot_dims);
  for (int idx = threadIdx.x; idx < H * per_head; idx += 256) {
    const int h = idx / per_head, i = idx % per_head;
    const T* src = q + t * tok_stride + h * head_stride + col0;
    float* dst = out + (t * H + h) * (int64_t)rot_w;
    if (i < half) {
      const float u = ldf(src + i), v = ldf(src + i + half);
      dst[i] = u * cs[i] - v * cs[half + i];
      dst[i + half] = v * cs[i] + u * cs[half + i];
    } else {
      const int k = rot_dims + (i - half);
      dst[k] = ldf(src + k);
    }
  }
}

#define LWA_WAVES 4
#define LWA_MAX_RF 16  // latent features per lane: rank <= 64 * LWA_MAX_RF

template <typename T, int RF>
__global__ __launch_bounds__(256) void latent_window_attention_kernel(
    float* __restrict__ out, const float* __restrict__ q_lat,
    const float* __restrict__ q_rot, const T* __restrict__ cache,
    const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ token_seq, const int* __restrict__ positions,
    int H, int rank, int rot_w, int block_size, int window, float scale) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = blockIdx.x;
  int h = blockIdx.y * LWA_WAVES + wave;
  const bool live = h < H;
  if (!live) h = H - 1;
  const int E = rank + rot_w;
  const int Ep = (E + 1) & ~1;  // keeps the int64 row offsets 8-byte aligned
  // per wave: q [Ep] | p [64] | row offsets [64] (as int64 -> 128 floats)
  float* qs = lds + wave * (Ep + 64 + 128);
  float* ps = qs + Ep;
  int64_t* rows = reinterpret_cast<int64_t*>(ps + 64);

  const float* ql = q_lat + (t * H + h) * (int64_t)rank;
  const float* qr = q_rot + (t * H + h) * (int64_t)rot_w;
  for (int f = lane; f < rank; f += 64) qs[f] = ql[f];
  for (int f = lane; f < rot_w; f += 64) qs[rank + f] = qr[f];

  const int b = token_seq ? token_seq[t] : (int)t;
  const int pos = positions[t];
  const int lo = max(0, pos - window + 1);
  const int* bt = block_tables + (int64_t)b * bt_stride;

  float m = -INFINITY, l = 0.f;
  float acc[RF];
#pragma unroll
  for (int k = 0; k < RF; ++k) acc[k] = 0.f;
  __syncthreads();

  for (int j0 = lo; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s = -INFINITY;
    int64_t off = 0;
    if (valid) {
      off = ((int64_t)bt[j / block_size] * block_size + j % block_size) * E;
      const T* row = cache + off;
      float d = 0.f;
      for (int f = 0; f < E; ++f) d = fmaf(qs[f], ldf(row + f), d);
      s = d * scale;
    }
    const float m_new = fmaxf(m, wave_reduce_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf at first: exp(-inf) = 0
    l = l * corr + wave_reduce_sum(p);
    m = m_new;
    ps[lane] = p;
    rows[lane] = off;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < RF; ++k) acc[k] *= corr;
    const int cnt = min(64, pos - j0 + 1);
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = ps[jj];
      const T* row = cache + rows[jj];
#pragma unroll
      for (int k = 0; k < RF; ++k) {
        const int f = lane + 64 * k;
        if (f < rank) acc[k] = fmaf(pj, ldf(row + f), acc[k]);
      }
    }
    __syncthreads();
  }
  if (live) {
    const float inv = 1.0f / l;
    float* o = out + (t * H + h) * (int64_t)rank;
#pragma unroll
    for (int k = 0; k < RF; ++k) {
      const int f = lane + 64 * k;
      if (f < rank) o[f] = acc[k] * inv;
    }
  }
}

extern "C" void launch_latent_kv_store(const void* dkv, int64_t dkv_stride,
                                       const void* norm_w, float eps,
                                       const float* freq, float mult,
                                       int rot_dims, const int* positions,
                                       const int64_t* slots, void* cache,
                                       int rank, int rot_w, int T, int kind,
                                       hipStream_t stream) {
  if (T == 0) return;
  if (kind == 0)
    hipLaunchKernelGGL((latent_kv_store_kernel<bf16_t>), dim3(T), dim3(128), 0,
                       stream, (const bf16_t*)dkv, dkv_stride,
                       (const bf16_t*)norm_w, eps, freq, mult, rot_dims,
                       positions, slots, (bf16_t*)cache, rank, rot_w);
  else
    hipLaunchKernelGGL((latent_kv_store_kernel<float>), dim3(T), dim3(128), 0,
                       stream, (const float*)dkv, dkv_stride,
                       (const float*)norm_w, eps, freq, mult, rot_dims,
                       positions, slots, (float*)cache, rank, rot_w);
}

extern "C" void launch_rope_rows(float* out, const void* q, int64_t tok_stride,
                                 int64_t head_stride, int col0,
                                 const float* freq, float mult, int rot_dims,
                                 const int* positions, int H, int rot_w, int T,
                                 int kind, hipStream_t stream) {
  if (T == 0) return;
  const size_t shm = sizeof(float) * (size_t)rot_dims;
  if (kind == 0)
    hipLaunchKernelGGL((rope_rows_kernel<bf16_t>), dim3(T), dim3(256), shm,
                       stream, out, (const bf16_t*)q, tok_stride, head_stride,
                       col0, freq, mult, rot_dims, positions, H, rot_w);
  else
    hipLaunchKernelGGL((rope_rows_kernel<float>), dim3(T), dim3(256), shm,
                       stream, out, (const float*)q, tok_stride, head_stride,
                       col0, freq, mult, rot_dims, positions, H, rot_w);
}

template <typename T>
static void launch_lwa_t(float* out, const float* q_lat, const float* q_rot,
                         const void* cache, const int* block_tables,
                         int bt_stride, const int* token_seq,
                         const int* positions, int T_, int H, int rank,
                         int rot_w, int block_size, int window, float scale,
                         hipStream_t stream) {
  const dim3 grid(T_, (H + LWA_WAVES - 1) / LWA_WAVES);
  const size_t shm =
      sizeof(float) * LWA_WAVES * (size_t)(((rank + rot_w + 1) & ~1) + 64 + 128);
  const int rf = (rank + 63) / 64;
#define LWA_LAUNCH(RF)                                                        \
  hipLaunchKernelGGL((latent_window_attention_kernel<T, RF>), grid, dim3(256), \
                     shm, stream, out, q_lat, q_rot, (const T*)cache,          \
                     block_tables, bt_stride, token_seq, positions, H, rank,   \
                     rot_w, block_size, window, scale)
  if (rf <= 1) LWA_LAUNCH(1);
  else if (rf <= 2) LWA_LAUNCH(2);
  else if (rf <= 4) LWA_LAUNCH(4);
  else if (rf <= 8) LWA_LAUNCH(8);
  else LWA_LAUNCH(LWA_MAX_RF);
#undef LWA_LAUNCH
}

extern "C" void launch_latent_window_attention(
    float* out, const float* q_lat, const float* q_rot, const void* cache,
    const int* block_tables, int bt_stride, const int* token_seq,
    const int* positions, int T, int H, int rank, int rot_w, int block_size,
    int window, float scale, int kind, hipStream_t stream) {
  if (T == 0) return;
  if (kind == 0)
    launch_lwa_t<bf16_t>(out, q_lat, q_rot, cache, block_tables, bt_stride,
                         token_seq, positions, T, H, rank, rot_w, block_size,
                         window, scale, stream);
  else
    launch_lwa_t<float>(out, q_lat, q_rot, cache, block_tables, bt_stride,
                        token_seq, positions, T, H, rank, rot_w, block_size,
                        window, scale, stream);
}
