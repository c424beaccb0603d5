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
//   latent_window_attention : a workgroup per (token, group of heads, share of
//                     the keys); 64 keys per wave and pass, online softmax,
//                     every cache row converted once for all heads of the
//                     group. A token sees keys j with 0 <= pos - j < window.
//                     Prompt portions run one share per token; decode rows
//                     split their window over several workgroups (fixed by
//                     host-known sizes, so captured graphs stay valid) and a
//                     small kernel joins the partial results.
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

// 8 consecutive cache elements as floats (one 16-byte load for bf16, two for
// float); p must be 16-byte aligned.
template <typename T>
DEVINL void load8(const T* p, float* v);
template <>
DEVINL void load8<bf16_t>(const bf16_t* p, float* v) {
  const bf16x8 raw = load_bf16x8(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = bf16x8_get(raw, i);
}
template <>
DEVINL void load8<float>(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// One workgroup = one token x one group of HB heads x one share of the keys.
// All heads read the same cache rows, so a row is loaded and converted once
// and used for HB heads. Score pass: a lane owns one key of a 64-key tile and
// walks the row's features in 16-byte steps against the HB queries in LDS.
// Value pass: a lane owns 8 consecutive latent features (x RC chunks of 512)
// and walks the tile's keys. The window's tiles are dealt round-robin to the
// 4 waves (x `splits` workgroups); each wave keeps its own online-softmax
// state and they merge at the end (through `part` when splits > 1).
// VEC: rows start 16-byte aligned and E is a multiple of 8 (else scalar loads).
template <typename T, int HB, int RC, bool VEC>
__global__ __launch_bounds__(256) void latent_window_attention_kernel(
    float* __restrict__ out, float* __restrict__ part,
    const float* __restrict__ q_lat, const float* __restrict__ q_rot,
    const T* __restrict__ cache, const int* __restrict__ block_tables,
    int bt_stride, const int* __restrict__ token_seq,
    const int* __restrict__ positions, int H, int rank, int rot_w,
    int block_size, int window, float scale, int splits) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = blockIdx.x;
  const int h0 = blockIdx.y * HB;
  const int split = blockIdx.z;
  const int E = rank + rot_w;
  const int Ep = (E + 7) & ~7;
  // LDS: q [HB][Ep] | per wave: p [HB][64], row offsets [64] (int64)
  float* qs = lds;
  float* ps = qs + HB * Ep + wave * (HB * 64 + 128);
  int64_t* rows = reinterpret_cast<int64_t*>(ps + HB * 64);

  for (int idx = threadIdx.x; idx < HB * Ep; idx += 256) {
    const int hh = idx / Ep, f = idx % Ep;
    const int h = min(h0 + hh, H - 1);
    float v = 0.f;
    if (f < rank) v = q_lat[(t * H + h) * (int64_t)rank + f];
    else if (f < E) v = q_rot[(t * H + h) * (int64_t)rot_w + (f - rank)];
    qs[idx] = v;
  }

  const int b = token_seq ? token_seq[t] : (int)t;
  const int pos = positions[t];
  const int lo = max(0, pos - window + 1);
  const int* bt = block_tables + (int64_t)b * bt_stride;

  float m[HB], l[HB], acc[HB][RC][8];
#pragma unroll
  for (int h = 0; h < HB; ++h) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int c = 0; c < RC; ++c)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[h][c][i] = 0.f;
  }
  __syncthreads();

  const int stride = 64 * LWA_WAVES * splits;
  for (int j0 = lo + 64 * (split * LWA_WAVES + wave); j0 <= pos; j0 += stride) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    int64_t off = 0;
    float s[HB];
#pragma unroll
    for (int h = 0; h < HB; ++h) s[h] = 0.f;
    if (valid) {
      off = ((int64_t)bt[j / block_size] * block_size + j % block_size) * E;
      const T* row = cache + off;
      if (VEC) {
        for (int f = 0; f < E; f += 8) {
          float kv[8];
          load8<T>(row + f, kv);
#pragma unroll
          for (int h = 0; h < HB; ++h) {
            const float4 qa = *reinterpret_cast<const float4*>(qs + h * Ep + f);
            const float4 qb = *reinterpret_cast<const float4*>(qs + h * Ep + f + 4);
            s[h] = fmaf(qa.x, kv[0], s[h]);
            s[h] = fmaf(qa.y, kv[1], s[h]);
            s[h] = fmaf(qa.z, kv[2], s[h]);
            s[h] = fmaf(qa.w, kv[3], s[h]);
            s[h] = fmaf(qb.x, kv[4], s[h]);
            s[h] = fmaf(qb.y, kv[5], s[h]);
            s[h] = fmaf(qb.z, kv[6], s[h]);
            s[h] = fmaf(qb.w, kv[7], s[h]);
          }
        }
      } else {
        for (int f = 0; f < E; ++f) {
          const float kv = ldf(row + f);
#pragma unroll
          for (int h = 0; h < HB; ++h) s[h] = fmaf(qs[h * Ep + f], kv, s[h]);
        }
      }
    }
    float corr[HB];
#pragma unroll
    for (int h = 0; h < HB; ++h) {
      const float sc = valid ? s[h] * scale : -INFINITY;
      const float m_new = fmaxf(m[h], wave_reduce_max(sc));  // finite: key j0 is valid
      const float p = valid ? expf(sc - m_new) : 0.f;
      corr[h] = expf(m[h] - m_new);  // exp(-inf) = 0 on the first tile
      l[h] = l[h] * corr[h] + wave_reduce_sum(p);
      m[h] = m_new;
      ps[h * 64 + lane] = p;
    }
    rows[lane] = off;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int h = 0; h < HB; ++h)
#pragma unroll
      for (int c = 0; c < RC; ++c)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[h][c][i] *= corr[h];
    const int cnt = min(64, pos - j0 + 1);
    for (int jj = 0; jj < cnt; ++jj) {
      const T* row = cache + rows[jj];
#pragma unroll
      for (int c = 0; c < RC; ++c) {
        const int f = c * 512 + lane * 8;
        if (f < rank) {
          float cv[8];
          if (VEC) {
            load8<T>(row + f, cv);
          } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) cv[i] = (f + i < rank) ? ldf(row + f + i) : 0.f;
          }
#pragma unroll
          for (int h = 0; h < HB; ++h) {
            const float pj = ps[h * 64 + jj];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[h][c][i] = fmaf(pj, cv[i], acc[h][c][i]);
          }
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }

  // ---- merge the 4 waves: common max, rescale, add up through LDS ----------------
  __syncthreads();  // q and the per-wave regions are free from here on
  float* wm = lds;                       // [4][HB]
  float* wl = wm + LWA_WAVES * HB;       // [4][HB]
  float* oacc = wl + LWA_WAVES * HB;     // [HB][rank_p], rank_p = RC * 512 cap
  if (lane == 0) {
#pragma unroll
    for (int h = 0; h < HB; ++h) wm[wave * HB + h] = m[h];
  }
  __syncthreads();
  float mg[HB], sc_w[HB];
#pragma unroll
  for (int h = 0; h < HB; ++h) {
    float x = wm[h];
    for (int w = 1; w < LWA_WAVES; ++w) x = fmaxf(x, wm[w * HB + h]);
    mg[h] = x;
    sc_w[h] = (m[h] == -INFINITY) ? 0.f : expf(m[h] - x);
  }
  if (lane == 0) {
#pragma unroll
    for (int h = 0; h < HB; ++h) wl[wave * HB + h] = l[h] * sc_w[h];
  }
  const int rank8 = (rank + 7) & ~7;
  for (int w = 0; w < LWA_WAVES; ++w) {
    if (wave == w) {
#pragma unroll
      for (int h = 0; h < HB; ++h)
#pragma unroll
        for (int c = 0; c < RC; ++c) {
          const int f = c * 512 + lane * 8;
          if (f < rank) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              float* dst = oacc + h * rank8 + f + i;
              const float v = acc[h][c][i] * sc_w[h];
              *dst = (w == 0) ? v : *dst + v;
            }
          }
        }
    }
    __syncthreads();
  }
  // every thread: write the merged result
  for (int idx = threadIdx.x; idx < HB * rank; idx += 256) {
    const int hh = idx / rank, f = idx % rank;
    const int h = h0 + hh;
    if (h >= H) continue;
    float lg = 0.f;
    for (int w = 0; w < LWA_WAVES; ++w) lg += wl[w * HB + hh];
    float mgh = wm[hh];
    for (int w = 1; w < LWA_WAVES; ++w) mgh = fmaxf(mgh, wm[w * HB + hh]);
    const float v = oacc[hh * rank8 + f];
    if (splits == 1) {
      out[(t * H + h) * (int64_t)rank + f] = v / lg;
    } else {
      float* pr = part + (((t * H + h) * (int64_t)splits + split) * (rank + 2));
      pr[2 + f] = v;
      if (f == 0) {
        pr[0] = mgh;
        pr[1] = lg;
      }
    }
  }
}

// out[t, h, :] from `splits` partial results [T, H, splits, 2 + rank]
__global__ __launch_bounds__(256) void latent_window_reduce_kernel(
    float* __restrict__ out, const float* __restrict__ part, int rank,
    int splits) {
  const int64_t th = blockIdx.x;
  const float* pr = part + th * splits * (int64_t)(rank + 2);
  float mg = -INFINITY;
  for (int s = 0; s < splits; ++s) mg = fmaxf(mg, pr[s * (rank + 2)]);
  float lg = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float ms = pr[s * (rank + 2)];
    lg += (ms == -INFINITY) ? 0.f : pr[s * (rank + 2) + 1] * expf(ms - mg);
  }
  for (int f = threadIdx.x; f < rank; f += 256) {
    float v = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float ms = pr[s * (rank + 2)];
      if (ms != -INFINITY) v += pr[s * (rank + 2) + 2 + f] * expf(ms - mg);
    }
    out[th * rank + f] = v / lg;
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

template <typename T, int HB, int RC>
static void launch_lwa_hb(float* out, float* part, const float* q_lat,
                          const float* q_rot, const void* cache,
                          const int* block_tables, int bt_stride,
                          const int* token_seq, const int* positions, int T_,
                          int H, int rank, int rot_w, int block_size, int window,
                          float scale, int splits, hipStream_t stream) {
  const int E = rank + rot_w;
  const int Ep = (E + 7) & ~7;
  const int rank8 = (rank + 7) & ~7;
  const size_t run = (size_t)HB * Ep + LWA_WAVES * (HB * 64 + 128);
  const size_t merge = 2 * LWA_WAVES * HB + (size_t)HB * rank8;
  const size_t shm = sizeof(float) * (run > merge ? run : merge);
  const dim3 grid(T_, (H + HB - 1) / HB, splits);
  const bool vec = (E % 8 == 0) && (sizeof(T) == 2 || E % 4 == 0);
  if (vec)
    hipLaunchKernelGGL((latent_window_attention_kernel<T, HB, RC, true>), grid,
                       dim3(256), shm, stream, out, part, q_lat, q_rot,
                       (const T*)cache, block_tables, bt_stride, token_seq,
                       positions, H, rank, rot_w, block_size, window, scale,
                       splits);
  else
    hipLaunchKernelGGL((latent_window_attention_kernel<T, HB, RC, false>), grid,
                       dim3(256), shm, stream, out, part, q_lat, q_rot,
                       (const T*)cache, block_tables, bt_stride, token_seq,
                       positions, H, rank, rot_w, block_size, window, scale,
                       splits);
  if (splits > 1)
    hipLaunchKernelGGL(latent_window_reduce_kernel, dim3(T_ * H), dim3(256), 0,
                       stream, out, part, rank, splits);
}

template <typename T>
static void launch_lwa_t(float* out, float* part, const float* q_lat,
                         const float* q_rot, const void* cache,
                         const int* block_tables, int bt_stride,
                         const int* token_seq, const int* positions, int T_,
                         int H, int rank, int rot_w, int block_size, int window,
                         float scale, int splits, hipStream_t stream) {
#define LWA_ARGS                                                             \
  out, part, q_lat, q_rot, cache, block_tables, bt_stride, token_seq,         \
      positions, T_, H, rank, rot_w, block_size, window, scale, splits, stream
  // heads per workgroup: 8 where the latent accumulators fit the registers
  // (rank <= 512), 4 above; fewer when the model has fewer heads
  if (rank <= 512) {
    if (H >= 8) launch_lwa_hb<T, 8, 1>(LWA_ARGS);
    else if (H >= 4) launch_lwa_hb<T, 4, 1>(LWA_ARGS);
    else if (H >= 2) launch_lwa_hb<T, 2, 1>(LWA_ARGS);
    else launch_lwa_hb<T, 1, 1>(LWA_ARGS);
  } else {
    if (H >= 4) launch_lwa_hb<T, 4, 2>(LWA_ARGS);
    else if (H >= 2) launch_lwa_hb<T, 2, 2>(LWA_ARGS);
    else launch_lwa_hb<T, 1, 2>(LWA_ARGS);
  }
#undef LWA_ARGS
}

extern "C" void launch_latent_window_attention(
    float* out, float* part, const float* q_lat, const float* q_rot,
    const void* cache, const int* block_tables, int bt_stride,
    const int* token_seq, const int* positions, int T, int H, int rank,
    int rot_w, int block_size, int window, float scale, int splits, int kind,
    hipStream_t stream) {
  if (T == 0) return;
  if (kind == 0)
    launch_lwa_t<bf16_t>(out, part, q_lat, q_rot, cache, block_tables,
                         bt_stride, token_seq, positions, T, H, rank, rot_w,
                         block_size, window, scale, splits, stream);
  else
    launch_lwa_t<float>(out, part, q_lat, q_rot, cache, block_tables, bt_stride,
                        token_seq, positions, T, H, rank, rot_w, block_size,
                        window, scale, splits, stream);
}
