// Attention over one narrow vector a token ("latent attention") and the rotation of neighbouring pairs.
//
// A token keeps one row of D = R + Dr entries in the cache: R entries of a normalised latent c, from which
// every head's keys and values are linear maps, and Dr entries of a key piece that is turned by the position
// and shared by all heads.  With the heads' key maps folded into the queries (q'_h = [Wk_h^T q_h | turned
// q_h]) the score of head h is q'_h . row, and with the value maps applied afterwards the weighted sum is
// taken over the first R entries of the rows: all heads read the same rows, once as keys and once as values.
//
//   da_rotary          dst[n, h, :] = src[n, h, :] with the first `dims` entries turned in pairs by the position
//   da_latent_prepare  from the down-projection's row [ query latent | c | key piece ]: both norms, the turn of
//                      the key piece, the cache write, and the normalised query latent
//   da_attn_latent_ref plain attention over the rows, one wavefront per (token, head), any dtype
//
// A latent cache slot is [n_pages][page][D], rows of D entries.  Angles are position * speed_i with the
// speeds given in double precision; sine and cosine are taken of the double angle and used in 32-bit.
#include "common.h"

#define LAT_MAX_D 1024
#define ROT_MAX_HALF 256

// (2i, 2i + 1) -> (u cos - v sin, v cos + u sin) when `interleaved`, else the pair is (i, i + dims / 2)
template <typename T>
__global__ void __launch_bounds__(128)
rotary_kernel(const T* __restrict__ src, int src_ld, int src_hs, T* __restrict__ dst, int dst_ld, int dst_hs,
              const int* __restrict__ positions, const double* __restrict__ speeds, int H, int width, int dims,
              int interleaved, float mag) {
  __shared__ float cs[ROT_MAX_HALF], sn[ROT_MAX_HALF];
  const int n = blockIdx.x, half = dims / 2;
  const double p = (double)positions[n];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    double s, c;
    sincos(p * speeds[i], &s, &c);
    cs[i] = (float)c * mag;                             // (mag: the length that a turned pair gains; 1 as a rule)
    sn[i] = (float)s * mag;
  }
  __syncthreads();
  const T* in = src + (size_t)n * src_ld;
  T* out = dst + (size_t)n * dst_ld;
  // a thread owns a whole pair (both reads come before both writes), so src and dst may be one place
  for (int idx = threadIdx.x; idx < H * width; idx += blockDim.x) {
    const int h = idx / width, d = idx % width;
    const T* v = in + (size_t)h * src_hs;
    T* o = out + (size_t)h * dst_hs;
    if (d >= dims) {
      from_f32(&o[d], to_f32(v[d]));
      continue;
    }
    const bool first = interleaved ? (d & 1) == 0 : d < half;
    if (!first) continue;
    const int i = interleaved ? d >> 1 : d;
    const int other = interleaved ? d + 1 : d + half;
    const float a = to_f32(v[d]), b = to_f32(v[other]);
    from_f32(&o[d], a * cs[i] - b * sn[i]);
    from_f32(&o[other], b * cs[i] + a * sn[i]);
  }
}

extern "C" int da_rotary(const void* src, int src_ld, int src_hs, void* dst, int dst_ld, int dst_hs, int dtype,
                         const int* positions, const double* speeds, int N, int H, int width, int dims, int interleaved,
                         float mag, void* stream) {
  DA_REQUIRE(N >= 0 && H > 0 && width > 0 && dims >= 0 && dims <= width && dims % 2 == 0, "rotary: bad sizes");
  DA_REQUIRE(dims / 2 <= ROT_MAX_HALF, "rotary: %d turned entries, %d are taken", dims, 2 * ROT_MAX_HALF);
  DA_REQUIRE(src_ld >= (H - 1) * src_hs + width && dst_ld >= (H - 1) * dst_hs + width && src_hs >= width && dst_hs >= width,
             "rotary: the heads leave the row");
  if (N == 0) return 0;
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(rotary_kernel<bf16_t>, dim3(N), dim3(128), 0, (hipStream_t)stream, (const bf16_t*)src, src_ld, src_hs,
                       (bf16_t*)dst, dst_ld, dst_hs, positions, speeds, H, width, dims, interleaved, mag);
  else
    hipLaunchKernelGGL(rotary_kernel<float>, dim3(N), dim3(128), 0, (hipStream_t)stream, (const float*)src, src_ld, src_hs,
                       (float*)dst, dst_ld, dst_hs, positions, speeds, H, width, dims, interleaved, mag);
  DA_CHECK_LAUNCH("rotary");
  return 0;
}

// One workgroup of two wavefronts a token.  Wavefront 0: cq = rms(row[0 .. Rq)) * gq.  Wavefront 1: the cache
// row [ rms(row[Rq .. Rq + R)) * gc | turn(row[Rq + R .. Rq + R + Dr)) ].  Norms in 32-bit, eps under the root.
template <typename TIN, typename TOUT>
__global__ void __launch_bounds__(128)
latent_prepare_kernel(const TIN* __restrict__ down, int ld, int Rq, int R, int Dr, const void* __restrict__ gq,
                      int gq_dtype, const void* __restrict__ gc, int gc_dtype, float eps,
                      const int* __restrict__ positions, const int* __restrict__ slot_map,
                      const double* __restrict__ speeds, int dims, int interleaved, float mag, TOUT* __restrict__ cq,
                      int cq_ld, TOUT* __restrict__ cache, int page) {
  const int n = blockIdx.x, lane = threadIdx.x % DA_WAVE, wave = threadIdx.x / DA_WAVE;
  const TIN* row = down + (size_t)n * ld;
  if (wave == 0) {
    if (Rq <= 0) return;
    float ss = 0.f;
    for (int d = lane; d < Rq; d += DA_WAVE) { const float v = to_f32(row[d]); ss = fmaf(v, v, ss); }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)Rq + eps);
    for (int d = lane; d < Rq; d += DA_WAVE)
      from_f32(&cq[(size_t)n * cq_ld + d], to_f32(row[d]) * inv * load_param(gq, gq_dtype, d));
    return;
  }
  const int slot = slot_map ? slot_map[n] : -1;
  if (slot < 0) return;                               // a row whose keys are not kept
  TOUT* dst = cache + (size_t)slot * (R + Dr);       // slot = page id * page + row, rows of D entries
  const TIN* c = row + Rq;
  float ss = 0.f;
  for (int d = lane; d < R; d += DA_WAVE) { const float v = to_f32(c[d]); ss = fmaf(v, v, ss); }
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)R + eps);
  for (int d = lane; d < R; d += DA_WAVE) from_f32(&dst[d], to_f32(c[d]) * inv * load_param(gc, gc_dtype, d));
  const TIN* kr = c + R;
  const int half = dims / 2;
  const double p = (double)positions[n];
  for (int d = lane; d < Dr; d += DA_WAVE) {
    float r;
    if (d >= dims) {
      r = to_f32(kr[d]);
    } else {
      int i, other;
      bool first;
      if (interleaved) { i = d >> 1; first = (d & 1) == 0; other = d ^ 1; }
      else { first = d < half; i = first ? d : d - half; other = first ? d + half : d - half; }
      double s, co;
      sincos(p * speeds[i], &s, &co);
      const float a = to_f32(kr[d]), b = to_f32(kr[other]);
      const float cf = (float)co * mag, sf = (float)s * mag;
      r = first ? a * cf - b * sf : a * cf + b * sf;
    }
    from_f32(&dst[R + d], r);
  }
}

extern "C" int da_latent_prepare(const void* down, int in_dtype, int ld, int Rq, int R, int Dr, const void* gq, int gq_dtype,
                                 const void* gc, int gc_dtype, float eps, const int* positions, const int* slot_map,
                                 const double* speeds, int dims, int interleaved, float mag, void* cq, int cq_ld,
                                 void* cache, int out_dtype, int page, int N, void* stream) {
  DA_REQUIRE(N >= 0 && Rq >= 0 && R > 0 && Dr >= 0 && ld >= Rq + R + Dr && page > 0, "latent_prepare: bad sizes");
  DA_REQUIRE(dims >= 0 && dims <= Dr && dims % 2 == 0, "latent_prepare: %d turned entries of %d", dims, Dr);
  DA_REQUIRE(Rq == 0 || (cq != nullptr && cq_ld >= Rq && gq != nullptr), "latent_prepare: the query latent needs a gain and a place");
  DA_REQUIRE(eps > 0.f && gc != nullptr && positions != nullptr, "latent_prepare: missing operands");
  if (N == 0) return 0;
#define DA_LP_GO(TIN, TOUT)                                                                                              \
  hipLaunchKernelGGL((latent_prepare_kernel<TIN, TOUT>), dim3(N), dim3(128), 0, (hipStream_t)stream, (const TIN*)down, ld, \
                     Rq, R, Dr, gq, gq_dtype, gc, gc_dtype, eps, positions, slot_map, speeds, dims, interleaved, mag,     \
                     (TOUT*)cq, cq_ld, (TOUT*)cache, page)
  if (in_dtype == DA_F32 && out_dtype == DA_F32) DA_LP_GO(float, float);
  else if (in_dtype == DA_F32) DA_LP_GO(float, bf16_t);
  else if (out_dtype == DA_BF16) DA_LP_GO(bf16_t, bf16_t);
  else DA_REQUIRE(false, "latent_prepare: a bfloat16 row into a 32-bit cache is not taken");
#undef DA_LP_GO
  DA_CHECK_LAUNCH("latent_prepare");
  return 0;
}

// For the token at position p, head h, rows j in [lo, p] of its sequence:
//   s_j = (q'[n, h, :] . row_j) * scale,  w = softmax(s),  o[n, h, :] = sum_j w_j row_j[0 .. Dv)        (32-bit)
// With `sink` ([Hq], 32-bit) the softmax's denominator also holds exp(sink[h]): no key, no value, not scaled.
// Rows are walked in chunks of 64 from lo, so the order of the sums depends on the token's position only.
template <typename T>
__global__ void __launch_bounds__(DA_WAVE)
attn_latent_ref_kernel(const T* __restrict__ q, int q_ld, const T* __restrict__ cache, const int* __restrict__ block_table,
                       int max_blocks, const int* __restrict__ seq_of_token, const int* __restrict__ positions, int Hq,
                       int D, int Dv, int page, float scale, int window, const float* __restrict__ sink,
                       T* __restrict__ out, int out_ld) {
  __shared__ float qs[LAT_MAX_D];
  __shared__ float ps[DA_WAVE];
  __shared__ long long roff[DA_WAVE];
  const int lane = threadIdx.x;
  const int n = blockIdx.x / Hq, h = blockIdx.x % Hq;
  const int p = positions[n];
  const int* bt = block_table + (size_t)seq_of_token[n] * max_blocks;
  for (int d = lane; d < D; d += DA_WAVE) qs[d] = to_f32(q[(size_t)n * q_ld + (size_t)h * D + d]);
  __syncthreads();
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  float m = -INFINITY, l = 0.f;
  float acc[LAT_MAX_D / DA_WAVE];
#pragma unroll
  for (int i = 0; i < LAT_MAX_D / DA_WAVE; ++i) acc[i] = 0.f;
  for (int c0 = lo; c0 <= p; c0 += DA_WAVE) {
    const int key = c0 + lane;
    const bool valid = key <= p && bt[key / page] >= 0;
    float s = -INFINITY;
    if (valid) {
      const long long off = ((long long)bt[key / page] * page + key % page) * D;
      roff[lane] = off;
      const T* kr = cache + off;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f32(kr[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float e = valid ? expf(s - m_new) : 0.f;
    const float alpha = m_new == -INFINITY ? 1.f : expf(m - m_new);
    l = l * alpha + wave_sum(e);
    m = m_new;
    ps[lane] = e;
    __syncthreads();
    const int cnt = (p - c0 + 1 < DA_WAVE) ? p - c0 + 1 : DA_WAVE;
#pragma unroll
    for (int i = 0; i < LAT_MAX_D / DA_WAVE; ++i) {
      const int d = lane + i * DA_WAVE;
      if (d < Dv) {
        float a = acc[i] * alpha;
        for (int j = 0; j < cnt; ++j) {
          const float pj = ps[j];                  // 0 for a row that is not seen: it is not read
          if (pj != 0.f) a = fmaf(pj, to_f32(cache[roff[j] + d]), a);
        }
        acc[i] = a;
      }
    }
    __syncthreads();
  }
  float shrink = 1.f;
  if (sink) {
    const float s0 = sink[h];
    const float m_all = fmaxf(m, s0);
    shrink = m == -INFINITY ? 0.f : expf(m - m_all);
    l = l * shrink + expf(s0 - m_all);
  }
  const float inv = l > 0.f ? shrink / l : 0.f;
#pragma unroll
  for (int i = 0; i < LAT_MAX_D / DA_WAVE; ++i) {
    const int d = lane + i * DA_WAVE;
    if (d < Dv) from_f32(&out[(size_t)n * out_ld + (size_t)h * Dv + d], acc[i] * inv);
  }
}

extern "C" int da_attn_latent_ref(const void* q, int q_ld, const void* cache, int dtype, const int* block_table,
                                  int max_blocks, const int* seq_of_token, const int* positions, int N, int Hq, int D,
                                  int Dv, int page, float scale, int window, const float* sink, void* out, int out_ld,
                                  void* stream) {
  DA_REQUIRE(N >= 0 && Hq > 0 && D > 0 && Dv > 0 && Dv <= D && page > 0, "attn_latent_ref: bad sizes");
  DA_REQUIRE(D <= LAT_MAX_D, "attn_latent_ref: rows of %d entries, %d are taken", D, LAT_MAX_D);
  DA_REQUIRE(q_ld >= Hq * D && out_ld >= Hq * Dv, "attn_latent_ref: row lengths too small");
  DA_REQUIRE(window >= 0 && max_blocks > 0, "attn_latent_ref: bad window or block table");
  if (N == 0) return 0;
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(attn_latent_ref_kernel<bf16_t>, dim3(N * Hq), dim3(DA_WAVE), 0, (hipStream_t)stream, (const bf16_t*)q,
                       q_ld, (const bf16_t*)cache, block_table, max_blocks, seq_of_token, positions, Hq, D, Dv, page, scale,
                       window, sink, (bf16_t*)out, out_ld);
  else
    hipLaunchKernelGGL(attn_latent_ref_kernel<float>, dim3(N * Hq), dim3(DA_WAVE), 0, (hipStream_t)stream, (const float*)q,
                       q_ld, (const float*)cache, block_table, max_blocks, seq_of_token, positions, Hq, D, Dv, page, scale,
                       window, sink, (float*)out, out_ld);
  DA_CHECK_LAUNCH("attn_latent_ref");
  return 0;
}
