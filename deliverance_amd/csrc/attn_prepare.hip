// Queries, keys and values on their way from the q | k | v product to the attention kernels, in one pass over the
// product's 32-bit rows: the root-mean-square norm of queries and of keys (optional), the turn by the position
// (optional), the queries stored in the step's dtype, keys and values written to their cache rows.
//
//   norm, whole:     x <- x / sqrt(mean over all of the token's query (key) entries of x^2 + eps) * gain[entry]
//   norm, per head:  the same head by head, gain[entry within the head]
//   turn:            the first `dims` entries of every head in pairs, (2i, 2i + 1) when interleaved, else
//                    (i, i + dims / 2): (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * speeds[i]
//                    (speeds in double precision; sine and cosine of the double angle, used in 32-bit)
//
// `v_from_k`: the rows hold no values; a key as it was projected (normalised, not turned) is also the value (Dv = D).
// `pass_cols`: so many columns behind q | k | v of the rows (a gate's, say) go over into the queries' rows behind the
// queries, converted.  `mag` multiplies sine and cosine (the length that a turned pair gains; 1 as a rule).
//
// A page of the cache slot holds Hkv * page * D keys (rows of D), then Hkv * Dv * page values (dimension-major);
// slot_map[n] = page id * page + row, or -1 for a token whose keys are not kept.  One workgroup a token.
#include "common.h"

#define PREP_THREADS 256
#define PREP_MAX_HALF 128
#define PREP_MAX_GROUPS 256

template <typename T>
__global__ void __launch_bounds__(PREP_THREADS)
attn_prepare_kernel(const float* __restrict__ raw, int ld, int Hq, int Hkv, int D, int Dv, const void* __restrict__ gq,
                    int gq_dtype, const void* __restrict__ gk, int gk_dtype, float eps, int whole,
                    const int* __restrict__ positions, const double* __restrict__ speeds, int dims, int interleaved,
                    T* __restrict__ q_out, int q_ld, T* __restrict__ cache, const int* __restrict__ slot_map, int page,
                    int v_from_k, int pass_cols, float mag) {
  __shared__ float cs[PREP_MAX_HALF], sn[PREP_MAX_HALF];
  __shared__ float inv[PREP_MAX_GROUPS];               // queries' groups first, then the keys'
  const int n = blockIdx.x, lane = threadIdx.x % DA_WAVE, wave = threadIdx.x / DA_WAVE;
  const float* row = raw + (size_t)n * ld;
  const int half = dims / 2;
  const bool normed = gq != nullptr;
  const int q_groups = whole ? 1 : Hq, k_groups = whole ? 1 : Hkv;
  const int q_len = whole ? Hq * D : D, k_len = whole ? Hkv * D : D;
  if (dims > 0) {
    const double p = (double)positions[n];
    for (int i = threadIdx.x; i < half; i += PREP_THREADS) {
      double s, c;
      sincos(p * speeds[i], &s, &c);
      cs[i] = (float)c * mag;
      sn[i] = (float)s * mag;
    }
  }
  if (normed) {
    for (int g = wave; g < q_groups + k_groups; g += PREP_THREADS / DA_WAVE) {
      const bool is_q = g < q_groups;
      const float* v = is_q ? row + (size_t)g * q_len : row + Hq * D + (size_t)(g - q_groups) * k_len;
      const int len = is_q ? q_len : k_len;
      float ss = 0.f;
      for (int d = lane; d < len; d += DA_WAVE) ss = fmaf(v[d], v[d], ss);
      ss = wave_sum(ss);
      if (lane == 0) inv[g] = 1.0f / sqrtf(ss / (float)len + eps);
    }
  }
  __syncthreads();
  const int slot = (cache != nullptr && slot_map != nullptr) ? slot_map[n] : -1;
  const long long pg = slot >= 0 ? slot / page : 0;
  const int prow = slot >= 0 ? slot % page : 0;
  T* kbase = cache + pg * ((long long)Hkv * page * (D + Dv));
  // entries of queries, then of keys: entry d of head h, normalised, and its partner when it is turned
  const int total = (Hq + Hkv) * D;
  for (int idx = threadIdx.x; idx < total; idx += PREP_THREADS) {
    const bool is_q = idx < Hq * D;
    const int e = is_q ? idx : idx - Hq * D;           // entry within the queries / the keys
    const int h = e / D, d = e % D;
    if (!is_q && slot < 0) continue;
    const float* src = row + (is_q ? 0 : Hq * D);
    const void* gain = is_q ? gq : gk;
    const int gdt = is_q ? gq_dtype : gk_dtype;
    const float gi = normed ? inv[is_q ? (whole ? 0 : h) : q_groups + (whole ? 0 : h)] : 1.f;
    float val = src[e] * gi;
    if (normed) val *= load_param(gain, gdt, whole ? e : d);
    if (d < dims) {
      int i, other;
      bool first;
      if (interleaved) { i = d >> 1; first = (d & 1) == 0; other = d ^ 1; }
      else { first = d < half; i = first ? d : d - half; other = first ? d + half : d - half; }
      const int eo = h * D + other;
      float b = src[eo] * gi;
      if (normed) b *= load_param(gain, gdt, whole ? eo : other);
      val = first ? val * cs[i] - b * sn[i] : val * cs[i] + b * sn[i];
    }
    if (is_q) from_f32(&q_out[(size_t)n * q_ld + e], val);
    else from_f32(&kbase[((long long)h * page + prow) * D + d], val);
  }
  if (slot >= 0) {
    const float* v = row + (v_from_k ? Hq : Hq + Hkv) * D;
    T* vb = kbase + (long long)Hkv * page * D;
    for (int idx = threadIdx.x; idx < Hkv * Dv; idx += PREP_THREADS) {
      const int h = idx / Dv, d = idx % Dv;
      float val = v[idx];
      if (v_from_k && normed) val *= inv[q_groups + (whole ? 0 : h)] * load_param(gk, gk_dtype, whole ? idx : d);
      from_f32(&vb[((long long)h * Dv + d) * page + prow], val);
    }
  }
  const float* extra = row + (Hq + Hkv) * D + (v_from_k ? 0 : Hkv * Dv);
  for (int idx = threadIdx.x; idx < pass_cols; idx += PREP_THREADS) from_f32(&q_out[(size_t)n * q_ld + Hq * D + idx], extra[idx]);
}

extern "C" int da_attn_prepare(const float* raw, int ld, int Hq, int Hkv, int D, int Dv, const void* gq, int gq_dtype,
                               const void* gk, int gk_dtype, float eps, int whole, const int* positions,
                               const double* speeds, int dims, int interleaved, void* q_out, int out_dtype, int q_ld,
                               void* cache, const int* slot_map, int page, int N, int v_from_k, int pass_cols, float mag,
                               void* stream) {
  DA_REQUIRE(N >= 0 && Hq > 0 && Hkv > 0 && D > 0 && Dv > 0 && page > 0 && pass_cols >= 0, "attn_prepare: bad sizes");
  DA_REQUIRE(!v_from_k || Dv == D, "attn_prepare: values that are the keys have the keys' size %d, not %d", D, Dv);
  DA_REQUIRE(ld >= (Hq + Hkv) * D + (v_from_k ? 0 : Hkv * Dv) + pass_cols && q_ld >= Hq * D + pass_cols,
             "attn_prepare: row lengths too small");
  DA_REQUIRE((gq == nullptr) == (gk == nullptr), "attn_prepare: a norm needs both gains");
  DA_REQUIRE(gq == nullptr || eps > 0.f, "attn_prepare: the norm needs a positive eps");
  DA_REQUIRE(dims >= 0 && dims <= D && dims % 2 == 0 && dims / 2 <= PREP_MAX_HALF, "attn_prepare: %d turned entries of %d", dims, D);
  DA_REQUIRE(dims == 0 || (positions != nullptr && speeds != nullptr), "attn_prepare: a turn needs positions and speeds");
  DA_REQUIRE(whole || Hq + Hkv <= PREP_MAX_GROUPS, "attn_prepare: %d heads, %d norms are taken", Hq + Hkv, PREP_MAX_GROUPS);
  DA_REQUIRE(q_out != nullptr, "attn_prepare: the queries need a place");
  if (N == 0) return 0;
  if (out_dtype == DA_BF16)
    hipLaunchKernelGGL(attn_prepare_kernel<bf16_t>, dim3(N), dim3(PREP_THREADS), 0, (hipStream_t)stream, raw, ld, Hq, Hkv, D,
                       Dv, gq, gq_dtype, gk, gk_dtype, eps, whole, positions, speeds, dims, interleaved, (bf16_t*)q_out, q_ld,
                       (bf16_t*)cache, slot_map, page, v_from_k, pass_cols, mag);
  else
    hipLaunchKernelGGL(attn_prepare_kernel<float>, dim3(N), dim3(PREP_THREADS), 0, (hipStream_t)stream, raw, ld, Hq, Hkv, D,
                       Dv, gq, gq_dtype, gk, gk_dtype, eps, whole, positions, speeds, dims, interleaved, (float*)q_out, q_ld,
                       (float*)cache, slot_map, page, v_from_k, pass_cols, mag);
  DA_CHECK_LAUNCH("attn_prepare");
  return 0;
}
