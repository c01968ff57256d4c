// Plain paged attention with the extras that some designs put on the scores, and with keys and values
// of different sizes.  One wavefront per (token, query head), any mix of prompt rows and decode rows; it
// is this attention's true 32-bit path and the reference beside the matrix-core kernels.
//
// For the token at position p of its sequence, head h, key j in [lo, p]:
//   s_j = cap((q . k_j) * scale * temp(p)) + bias[h][min(p - j, n_dist - 1)]
//   temp(p) = 1 + t_coef * ln(floor((p + 1) / t_every) + 1)          (1 when t_every is 0)
//   cap(s) = softcap * tanh(s / softcap)                              (s itself when softcap is 0)
// With a window w the keys are j in [p - w + 1, p] and, with keep_first, also j < keep_first: the first keys of a
// sequence stay visible at their true positions.
//   w = softmax(s),  o = sum_j w_j v_j                                 (all in 32-bit)
// `sink` (optional, [Hq], 32-bit): the softmax's denominator also holds exp(sink[h]), a term without a key or a
// value that is not scaled.  `gate` (optional, rows like out): o <- o * logistic(gate).
// `bias` (optional) is a table by distance, [Hq][n_dist], 32-bit: whoever owns the rule that turns a
// distance into a learned value (buckets, slopes) writes it out once per layer up to the distance from
// which it no longer changes.
//
// One cache slot is [n_pages][ Hkv * page * D keys | Hkv * Dv * page values ]: keys of a (page, head) are
// page rows of D, values are Dv runs of `page` (dimension-major).  With D == Dv this is the layout of
// common.h.  Keys are walked in chunks of 64 starting at lo, so the order of the sums depends only on the
// token's own position.
#include "common.h"

#define REL_MAX_D 256

template <typename T>
__global__ void __launch_bounds__(DA_WAVE)
attn_rel_ref_kernel(const T* __restrict__ q, int q_ld, const T* __restrict__ cache,
                    const int* __restrict__ block_table, int max_blocks,
                    const int* __restrict__ seq_of_token, const int* __restrict__ positions,
                    int Hq, int Hkv, int D, int Dv, int page, float scale, int window,
                    const float* __restrict__ bias, int n_dist, float t_coef, int t_every, float softcap, int keep_first,
                    const float* __restrict__ sink, const T* __restrict__ gate, int gate_ld,
                    T* __restrict__ out, int out_ld) {
  __shared__ float qs[REL_MAX_D];
  __shared__ float ps[DA_WAVE];
  __shared__ long long voff[DA_WAVE];
  const int lane = threadIdx.x;
  const int n = blockIdx.x / Hq, h = blockIdx.x % Hq;
  const int hk = h / (Hq / Hkv);
  const int p = positions[n];
  const int* bt = block_table + (size_t)seq_of_token[n] * max_blocks;
  const long long page_elems = (long long)Hkv * page * (D + Dv);
  const long long v0 = (long long)Hkv * page * D + (long long)hk * page * Dv;
  const float* brow = bias ? bias + (size_t)h * n_dist : nullptr;
  const float temp = t_every > 0 ? 1.0f + t_coef * logf((float)((p + 1) / t_every + 1)) : 1.0f;
  const float qscale = scale * temp;

  for (int d = lane; d < D; d += DA_WAVE) qs[d] = to_f32(q[(size_t)n * q_ld + h * D + d]);
  __syncthreads();

  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  float m = -INFINITY, l = 0.f;
  float acc[REL_MAX_D / DA_WAVE];
#pragma unroll
  for (int i = 0; i < REL_MAX_D / DA_WAVE; ++i) acc[i] = 0.f;

  // two runs of keys: the kept first ones that the window has left behind, then the window itself
  const int kept = keep_first < lo ? keep_first : lo;
  for (int run = 0; run < 2; ++run) {
  const int first = run == 0 ? 0 : lo, last = run == 0 ? kept - 1 : p;
  for (int c0 = first; c0 <= last; c0 += DA_WAVE) {
    const int key = c0 + lane;
    const bool valid = key <= last && bt[key / page] >= 0;
    float s = -INFINITY;
    if (valid) {
      const long long pg = bt[key / page];
      const int row = key % page;
      const T* kr = cache + pg * page_elems + ((long long)hk * page + row) * D;
      voff[lane] = pg * page_elems + v0 + row;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f32(kr[d]), dot);
      s = dot * qscale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      if (brow) {
        const int dist = p - key;
        s += brow[dist < n_dist ? dist : n_dist - 1];
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float e = valid ? expf(s - m_new) : 0.f;
    const float alpha = m_new == -INFINITY ? 1.f : expf(m - m_new);
    l = l * alpha + wave_sum(e);
    m = m_new;
    ps[lane] = e;
    __syncthreads();
    const int cnt = (last - c0 + 1 < DA_WAVE) ? last - c0 + 1 : DA_WAVE;
#pragma unroll
    for (int i = 0; i < REL_MAX_D / DA_WAVE; ++i) {
      const int d = lane + i * DA_WAVE;
      if (d < Dv) {
        float a = acc[i] * alpha;
        for (int j = 0; j < cnt; ++j) {
          const float pj = ps[j];                  // 0 for a key that is not seen: its row is not read
          if (pj != 0.f) a = fmaf(pj, to_f32(cache[voff[j] + (long long)d * page]), a);
        }
        acc[i] = a;
      }
    }
    __syncthreads();
  }
  }
  float shrink = 1.f;
  if (sink) {                                            // one more term of the denominator, counted once
    const float s0 = sink[h];
    const float m_all = fmaxf(m, s0);
    shrink = m == -INFINITY ? 0.f : expf(m - m_all);
    l = l * shrink + expf(s0 - m_all);
  }
  const float inv = l > 0.f ? shrink / l : 0.f;
#pragma unroll
  for (int i = 0; i < REL_MAX_D / DA_WAVE; ++i) {
    const int d = lane + i * DA_WAVE;
    if (d < Dv) {
      float r = acc[i] * inv;
      if (gate) r *= 1.0f / (1.0f + expf(-to_f32(gate[(size_t)n * gate_ld + h * Dv + d])));
      from_f32(&out[(size_t)n * out_ld + h * Dv + d], r);
    }
  }
}

extern "C" int da_attn_rel_ref(const void* q, int q_ld, const void* cache, int dtype, const int* block_table,
                               int max_blocks, const int* seq_of_token, const int* positions, int N, int Hq, int Hkv,
                               int D, int Dv, int page, float scale, int window, const float* bias, int n_dist,
                               float t_coef, int t_every, float softcap, int keep_first, const float* sink,
                               const void* gate, int gate_ld, void* out, int out_ld, void* stream) {
  DA_REQUIRE(N >= 0 && Hq > 0 && Hkv > 0 && D > 0 && Dv > 0 && page > 0, "attn_rel_ref: bad sizes");
  DA_REQUIRE(Hq % Hkv == 0, "attn_rel_ref: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  DA_REQUIRE(D <= REL_MAX_D && Dv <= REL_MAX_D, "attn_rel_ref: head sizes %d, %d exceed %d", D, Dv, REL_MAX_D);
  DA_REQUIRE(q_ld >= Hq * D && out_ld >= Hq * Dv, "attn_rel_ref: row lengths too small");
  DA_REQUIRE(window >= 0 && max_blocks > 0, "attn_rel_ref: bad window or block table");
  DA_REQUIRE(!bias || n_dist > 0, "attn_rel_ref: a bias table without entries");
  DA_REQUIRE(t_every >= 0, "attn_rel_ref: bad temperature period %d", t_every);
  DA_REQUIRE(softcap >= 0.f && keep_first >= 0, "attn_rel_ref: bad score cap or kept first keys");
  DA_REQUIRE(!gate || gate_ld >= Hq * Dv, "attn_rel_ref: the gate's rows are too short");
  if (N == 0) return 0;
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(attn_rel_ref_kernel<bf16_t>, dim3(N * Hq), dim3(DA_WAVE), 0, (hipStream_t)stream,
                       (const bf16_t*)q, q_ld, (const bf16_t*)cache, block_table, max_blocks, seq_of_token, positions,
                       Hq, Hkv, D, Dv, page, scale, window, bias, n_dist, t_coef, t_every, softcap, keep_first, sink,
                       (const bf16_t*)gate, gate_ld, (bf16_t*)out, out_ld);
  else
    hipLaunchKernelGGL(attn_rel_ref_kernel<float>, dim3(N * Hq), dim3(DA_WAVE), 0, (hipStream_t)stream,
                       (const float*)q, q_ld, (const float*)cache, block_table, max_blocks, seq_of_token, positions,
                       Hq, Hkv, D, Dv, page, scale, window, bias, n_dist, t_coef, t_every, softcap, keep_first, sink,
                       (const float*)gate, gate_ld, (float*)out, out_ld);
  DA_CHECK_LAUNCH("attn_rel_ref");
  return 0;
}

// Keys (D a head) and values (Dv a head) of the step's tokens go to their cache rows; slot_map[n] is
// page_id * page + row, or -1 for a token whose keys are not kept.  One workgroup a token.
template <typename T>
__global__ void kv_write_split_kernel(const T* __restrict__ qkv, int ld, int k_off, int v_off, T* __restrict__ cache,
                                      const int* __restrict__ slot_map, int Hkv, int D, int Dv, int page) {
  const int n = blockIdx.x;
  const int slot = slot_map[n];
  if (slot < 0) return;
  const long long pg = slot / page;
  const int row = slot % page;
  T* base = cache + pg * ((long long)Hkv * page * (D + Dv));
  const T* src = qkv + (size_t)n * ld;
  for (int i = threadIdx.x; i < Hkv * D; i += blockDim.x) {
    const int hk = i / D, d = i % D;
    base[((long long)hk * page + row) * D + d] = src[k_off + i];
  }
  T* vb = base + (long long)Hkv * page * D;
  for (int i = threadIdx.x; i < Hkv * Dv; i += blockDim.x) {
    const int hk = i / Dv, d = i % Dv;
    vb[((long long)hk * Dv + d) * page + row] = src[v_off + i];
  }
}

extern "C" int da_kv_write_split(const void* qkv, int dtype, int ld, int k_off, int v_off, void* cache,
                                 const int* slot_map, int N, int Hkv, int D, int Dv, int page, void* stream) {
  DA_REQUIRE(N >= 0 && Hkv > 0 && D > 0 && Dv > 0 && page > 0, "kv_write_split: bad sizes");
  DA_REQUIRE(k_off >= 0 && v_off >= 0 && k_off + Hkv * D <= ld && v_off + Hkv * Dv <= ld,
             "kv_write_split: the key or value columns leave the row");
  if (N == 0) return 0;
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(kv_write_split_kernel<bf16_t>, dim3(N), dim3(128), 0, (hipStream_t)stream, (const bf16_t*)qkv, ld,
                       k_off, v_off, (bf16_t*)cache, slot_map, Hkv, D, Dv, page);
  else
    hipLaunchKernelGGL(kv_write_split_kernel<float>, dim3(N), dim3(128), 0, (hipStream_t)stream, (const float*)qkv, ld,
                       k_off, v_off, (float*)cache, slot_map, Hkv, D, Dv, page);
  DA_CHECK_LAUNCH("kv_write_split");
  return 0;
}
