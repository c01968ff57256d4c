// Latent attention on the matrix cores (bfloat16): prompt portions and single decoded tokens in one form.
//
// All heads of a token read the same cache rows, so the query rows of a workgroup are (token, head) pairs of one
// sequence: 64 of them, 16 a wavefront, which for decoding is up to 64 heads of one token.  The rows of a tile of
// 32 cached tokens go from memory into LDS once, row-major for the scores S = Q' K^T and, their first R entries,
// dimension-major for O = P V (the matrix cores contract over 8 consecutive entries of a lane, which are entries of
// a row for the scores and tokens for the weighted sums).  MFMA 16x16x32: a lane's fragment is 8 consecutive k of
// row (or column) lane % 16, k starting at 8 (lane / 16); result r of a lane is row 4 (lane / 16) + r, column
// lane % 16.  The softmax runs over a wavefront's own 16 rows in 32-bit; the weights pass through LDS to become
// the first operand of the second product.  The next tile's rows are asked for before this tile's arithmetic.
// Tiles are walked from the first visible key in steps of 32, so the order of a row's sums depends on the row's
// own sequence only.  With `sink` ([H], 32-bit) the softmax's denominator also holds exp(sink[head]), which has no
// key and no value and is not scaled; it joins once, where a row's result is final (here, or in the merge).
#include "gemm_common.h"

#define LM_ROWS 64            // query rows a workgroup
#define LM_KEYS 32            // cached tokens a tile
#define LM_PAD 8
#define LM_BT 2048            // entries of a block table that LDS holds

template <int DB, int RB>     // DB: blocks of 32 entries of a cache row (padded), RB: blocks of 16 entries of R
__global__ void __launch_bounds__(256)
attn_latent_mfma_kernel(const bf16_t* __restrict__ q, int q_ld, const bf16_t* __restrict__ cache,
                        const int* __restrict__ block_table, int max_blocks, const int* __restrict__ q_start,
                        const int* __restrict__ seq_lens, int H, int D, int R, int page, float scale_log2e, int window,
                        bf16_t* __restrict__ out, int out_ld, int seq0, int n_splits, float* __restrict__ partial,
                        const float* __restrict__ sink) {
  constexpr int D32 = DB * 32;
  constexpr int ldk = D32 + LM_PAD;                   // entries of a row of the key tile
  constexpr int ldv = LM_KEYS + LM_PAD;               // entries of a row of the value tile (one entry of R)
  __shared__ __attribute__((aligned(16))) bf16_t Ks[LM_KEYS * ldk];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[16 * RB * ldv];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4 * 16 * ldv];
  __shared__ int pages[LM_BT];                        // the sequence's block table (its first LM_BT entries)

  const int s = seq0 + blockIdx.y;
  const int first = q_start[s], T = q_start[s + 1] - first;
  const int row0 = blockIdx.x * LM_ROWS;
  if (row0 >= T * H) return;
  const int len = seq_lens[s];                        // the sequence's length after this step
  const int past = len - T;                           // position of the portion's first token
  const int t = threadIdx.x, lane = t % DA_WAVE, wave = t / DA_WAVE;
  const int fr = lane % 16, fg = lane / 16;
  const int* bt = block_table + (size_t)s * max_blocks;
  const int page_shift = 31 - __builtin_clz(page);    // (a page holds a power of two of tokens)

  // this lane's fragment row, and the four rows whose results it holds
  const int arow = row0 + wave * 16 + fr;
  const bool arow_ok = arow < T * H;
  const bf16_t* qp = q + (size_t)(first + (arow_ok ? arow / H : 0)) * q_ld + (size_t)(arow_ok ? arow % H : 0) * D + fg * 8;
  uint4 qf[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)                        // all asked for at once, from places that exist; masked below
    qf[i] = load16(i * 32 + fg * 8 < D ? qp + i * 32 : qp - fg * 8);
#pragma unroll
  for (int i = 0; i < DB; ++i)
    if (!(arow_ok && i * 32 + fg * 8 < D)) qf[i] = make_uint4(0, 0, 0, 0);
  int pos[4];                                         // positions of the rows whose results this lane holds (-1: none)
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = row0 + wave * 16 + 4 * fg + r;
    pos[r] = row < T * H ? past + row / H : -1;
  }
  // the keys this workgroup walks: from the first one its first row sees to the last one its last row sees
  const int last_row = (row0 + LM_ROWS < T * H ? row0 + LM_ROWS : T * H) - 1;
  const int p_first = past + row0 / H, p_last = past + last_row / H;
  const int key_lo = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;

  floatx4 o[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) o[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m[4], l[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) { m[r] = -INFINITY; l[r] = 0.f; }

  // the block table goes to LDS once: a tile's loads then wait for one trip to memory, not for two in a row
  const int n_bt = (p_last / page + 1 < LM_BT) ? p_last / page + 1 : LM_BT;
  for (int i = t; i < n_bt; i += 256) pages[i] = bt[i];
  // zero the padding entries of the key tile once (entries D .. D32 of every row)
  for (int i = t; i < LM_KEYS * (D32 - D); i += 256) Ks[(i / (D32 - D)) * ldk + D + i % (D32 - D)] = 0;
  // ... and the rows of the value tile behind R, up to a whole block of 16
  for (int i = t; i < ((R + 15) / 16 * 16 - R) * ldv; i += 256) Vs[R * ldv + i] = 0;

  const int chunks = D / 8;                           // 16-byte pieces of a cache row
  // a unit: the same piece of two neighbouring tokens.  Neighbouring lanes take neighbouring pairs of tokens, so
  // that their words of the dimension-major tile lie side by side (lanes along a row's pieces would all meet in
  // two LDS banks there); four lanes still read 64 consecutive bytes of a row.
  const int n_units = (LM_KEYS / 2) * chunks;
  constexpr int PER = ((LM_KEYS / 2) * DB * 4 + 255) / 256;
  uint4 stage[PER][2];
  unsigned stage_ok = 0;                              // bit 2 i + e: stage[i][e] holds a row that exists
  // Every load is asked for without a condition, from the row's place or, for a row that does not exist (behind the
  // last key, or in a page that was given back), from the cache's first row; what came back is looked at only when it
  // is parked, a tile later.  (A load under a condition, or a value replaced right after its load, makes the
  // wavefront wait for that load on the spot, one after the other, and nothing would run ahead.)
  auto fetch = [&](int k0) {
    stage_ok = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int u = t + i * 256;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int key = k0 + 2 * (u % (LM_KEYS / 2)) + e;
        const int blk = key >> page_shift;
        const bool want = u < n_units && key <= p_last;
        const int pg = want ? (blk < LM_BT ? pages[blk] : bt[blk]) : -1;
        const bool ok = pg >= 0;
        const size_t row = ok ? (size_t)pg * page + (key & (page - 1)) : 0;
        const int piece = u < n_units ? u / (LM_KEYS / 2) : 0;
        stage[i][e] = load16(cache + row * D + piece * 8);
        stage_ok |= (unsigned)ok << (2 * i + e);
      }
    }
  };
  auto park = [&]() {
    const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int u = t + i * 256;
      if (u < n_units) {
        const int kk = 2 * (u % (LM_KEYS / 2)), d = (u / (LM_KEYS / 2)) * 8;
        const uint4 v0 = (stage_ok >> (2 * i)) & 1u ? stage[i][0] : zero;      // rows nobody wrote read as zeros
        const uint4 v1 = (stage_ok >> (2 * i + 1)) & 1u ? stage[i][1] : zero;
        *(uint4*)(Ks + kk * ldk + d) = v0;
        *(uint4*)(Ks + (kk + 1) * ldk + d) = v1;
        if (d < R) {                                  // dimension-major: the two tokens' entries side by side, one word
          const bf16_t* e0 = (const bf16_t*)&v0;
          const bf16_t* e1 = (const bf16_t*)&v1;
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (d + j < R) *(uint32_t*)(Vs + (d + j) * ldv + kk) = (uint32_t)e0[j] | ((uint32_t)e1[j] << 16);
        }
      }
    }
  };

  // the tiles of this workgroup: all of them, or its share when several workgroups split a block's keys
  const int n_tiles = (p_last - key_lo) / LM_KEYS + 1;
  const int share = (n_tiles + n_splits - 1) / n_splits;
  const int k_begin = key_lo + (int)blockIdx.z * share * LM_KEYS;
  const int k_stop = (k_begin + share * LM_KEYS < p_last + 1) ? k_begin + share * LM_KEYS : p_last + 1;
  __syncthreads();                                    // the block table's copy is there
  if (k_begin < k_stop) fetch(k_begin);
  for (int k0 = k_begin; k0 < k_stop; k0 += LM_KEYS) {
    __syncthreads();                                  // the tile before has been read by everyone
    park();
    __syncthreads();
    if (k0 + LM_KEYS < k_stop) fetch(k0 + LM_KEYS);
    // ---- scores of this wavefront's 16 rows against the tile's 32 tokens
    floatx4 sc[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      sc[b] = floatx4{0.f, 0.f, 0.f, 0.f};
      const bf16_t* kp = Ks + (b * 16 + fr) * ldk + fg * 8;
#pragma unroll
      for (int i = 0; i < DB; ++i) {
        if (i * 32 < D) {
          const uint4 kf = *(const uint4*)(kp + i * 32);
          sc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, qf[i]), __builtin_bit_cast(bf16x8_t, kf),
                                                          sc[b], 0, 0, 0);
        }
      }
    }
    // ---- the softmax's running maximum and sum, per row, in 32-bit
    float alpha[4];
    bf16_t* pw = Ps + wave * 16 * ldv;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float v[2];
      float mx = -INFINITY;
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int key = k0 + b * 16 + fr;
        const bool seen = key <= pos[r] && (window <= 0 || key > pos[r] - window);
        v[b] = seen ? sc[b][r] * scale_log2e : -INFINITY;
        mx = fmaxf(mx, v[b]);
      }
      mx = fmaxf(mx, dpp_move<0xB1, 0xF>(mx, mx));
      mx = fmaxf(mx, dpp_move<0x4E, 0xF>(mx, mx));
      mx = fmaxf(mx, dpp_move<0x141, 0xF>(mx, mx));
      mx = fmaxf(mx, dpp_move<0x140, 0xF>(mx, mx));
      const float m_new = fmaxf(m[r], mx);
      const bool none = m_new == -INFINITY;
      alpha[r] = none ? 1.f : __builtin_amdgcn_exp2f(m[r] - m_new);
      float sum = 0.f;
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const float e = none ? 0.f : __builtin_amdgcn_exp2f(v[b] - m_new);
        const bf16_t eb = f32_to_bf16(e);
        pw[(4 * fg + r) * ldv + b * 16 + fr] = eb;
        sum += bf16_to_f32(eb);                        // the sum of what the second product really uses
      }
      sum = group_sum<16>(sum);
      l[r] = l[r] * alpha[r] + sum;
      m[r] = m_new;
    }
    // (the weights were written and are read by this wavefront only; LDS operations of a wavefront stay in order)
    const uint4 pf = *(const uint4*)(pw + fr * ldv + fg * 8);
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      if (i * 16 < R) {
#pragma unroll
        for (int r = 0; r < 4; ++r) o[i][r] *= alpha[r];
        const uint4 vf = *(const uint4*)(Vs + (i * 16 + fr) * ldv + fg * 8);
        o[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, pf), __builtin_bit_cast(bf16x8_t, vf), o[i],
                                                       0, 0, 0);
      }
    }
  }
  if (n_splits > 1) {
    // ---- this share's maximum, sum and unscaled sums: [sequence][row][share][2 + R], merged by another kernel
    const int rows_cap = gridDim.x * LM_ROWS;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = row0 + wave * 16 + 4 * fg + r;
      if (row >= T * H) continue;
      float* pp = partial + (((size_t)blockIdx.y * rows_cap + row) * n_splits + blockIdx.z) * (R + 2);
      if (fr == 0) { pp[0] = m[r]; pp[1] = l[r]; }
#pragma unroll
      for (int i = 0; i < RB; ++i)
        if (i * 16 + fr < R) pp[2 + i * 16 + fr] = o[i][r];
    }
    return;
  }
  // ---- out[token, head, :R] = O / l
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = row0 + wave * 16 + 4 * fg + r;
    if (row >= T * H) continue;
    float shrink = 1.f, lr = l[r];
    if (sink) {                                       // base-2 domain, as the maxima are
      const float s0 = sink[row % H] * 1.4426950408889634f;
      const float m_all = fmaxf(m[r], s0);
      shrink = m[r] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[r] - m_all);
      lr = lr * shrink + __builtin_amdgcn_exp2f(s0 - m_all);
    }
    const float inv = lr > 0.f ? shrink / lr : 0.f;
    bf16_t* op = out + (size_t)(first + row / H) * out_ld + (size_t)(row % H) * R;
#pragma unroll
    for (int i = 0; i < RB; ++i)
      if (i * 16 + fr < R) op[i * 16 + fr] = f32_to_bf16(o[i][r] * inv);
  }
}

// The shares of a row's keys become one: out = sum_z O_z 2^(m_z - M) / sum_z l_z 2^(m_z - M), shares in ascending order.
#define LM_MAX_SPLITS 64
__global__ void __launch_bounds__(128)
attn_latent_merge_kernel(const float* __restrict__ partial, int rows_cap, int n_splits, const int* __restrict__ q_start,
                         int seq0, int H, int R, bf16_t* __restrict__ out, int out_ld, const float* __restrict__ sink) {
  __shared__ float wz[LM_MAX_SPLITS];
  const int s_local = blockIdx.y, row = blockIdx.x;
  const int first = q_start[seq0 + s_local], T = q_start[seq0 + s_local + 1] - first;
  if (row >= T * H) return;
  const float* pp = partial + ((size_t)s_local * rows_cap + row) * n_splits * (R + 2);
  if (threadIdx.x < DA_WAVE) {                      // one wavefront: a lane a share
    const int z = threadIdx.x;
    const float mz = z < n_splits ? pp[(size_t)z * (R + 2)] : -INFINITY;
    const float lz = z < n_splits ? pp[(size_t)z * (R + 2) + 1] : 0.f;
    const float s0 = sink ? sink[row % H] * 1.4426950408889634f : -INFINITY;
    const float M = fmaxf(wave_max(mz), s0);
    const float e = mz == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mz - M);
    const float L = wave_sum(lz * e) + (sink ? __builtin_amdgcn_exp2f(s0 - M) : 0.f);
    if (z < n_splits) wz[z] = L > 0.f ? e / L : 0.f;
  }
  __syncthreads();
  bf16_t* op = out + (size_t)(first + row / H) * out_ld + (size_t)(row % H) * R;
  for (int c = threadIdx.x; c < R; c += blockDim.x) {
    float acc = 0.f;
#pragma unroll 4
    for (int z = 0; z < n_splits; ++z)               // (a share without keys wrote zeros and has the weight 0)
      acc = fmaf(pp[(size_t)z * (R + 2) + 2 + c], wz[z], acc);
    op[c] = f32_to_bf16(acc);
  }
}

// Whether the matrix-core form takes these sizes: rows of whole 16-byte pieces, up to the largest form's.
extern "C" int da_attn_latent_mfma_takes(int D, int R) {
  return D % 8 == 0 && R >= 1 && R <= D && D <= 576 && R <= 512;
}

// How many workgroups share the keys of a block of query rows when every sequence brings one token (decoding): as
// many as fill the chip, none with less than two tiles of the longest context that the block table can hold.  From
// the step's shape only, so that a recorded step keeps it.
extern "C" int da_attn_latent_splits(int n_seqs, int H, int max_blocks, int page) {
  const long groups = (long)n_seqs * da_ceil_div(H, LM_ROWS);
  long n = 384 / (groups > 0 ? groups : 1);
  const long by_keys = ((long)max_blocks * page) / (2 * LM_KEYS);
  if (n > by_keys) n = by_keys;
  if (n > 16) n = 16;                                 // (every share costs the merge a pass)
  return n >= 2 ? (int)n : 1;
}

extern "C" long da_attn_latent_partial_floats(int S, int max_query_len, int H, int R, int n_splits) {
  return (long)S * da_ceil_div((long)max_query_len * H, LM_ROWS) * LM_ROWS * n_splits * (R + 2);
}

// Sequences seq0 .. seq0 + S - 1 of the step.  n_splits > 1: the keys of every block of rows are shared out over
// that many workgroups, whose results pass through `partial` (32-bit, da_attn_latent_partial_floats entries).
extern "C" int da_attn_latent_mfma(const void* q, int q_ld, const void* cache, const int* block_table, int max_blocks,
                                   const int* q_start, const int* seq_lens, int seq0, int S, int max_query_len, int H, int D,
                                   int R, int page, float scale, int window, void* out, int out_ld, int n_splits,
                                   float* partial, long partial_floats, const float* sink, void* stream) {
  DA_REQUIRE(S >= 0 && seq0 >= 0 && H > 0 && page > 0 && max_blocks > 0 && max_query_len > 0 && window >= 0 && n_splits >= 1,
             "attn_latent_mfma: bad sizes");
  DA_REQUIRE(da_attn_latent_mfma_takes(D, R), "attn_latent_mfma: rows of %d entries with %d of them values are not taken", D, R);
  DA_REQUIRE(q_ld >= H * D && out_ld >= H * R && q_ld % 8 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)cache % 16 == 0,
             "attn_latent_mfma: q must hold H * D entries a row in 16-byte pieces");
  DA_REQUIRE((page & (page - 1)) == 0, "attn_latent_mfma: a page of %d tokens is no power of two", page);
  DA_REQUIRE(n_splits <= LM_MAX_SPLITS, "attn_latent_mfma: %d shares, %d are taken", n_splits, LM_MAX_SPLITS);
  DA_REQUIRE(n_splits == 1 || (partial && partial_floats >= da_attn_latent_partial_floats(S, max_query_len, H, R, n_splits)),
             "attn_latent_mfma: the scratch for %d shares is too small", n_splits);
  if (S == 0) return 0;
  const dim3 grid(da_ceil_div((long)max_query_len * H, LM_ROWS), S, n_splits), block(256);
  const float sl2 = scale * 1.4426950408889634f;
  hipStream_t st = (hipStream_t)stream;
#define DA_LM_GO(DB, RB)                                                                                                  \
  hipLaunchKernelGGL((attn_latent_mfma_kernel<DB, RB>), grid, block, 0, st, (const bf16_t*)q, q_ld, (const bf16_t*)cache,   \
                     block_table, max_blocks, q_start, seq_lens, H, D, R, page, sl2, window, (bf16_t*)out, out_ld, seq0,   \
                     n_splits, partial, sink)
  if (D <= 128 && R <= 128) DA_LM_GO(4, 8);
  else if (D <= 256 && R <= 256) DA_LM_GO(8, 16);
  else if (D <= 384 && R <= 384) DA_LM_GO(12, 24);
  else DA_LM_GO(18, 32);
#undef DA_LM_GO
  DA_CHECK_LAUNCH("attn_latent_mfma");
  if (n_splits > 1) {
    hipLaunchKernelGGL(attn_latent_merge_kernel, dim3(max_query_len * H, S), dim3(128), 0, st, partial, (int)grid.x * LM_ROWS,
                       n_splits, q_start, seq0, H, R, (bf16_t*)out, out_ld, sink);
    DA_CHECK_LAUNCH("attn_latent_merge");
  }
  return 0;
}
