// Feed-forward layers made of experts: every token's rows go through `top` of `n_experts` small gated
// feed-forwards, and the results are added with weights.
//
//   da_moe_route    from each token's expert ids (read from a table by token id, or given) to a layout in
//                   which every expert's (token, choice) pairs lie together: pairs get slots, an expert's
//                   slots start at a multiple of `tile` rows, so that a tile of rows has one expert; weights
//                   given a pair are also written out a slot
//   da_moe_gated    mid[slot] = act(Wg_e a[row]) * (Wu_e a[row])      (plain kernel, any dtype)
//   da_moe_down     out[slot] = Wd_e mid[slot]                        (plain kernel, 32-bit out)
//   da_moe_combine  y[n] (+)= sum_k weight_k * out[slot(n, k)]        k ascending
//
// Everything the grid depends on comes from the step's shape (tokens x top, experts); which tiles are
// used is decided on the device, so a step can be recorded.  A pair's result does not depend on its slot:
// sums over k run in the same order for every row.  Expert weights are stacked: gate | up as
// [n_experts][2 F][K] (gate rows first), down as [n_experts][width][F].
#include "gemm_common.h"

#define MOE_MAX_EXPERTS 1024

__global__ void __launch_bounds__(1024)
moe_route_kernel(const int* __restrict__ tokens, const int* __restrict__ table, int vocab, const int* __restrict__ ids,
                 int N, int top, int n_experts, int tile, int* __restrict__ slot_of_pair,
                 int* __restrict__ row_of_slot, int* __restrict__ tile_expert, int P_cap, int T_cap,
                 const float* __restrict__ pair_weights, float* __restrict__ slot_weight) {
  __shared__ int counts[MOE_MAX_EXPERTS], start[MOE_MAX_EXPERTS], cursor[MOE_MAX_EXPERTS];
  const int t = threadIdx.x, nt = blockDim.x;
  const int P = N * top;
  for (int e = t; e < n_experts; e += nt) counts[e] = cursor[e] = 0;
  for (int i = t; i < P_cap; i += nt) row_of_slot[i] = -1;
  for (int i = t; i < T_cap; i += nt) tile_expert[i] = -1;
  __syncthreads();
  auto expert_of = [&](int i) -> int {
    int e;
    if (table) {
      const int tok = tokens[i / top];
      e = (tok >= 0 && tok < vocab) ? table[(size_t)tok * top + i % top] : -1;
    } else {
      e = ids[i];
    }
    return (e >= 0 && e < n_experts) ? e : -1;
  };
  for (int i = t; i < P; i += nt) {
    const int e = expert_of(i);
    if (e >= 0) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (t == 0) {
    int run = 0;
    for (int e = 0; e < n_experts; ++e) {
      start[e] = run;
      const int tiles = (counts[e] + tile - 1) / tile;
      for (int k = 0; k < tiles; ++k) tile_expert[run / tile + k] = e;
      run += tiles * tile;
    }
  }
  __syncthreads();
  for (int i = t; i < P; i += nt) {
    const int e = expert_of(i);
    int slot = -1;
    if (e >= 0) {
      slot = start[e] + atomicAdd(&cursor[e], 1);
      row_of_slot[slot] = i / top;
      if (pair_weights) slot_weight[slot] = pair_weights[i];      // the pair's weight where its slot's row is
    }
    slot_of_pair[i] = slot;
  }
}

extern "C" int da_moe_route(const int* tokens, const int* table, int vocab, const int* ids, int N, int top,
                            int n_experts, int tile, int* slot_of_pair, int* row_of_slot, int* tile_expert, int P_cap,
                            int T_cap, void* stream, const float* pair_weights, float* slot_weight) {
  DA_REQUIRE(N >= 0 && top > 0 && n_experts > 0 && tile > 0, "moe_route: bad sizes");
  DA_REQUIRE(n_experts <= MOE_MAX_EXPERTS, "moe_route: %d experts, %d are taken", n_experts, MOE_MAX_EXPERTS);
  DA_REQUIRE((table != nullptr && tokens != nullptr) != (ids != nullptr), "moe_route: a table with tokens, or expert ids");
  DA_REQUIRE((pair_weights == nullptr) == (slot_weight == nullptr), "moe_route: weights a pair need a place a slot");
  DA_REQUIRE(T_cap >= da_ceil_div((long)N * top, tile) + n_experts && P_cap >= T_cap * tile,
             "moe_route: the slot space (%d rows, %d tiles) is too small for %d pairs", P_cap, T_cap, N * top);
  if (N == 0) return 0;
  hipLaunchKernelGGL(moe_route_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, tokens, table, vocab, ids, N, top,
                     n_experts, tile, slot_of_pair, row_of_slot, tile_expert, P_cap, T_cap, pair_weights, slot_weight);
  DA_CHECK_LAUNCH("moe_route");
  return 0;
}

// ---- plain grouped products: tiles of 64 x 64, sums in two levels as the plain product has them ------------
#define MT 64
#define MBK 16
#define MCHUNK 8

// MOE_GATED: two products (gate and up rows of the expert's stacked matrix), out = act(g) * u in T; MOE_UP: one
// product, out = act(.) in T; MOE_DOWN: one product, 32-bit out.  The first two gather: row r of the tile is
// a[row_of_slot[slot]] (times slot_scale[slot] when given: the sums are scaled, which is the same number),
// MOE_DOWN reads a[slot].
#define MOE_DOWN 0
#define MOE_GATED 1
#define MOE_UP 2
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
moe_product_ref_kernel(const T* __restrict__ a, int lda, const int* __restrict__ row_of_slot,
                       const int* __restrict__ tile_expert, const T* __restrict__ w, void* __restrict__ out, int ldo,
                       int K, int F, int act, const float* __restrict__ slot_scale, float limit) {
  constexpr bool GATED = MODE == MOE_GATED, GATHER = MODE != MOE_DOWN;
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  __shared__ float As[MBK][MT + 4];
  __shared__ float Ws[GATED ? 2 : 1][MBK][MT + 4];
  __shared__ int srow[MT];
  const int t = threadIdx.x;
  const int tx = t % 16, ty = t / 16;
  const int m0 = blockIdx.y * MT, n0 = blockIdx.x * MT;
  const int lrow = t / 4, lk = (t % 4) * 4;
  if (t < MT) srow[t] = row_of_slot[m0 + t];
  __syncthreads();
  const T* wg = w + (size_t)e * (GATED ? 2 : 1) * F * K;
  const T* wu = wg + (size_t)F * K;
  float acc[GATED ? 2 : 1][4][4], part[GATED ? 2 : 1][4][4];
#pragma unroll
  for (int g = 0; g < (GATED ? 2 : 1); ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[g][i][j] = part[g][i][j] = 0.f;
  const int arow = GATHER ? srow[lrow] : (srow[lrow] >= 0 ? m0 + lrow : -1);
  int slab = 0;
  for (int k0 = 0; k0 < K; k0 += MBK) {
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int k = k0 + lk + x;
      const int wn = n0 + lrow;
      As[lk + x][lrow] = (arow >= 0 && k < K) ? to_f32(a[(size_t)arow * lda + k]) : 0.f;
      Ws[0][lk + x][lrow] = (wn < F && k < K) ? to_f32(wg[(size_t)wn * K + k]) : 0.f;
      if (GATED) Ws[1][lk + x][lrow] = (wn < F && k < K) ? to_f32(wu[(size_t)wn * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < MBK; ++k) {
      float av[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int g = 0; g < (GATED ? 2 : 1); ++g) {
        float wv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) wv[j] = Ws[g][k][tx * 4 + j];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) part[g][i][j] = fmaf(av[i], wv[j], part[g][i][j]);
      }
    }
    if (++slab == MCHUNK) {
      slab = 0;
#pragma unroll
      for (int g = 0; g < (GATED ? 2 : 1); ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc[g][i][j] += part[g][i][j];
            part[g][i][j] = 0.f;
          }
    }
    __syncthreads();
  }
#pragma unroll
  for (int g = 0; g < (GATED ? 2 : 1); ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[g][i][j] += part[g][i][j];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (srow[r] < 0) continue;
    const float sc = (GATHER && slot_scale) ? slot_scale[m0 + r] : 1.0f;      // the row of a times its weight
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= F) continue;
      const size_t o = (size_t)(m0 + r) * ldo + n;
      if (GATED) {
        from_f32(&((T*)out)[o], gated_mid<DTypeOf<T>::value == DA_BF16>(sc * acc[0][i][j], sc * acc[1][i][j], act, limit));
      } else if (MODE == MOE_UP) {
        from_f32(&((T*)out)[o], DTypeOf<T>::value == DA_BF16 ? apply_act_bf16(sc * acc[0][i][j], act) : apply_act(sc * acc[0][i][j], act));
      } else {
        ((float*)out)[o] = acc[0][i][j];
      }
    }
  }
}

extern "C" int da_moe_gated_ref(const void* a, int lda, int dtype, const int* row_of_slot, const int* tile_expert,
                                const void* w, void* mid, int ldm, int T_cap, int K, int F, int act, float limit,
                                void* stream) {
  DA_REQUIRE(T_cap >= 0 && K > 0 && F > 0 && lda >= K && ldm >= F, "moe_gated_ref: bad sizes");
  DA_REQUIRE(act != DA_ACT_GLU_CAPPED || limit > 0.f, "moe_gated_ref: the capped form needs a positive limit");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_LAST, "moe_gated_ref: unknown activation %d", act);
  if (T_cap == 0) return 0;
  dim3 grid(da_ceil_div(F, MT), T_cap);
  if (dtype == DA_BF16)
    hipLaunchKernelGGL((moe_product_ref_kernel<bf16_t, MOE_GATED>), grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t*)a,
                       lda, row_of_slot, tile_expert, (const bf16_t*)w, mid, ldm, K, F, act, nullptr, limit);
  else
    hipLaunchKernelGGL((moe_product_ref_kernel<float, MOE_GATED>), grid, dim3(256), 0, (hipStream_t)stream, (const float*)a,
                       lda, row_of_slot, tile_expert, (const float*)w, mid, ldm, K, F, act, nullptr, limit);
  DA_CHECK_LAUNCH("moe_gated_ref");
  return 0;
}

extern "C" int da_moe_down_ref(const void* mid, int ldm, int dtype, const int* row_of_slot, const int* tile_expert,
                               const void* w, float* out, int ldo, int T_cap, int F, int width, void* stream) {
  DA_REQUIRE(T_cap >= 0 && F > 0 && width > 0 && ldm >= F && ldo >= width, "moe_down_ref: bad sizes");
  if (T_cap == 0) return 0;
  dim3 grid(da_ceil_div(width, MT), T_cap);
  if (dtype == DA_BF16)
    hipLaunchKernelGGL((moe_product_ref_kernel<bf16_t, MOE_DOWN>), grid, dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)mid, ldm, row_of_slot, tile_expert, (const bf16_t*)w, out, ldo, F, width, 0, nullptr, 0.f);
  else
    hipLaunchKernelGGL((moe_product_ref_kernel<float, MOE_DOWN>), grid, dim3(256), 0, (hipStream_t)stream,
                       (const float*)mid, ldm, row_of_slot, tile_expert, (const float*)w, out, ldo, F, width, 0, nullptr, 0.f);
  DA_CHECK_LAUNCH("moe_down_ref");
  return 0;
}

// mid[slot] = act(scale[slot] * (W_e a[row_of_slot[slot]])): the first product of experts without a gate; w: [experts, F, K]
extern "C" int da_moe_up_ref(const void* a, int lda, int dtype, const int* row_of_slot, const int* tile_expert,
                             const void* w, const float* slot_scale, void* mid, int ldm, int T_cap, int K, int F, int act,
                             void* stream) {
  DA_REQUIRE(T_cap >= 0 && K > 0 && F > 0 && lda >= K && ldm >= F, "moe_up_ref: bad sizes");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_LAST, "moe_up_ref: unknown activation %d", act);
  if (T_cap == 0) return 0;
  dim3 grid(da_ceil_div(F, MT), T_cap);
  if (dtype == DA_BF16)
    hipLaunchKernelGGL((moe_product_ref_kernel<bf16_t, MOE_UP>), grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t*)a,
                       lda, row_of_slot, tile_expert, (const bf16_t*)w, mid, ldm, K, F, act, slot_scale, 0.f);
  else
    hipLaunchKernelGGL((moe_product_ref_kernel<float, MOE_UP>), grid, dim3(256), 0, (hipStream_t)stream, (const float*)a,
                       lda, row_of_slot, tile_expert, (const float*)w, mid, ldm, K, F, act, slot_scale, 0.f);
  DA_CHECK_LAUNCH("moe_up_ref");
  return 0;
}

// The router's choice from 32-bit logits z (+ bias, when given): every token's `top` largest (the lower index wins a
// tie), ids[n, k] and weights[n, k] in descending order.  mode 0: the weights are logistic(z) (`renorm`: divided by
// their sum); mode 1: the softmax over the chosen logits only.
__global__ void moe_top_kernel(const float* __restrict__ z, int ldz, const void* __restrict__ bias, int bias_dtype, int N,
                               int E, int top, int mode, int renorm, int* __restrict__ ids, float* __restrict__ weights) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  const float* row = z + (size_t)n * ldz;
  float sum = 0.f, first = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bz = -INFINITY;
    for (int e = 0; e < E; ++e) {
      const float v = row[e] + (bias ? load_param(bias, bias_dtype, e) : 0.f);
      bool taken = false;
      for (int j = 0; j < k; ++j) taken |= ids[(size_t)n * top + j] == e;
      if (!taken && (best < 0 || v > bz)) { best = e; bz = v; }
    }
    if (k == 0) first = bz;
    const float sc = mode == 1 ? expf(bz - first) : 1.0f / (1.0f + expf(-bz));
    ids[(size_t)n * top + k] = best;
    weights[(size_t)n * top + k] = sc;
    sum += sc;
  }
  if (renorm || mode == 1)
    for (int k = 0; k < top; ++k) weights[(size_t)n * top + k] /= sum;
}

extern "C" int da_moe_top(const float* z, int ldz, const void* bias, int bias_dtype, int N, int E, int top, int mode,
                          int renorm, int* ids, float* weights, void* stream) {
  DA_REQUIRE(N >= 0 && E > 0 && top > 0 && top <= E && ldz >= E, "moe_top: bad sizes");
  DA_REQUIRE(mode == 0 || mode == 1, "moe_top: mode %d (0: logistic scores, 1: softmax over the chosen)", mode);
  if (N == 0) return 0;
  hipLaunchKernelGGL(moe_top_kernel, dim3(da_ceil_div(N, 64)), dim3(64), 0, (hipStream_t)stream, z, ldz, bias, bias_dtype, N,
                     E, top, mode, renorm, ids, weights);
  DA_CHECK_LAUNCH("moe_top");
  return 0;
}

extern "C" int da_moe_top_logistic(const float* z, int ldz, int N, int E, int top, int renorm, int* ids, float* weights,
                                   void* stream) {
  return da_moe_top(z, ldz, nullptr, 0, N, E, top, 0, renorm, ids, weights, stream);
}

// slot_weight[slot_of_pair[i]] = weights[i]: a pair's weight where its slot's row is
__global__ void moe_slot_weights_kernel(const int* __restrict__ slot_of_pair, const float* __restrict__ weights, int P,
                                        float* __restrict__ slot_weight) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  const int slot = slot_of_pair[i];
  if (slot >= 0) slot_weight[slot] = weights[i];
}

extern "C" int da_moe_slot_weights(const int* slot_of_pair, const float* weights, int P, float* slot_weight, void* stream) {
  DA_REQUIRE(P >= 0, "moe_slot_weights: bad size");
  if (P == 0) return 0;
  hipLaunchKernelGGL(moe_slot_weights_kernel, dim3(da_ceil_div(P, 256)), dim3(256), 0, (hipStream_t)stream, slot_of_pair,
                     weights, P, slot_weight);
  DA_CHECK_LAUNCH("moe_slot_weights");
  return 0;
}

// y[n] (+)= sum_k weight(n, k) * out[slot_of_pair[n * top + k]]; weights: per pair, or one for all
__global__ void moe_combine_kernel(const float* __restrict__ out, int ldo, const int* __restrict__ slot_of_pair,
                                   const float* __restrict__ weights, float uniform, int top, float* __restrict__ y,
                                   int ldy, int N, int width, int accumulate) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)N * width) return;
  const int n = (int)(i / width), c = (int)(i % width);
  float s = 0.f;
  for (int k = 0; k < top; ++k) {
    const int slot = slot_of_pair[n * top + k];
    if (slot >= 0) s += (weights ? weights[n * top + k] : uniform) * out[(size_t)slot * ldo + c];
  }
  float* dst = y + (size_t)n * ldy + c;
  *dst = accumulate ? *dst + s : s;
}

extern "C" int da_moe_combine(const float* out, int ldo, const int* slot_of_pair, const float* weights, float uniform,
                              int top, float* y, int ldy, int N, int width, int accumulate, void* stream) {
  DA_REQUIRE(N >= 0 && width > 0 && top > 0 && ldo >= width && ldy >= width, "moe_combine: bad sizes");
  if (N == 0) return 0;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(da_ceil_div((long)N * width, 256)), dim3(256), 0, (hipStream_t)stream, out,
                     ldo, slot_of_pair, weights, uniform, top, y, ldy, N, width, accumulate);
  DA_CHECK_LAUNCH("moe_combine");
  return 0;
}

// ---- the grouped products on the matrix cores (bfloat16) ---------------------------------------------------
// A workgroup of four wavefronts owns a tile of 32 slots x 64 columns of one expert: wavefront v the columns
// 16 v .. 16 v + 15 of both blocks of 16 rows, with MFMA 16x16x32.  Operands go from memory into the lanes'
// fragments (a lane's 16 bytes are 8 consecutive k of one row), four k-steps of 32 asked for at once; with
// few rows an expert, as in decoding, the kernel streams the expert's weights once.  GATED: the gate and up
// rows of the same columns are multiplied side by side and out = act(g) * u leaves in bfloat16; else one
// product leaves in 32-bit.  A row's sums run over k in ascending order whatever else is in the step.
#define MM_ROWS 32
#define MM_COLS 64
#define MM_UNROLL 4

template <int MODE>
__global__ void __launch_bounds__(256)
moe_mfma_kernel(const bf16_t* __restrict__ a, int lda, const int* __restrict__ row_of_slot,
                const int* __restrict__ tile_expert, const bf16_t* __restrict__ w, void* __restrict__ out, int ldo,
                int K, int F, int act, const float* __restrict__ slot_scale, float limit) {
  constexpr bool GATED = MODE == MOE_GATED, GATHER = MODE != MOE_DOWN;
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  const int t = threadIdx.x, lane = t % DA_WAVE, wave = t / DA_WAVE;
  const int fr = lane % 16, fk = (lane / 16) * 8;
  const int m0 = blockIdx.y * MM_ROWS, n0 = blockIdx.x * MM_COLS + wave * 16;
  if (n0 >= F) return;
  // the rows of a: gathered by slot for the first product (a padding slot reads row 0 and is never stored),
  // the slot's own row for the second
  const bf16_t* ap[2];
  int srow[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    srow[i] = row_of_slot[m0 + i * 16 + fr];
    const int r = GATHER ? (srow[i] >= 0 ? srow[i] : 0) : m0 + i * 16 + fr;
    ap[i] = a + (size_t)r * lda + fk;
  }
  const int wcol = n0 + fr < F ? n0 + fr : 0;
  const bf16_t* wg = w + ((size_t)e * (GATED ? 2 : 1) * F + wcol) * K + fk;
  const bf16_t* wu = wg + (size_t)F * K;
  floatx4 acc[2][GATED ? 2 : 1];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int g = 0; g < (GATED ? 2 : 1); ++g) acc[i][g] = floatx4{0.f, 0.f, 0.f, 0.f};
  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (int k0 = 0; k0 < K; k0 += 32 * MM_UNROLL) {
    uint4 av[MM_UNROLL][2], wv[MM_UNROLL][GATED ? 2 : 1];
#pragma unroll
    for (int u = 0; u < MM_UNROLL; ++u) {
      const int k = k0 + u * 32;
      const int ks = (k + fk < K) ? k : -fk;            // past K: the row's first chunk, met by zeros in a
      av[u][0] = load16(ap[0] + ks);
      av[u][1] = load16(ap[1] + ks);
      wv[u][0] = load16(wg + ks);
      if (GATED) wv[u][GATED ? 1 : 0] = load16(wu + ks);
    }
#pragma unroll
    for (int u = 0; u < MM_UNROLL; ++u) {
      const bool kin = k0 + u * 32 + fk < K;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint4 x = kin ? av[u][i] : zero;
#pragma unroll
        for (int g = 0; g < (GATED ? 2 : 1); ++g)
          acc[i][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, x),
                                                              __builtin_bit_cast(bf16x8_t, wv[u][g]), acc[i][g], 0, 0, 0);
      }
    }
  }
  // acc[i][.][r] is row 16 i + 4 (lane / 16) + r of the tile, column n0 + fr
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 4 * (lane / 16) + r;
      const int used = row_of_slot[m0 + i * 16 + row];
      if (used < 0 || n0 + fr >= F) continue;
      const size_t o = (size_t)(m0 + i * 16 + row) * ldo + n0 + fr;
      const float sc = (GATHER && slot_scale) ? slot_scale[m0 + i * 16 + row] : 1.0f;
      if (GATED) ((bf16_t*)out)[o] = f32_to_bf16(gated_mid<true>(sc * acc[i][0][r], sc * acc[i][GATED ? 1 : 0][r], act, limit));
      else if (MODE == MOE_UP) ((bf16_t*)out)[o] = f32_to_bf16(apply_act_bf16(sc * acc[i][0][r], act));
      else ((float*)out)[o] = acc[i][0][r];
    }
}

static int moe_mfma_checks(const void* a, int lda, const void* w, int K, const char* name) {
  DA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0,
             "%s: K and the row length of a must be multiples of 8, operands 16-byte aligned", name);
  return 0;
}

extern "C" int da_moe_tile_rows_mfma() { return MM_ROWS; }

extern "C" int da_moe_gated_mfma(const void* a, int lda, const int* row_of_slot, const int* tile_expert, const void* w,
                                 void* mid, int ldm, int T_cap, int K, int F, int act, float limit, void* stream) {
  DA_REQUIRE(T_cap >= 0 && K > 0 && F > 0 && lda >= K && ldm >= F, "moe_gated_mfma: bad sizes");
  DA_REQUIRE(act != DA_ACT_GLU_CAPPED || limit > 0.f, "moe_gated_mfma: the capped form needs a positive limit");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_LAST, "moe_gated_mfma: unknown activation %d", act);
  if (moe_mfma_checks(a, lda, w, K, "moe_gated_mfma")) return 1;
  if (T_cap == 0) return 0;
  hipLaunchKernelGGL((moe_mfma_kernel<MOE_GATED>), dim3(da_ceil_div(F, MM_COLS), T_cap), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)a, lda, row_of_slot, tile_expert, (const bf16_t*)w, mid, ldm, K, F, act, nullptr, limit);
  DA_CHECK_LAUNCH("moe_gated_mfma");
  return 0;
}

extern "C" int da_moe_up_mfma(const void* a, int lda, const int* row_of_slot, const int* tile_expert, const void* w,
                              const float* slot_scale, void* mid, int ldm, int T_cap, int K, int F, int act, void* stream) {
  DA_REQUIRE(T_cap >= 0 && K > 0 && F > 0 && lda >= K && ldm >= F, "moe_up_mfma: bad sizes");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_LAST, "moe_up_mfma: unknown activation %d", act);
  if (moe_mfma_checks(a, lda, w, K, "moe_up_mfma")) return 1;
  if (T_cap == 0) return 0;
  hipLaunchKernelGGL((moe_mfma_kernel<MOE_UP>), dim3(da_ceil_div(F, MM_COLS), T_cap), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)a, lda, row_of_slot, tile_expert, (const bf16_t*)w, mid, ldm, K, F, act, slot_scale, 0.f);
  DA_CHECK_LAUNCH("moe_up_mfma");
  return 0;
}

extern "C" int da_moe_down_mfma(const void* mid, int ldm, const int* row_of_slot, const int* tile_expert, const void* w,
                                float* out, int ldo, int T_cap, int F, int width, void* stream) {
  DA_REQUIRE(T_cap >= 0 && F > 0 && width > 0 && ldm >= F && ldo >= width, "moe_down_mfma: bad sizes");
  if (moe_mfma_checks(mid, ldm, w, F, "moe_down_mfma")) return 1;
  if (T_cap == 0) return 0;
  hipLaunchKernelGGL((moe_mfma_kernel<MOE_DOWN>), dim3(da_ceil_div(width, MM_COLS), T_cap), dim3(256), 0,
                     (hipStream_t)stream, (const bf16_t*)mid, ldm, row_of_slot, tile_expert, (const bf16_t*)w, out, ldo, F,
                     width, 0, nullptr, 0.f);
  DA_CHECK_LAUNCH("moe_down_mfma");
  return 0;
}

// rows of a in the order of the slots (zeros for slots that hold no pair): the operand of the grouped block-tile
// product, 16 bytes a thread
__global__ void moe_gather_kernel(const bf16_t* __restrict__ a, int lda, const int* __restrict__ row_of_slot,
                                  bf16_t* __restrict__ out, int rows, int width8, const float* __restrict__ slot_scale) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)rows * width8) return;
  const int slot = (int)(i / width8), c = (int)(i % width8) * 8;
  const int r = row_of_slot[slot];
  uint4 v = make_uint4(0, 0, 0, 0);
  if (r >= 0) v = *(const uint4*)(a + (size_t)r * lda + c);
  if (slot_scale && r >= 0) {                     // the row times its pair's weight, rounded once
    const float sc = slot_scale[slot];
    uint32_t* w2 = (uint32_t*)&v;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      w2[e] = pack2_bf16(sc * bf16_to_f32((bf16_t)(w2[e] & 0xffffu)), sc * bf16_to_f32((bf16_t)(w2[e] >> 16)));
  }
  *(uint4*)(out + (size_t)slot * width8 * 8 + c) = v;
}

extern "C" int da_moe_gather(const void* a, int lda, const int* row_of_slot, void* out, int rows, int width, void* stream,
                             const float* slot_scale) {
  DA_REQUIRE(rows >= 0 && width > 0 && width % 8 == 0 && lda % 8 == 0 && lda >= width, "moe_gather: the width must be a multiple of 8");
  DA_REQUIRE((uintptr_t)a % 16 == 0 && (uintptr_t)out % 16 == 0, "moe_gather: operands must be 16-byte aligned");
  if (rows == 0) return 0;
  const long n = (long)rows * (width / 8);
  hipLaunchKernelGGL(moe_gather_kernel, dim3(da_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)a, lda,
                     row_of_slot, (bf16_t*)out, rows, width / 8, slot_scale);
  DA_CHECK_LAUNCH("moe_gather");
  return 0;
}
