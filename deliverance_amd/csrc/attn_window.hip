// Paged attention in bfloat16 on the matrix cores for what the two tuned kernels leave out: keys and values of
// different sizes, a cap on the scores, and a window that keeps a sequence's first keys.  Prompt portions and
// decode rows alike; scores never leave the chip.
//
// For the row at position p, key j is seen when j <= p and (no window, or p - j < window, or j < keep_first);
//   s_j = cap((q . k_j) * scale),  cap(s) = softcap * tanh(s / softcap)   (s itself when softcap is 0)
//   o   = sum_j softmax(s)_j v_j                                           (scores, weights and sums in 32-bit)
// `sink` (optional, [Hq], 32-bit): the softmax's denominator also holds exp(sink[h]), a term without a key or a
// value that is not scaled; it joins once, after the phases have been merged.  `gate` (optional, rows like out):
// o <- o * logistic(gate), in the store.
//
// One workgroup of four wavefronts per (sequence, query head, 32 * RB rows).  A wavefront owns a row block of 32
// rows and one of KP = 4 / RB key phases: keys come in aligned tiles of 32, tile a (keys 32 a ..) belongs to phase
// a mod KP whatever the workgroup, and at the end the phases' partial results (maximum, sum of weights, weighted
// sum) are merged in LDS in the order of the phases.  A wavefront's tiles are the ones that hold kept first keys
// below its window, then the window's; a row's sums run over its tiles in ascending order, so they depend on the
// row's position, the window and KP only, never on how the prompt was cut or on the batch.  Decode rows take
// RB = 1 (four phases share out the keys), portions up to 64 rows RB = 2, longer ones RB = 4, or fewer where 128 rows
// a workgroup would leave compute units idle.
//
// Per tile, with MFMA 32x32x16 (the operand layouts of attn_prefill.hip):
//   S^T[key, row] = K . Q^T      key rows straight from the pages, 16 bytes a lane and 16 dimensions
//   cap, mask, online softmax    a lane holds one row's scores of 16 keys; the halves meet by one exchange
//   O^T[dim, row] += V^T . P^T   values are dimension-major in the pages: 4 consecutive keys are 8 bytes
// The next tile's keys and values are asked for before this tile's arithmetic.  Nothing is parked in LDS: the row
// blocks of a workgroup read the same pages one after the other and find them in the caches.
//
// One cache slot is [n_pages][ Hkv * page * D keys | Hkv * Dv * page values ] (attn_rel.hip).  A key that a
// wavefront does not see (past its last row, or between the kept keys and the window, where the page may be gone)
// reads a key that exists instead, and its values count as zero.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 aw_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float aw_floatx16;

#define AW_BK 32
#define AW_WAVES 4
#define AW_FEW_WORKGROUPS 1024    // 128-row workgroups below which smaller ones are ahead (see the launch)
#define AW_LOG2E 1.4426950408889634f

// D16: the key size rounded up, in sixteens; DT: 32-dimension tiles of the values
template <int D16, int DT>
struct AwTile {
  uint4 k[D16];
  uint2 v[DT][4];      // [value tile][16-key block * 2 + half]: 4 keys of one dimension
};

template <int D16, int DT>
__global__ void __launch_bounds__(AW_WAVES * DA_WAVE)
attn_window_kernel(const bf16_t* __restrict__ q, int q_ld, const bf16_t* __restrict__ cache,
                   const int* __restrict__ block_table, int max_blocks, const int* __restrict__ q_start,
                   const int* __restrict__ seq_lens, int seq0, int Hq, int Hkv, int D, int Dv, int page, float scale,
                   int window, int keep_first, float softcap, const float* __restrict__ sink,
                   const bf16_t* __restrict__ gate, int gate_ld, bf16_t* __restrict__ out, int out_ld, int RB) {
  constexpr int PER = DT * 16 + 2;
  __shared__ float mg[3 * PER * DA_WAVE];              // (KP - 1) * RB <= 3 partial results
  const int KP = AW_WAVES / RB;
  const int s = seq0 + (int)blockIdx.x / Hq, h = (int)blockIdx.x % Hq;
  const int row0 = q_start[s], T = q_start[s + 1] - row0;
  const int i0 = (int)blockIdx.y * 32 * RB;
  if (i0 >= T) return;                                 // (the whole workgroup)
  const int past = seq_lens[s] - T;
  const int hk = h / (Hq / Hkv);
  const int* bt = block_table + (size_t)s * max_blocks;
  const int t = threadIdx.x, lane = t % DA_WAVE, wave = t / DA_WAVE;
  const int col = lane % 32, hf = lane / 32;
  const int rbi = wave % RB, kp = wave / RB;
  const int wrow = i0 + rbi * 32;
  const int lg = 31 - __builtin_clz(page), pmask = page - 1;
  const long long page_elems = (long long)Hkv * page * (D + Dv);
  const bf16_t* kbase = cache + (long long)hk * page * D;
  const bf16_t* vbase = cache + (long long)Hkv * page * D + (long long)hk * Dv * page;
  const int kfw = window > 0 ? keep_first : 0;

  // this lane's query row (a column of Q^T) and its position; a row that does not exist sees nothing
  const int qi = wrow + col;
  const bool q_ok = qi < T && past + qi >= 0;
  const int pq = q_ok ? past + qi : -1;
  aw_bf16x8_t qf[D16];
#pragma unroll
  for (int kd = 0; kd < D16; ++kd) {
    // (unconditional, from a row and a place that exist, replaced afterwards: see the keys' loads below)
    const int off = kd * 16 + hf * 8;
    uint4 v = *(const uint4*)(q + (size_t)(row0 + (qi < T ? qi : T - 1)) * q_ld + h * D + (off < D ? off : 0));
    if (!q_ok || off >= D) v = make_uint4(0, 0, 0, 0);
    qf[kd] = __builtin_bit_cast(aw_bf16x8_t, v);
  }
  // the wavefront's rows span positions w_first .. w_last; its keys are w_lo .. w_last and those below kfw
  const int w_first = past + wrow;
  const int w_last = past + ((wrow + 31 < T - 1) ? wrow + 31 : T - 1);
  const bool wave_on = wrow < T && w_last >= 0 && w_first >= 0;
  const int w_lo = (window > 0 && w_first - window + 1 > 0) ? w_first - window + 1 : 0;
  const int t_lo = w_lo / AW_BK, t_hi = wave_on ? w_last / AW_BK : -1;
  const int kept_tiles = (kfw + AW_BK - 1) / AW_BK;
  const int n_kept = kept_tiles < t_lo ? kept_tiles : t_lo;       // tiles below the window's first that hold kept keys
  const int safe_key = w_last > 0 ? w_last : 0;

  aw_floatx16 acc_o[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_o[i][r] = 0.f;
  float m = -INFINITY, l = 0.f;       // running maximum (base-2 domain); sum of the weights of this lane half's keys

  auto key_ok = [&](int j) -> bool { return j <= w_last && (j >= w_lo || j < kfw); };
  auto page_of = [&](int j) -> long long {
    const int pg = bt[j >> lg];
    return (long long)(pg >= 0 ? pg : 0) * page_elems;
  };
  // tile a's keys and values into registers
  auto load = [&](AwTile<D16, DT>& tl, int a) {
    const int kt = a * AW_BK;
    const bool whole = kt + AW_BK - 1 <= w_last && (kt >= w_lo || kt + AW_BK - 1 < kfw);   // the same for the wavefront
    {
      const int j = kt + col, jj = (whole || key_ok(j)) ? j : safe_key;
      const bf16_t* kr = kbase + page_of(jj) + (long long)(jj & pmask) * D;
      // (unconditional loads, replaced afterwards where the head has no such entries: a load under a condition
      // becomes a branch, and the loads would wait for each other)
#pragma unroll
      for (int kd = 0; kd < D16; ++kd) {
        const int off = kd * 16 + hf * 8;
        uint4 v = *(const uint4*)(kr + (off < D ? off : 0));
        if (off >= D) v = make_uint4(0, 0, 0, 0);
        tl.k[kd] = v;
      }
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int k4 = kt + (g / 2) * 16 + (g % 2) * 8 + 4 * hf;       // 4 keys that share a page
      bool ok[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) ok[e] = whole || key_ok(k4 + e);
      const bool any = ok[0] || ok[1] || ok[2] || ok[3];
      const int ka = any ? k4 : (safe_key & ~3);
      const bf16_t* vp = vbase + page_of(ka) + (ka & pmask);
#pragma unroll
      for (int i = 0; i < DT; ++i) {
        const int d = i * 32 + col;
        uint2 v = *(const uint2*)(vp + (long long)(d < Dv ? d : 0) * page);
        if (!whole) {                                  // rows that were never written for this wavefront may hold anything
          if (!ok[0]) v.x &= 0xffff0000u;
          if (!ok[1]) v.x &= 0x0000ffffu;
          if (!ok[2]) v.y &= 0xffff0000u;
          if (!ok[3]) v.y &= 0x0000ffffu;
        }
        tl.v[i][g] = v;
      }
    }
  };
  // scores, cap, mask, online softmax and the weighted sum of tile a
  auto weigh = [&](const AwTile<D16, DT>& tl, int a) {
    const int kt = a * AW_BK;
    aw_floatx16 sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
    for (int kd = 0; kd < D16; ++kd)
      sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(aw_bf16x8_t, tl.k[kd]), qf[kd], sc, 0, 0, 0);
    float tmax = -INFINITY;
    const float cap2 = softcap * AW_LOG2E, in2 = softcap > 0.f ? 2.0f * AW_LOG2E * scale / softcap : 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = kt + 8 * (r / 4) + 4 * hf + (r % 4);
      float v;
      if (softcap > 0.f) {
        // cap * tanh(x / cap) in the base-2 domain: tanh(y) = 1 - 2 / (1 + e^(2y))
        const float e2 = __builtin_amdgcn_exp2f(sc[r] * in2);
        v = cap2 * (1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e2));
      } else {
        v = sc[r] * (scale * AW_LOG2E);
      }
      const bool seen = key <= pq && (window <= 0 || pq - key < window || key < keep_first);
      v = seen ? v : -INFINITY;
      sc[r] = v;
      tmax = fmaxf(tmax, v);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, DA_WAVE));        // both halves of the wavefront: all 32 keys of the row
    const float m_new = fmaxf(m, tmax);
    const float m_use = m_new != -INFINITY ? m_new : 0.f;     // a row that has seen no key yet keeps zeros
    const float alpha = __builtin_amdgcn_exp2f(m - m_use);
    float tsum = 0.f;
    aw_bf16x8_t pf[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      uint32_t u[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float p0 = __builtin_amdgcn_exp2f(sc[kb * 8 + 2 * e] - m_use);
        const float p1 = __builtin_amdgcn_exp2f(sc[kb * 8 + 2 * e + 1] - m_use);
        tsum += p0 + p1;
        u[e] = pack2_bf16(p0, p1);
      }
      pf[kb] = __builtin_bit_cast(aw_bf16x8_t, make_uint4(u[0], u[1], u[2], u[3]));
    }
    l = l * alpha + tsum;
    m = m_new;
#pragma unroll
    for (int i = 0; i < DT; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc_o[i][r] *= alpha;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const uint2 v0 = tl.v[i][kb * 2], v1 = tl.v[i][kb * 2 + 1];
        const aw_bf16x8_t vf = __builtin_bit_cast(aw_bf16x8_t, make_uint4(v0.x, v0.y, v1.x, v1.y));
        acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kb], acc_o[i], 0, 0, 0);
      }
    }
  };
  // this wavefront's tiles in ascending order: a mod KP == kp among 0 .. n_kept - 1, then among t_lo .. t_hi
  const int win0 = t_lo + ((kp - t_lo % KP) + KP) % KP;
  auto advance = [&](int a) -> int {
    const int b = a + KP;
    return (a < n_kept && b >= n_kept) ? win0 : b;
  };
  {
    AwTile<D16, DT> cur, nxt;
    int a = kp < n_kept ? kp : win0;
    if (a <= t_hi) load(cur, a);
    while (a <= t_hi) {
      const int an = advance(a);
      if (an <= t_hi) load(nxt, an);
      weigh(cur, a);
      cur = nxt;
      a = an;
    }
  }
  l += __shfl_xor(l, 32, DA_WAVE);                       // (both halves had the same maximum all along)
  if (KP > 1) {
    // the phases' partial results, merged by phase 0 in the order of the phases
    if (kp > 0) {
      float* mine = mg + (size_t)((kp - 1) * RB + rbi) * PER * DA_WAVE + lane;
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) mine[(i * 16 + r) * DA_WAVE] = acc_o[i][r];
      mine[(DT * 16) * DA_WAVE] = m;
      mine[(DT * 16 + 1) * DA_WAVE] = l;
    }
    lds_barrier();
    if (kp > 0) return;
    for (int k = 1; k < KP; ++k) {
      const float* theirs = mg + (size_t)((k - 1) * RB + rbi) * PER * DA_WAVE + lane;
      const float mk = theirs[(DT * 16) * DA_WAVE], lk = theirs[(DT * 16 + 1) * DA_WAVE];
      const float m_new = fmaxf(m, mk);
      const float m_use = m_new != -INFINITY ? m_new : 0.f;
      const float a0 = __builtin_amdgcn_exp2f(m - m_use), a1 = __builtin_amdgcn_exp2f(mk - m_use);
      l = l * a0 + lk * a1;
      m = m_new;
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] = acc_o[i][r] * a0 + theirs[(i * 16 + r) * DA_WAVE] * a1;
    }
  }
  if (qi < T) {
    float shrink = 1.f;
    if (sink) {                                          // the term without a key, in the base-2 domain
      const float s0 = sink[h] * AW_LOG2E;
      const float m_all = fmaxf(m, s0);
      shrink = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - m_all);
      l = l * shrink + __builtin_amdgcn_exp2f(s0 - m_all);
    }
    const float inv = l > 0.f ? shrink / l : 0.f;        // a sequence of length 0 (padding) gives zeros
    bf16_t* orow = out + (size_t)(row0 + qi) * out_ld + h * Dv;
    const bf16_t* grow = gate ? gate + (size_t)(row0 + qi) * gate_ld + h * Dv : nullptr;
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
      for (int r = 0; r < 16; r += 4) {
        const int d = i * 32 + 8 * (r / 4) + 4 * hf;     // four neighbouring entries
        if (d < Dv) {
          float g4[4] = {1.f, 1.f, 1.f, 1.f};
          if (grow) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (d + e < Dv) g4[e] = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-AW_LOG2E * bf16_to_f32(grow[d + e])));
          }
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (d + e < Dv) orow[d + e] = f32_to_bf16(acc_o[i][r + e] * inv * g4[e]);
        }
      }
  }
}

// 1 when da_attn_window takes these sizes
extern "C" int da_attn_window_takes(int D, int Dv, int page) {
  return D > 0 && D % 8 == 0 && D <= 128 && Dv > 0 && Dv <= 128 && page >= 8 && (page & (page - 1)) == 0;
}

// Sequences seq0 .. seq0 + n_seqs - 1 of the step; rows of sequence s are q_start[s] .. q_start[s + 1] - 1, the
// last of them at position seq_lens[s] - 1.  form: 0, or the row blocks a workgroup (1, 2, 4).
extern "C" int da_attn_window(const void* q, int q_ld, const void* cache, const int* block_table, int max_blocks,
                              const int* q_start, const int* seq_lens, int seq0, int n_seqs, int max_query_len, int Hq,
                              int Hkv, int D, int Dv, int page, float scale, int window, int keep_first, float softcap,
                              const float* sink, const void* gate, int gate_ld, void* out, int out_ld, int form,
                              void* stream) {
  DA_REQUIRE(n_seqs >= 0 && Hq > 0 && Hkv > 0 && max_query_len >= 0, "attn_window: bad sizes");
  DA_REQUIRE(form == 0 || form == 1 || form == 2 || form == 4, "attn_window: form %d (0 leaves the choice to the rule; 1, 2 or 4 row blocks)", form);
  DA_REQUIRE(Hq % Hkv == 0, "attn_window: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  DA_REQUIRE(da_attn_window_takes(D, Dv, page), "attn_window: head sizes %d and %d with pages of %d are not taken", D, Dv, page);
  DA_REQUIRE(q_ld >= Hq * D && q_ld % 8 == 0 && out_ld >= Hq * Dv, "attn_window: row lengths");
  DA_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)cache % 16 == 0), "attn_window: operands must be 16-byte aligned");
  DA_REQUIRE(window >= 0 && keep_first >= 0 && softcap >= 0.f && max_blocks > 0, "attn_window: bad window, kept keys, cap or block table");
  DA_REQUIRE(scale > 0.f, "attn_window: the score scale must be positive, found %g", (double)scale);
  DA_REQUIRE(!gate || gate_ld >= Hq * Dv, "attn_window: the gate's rows are too short");
  DA_REQUIRE((long)n_seqs * Hq < (1L << 31) && max_query_len <= 65535 * 32, "attn_window: too many sequences, heads or rows for one launch");
  if (n_seqs == 0 || max_query_len == 0) return 0;
  // Row blocks a workgroup by the longest portion; where that leaves few workgroups (a long prompt or two, few
  // heads), smaller workgroups whose wavefronts also share out the keys.  The step's shape only.  Measured on MI355X,
  // head size 64, a window of 512 keeping 4, microseconds with 128 / 64 / 32 rows a workgroup: 2 x 1,024 rows, 6 heads
  // 70 / - / 26.5; 8 heads - / 34.4 / 27.3; 4,096 rows, 16 heads 77.3 / 76.6 / -; 8 x 1,024 rows, 16 heads 113 / - / -.
  int RB = max_query_len <= 32 ? 1 : (max_query_len <= 64 ? 2 : 4);
  const long wg4 = (long)Hq * n_seqs * da_ceil_div(max_query_len, 128);
  if (RB == 4 && wg4 < AW_FEW_WORKGROUPS) RB = 2 * wg4 < AW_FEW_WORKGROUPS ? 1 : 2;
  if (form) RB = form;                                   // (tests walk every form at small sizes)
  const dim3 grid((unsigned)(Hq * n_seqs), (unsigned)da_ceil_div(max_query_len, 32 * RB)), block(AW_WAVES * DA_WAVE);
#define AW_GO(N, M)                                                                                                  \
  hipLaunchKernelGGL((attn_window_kernel<N, M>), grid, block, 0, (hipStream_t)stream, (const bf16_t*)q, q_ld,        \
                     (const bf16_t*)cache, block_table, max_blocks, q_start, seq_lens, seq0, Hq, Hkv, D, Dv, page,   \
                     scale, window, keep_first, softcap, sink, (const bf16_t*)gate, gate_ld, (bf16_t*)out, out_ld, RB)
#define AW_VALUES(N)                 \
  do {                               \
    if (Dv <= 32) AW_GO(N, 1);       \
    else if (Dv <= 64) AW_GO(N, 2);  \
    else AW_GO(N, 4);                \
  } while (0)
  if (D <= 32) AW_VALUES(2);
  else if (D <= 64) AW_VALUES(4);
  else AW_VALUES(8);
#undef AW_VALUES
#undef AW_GO
  DA_CHECK_LAUNCH("attn_window");
  return 0;
}
