// Retention: linear attention with a fixed decay per head, without softmax or denominator.
//
// Per head h a matrix S [D rows (key channels)][Dv columns (value channels)], 32-bit, token by token:
//     S <- decay[h] * S + k v^T
//     o  = S^T q            (after the write)
// q and k come turned by their positions already; k is multiplied by k_scale here (D^-1/2).
//
// The columns of S do not meet: column c needs q, k and v[c] only.  A column is shared out over 16 neighbouring
// lanes, lane j holding the RPL consecutive rows from j * RPL on in registers (so that a token's q and k entries are
// one 16-byte LDS read each where RPL is a multiple of 4); the sum over rows is taken inside the lane and then over
// the 16 lanes by DPP additions.  A wavefront holds 4 columns, a workgroup of 4 wavefronts 16; the grid is
// (column blocks x heads x sequences), each walking its sequence's portion in order.  Tokens come through LDS in
// blocks of TB (64 for key sizes up to 64, 32 up to 128, else 16: 32 KB of LDS): every thread asks for its share of
// the next block before it walks the block at hand, and a block's walk (about 3 us) is longer than the trip to
// memory.  Inside a block the walk goes in groups of 16 tokens of straight-line code; lane j keeps the result of a
// group's token j, so a group's results leave in one store a lane.  A token's result is the same bits however the
// sequence was cut into steps and whatever else the step holds: the walk is the recurrence itself, and the order of
// the sum over rows depends on D only.
//
// Long portions in chunks (`chunk` > 0; the bfloat16 path from 256 rows on): the recurrence is linear in the state, so
// chunk k of a portion is walked from a zero state (chunk 0 from the request's) by a workgroup of its own, all chunks
// side by side, and leaves its end state Q_k; a carry pass turns these into the true states at the chunks' starts,
// start_{k+1} = decay^len_k start_k + Q_k, and keeps the last as the request's; a third pass adds what the walk from
// zero left out, o_t += decay^(t - t_k + 1) start_k^T q_t, again all chunks side by side.  A row's result then depends
// on where its chunk starts in the portion, by 32-bit rounding only; the 32-bit path walks every portion in one piece.
//
// A request's state row holds S as [H][Dv][D] (a column's rows side by side) at its start; a sequence without a
// slot (a padding row of a fixed-shape step) starts from zeros and keeps nothing.
#include "common.h"

#define RET_LPC 16            // lanes that share a column
#define RET_CPB 16            // columns of a workgroup
#define RET_GROUP 16          // tokens whose results the 16 lanes of a column keep, one each
#define RET_MAX_D 256

struct RetArgs {
  const void* qkv; int ld;            // [N, ...]: q at q_off, k at k_off (H * D each), v at v_off (H * Dv)
  int q_off, k_off, v_off;
  const float* decay;                 // [H]
  float* state; long state_ld;        // [slots, >= H * Dv * D]
  const int* state_slots;             // [S]
  const int* q_start;                 // [S + 1]
  float* o; int o_ld;                 // [N, H * Dv]
  int H, D, Dv, write;
  float k_scale;
  int chunk, n_chunks;                // tokens of a chunk (0: portions in one piece), chunks of the longest portion
  float* ends;                        // [S * n_chunks, H * Dv * D]: the chunks' end states, then their start states
};

#define RET_WALK 0            // the recurrence
#define RET_ADD 1             // o += decay^(t + 1) start^T q for the chunks behind a portion's first

template <typename T, int RPL, int MODE>
__global__ void __launch_bounds__(RET_CPB * RET_LPC)
retention_kernel(RetArgs A) {
  constexpr int DP = RPL * RET_LPC;                 // D rounded up to what the lanes hold
  constexpr int TB = RPL <= 4 ? 64 : (RPL <= 8 ? 32 : 16);       // tokens of a block
  constexpr int PER = TB * RPL / RET_LPC;           // entries of q (and of k) of a block that a thread brings
  constexpr int PERV = TB / RET_GROUP;              // ... and of v
  __shared__ __attribute__((aligned(16))) float qs[TB][DP], ks[TB][DP], vs[TB][RET_CPB];
  const int t = threadIdx.x, j = t % RET_LPC, c = t / RET_LPC;
  const int h = blockIdx.y;
  const int s = A.chunk ? (int)blockIdx.z / A.n_chunks : (int)blockIdx.z;
  const int kc = A.chunk ? (int)blockIdx.z % A.n_chunks : 0;           // this workgroup's chunk of the portion
  const int col = blockIdx.x * RET_CPB + c;
  const bool col_ok = col < A.Dv;
  const int first = A.q_start[s] + kc * A.chunk;
  const int left = A.q_start[s + 1] - first;
  const int n_tok = A.chunk && left > A.chunk ? A.chunk : left;        // tokens of this chunk (of the portion)
  if (n_tok <= 0 || (MODE == RET_ADD && kc == 0)) return;
  const int row0 = first;
  const int slot = A.state_slots[s];
  const float g = A.decay[h];
  const T* base = (const T*)A.qkv;

  // the state at the start: the request's for a portion's first chunk, zeros for the walk of a later one (whose
  // true start the carry pass leaves in `ends`, where the adding pass finds it)
  float S[RPL];
  float* srow = (slot >= 0 && col_ok) ? A.state + (size_t)slot * A.state_ld + ((size_t)h * A.Dv + col) * A.D : nullptr;
  float* erow = (A.chunk && col_ok) ? A.ends + ((size_t)blockIdx.z * A.H * A.Dv + (size_t)h * A.Dv + col) * A.D : nullptr;
  const float* from = MODE == RET_ADD ? erow : (kc == 0 ? srow : nullptr);
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int r = j * RPL + i;
    S[i] = (from && r < A.D) ? from[r] : 0.f;
  }
  float pw = g;                                     // RET_ADD: decay^(t + 1) of the token at hand

  // this thread's share of a block: entries t + 256 i of [token][DP] for q and for k, of [token][16] for v
  T rq[PER], rk[PER], rv[PERV];
  unsigned long long ok = 0;                        // bit i: entry i of q and k exists; bit 60 + i: entry i of v
  auto fetch = [&](int t0) {
    ok = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = t + 256 * i, tok = idx / DP, r = idx % DP;
      const bool e = t0 + tok < n_tok && r < A.D;
      const size_t at = (size_t)(row0 + (e ? t0 + tok : 0)) * A.ld + (size_t)h * A.D + (e ? r : 0);
      rq[i] = base[at + A.q_off];                   // (unconditional, from a place that exists; looked at when parked)
      if (MODE == RET_WALK) rk[i] = base[at + A.k_off];
      ok |= (unsigned long long)e << i;
    }
    if (MODE == RET_WALK)
#pragma unroll
    for (int i = 0; i < PERV; ++i) {
      const int idx = t + 256 * i, tok = idx / RET_CPB, cc = blockIdx.x * RET_CPB + idx % RET_CPB;
      const bool e = t0 + tok < n_tok && cc < A.Dv;
      rv[i] = base[(size_t)(row0 + (e ? t0 + tok : 0)) * A.ld + A.v_off + (size_t)h * A.Dv + (e ? cc : 0)];
      ok |= (unsigned long long)e << (60 + i);
    }
  };
  auto park = [&](int nt) {                         // (tokens past the block's last are never read)
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = t + 256 * i, tok = idx / DP, r = idx % DP;
      const bool e = (ok >> i) & 1u;
      if (tok < nt) {
        qs[tok][r] = e ? to_f32(rq[i]) : 0.f;
        if (MODE == RET_WALK) ks[tok][r] = e ? to_f32(rk[i]) * A.k_scale : 0.f;
      }
    }
    if (MODE == RET_WALK)
#pragma unroll
    for (int i = 0; i < PERV; ++i) {
      const int idx = t + 256 * i;
      if (idx / RET_CPB < nt) vs[idx / RET_CPB][idx % RET_CPB] = ((ok >> (60 + i)) & 1u) ? to_f32(rv[i]) : 0.f;
    }
  };

  fetch(0);
  for (int t0 = 0; t0 < n_tok; t0 += TB) {
    const int nt = n_tok - t0 < TB ? n_tok - t0 : TB;
    __syncthreads();                                // the block before has been walked by everyone
    park(nt);
    __syncthreads();
    if (t0 + TB < n_tok) fetch(t0 + TB);
    for (int g0 = 0; g0 < nt; g0 += RET_GROUP) {
      const int ng = nt - g0 < RET_GROUP ? nt - g0 : RET_GROUP;
      float mine = 0.f;                             // lane j keeps the result of the group's token j
      auto token = [&](int k) {
        const int tk = g0 + k;
        float acc = 0.f;
        if (MODE == RET_WALK) {
          const float vv = vs[tk][c];
#pragma unroll
          for (int i = 0; i < RPL; ++i) {
            const int r = j * RPL + i;
            S[i] = fmaf(g, S[i], ks[tk][r] * vv);
            acc = fmaf(S[i], qs[tk][r], acc);
          }
          acc = group_sum<RET_LPC>(acc);
        } else {
#pragma unroll
          for (int i = 0; i < RPL; ++i) acc = fmaf(S[i], qs[tk][j * RPL + i], acc);
          acc = group_sum<RET_LPC>(acc) * pw;
          pw *= g;
        }
        mine = k == j ? acc : mine;
      };
      if (ng == RET_GROUP) {                        // a whole group: straight-line code, the LDS reads run ahead
#pragma unroll
        for (int k = 0; k < RET_GROUP; ++k) token(k);
      } else {
        for (int k = 0; k < ng; ++k) token(k);
      }
      if (j < ng && col_ok) {
        float* op = A.o + (size_t)(row0 + t0 + g0 + j) * A.o_ld + (size_t)h * A.Dv + col;
        *op = MODE == RET_ADD ? *op + mine : mine;
      }
    }
  }
  if (MODE == RET_ADD) return;
  float* keep = A.chunk ? erow : (A.write ? srow : nullptr);           // in chunks: every chunk's end state, for the carry pass
  if (keep) {
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      const int r = j * RPL + i;
      if (r < A.D) keep[r] = S[i];
    }
  }
}

// One thread an entry of a head's state: ends[s][k] holds chunk k's end state from its walk (chunk 0: the true one);
// afterwards ends[s][k] is the true state at chunk k's start (k >= 1), and the request's row the state at the
// portion's end.  decay^len by repeated multiplication, the same for every entry.
__global__ void retention_carry_kernel(RetArgs A, int S) {
  const long per = (long)A.H * A.Dv * A.D;
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= per * S) return;
  const int s = (int)(i / per);
  const long e = i % per;
  const int n_tok = A.q_start[s + 1] - A.q_start[s];
  if (n_tok <= 0) return;
  const float g = A.decay[e / ((long)A.Dv * A.D)];
  const int nk = (n_tok + A.chunk - 1) / A.chunk;
  float* ends = A.ends + (size_t)s * A.n_chunks * per + e;
  // decay^chunk and decay^(the last chunk's length), each by repeated multiplication, once
  const int last = n_tok - (nk - 1) * A.chunk;
  float p_last = 1.f, p_full = 1.f;
  for (int t = 0; t < A.chunk; ++t) {
    p_full *= g;
    p_last = t < last ? p_full : p_last;
  }
  float cur = ends[0];
  for (int k0 = 1; k0 < nk; k0 += 8) {              // eight chunks' end states asked for at once, then walked
    float q[8];
#pragma unroll
    for (int i2 = 0; i2 < 8; ++i2) q[i2] = ends[(size_t)(k0 + i2 < nk ? k0 + i2 : 0) * per];
#pragma unroll
    for (int i2 = 0; i2 < 8; ++i2) {
      const int k = k0 + i2;
      if (k < nk) {
        ends[(size_t)k * per] = cur;
        cur = fmaf(k == nk - 1 ? p_last : p_full, cur, q[i2]);
      }
    }
  }
  const int slot = A.state_slots[s];
  if (A.write && slot >= 0) A.state[(size_t)slot * A.state_ld + e] = cur;
}

template <typename T, int MODE>
static int retention_launch(const RetArgs& A, int S, void* stream) {
  const dim3 grid((unsigned)da_ceil_div(A.Dv, RET_CPB), (unsigned)A.H, (unsigned)(A.chunk ? S * A.n_chunks : S)), block(RET_CPB * RET_LPC);
  hipStream_t st = (hipStream_t)stream;
  const int rpl = da_ceil_div(A.D, RET_LPC);
  if (rpl <= 1) hipLaunchKernelGGL((retention_kernel<T, 1, MODE>), grid, block, 0, st, A);
  else if (rpl <= 2) hipLaunchKernelGGL((retention_kernel<T, 2, MODE>), grid, block, 0, st, A);
  else if (rpl <= 4) hipLaunchKernelGGL((retention_kernel<T, 4, MODE>), grid, block, 0, st, A);
  else if (rpl <= 8) hipLaunchKernelGGL((retention_kernel<T, 8, MODE>), grid, block, 0, st, A);
  else hipLaunchKernelGGL((retention_kernel<T, 16, MODE>), grid, block, 0, st, A);
  DA_CHECK_LAUNCH("retention");
  return 0;
}

template <typename T>
static int retention_go(const RetArgs& A, int S, void* stream) {
  if (retention_launch<T, RET_WALK>(A, S, stream)) return 2;
  if (!A.chunk) return 0;
  // (in chunks the walk leaves every end state in `ends`, a portion's only chunk included: the carry pass keeps it)
  const long n = (long)S * A.H * A.Dv * A.D;
  hipLaunchKernelGGL(retention_carry_kernel, dim3(da_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, A, S);
  DA_CHECK_LAUNCH("retention_carry");
  if (A.n_chunks < 2) return 0;
  return retention_launch<T, RET_ADD>(A, S, stream);
}

// Sequences 0 .. S - 1 of the step; rows of sequence s are q_start[s] .. q_start[s + 1] - 1.  The state row of
// state_slots[s] is read at the portion's start and, with `write`, written at its end.  chunk > 0: portions in
// chunks of so many tokens (a multiple of 16) that run side by side, n_chunks of them for the longest portion, their
// states passing through `ends` ([S * n_chunks, H * Dv * D], 32-bit).
extern "C" int da_retention(const void* qkv, int dtype, int ld, int q_off, int k_off, int v_off, const float* decay,
                            float k_scale, float* state, long state_ld, const int* state_slots, const int* q_start,
                            float* o, int o_ld, int S, int H, int D, int Dv, int write, int chunk, int n_chunks,
                            float* ends, long ends_floats, void* stream) {
  DA_REQUIRE(chunk >= 0 && (chunk == 0 || (chunk % RET_GROUP == 0 && n_chunks >= 1 && ends != nullptr &&
                                           ends_floats >= (long)S * n_chunks * H * Dv * D)),
             "retention: chunks of %d tokens need a multiple of %d and a scratch for %d x %d states", chunk, RET_GROUP, S, n_chunks);
  DA_REQUIRE(chunk == 0 || (long)S * n_chunks <= 65535, "retention: too many chunks for one launch");
  DA_REQUIRE(S >= 0 && H > 0 && D > 0 && Dv > 0, "retention: bad sizes");
  DA_REQUIRE(D <= RET_MAX_D, "retention: a key size of %d, %d are taken", D, RET_MAX_D);
  DA_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && ld >= q_off + H * D && ld >= k_off + H * D && ld >= v_off + H * Dv,
             "retention: q, k and v leave the row");
  DA_REQUIRE(o_ld >= H * Dv && state_ld >= (long)H * Dv * D, "retention: the rows of o or of the state are too short");
  DA_REQUIRE(H <= 65535 && S <= 65535, "retention: too many heads or sequences for one launch");
  if (S == 0) return 0;
  RetArgs A;
  A.qkv = qkv; A.ld = ld; A.q_off = q_off; A.k_off = k_off; A.v_off = v_off; A.decay = decay; A.state = state;
  A.state_ld = state_ld; A.state_slots = state_slots; A.q_start = q_start; A.o = o; A.o_ld = o_ld; A.H = H; A.D = D;
  A.Dv = Dv; A.write = write; A.k_scale = k_scale; A.chunk = chunk; A.n_chunks = chunk ? n_chunks : 1; A.ends = ends;
  if (dtype == DA_BF16) return retention_go<bf16_t>(A, S, stream);
  return retention_go<float>(A, S, stream);
}
