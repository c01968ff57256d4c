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
};

template <typename T, int RPL>
__global__ void __launch_bounds__(RET_CPB * RET_LPC)
retention_kernel(RetArgs A) {
  constexpr int DP = RPL * RET_LPC;                 // D rounded up to what the lanes hold
  constexpr int TB = RPL <= 4 ? 64 : (RPL <= 8 ? 32 : 16);       // tokens of a block
  constexpr int PER = TB * RPL / RET_LPC;           // entries of q (and of k) of a block that a thread brings
  constexpr int PERV = TB / RET_GROUP;              // ... and of v
  __shared__ __attribute__((aligned(16))) float qs[TB][DP], ks[TB][DP], vs[TB][RET_CPB];
  const int t = threadIdx.x, j = t % RET_LPC, c = t / RET_LPC;
  const int h = blockIdx.y, s = blockIdx.z;
  const int col = blockIdx.x * RET_CPB + c;
  const bool col_ok = col < A.Dv;
  const int row0 = A.q_start[s], n_tok = A.q_start[s + 1] - row0;
  if (n_tok <= 0) return;
  const int slot = A.state_slots[s];
  const float g = A.decay[h];
  const T* base = (const T*)A.qkv;

  float S[RPL];
  float* srow = (slot >= 0 && col_ok) ? A.state + (size_t)slot * A.state_ld + ((size_t)h * A.Dv + col) * A.D : nullptr;
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int r = j * RPL + i;
    S[i] = (srow && r < A.D) ? srow[r] : 0.f;
  }

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
      rk[i] = base[at + A.k_off];
      ok |= (unsigned long long)e << i;
    }
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
        ks[tok][r] = e ? to_f32(rk[i]) * A.k_scale : 0.f;
      }
    }
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
        const float vv = vs[tk][c];
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
          const int r = j * RPL + i;
          S[i] = fmaf(g, S[i], ks[tk][r] * vv);
          acc = fmaf(S[i], qs[tk][r], acc);
        }
        acc = group_sum<RET_LPC>(acc);
        mine = k == j ? acc : mine;
      };
      if (ng == RET_GROUP) {                        // a whole group: straight-line code, the LDS reads run ahead
#pragma unroll
        for (int k = 0; k < RET_GROUP; ++k) token(k);
      } else {
        for (int k = 0; k < ng; ++k) token(k);
      }
      if (j < ng && col_ok) A.o[(size_t)(row0 + t0 + g0 + j) * A.o_ld + (size_t)h * A.Dv + col] = mine;
    }
  }
  if (A.write && srow) {
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      const int r = j * RPL + i;
      if (r < A.D) srow[r] = S[i];
    }
  }
}

template <typename T>
static int retention_launch(const RetArgs& A, int S, void* stream) {
  const dim3 grid((unsigned)da_ceil_div(A.Dv, RET_CPB), (unsigned)A.H, (unsigned)S), block(RET_CPB * RET_LPC);
  hipStream_t st = (hipStream_t)stream;
  const int rpl = da_ceil_div(A.D, RET_LPC);
  if (rpl <= 1) hipLaunchKernelGGL((retention_kernel<T, 1>), grid, block, 0, st, A);
  else if (rpl <= 2) hipLaunchKernelGGL((retention_kernel<T, 2>), grid, block, 0, st, A);
  else if (rpl <= 4) hipLaunchKernelGGL((retention_kernel<T, 4>), grid, block, 0, st, A);
  else if (rpl <= 8) hipLaunchKernelGGL((retention_kernel<T, 8>), grid, block, 0, st, A);
  else hipLaunchKernelGGL((retention_kernel<T, 16>), grid, block, 0, st, A);
  DA_CHECK_LAUNCH("retention");
  return 0;
}

// Sequences 0 .. S - 1 of the step; rows of sequence s are q_start[s] .. q_start[s + 1] - 1.  The state row of
// state_slots[s] is read at the portion's start and, with `write`, written at its end.
extern "C" int da_retention(const void* qkv, int dtype, int ld, int q_off, int k_off, int v_off, const float* decay,
                            float k_scale, float* state, long state_ld, const int* state_slots, const int* q_start,
                            float* o, int o_ld, int S, int H, int D, int Dv, int write, void* stream) {
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
  A.Dv = Dv; A.write = write; A.k_scale = k_scale;
  if (dtype == DA_BF16) return retention_launch<bf16_t>(A, S, stream);
  return retention_launch<float>(A, S, stream);
}
