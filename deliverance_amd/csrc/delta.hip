// A gated delta rule's own kernels: the recurrence over a step's tokens and the gated norm of its read-out.
//
// Per value head h a matrix S [D rows (key channels)][Dv columns (value channels)], 32-bit, token by token:
//     S <- g * S            g: one decay a head, or one a head and row
//     u  = beta * (v - S^T k)
//     S <- S + k u^T
//     o  = S^T q            (after the write)
// with k and q scaled to unit length per key head here (1 / sqrt(sum x^2 + unit_eps); q also times D^-1/2),
// beta = 1 / (1 + exp(-braw)), g = exp(-rate[h] * softplus(araw + dt_bias)).  Key head of value head h: h / (H / G).
//
// The columns of S do not meet: column j needs k, q, g, beta and v[j] only.  A column is shared out over 16
// neighbouring lanes, each with RPL consecutive rows in registers; the two sums over rows are taken inside the
// lane and then over the 16 lanes by DPP additions.  A wavefront holds 4 columns, a workgroup's 4 walking wavefronts 16;
// the grid is (sequences x heads x column blocks), each walking its sequence's portion in order; the tokens' numbers
// come through LDS in blocks (see the kernel).  The order of every sum depends on D and on the token's place among
// its portion's groups of four, so a token's result does not depend on its neighbours in the batch, and on how the
// sequence was cut into steps by 32-bit rounding only.
//
// A request's state row holds S as [H][Dv][D] (a column's rows side by side) at its start; a sequence without a
// slot (a padding row of a fixed-shape step) starts from zeros and keeps nothing.
//
//   da_delta_rule        the recurrence; q | k | v rows in the step's dtype, braw/araw 32-bit, o 32-bit
//   da_delta_gate_norm   y[n, h, :] = o[n, h, :] / sqrt(mean(o[n, h, :]^2) + eps) * gain[:] * act(gate[n, h, :])
#include "common.h"

#define DELTA_LPC 16          // lanes that share a column
#define DELTA_CPB 16          // columns of a workgroup (4 wavefronts of 4)
#define DELTA_MAX_D 256

template <bool FAST>
__device__ __forceinline__ float delta_softplus(float v) {
  if (!FAST) return v > 20.f ? v : log1pf(expf(v));
  const float e = __builtin_amdgcn_exp2f(v * 1.4426950408889634f);
  return v > 20.f ? v : 0.6931471805599453f * __builtin_amdgcn_logf(1.0f + e);
}
template <bool FAST>
__device__ __forceinline__ float delta_exp(float v) {
  return FAST ? __builtin_amdgcn_exp2f(v * 1.4426950408889634f) : expf(v);
}
template <bool FAST>
__device__ __forceinline__ float delta_logistic(float v) {
  return FAST ? __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v)) : 1.0f / (1.0f + expf(-v));
}

struct DeltaArgs {
  const void* qkv; int ld;            // [N, >= v_off + H * Dv]: q at 0, k at k_off, v at v_off
  int k_off, v_off;
  const float* braw; int b_ld;        // [N, H]
  const float* araw; int a_ld, a_off; // [N, a_off + H] or [N, a_off + H * D] (may be the rows of braw)
  const float* dt_bias;               // [H] or [H * D]
  const float* rate;                  // [H]: exp(A_log)
  float* state; long state_ld;        // [slots, >= H * Dv * D]
  const int* state_slots;             // [S]
  const int* q_start;                 // [S + 1]
  float* o; int o_ld;                 // [N, H * Dv]
  int H, G, D, Dv, channel, write;
  float unit_eps, q_scale;
};

// Tokens come through LDS in blocks of TB, and a workgroup is two teams: four walking wavefronts and up to eight
// helping ones.  The walkers hold the
// state (16 columns, a column over 16 lanes) and walk a block four tokens at a time; meanwhile the helpers make the
// next block ready in the other LDS buffer: a helper takes whole fours, loads their raw numbers (every load
// unconditional, from a place that exists), and works out in registers, a lane a key row, everything that does not
// depend on the state.  One barrier a block.  With S the state in front of tokens 1..4, P_ts the product of the decays
// of tokens s+1..t (row by row; P_tt = 1) and G_t = P_t0 the product of the decays of tokens 1..t:
//     u_t = beta_t (v_t - S^T (G_t k_t) - sum_{s<t} A_ts u_s)        A_ts = sum_d k_t k_s P_ts
//     o_t = S^T (G_t q_t) + sum_{s<=t} B_ts u_s                       B_ts = sum_d q_t k_s P_ts
//     S  <- G_4 S + sum_s (P_4s k_s) u_s^T
// which is the token-by-token rule written out (no quotient of decays anywhere: only products of numbers in (0, 1]).
// The helpers leave G_t q_t, G_t k_t, P_4s k_s, G_4, A, B, beta and the columns' values.  What is left on the path
// from one four's state to the next: eight sums over the rows of a column (independent of each other, so their lane
// exchanges overlap), ten multiply-adds on a column's four u, and the update.  A portion's last four is filled up
// with tokens that change nothing (decay 1, beta 0, k = q = 0).
#define DELTA_TEAM 256        // threads that walk
#define DELTA_HELPERS 8       // helping wavefronts: one a four of a block of 32 tokens (a four is a trip to memory and
                              // some arithmetic; two fours a helper in a row took as long as the walk of the block)
// SHORT: no sequence brings more than four tokens (decoding): one four a block, one buffer, one helping wavefront.
template <typename T, int RPL, bool FAST, bool SHORT>
__global__ void __launch_bounds__(DELTA_TEAM + DELTA_HELPERS * DA_WAVE)
delta_rule_kernel(DeltaArgs A) {
  constexpr int DP = RPL * DELTA_LPC;                        // key rows, padded
  constexpr int TB = SHORT ? 4 : (RPL <= 4 ? 32 : (RPL == 8 ? 16 : 8));    // tokens a block
  constexpr int NBUF = SHORT ? 1 : 2;
  constexpr int TS = 3 * DP + 20;                            // floats a token: G q | G k | P k | 16 values | beta
  constexpr int NF = TB / 4, FS = DP + 16;                   // fours a block; floats a four: G_4 | A (6) | B (10)
  constexpr int EL = (DP + DA_WAVE - 1) / DA_WAVE;           // key rows a helper's lane
  __shared__ __attribute__((aligned(16))) float stage[NBUF][TB * TS];
  __shared__ __attribute__((aligned(16))) float fours[NBUF][NF * FS];
  const int blocks_per_head = (A.Dv + DELTA_CPB - 1) / DELTA_CPB;
  const int cb = blockIdx.x % blocks_per_head;
  const int h = (blockIdx.x / blocks_per_head) % A.H;
  const int s = blockIdx.x / (blocks_per_head * A.H);
  const int kh = h / (A.H / A.G);
  const int tid = threadIdx.x, lane = tid % DA_WAVE;          // (tid: a walker's)
  const bool helper = threadIdx.x >= DELTA_TEAM;             // (the same for a whole wavefront)
  const int hw = ((int)threadIdx.x - DELTA_TEAM) / DA_WAVE;  // a helper's number
  const int n_helpers = ((int)blockDim.x - DELTA_TEAM) / DA_WAVE;
  const int sub = tid % DELTA_LPC;
  const int col = cb * DELTA_CPB + tid / DELTA_LPC;
  const bool col_ok = col < A.Dv;
  const int row0 = sub * RPL;
  const int first = A.q_start[s], last = A.q_start[s + 1];
  const int n_blocks = (last - first + TB - 1) / TB;
  const float rate = A.rate[h];

  // a helper: fours hw, hw + 4, ... of block b, from memory to the block's LDS buffer
  auto prepare = [&](int b) {
    const int n0 = first + b * TB;
    const int cnt = last - n0 < TB ? last - n0 : TB;
    float* st = stage[b & (NBUF - 1)];
    float* fo = fours[b & (NBUF - 1)];
    for (int f = hw; f * 4 < cnt; f += n_helpers) {
      float q[EL][4], k[EL][4], g[EL][4], vv[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int tok = f * 4 + t, tc = tok < cnt ? tok : cnt - 1;
        const T* row = (const T*)A.qkv + (size_t)(n0 + tc) * A.ld;
#pragma unroll
        for (int e = 0; e < EL; ++e) {
          const int d = lane + e * DA_WAVE, dc = d < A.D ? d : A.D - 1;
          const int ac = A.channel ? h * A.D + dc : h;
          q[e][t] = to_f32(row[kh * A.D + dc]);
          k[e][t] = to_f32(row[A.k_off + kh * A.D + dc]);
          g[e][t] = A.araw[(size_t)(n0 + tc) * A.a_ld + A.a_off + ac] + A.dt_bias[ac];
        }
        const int c = cb * DELTA_CPB + lane % DELTA_CPB;
        vv[t] = to_f32(row[A.v_off + h * A.Dv + (c < A.Dv ? c : A.Dv - 1)]);
      }
      const int bt = f * 4 + lane % 4;                         // the token whose beta this lane takes
      const float braw = A.braw[(size_t)(n0 + (bt < cnt ? bt : cnt - 1)) * A.b_ld + h];
      // q and k to unit length (q also times D^-1/2), decays; tokens past the block's last and rows past D change nothing
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const bool tok_ok = f * 4 + t < cnt;
        float qq = 0.f, kk = 0.f;
#pragma unroll
        for (int e = 0; e < EL; ++e) {
          const bool ok = tok_ok && lane + e * DA_WAVE < A.D;
          q[e][t] = ok ? q[e][t] : 0.f;
          k[e][t] = ok ? k[e][t] : 0.f;
          g[e][t] = ok ? delta_exp<FAST>(-rate * delta_softplus<FAST>(g[e][t])) : 1.f;
          qq = fmaf(q[e][t], q[e][t], qq);
          kk = fmaf(k[e][t], k[e][t], kk);
        }
        qq = wave_sum(qq);
        kk = wave_sum(kk);
        const float qinv = (FAST ? __builtin_amdgcn_rsqf(qq + A.unit_eps) : 1.0f / sqrtf(qq + A.unit_eps)) * A.q_scale;
        const float kinv = FAST ? __builtin_amdgcn_rsqf(kk + A.unit_eps) : 1.0f / sqrtf(kk + A.unit_eps);
#pragma unroll
        for (int e = 0; e < EL; ++e) { q[e][t] *= qinv; k[e][t] *= kinv; }
      }
      float ab[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) ab[i] = 0.f;
#pragma unroll
      for (int e = 0; e < EL; ++e) {
        const int d = lane + e * DA_WAVE;
        const float* qe = q[e];
        const float* ke = k[e];
        const float* ge = g[e];
        const float p21 = ge[1], p32 = ge[2], p43 = ge[3], p31 = ge[1] * ge[2], p42 = ge[2] * ge[3], p41 = p31 * ge[3];
        const float G1 = ge[0], G2 = G1 * ge[1], G3 = G2 * ge[2], G4 = G3 * ge[3];
        ab[0] = fmaf(ke[1] * ke[0], p21, ab[0]);                 // A21 A31 A32 A41 A42 A43
        ab[1] = fmaf(ke[2] * ke[0], p31, ab[1]);
        ab[2] = fmaf(ke[2] * ke[1], p32, ab[2]);
        ab[3] = fmaf(ke[3] * ke[0], p41, ab[3]);
        ab[4] = fmaf(ke[3] * ke[1], p42, ab[4]);
        ab[5] = fmaf(ke[3] * ke[2], p43, ab[5]);
        ab[6] = fmaf(qe[0], ke[0], ab[6]);                       // B11 | B21 B22 | B31 B32 B33 | B41 B42 B43 B44
        ab[7] = fmaf(qe[1] * ke[0], p21, ab[7]);
        ab[8] = fmaf(qe[1], ke[1], ab[8]);
        ab[9] = fmaf(qe[2] * ke[0], p31, ab[9]);
        ab[10] = fmaf(qe[2] * ke[1], p32, ab[10]);
        ab[11] = fmaf(qe[2], ke[2], ab[11]);
        ab[12] = fmaf(qe[3] * ke[0], p41, ab[12]);
        ab[13] = fmaf(qe[3] * ke[1], p42, ab[13]);
        ab[14] = fmaf(qe[3] * ke[2], p43, ab[14]);
        ab[15] = fmaf(qe[3], ke[3], ab[15]);
        if (d < DP) {
          float* t0 = st + (f * 4) * TS + d;
          t0[0] = qe[0] * G1;          t0[DP] = ke[0] * G1;          t0[2 * DP] = ke[0] * p41;
          t0[TS] = qe[1] * G2;         t0[TS + DP] = ke[1] * G2;     t0[TS + 2 * DP] = ke[1] * p42;
          t0[2 * TS] = qe[2] * G3;     t0[2 * TS + DP] = ke[2] * G3; t0[2 * TS + 2 * DP] = ke[2] * p43;
          t0[3 * TS] = qe[3] * G4;     t0[3 * TS + DP] = ke[3] * G4; t0[3 * TS + 2 * DP] = ke[3];
          fo[f * FS + d] = G4;
        }
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) ab[i] = wave_sum(ab[i]);
      if (lane == 0) {
#pragma unroll
        for (int i = 0; i < 16; ++i) fo[f * FS + DP + i] = ab[i];
      }
      if (lane < DELTA_CPB) {
        const bool c_ok = cb * DELTA_CPB + lane < A.Dv;
#pragma unroll
        for (int t = 0; t < 4; ++t) st[(f * 4 + t) * TS + 3 * DP + lane] = (c_ok && f * 4 + t < cnt) ? vv[t] : 0.f;
      }
      if (lane < 4) st[(f * 4 + lane) * TS + 3 * DP + DELTA_CPB] = bt < cnt ? delta_logistic<FAST>(braw) : 0.f;
    }
  };

  if (helper) {
    if (n_blocks > 0) prepare(0);
    lds_barrier();
    for (int b = 0; b < n_blocks; ++b) {
      if (b + 1 < n_blocks) prepare(b + 1);
      lds_barrier();
    }
    return;
  }

  const int slot = A.state_slots[s];
  float* srow = slot >= 0 ? A.state + (size_t)slot * A.state_ld + ((size_t)h * A.Dv + (col_ok ? col : 0)) * A.D : nullptr;
  float S[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) S[r] = (srow && col_ok && row0 + r < A.D) ? srow[row0 + r] : 0.f;
  lds_barrier();
  for (int b = 0; b < n_blocks; ++b) {
    const int n0 = first + b * TB;
    const int cnt = last - n0 < TB ? last - n0 : TB;
    const int n_fours = (cnt + 3) / 4;
    for (int f = 0; f < n_fours; ++f) {
      const float* t0 = stage[b & (NBUF - 1)] + (f * 4) * TS;
      const float* fd = fours[b & (NBUF - 1)] + f * FS;
      float dk[4], eq[4], v[4], be[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        dk[t] = 0.f; eq[t] = 0.f;
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
          dk[t] = fmaf(S[r], t0[t * TS + DP + row0 + r], dk[t]);
          eq[t] = fmaf(S[r], t0[t * TS + row0 + r], eq[t]);
        }
        v[t] = t0[t * TS + 3 * DP + tid / DELTA_LPC];
        be[t] = t0[t * TS + 3 * DP + DELTA_CPB];
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) { dk[t] = group_sum<DELTA_LPC>(dk[t]); eq[t] = group_sum<DELTA_LPC>(eq[t]); }
      const float* ab = fd + DP;
      const float u0 = be[0] * (v[0] - dk[0]);
      const float u1 = be[1] * (v[1] - dk[1] - ab[0] * u0);
      const float u2 = be[2] * (v[2] - dk[2] - ab[1] * u0 - ab[2] * u1);
      const float u3 = be[3] * (v[3] - dk[3] - ab[3] * u0 - ab[4] * u1 - ab[5] * u2);
      const float o0 = eq[0] + ab[6] * u0;
      const float o1 = eq[1] + ab[7] * u0 + ab[8] * u1;
      const float o2 = eq[2] + ab[9] * u0 + ab[10] * u1 + ab[11] * u2;
      const float o3 = eq[3] + ab[12] * u0 + ab[13] * u1 + ab[14] * u2 + ab[15] * u3;
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        float x = fd[row0 + r] * S[r];
        x = fmaf(t0[2 * DP + row0 + r], u0, x);
        x = fmaf(t0[TS + 2 * DP + row0 + r], u1, x);
        x = fmaf(t0[2 * TS + 2 * DP + row0 + r], u2, x);
        x = fmaf(t0[3 * TS + 2 * DP + row0 + r], u3, x);
        S[r] = x;
      }
      // lanes 0..3 of a column's 16 write its four read-outs
      const int tok = f * 4 + sub;
      if (sub < 4 && tok < cnt && col_ok)
        A.o[(size_t)(n0 + tok) * A.o_ld + h * A.Dv + col] = sub == 0 ? o0 : (sub == 1 ? o1 : (sub == 2 ? o2 : o3));
    }
    lds_barrier();
  }
  if (srow && col_ok && A.write) {
#pragma unroll
    for (int r = 0; r < RPL; ++r)
      if (row0 + r < A.D) srow[row0 + r] = S[r];
  }
}

template <typename T, bool FAST>
static int delta_launch(const DeltaArgs& A, int S, int max_rows, void* stream) {
  const int rpl = (A.D + DELTA_LPC - 1) / DELTA_LPC;
  const bool brief = max_rows > 0 && max_rows <= 4;
  const dim3 grid((unsigned)(S * A.H * ((A.Dv + DELTA_CPB - 1) / DELTA_CPB))), block(DELTA_TEAM + (brief ? 1 : DELTA_HELPERS) * DA_WAVE);
#define DA_DELTA_GO(R)                                                                                          \
  do {                                                                                                          \
    if (brief) hipLaunchKernelGGL((delta_rule_kernel<T, R, FAST, true>), grid, block, 0, (hipStream_t)stream, A); \
    else hipLaunchKernelGGL((delta_rule_kernel<T, R, FAST, false>), grid, block, 0, (hipStream_t)stream, A);    \
  } while (0)
  if (rpl <= 1) DA_DELTA_GO(1);
  else if (rpl <= 2) DA_DELTA_GO(2);
  else if (rpl <= 4) DA_DELTA_GO(4);
  else if (rpl <= 8) DA_DELTA_GO(8);
  else DA_DELTA_GO(16);
#undef DA_DELTA_GO
  DA_CHECK_LAUNCH("delta_rule");
  return 0;
}

// max_rows: the most tokens a sequence of the step brings (0: not known)
extern "C" int da_delta_rule(const void* qkv, int dtype, int ld, int k_off, int v_off, const float* braw, int b_ld,
                             const float* araw, int a_ld, int a_off, const float* dt_bias, const float* rate, float* state,
                             long state_ld, const int* state_slots, const int* q_start, float* o, int o_ld, int S, int H,
                             int G, int D, int Dv, int channel, float unit_eps, int write, int max_rows, void* stream) {
  DA_REQUIRE(S >= 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0, "delta_rule: bad sizes");
  DA_REQUIRE(D <= DELTA_MAX_D, "delta_rule: a key size of %d, %d are taken", D, DELTA_MAX_D);
  DA_REQUIRE(k_off >= G * D && v_off >= k_off + G * D && ld >= v_off + H * Dv, "delta_rule: q, k and v leave the row");
  DA_REQUIRE(b_ld >= H && a_off >= 0 && a_ld >= a_off + (channel ? H * D : H) && o_ld >= H * Dv, "delta_rule: row lengths too small");
  DA_REQUIRE(state_ld >= (long)H * Dv * D, "delta_rule: the state row is too short");
  DA_REQUIRE(unit_eps > 0.f, "delta_rule: the unit norm needs a positive eps");
  if (S == 0) return 0;
  DeltaArgs A;
  A.qkv = qkv; A.ld = ld; A.k_off = k_off; A.v_off = v_off; A.braw = braw; A.b_ld = b_ld; A.araw = araw; A.a_ld = a_ld; A.a_off = a_off;
  A.dt_bias = dt_bias; A.rate = rate; A.state = state; A.state_ld = state_ld; A.state_slots = state_slots;
  A.q_start = q_start; A.o = o; A.o_ld = o_ld; A.H = H; A.G = G; A.D = D; A.Dv = Dv; A.channel = channel; A.write = write;
  A.unit_eps = unit_eps; A.q_scale = 1.0f / sqrtf((float)D);
  if (dtype == DA_BF16) return delta_launch<bf16_t, true>(A, S, max_rows, stream);
  return delta_launch<float, false>(A, S, max_rows, stream);
}

// One wavefront per (token, head): the read-out divided by its root mean square, times the gain, times the gate.
template <typename T, bool FAST>
__global__ void __launch_bounds__(256)
delta_gate_norm_kernel(const float* __restrict__ o, int o_ld, const T* __restrict__ gate, int g_ld,
                       const void* __restrict__ gain, int gain_dtype, float eps, int act, T* __restrict__ y, int y_ld,
                       int N, int H, int Dv) {
  const int lane = threadIdx.x % DA_WAVE;
  const long pair = (long)blockIdx.x * (blockDim.x / DA_WAVE) + threadIdx.x / DA_WAVE;
  if (pair >= (long)N * H) return;
  const int n = (int)(pair / H), h = (int)(pair % H);
  const float* src = o + (size_t)n * o_ld + h * Dv;
  float ss = 0.f;
  for (int d = lane; d < Dv; d += DA_WAVE) ss = fmaf(src[d], src[d], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)Dv + eps);
  for (int d = lane; d < Dv; d += DA_WAVE) {
    const float z = to_f32(gate[(size_t)n * g_ld + h * Dv + d]);
    const float gt = act == DA_ACT_SILU ? z * delta_logistic<FAST>(z) : delta_logistic<FAST>(z);
    from_f32(&y[(size_t)n * y_ld + h * Dv + d], src[d] * inv * load_param(gain, gain_dtype, d) * gt);
  }
}

// act: DA_ACT_SILU, or DA_ACT_NONE for the logistic function.
extern "C" int da_delta_gate_norm(const float* o, int o_ld, const void* gate, int dtype, int g_ld, const void* gain,
                                  int gain_dtype, float eps, int act, void* y, int y_ld, int N, int H, int Dv,
                                  void* stream) {
  DA_REQUIRE(N >= 0 && H > 0 && Dv > 0 && o_ld >= H * Dv && g_ld >= H * Dv && y_ld >= H * Dv, "delta_gate_norm: bad sizes");
  DA_REQUIRE(eps > 0.f && (act == DA_ACT_SILU || act == DA_ACT_NONE), "delta_gate_norm: bad eps or gate");
  if (N == 0) return 0;
  const dim3 grid((unsigned)da_ceil_div((long)N * H, 4)), block(256);
  if (dtype == DA_BF16)
    hipLaunchKernelGGL((delta_gate_norm_kernel<bf16_t, true>), grid, block, 0, (hipStream_t)stream, o, o_ld,
                       (const bf16_t*)gate, g_ld, gain, gain_dtype, eps, act, (bf16_t*)y, y_ld, N, H, Dv);
  else
    hipLaunchKernelGGL((delta_gate_norm_kernel<float, false>), grid, block, 0, (hipStream_t)stream, o, o_ld,
                       (const float*)gate, g_ld, gain, gain_dtype, eps, act, (float*)y, y_ld, N, H, Dv);
  DA_CHECK_LAUNCH("delta_gate_norm");
  return 0;
}
