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
// lane and then over the 16 lanes by DPP additions.  A wavefront holds 4 columns, a workgroup of 4 wavefronts 16;
// the grid is (sequences x heads x column blocks), each walking its sequence's portion in order; the tokens' numbers
// come through LDS in blocks (see the kernel).  The order of every sum depends on D only, so a token's result
// does not depend on how the sequence was cut into steps or on its neighbours in the batch.
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

// What a lane needs of one token, as it stands in LDS.
template <int RPL>
struct DeltaToken {
  float k[RPL], q[RPL], g[RPL];       // unit k, unit q * D^-1/2, the decay a row (channel-wise decays only)
  float v, b, gh;                     // the column's value, beta, the head's decay
};

// Tokens come through LDS in blocks of TB: the whole workgroup loads a block (every number once, coalesced), turns
// the raw numbers into what the recurrence takes (decays, beta, q and k at unit length: all of that is independent
// of the state and done for the block's tokens side by side), and only then walks the block token by token.  The
// next block's loads are in flight meanwhile.  What is left on the path from one token's state to the next is a
// product, a sum over 16 lanes and a multiply-add.
template <typename T, int RPL, bool FAST>
__global__ void __launch_bounds__(256)
delta_rule_kernel(DeltaArgs A) {
  constexpr int DP = RPL * DELTA_LPC;                        // key rows, padded
  constexpr int TB = RPL <= 4 ? 32 : (RPL == 8 ? 16 : 8);    // tokens a block
  constexpr int TS = 3 * DP + 20;                            // floats a token: q | k | g | 16 values | beta | head decay
  constexpr int PT = (TB * DP + 255) / 256, PV = (TB * DELTA_CPB + 255) / 256;
  __shared__ __attribute__((aligned(16))) float stage[TB * TS];
  const int blocks_per_head = (A.Dv + DELTA_CPB - 1) / DELTA_CPB;
  const int cb = blockIdx.x % blocks_per_head;
  const int h = (blockIdx.x / blocks_per_head) % A.H;
  const int s = blockIdx.x / (blocks_per_head * A.H);
  const int kh = h / (A.H / A.G);
  const int tid = threadIdx.x, lane = tid % DA_WAVE, wave = tid / DA_WAVE;
  const int sub = tid % DELTA_LPC;
  const int col = cb * DELTA_CPB + tid / DELTA_LPC;
  const bool col_ok = col < A.Dv;
  const int row0 = sub * RPL;
  const int first = A.q_start[s], last = A.q_start[s + 1];
  const int slot = A.state_slots[s];
  float* srow = slot >= 0 ? A.state + (size_t)slot * A.state_ld + ((size_t)h * A.Dv + (col_ok ? col : 0)) * A.D : nullptr;
  const float rate = A.rate[h];

  float S[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) S[r] = (srow && col_ok && row0 + r < A.D) ? srow[row0 + r] : 0.f;

  // a thread's share of a block, from memory into registers
  float rq[PT], rk[PT], ra[PT], rv[PV], rb = 0.f, rh = 0.f;
  auto fetch = [&](int n0) {
    const int cnt = last - n0 < TB ? last - n0 : TB;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      const int idx = tid + i * 256, tok = idx / DP, d = idx % DP;
      const bool ok = tok < cnt && d < A.D;
      const T* row = (const T*)A.qkv + (size_t)(n0 + (ok ? tok : 0)) * A.ld;
      const int dc = ok ? d : 0;
      rq[i] = ok ? to_f32(row[kh * A.D + dc]) : 0.f;
      rk[i] = ok ? to_f32(row[A.k_off + kh * A.D + dc]) : 0.f;
      ra[i] = (ok && A.channel) ? A.araw[(size_t)(n0 + tok) * A.a_ld + A.a_off + h * A.D + dc] + A.dt_bias[h * A.D + dc] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < PV; ++i) {
      const int idx = tid + i * 256, tok = idx / DELTA_CPB, c = cb * DELTA_CPB + idx % DELTA_CPB;
      const bool ok = tok < cnt && c < A.Dv && idx < TB * DELTA_CPB;
      rv[i] = ok ? to_f32(((const T*)A.qkv)[(size_t)(n0 + tok) * A.ld + A.v_off + h * A.Dv + c]) : 0.f;
    }
    if (tid < cnt) {
      rb = A.braw[(size_t)(n0 + tid) * A.b_ld + h];
      rh = A.channel ? 0.f : A.araw[(size_t)(n0 + tid) * A.a_ld + A.a_off + h] + A.dt_bias[h];
    }
  };
  // ... and from registers into LDS, the decays and beta worked out on the way
  auto park = [&]() {
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      const int idx = tid + i * 256, tok = idx / DP, d = idx % DP;
      if (PT * 256 == TB * DP || idx < TB * DP) {
        float* at = stage + tok * TS + d;
        at[0] = rq[i];
        at[DP] = rk[i];
        if (A.channel) at[2 * DP] = delta_exp<FAST>(-rate * delta_softplus<FAST>(ra[i]));
      }
    }
#pragma unroll
    for (int i = 0; i < PV; ++i) {
      const int idx = tid + i * 256;
      if (idx < TB * DELTA_CPB) stage[(idx / DELTA_CPB) * TS + 3 * DP + idx % DELTA_CPB] = rv[i];
    }
    if (tid < TB) {
      stage[tid * TS + 3 * DP + DELTA_CPB] = delta_logistic<FAST>(rb);
      stage[tid * TS + 3 * DP + DELTA_CPB + 1] = A.channel ? 1.f : delta_exp<FAST>(-rate * delta_softplus<FAST>(rh));
    }
  };
  auto take = [&](int tok, DeltaToken<RPL>& t) {
    const float* at = stage + tok * TS;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      t.q[r] = at[row0 + r];
      t.k[r] = at[DP + row0 + r];
      t.g[r] = A.channel ? at[2 * DP + row0 + r] : 0.f;
    }
    t.v = at[3 * DP + tid / DELTA_LPC];
    t.b = at[3 * DP + DELTA_CPB];
    t.gh = at[3 * DP + DELTA_CPB + 1];
  };

  if (first < last) fetch(first);
  for (int n0 = first; n0 < last; n0 += TB) {
    const int cnt = last - n0 < TB ? last - n0 : TB;
    __syncthreads();                                 // the block before has been walked
    park();
    __syncthreads();
    // q and k to unit length (q also times D^-1/2): wavefront w takes tokens w, w + 4, ...
    for (int tok = wave; tok < cnt; tok += 256 / DA_WAVE) {
      float* at = stage + tok * TS;
      float qq = 0.f, kk = 0.f;
      for (int d = lane; d < DP; d += DA_WAVE) { qq = fmaf(at[d], at[d], qq); kk = fmaf(at[DP + d], at[DP + d], kk); }
      qq = wave_sum(qq);
      kk = wave_sum(kk);
      const float qinv = (FAST ? __builtin_amdgcn_rsqf(qq + A.unit_eps) : 1.0f / sqrtf(qq + A.unit_eps)) * A.q_scale;
      const float kinv = FAST ? __builtin_amdgcn_rsqf(kk + A.unit_eps) : 1.0f / sqrtf(kk + A.unit_eps);
      for (int d = lane; d < DP; d += DA_WAVE) { at[d] *= qinv; at[DP + d] *= kinv; }
    }
    __syncthreads();
    if (n0 + TB < last) fetch(n0 + TB);              // in flight while this block is walked
    DeltaToken<RPL> cur, nxt;
    take(0, cur);
    for (int tok = 0; tok < cnt; ++tok) {
      take(tok + 1 < TB ? tok + 1 : tok, nxt);       // the next token's numbers, ahead
      float dot = 0.f;
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        S[r] *= A.channel ? cur.g[r] : cur.gh;
        dot = fmaf(S[r], cur.k[r], dot);
      }
      dot = group_sum<DELTA_LPC>(dot);
      const float u = cur.b * (cur.v - dot);
      float out = 0.f;
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        S[r] = fmaf(cur.k[r], u, S[r]);
        out = fmaf(S[r], cur.q[r], out);
      }
      out = group_sum<DELTA_LPC>(out);
      if (sub == 0 && col_ok) A.o[(size_t)(n0 + tok) * A.o_ld + h * A.Dv + col] = out;
      cur = nxt;
    }
  }
  if (srow && col_ok && A.write) {
#pragma unroll
    for (int r = 0; r < RPL; ++r)
      if (row0 + r < A.D) srow[row0 + r] = S[r];
  }
}

template <typename T, bool FAST>
static int delta_launch(const DeltaArgs& A, int S, void* stream) {
  const int rpl = (A.D + DELTA_LPC - 1) / DELTA_LPC;
  const dim3 grid((unsigned)(S * A.H * ((A.Dv + DELTA_CPB - 1) / DELTA_CPB))), block(256);
#define DA_DELTA_GO(R) hipLaunchKernelGGL((delta_rule_kernel<T, R, FAST>), grid, block, 0, (hipStream_t)stream, A)
  if (rpl <= 1) DA_DELTA_GO(1);
  else if (rpl <= 2) DA_DELTA_GO(2);
  else if (rpl <= 4) DA_DELTA_GO(4);
  else if (rpl <= 8) DA_DELTA_GO(8);
  else DA_DELTA_GO(16);
#undef DA_DELTA_GO
  DA_CHECK_LAUNCH("delta_rule");
  return 0;
}

extern "C" int da_delta_rule(const void* qkv, int dtype, int ld, int k_off, int v_off, const float* braw, int b_ld,
                             const float* araw, int a_ld, int a_off, const float* dt_bias, const float* rate, float* state,
                             long state_ld, const int* state_slots, const int* q_start, float* o, int o_ld, int S, int H,
                             int G, int D, int Dv, int channel, float unit_eps, int write, void* stream) {
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
  if (dtype == DA_BF16) return delta_launch<bf16_t, true>(A, S, stream);
  return delta_launch<float, false>(A, S, stream);
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
