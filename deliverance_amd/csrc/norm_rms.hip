// Root-mean-square norms over rows of the 32-bit residual stream, all in 32-bit:
//
//   rms(x)[i] = x[i] / sqrt(mean(x^2) + eps) * (offset + w[i])
//
// `offset` is 0 for a gain stored as it is applied and 1 for a gain stored around zero.  One wavefront
// owns a row; where the width allows it the whole row sits in registers, so every load is in flight at
// once and the row is read once.
//
//   da_rmsnorm      y = rms(x[rows[r]] or x[r])                       (32-bit or bfloat16 out)
//   da_rmsnorm_add  x += rms_a(src);  h = rms_b(x), or x itself converted (optional)   the norm behind a part, the residual
//                   addition and the norm in front of the next part in one pass over the row
#include "common.h"

__device__ __forceinline__ float4 rms_param4(const void* p, int dtype, int i) {
  if (dtype == DA_BF16) {
    const uint2 u = *(const uint2*)((const bf16_t*)p + i);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                       __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
  }
  return *(const float4*)((const float*)p + i);
}

__device__ __forceinline__ void rms_store4(void* y, int y_dtype, size_t at, float4 o) {
  if (y_dtype == DA_BF16) {
    *(uint2*)((bf16_t*)y + at) = make_uint2(pack2_bf16(o.x, o.y), pack2_bf16(o.z, o.w));
  } else {
    *(float4*)((float*)y + at) = o;
  }
}

// VPL float4 a lane: E a multiple of 4, E <= 256 * VPL.  ADD: src is normalised with (wa), added into x,
// and (if h) the new x is normalised with (wb) into h.  !ADD: y = rms(x) with wa.
template <int VPL, bool ADD>
__global__ void __launch_bounds__(4 * DA_WAVE)
rmsnorm_row_kernel(const float* __restrict__ src, const int* __restrict__ rows, const void* __restrict__ wa, int wa_dtype,
                   float* __restrict__ x, const void* __restrict__ wb, int wb_dtype, float offset, float eps,
                   void* __restrict__ y, int y_dtype, int R, int E) {
  const int lane = threadIdx.x % DA_WAVE;
  const int r = blockIdx.x * (blockDim.x / DA_WAVE) + threadIdx.x / DA_WAVE;
  if (r >= R) return;
  const float* sr = src + (size_t)(rows ? rows[r] : r) * E;
  // Up to a width of 1,024 the gains are asked for beside the rows, so that the kernel costs one round trip
  // to memory and not one per norm; wider rows have no registers to spare for that and read them when needed.
  constexpr bool EARLY = VPL <= 4;
  float4 v[VPL], xv[VPL], ga[EARLY ? VPL : 1], gb[EARLY ? VPL : 1];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int c = (lane + i * DA_WAVE) * 4;
    v[i] = *(const float4*)(sr + (c < E ? c : 0));
    if (ADD) xv[i] = *(const float4*)(x + (size_t)r * E + (c < E ? c : 0));
  }
  if (EARLY) {
#pragma unroll
    for (int i = 0; i < (EARLY ? VPL : 1); ++i) {
      const int c = (lane + i * DA_WAVE) * 4, cc = c < E ? c : 0;
      ga[i] = rms_param4(wa, wa_dtype, cc);
      if (ADD && y && wb) gb[i] = rms_param4(wb, wb_dtype, cc);
    }
  }
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i)
    q += ((lane + i * DA_WAVE) * 4 < E ? 1.f : 0.f) * ((v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w));
  const float inv = 1.0f / sqrtf(wave_sum(q) / (float)E + eps);
  float q2 = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int c = (lane + i * DA_WAVE) * 4;
    if (c < E) {
      const float4 g = EARLY ? ga[EARLY ? i : 0] : rms_param4(wa, wa_dtype, c);
      float4 o = make_float4(v[i].x * inv * (offset + g.x), v[i].y * inv * (offset + g.y),
                             v[i].z * inv * (offset + g.z), v[i].w * inv * (offset + g.w));
      if (ADD) {
        o = make_float4(xv[i].x + o.x, xv[i].y + o.y, xv[i].z + o.z, xv[i].w + o.w);
        *(float4*)(x + (size_t)r * E + c) = o;
        xv[i] = o;
        q2 += (o.x * o.x + o.y * o.y) + (o.z * o.z + o.w * o.w);
      } else {
        rms_store4(y, y_dtype, (size_t)r * E + c, o);
      }
    }
  }
  if (ADD && y && !wb) {                               // no second norm: the new x itself, converted
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int c = (lane + i * DA_WAVE) * 4;
      if (c < E) rms_store4(y, y_dtype, (size_t)r * E + c, xv[i]);
    }
  } else if (ADD && y) {
    const float inv2 = 1.0f / sqrtf(wave_sum(q2) / (float)E + eps);
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int c = (lane + i * DA_WAVE) * 4;
      if (c < E) {
        const float4 g = EARLY ? gb[EARLY ? i : 0] : rms_param4(wb, wb_dtype, c);
        rms_store4(y, y_dtype, (size_t)r * E + c,
                   make_float4(xv[i].x * inv2 * (offset + g.x), xv[i].y * inv2 * (offset + g.y),
                               xv[i].z * inv2 * (offset + g.z), xv[i].w * inv2 * (offset + g.w)));
      }
    }
  }
}

// any width, any alignment
template <bool ADD>
__global__ void rmsnorm_any_kernel(const float* __restrict__ src, const int* __restrict__ rows, const void* __restrict__ wa,
                                   int wa_dtype, float* __restrict__ x, const void* __restrict__ wb, int wb_dtype,
                                   float offset, float eps, void* __restrict__ y, int y_dtype, int R, int E) {
  const int lane = threadIdx.x % DA_WAVE;
  const int r = blockIdx.x * (blockDim.x / DA_WAVE) + threadIdx.x / DA_WAVE;
  if (r >= R) return;
  const float* sr = src + (size_t)(rows ? rows[r] : r) * E;
  float q = 0.f;
  for (int i = lane; i < E; i += DA_WAVE) q += sr[i] * sr[i];
  const float inv = 1.0f / sqrtf(wave_sum(q) / (float)E + eps);
  float q2 = 0.f;
  for (int i = lane; i < E; i += DA_WAVE) {
    float o = sr[i] * inv * (offset + load_param(wa, wa_dtype, i));
    if (ADD) {
      o += x[(size_t)r * E + i];
      x[(size_t)r * E + i] = o;
      q2 += o * o;
    } else {
      store_out(y, y_dtype, (size_t)r * E + i, o);
    }
  }
  if (ADD && y && !wb) {
    for (int i = lane; i < E; i += DA_WAVE) store_out(y, y_dtype, (size_t)r * E + i, x[(size_t)r * E + i]);
  } else if (ADD && y) {
    const float inv2 = 1.0f / sqrtf(wave_sum(q2) / (float)E + eps);
    for (int i = lane; i < E; i += DA_WAVE)
      store_out(y, y_dtype, (size_t)r * E + i, x[(size_t)r * E + i] * inv2 * (offset + load_param(wb, wb_dtype, i)));
  }
}

template <bool ADD>
static void rms_launch(const float* src, const int* rows, const void* wa, int wa_dtype, float* x, const void* wb,
                       int wb_dtype, float offset, float eps, void* y, int y_dtype, int R, int E, hipStream_t st) {
  const bool aligned = ((uintptr_t)src % 16 == 0) && ((uintptr_t)y % 16 == 0) && ((uintptr_t)wa % 16 == 0) &&
                       ((uintptr_t)wb % 16 == 0) && ((uintptr_t)x % 16 == 0);
  const int wpb = R >= 512 ? 4 : 1;
#define RMS_LAUNCH(V)                                                                                                  \
  hipLaunchKernelGGL((rmsnorm_row_kernel<V, ADD>), dim3(da_ceil_div(R, wpb)), dim3(wpb * DA_WAVE), 0, st, src, rows, wa, \
                     wa_dtype, x, wb, wb_dtype, offset, eps, y, y_dtype, R, E)
  if (E % 4 == 0 && E <= 4096 && aligned) {
    if (E <= 256) RMS_LAUNCH(1);
    else if (E <= 512) RMS_LAUNCH(2);
    else if (E <= 1024) RMS_LAUNCH(4);
    else if (E <= 2048) RMS_LAUNCH(8);
    else RMS_LAUNCH(16);
  } else {
    hipLaunchKernelGGL((rmsnorm_any_kernel<ADD>), dim3(da_ceil_div(R, 4)), dim3(4 * DA_WAVE), 0, st, src, rows, wa,
                       wa_dtype, x, wb, wb_dtype, offset, eps, y, y_dtype, R, E);
  }
#undef RMS_LAUNCH
}

extern "C" int da_rmsnorm(const float* x, const int* rows, const void* w, int w_dtype, float offset, float eps, void* y,
                          int y_dtype, int R, int E, void* stream) {
  DA_REQUIRE(R >= 0 && E > 0, "rmsnorm: bad sizes R=%d E=%d", R, E);
  DA_REQUIRE(eps > 0.f, "rmsnorm: eps must be > 0");
  DA_REQUIRE(x && w && y, "rmsnorm: a null operand");
  if (R == 0) return 0;
  rms_launch<false>(x, rows, w, w_dtype, nullptr, nullptr, 0, offset, eps, y, y_dtype, R, E, (hipStream_t)stream);
  DA_CHECK_LAUNCH("rmsnorm");
  return 0;
}

extern "C" int da_rmsnorm_add(const float* src, const void* wa, int wa_dtype, float* x, const void* wb, int wb_dtype,
                              float offset, float eps, void* h, int h_dtype, int R, int E, void* stream) {
  DA_REQUIRE(R >= 0 && E > 0, "rmsnorm_add: bad sizes R=%d E=%d", R, E);
  DA_REQUIRE(eps > 0.f, "rmsnorm_add: eps must be > 0");
  DA_REQUIRE(src && wa && x && (const float*)x != src, "rmsnorm_add: a null operand, or the part's output is the stream itself");
  DA_REQUIRE(h != nullptr || wb == nullptr, "rmsnorm_add: the second norm needs an output");
  if (R == 0) return 0;
  rms_launch<true>(src, nullptr, wa, wa_dtype, x, wb, wb_dtype, offset, eps, h, h_dtype, R, E, (hipStream_t)stream);
  DA_CHECK_LAUNCH("rmsnorm_add");
  return 0;
}
