// Small elementwise kernels.
//   da_gated_act   mid[r, j] = act(gu[r, j]) * gu[r, inner + j]     the two halves of a fused gate | up product
//                  (or the capped form of common.h with its limit)
//   da_concat_rows dst[r, off + c] = src[r, c]                      a 32-bit matrix into columns of a wider one
//   da_softcap     v <- cap * tanh(v / cap)                         in place, 32-bit
//   da_scale_add_rows  dst[r, c] += mult * scale[c] * src[r, c]     a learned scale per channel, 32-bit
#include "common.h"

template <typename T, bool FAST>
__global__ void gated_act_kernel(const T* __restrict__ gu, int ld, T* __restrict__ mid, int ldm, int R, int inner, int act,
                                 float limit) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)R * inner) return;
  const int r = (int)(i / inner), j = (int)(i % inner);
  const float g = to_f32(gu[(size_t)r * ld + j]), u = to_f32(gu[(size_t)r * ld + inner + j]);
  from_f32(&mid[(size_t)r * ldm + j], gated_mid<FAST>(g, u, act, limit));
}

extern "C" int da_gated_act(const void* gu, int ld, int dtype, void* mid, int ldm, int R, int inner, int act, float limit,
                            void* stream) {
  DA_REQUIRE(R >= 0 && inner > 0 && ld >= 2 * inner && ldm >= inner, "gated_act: bad sizes R=%d inner=%d", R, inner);
  DA_REQUIRE(act != DA_ACT_GLU_CAPPED || limit > 0.f, "gated_act: the capped form needs a positive limit");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_LAST, "gated_act: unknown activation %d", act);
  if (R == 0) return 0;
  const long n = (long)R * inner;
  if (dtype == DA_BF16)
    hipLaunchKernelGGL((gated_act_kernel<bf16_t, true>), dim3(da_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)gu, ld, (bf16_t*)mid, ldm, R, inner, act, limit);
  else
    hipLaunchKernelGGL((gated_act_kernel<float, false>), dim3(da_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream,
                       (const float*)gu, ld, (float*)mid, ldm, R, inner, act, limit);
  DA_CHECK_LAUNCH("gated_act");
  return 0;
}

__global__ void softcap_kernel(float* __restrict__ v, long n, float cap) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) v[i] = cap * tanhf(v[i] / cap);
}

extern "C" int da_softcap(float* v, long n, float cap, void* stream) {
  DA_REQUIRE(n >= 0 && cap > 0.f, "softcap: bad size or cap");
  if (n == 0) return 0;
  hipLaunchKernelGGL(softcap_kernel, dim3(da_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, v, n, cap);
  DA_CHECK_LAUNCH("softcap");
  return 0;
}

__global__ void scale_add_rows_kernel(const float* __restrict__ src, const float* __restrict__ scale,
                                      float* __restrict__ dst, long n, int E, float mult) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = fmaf(mult * scale[i % E], src[i], dst[i]);
}

extern "C" int da_scale_add_rows(const float* src, const float* scale, float* dst, int R, int E, float mult, void* stream) {
  DA_REQUIRE(R >= 0 && E > 0, "scale_add_rows: bad sizes");
  if (R == 0) return 0;
  const long n = (long)R * E;
  hipLaunchKernelGGL(scale_add_rows_kernel, dim3(da_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, src, scale, dst, n,
                     E, mult);
  DA_CHECK_LAUNCH("scale_add_rows");
  return 0;
}

template <typename T>
__global__ void concat_rows_kernel(const float* __restrict__ src, T* __restrict__ dst, int ld, int off, long n, int E) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) from_f32(&dst[(i / E) * ld + off + i % E], src[i]);
}

extern "C" int da_concat_rows(const float* src, void* dst, int dtype, int ld, int off, int R, int E, void* stream) {
  DA_REQUIRE(R >= 0 && E > 0 && off >= 0 && ld >= off + E, "concat_rows: the columns leave the row");
  if (R == 0) return 0;
  const long n = (long)R * E;
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(concat_rows_kernel<bf16_t>, dim3(da_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, src,
                       (bf16_t*)dst, ld, off, n, E);
  else
    hipLaunchKernelGGL(concat_rows_kernel<float>, dim3(da_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, src,
                       (float*)dst, ld, off, n, E);
  DA_CHECK_LAUNCH("concat_rows");
  return 0;
}
