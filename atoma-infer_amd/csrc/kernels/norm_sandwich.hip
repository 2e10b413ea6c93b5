// A sublayer's output normed before it joins the residual stream, fused with the sum and with the norm that reads
// the stream next:
//
//   d     = sum_i scale_i * (sum over planes of delta_i)          (up to two terms: mixers that run side by side)
//   resid += d / sqrt(mean(d^2) + eps) * w_post                   (float32, in place)
//   out   = resid / sqrt(mean(resid^2) + eps) * w_next            (optional, in the activation dtype)
//
// One workgroup a row; the row waits in LDS between the passes, so every operand is read once.  All statistics and
// sums are float32.  The planes of a term are added in the order of their index and the terms in theirs, so a row's
// result does not depend on its place in the batch.
#include "common.h"

using namespace atoma;

struct Term {
  const void* data;      // [planes, T, width]
  int dtype;             // kF32 or kBF16
  int planes;
  size_t plane_stride;   // elements between planes
  float scale;
};

__device__ __forceinline__ float term_at(const Term& t, size_t idx) {
  float v = 0.f;
  if (t.dtype == kF32) {
    const float* p = (const float*)t.data;
    for (int s = 0; s < t.planes; ++s) v += p[s * t.plane_stride + idx];
  } else {
    const bf16_t* p = (const bf16_t*)t.data;
    for (int s = 0; s < t.planes; ++s) v += to_f32(p[s * t.plane_stride + idx]);
  }
  return v * t.scale;
}

template <typename TO>
__global__ void __launch_bounds__(256)
add_normed_kernel(float* __restrict__ resid, Term a, Term b, int n_terms, const float* __restrict__ w_post,
                  const float* __restrict__ w_next, TO* __restrict__ out, int width, float eps_post, float eps_next) {
  extern __shared__ float row[];
  __shared__ float scratch[4];
  const size_t base = (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    float d = term_at(a, base + i);
    if (n_terms > 1) d += term_at(b, base + i);
    row[i] = d;
    ss += d * d;
  }
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps_post);
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float x = resid[base + i] + row[i] * inv * w_post[i];
    resid[base + i] = x;
    row[i] = x;
    ss2 += x * x;
  }
  if (out == nullptr) return;
  ss2 = block_sum<4>(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
  for (int i = threadIdx.x; i < width; i += 256) out[base + i] = from_f32<TO>(row[i] * inv2 * w_next[i]);
}

// terms: data pointers, dtypes, planes, plane strides and scales of one or two terms, each [planes, n_rows, width]
extern "C" int atoma_add_normed(float* resid, const void* d0, int dtype0, int planes0, size_t stride0, float scale0,
                                const void* d1, int dtype1, int planes1, size_t stride1, float scale1,
                                const float* w_post, float eps_post, const float* w_next, float eps_next, void* out,
                                int out_dtype, int n_rows, int width, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || width > 16384 || d0 == nullptr || planes0 <= 0 || (d1 != nullptr && planes1 <= 0)) return ATOMA_ERR_SHAPE;
  if ((dtype0 != kF32 && dtype0 != kBF16) || (d1 != nullptr && dtype1 != kF32 && dtype1 != kBF16)) return ATOMA_ERR_DTYPE;
  Term a{d0, dtype0, planes0, stride0, scale0}, b{d1, dtype1, planes1, stride1, scale1};
  const int n_terms = d1 != nullptr ? 2 : 1;
  const size_t lds = (size_t)width * sizeof(float);
  dim3 grid(n_rows), block(256);
  if (out == nullptr || out_dtype == kF32)
    hipLaunchKernelGGL((add_normed_kernel<float>), grid, block, lds, stream, resid, a, b, n_terms, w_post, w_next,
                       (float*)out, width, eps_post, eps_next);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL((add_normed_kernel<bf16_t>), grid, block, lds, stream, resid, a, b, n_terms, w_post, w_next,
                       (bf16_t*)out, width, eps_post, eps_next);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}
