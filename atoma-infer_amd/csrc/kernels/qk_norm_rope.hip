// Queries and keys normed over their whole projection, rotated in neighbouring pairs, and the cache write, in one pass.
//
// Per token, from the float32 result of the fused q, k projection [T, (nh + nkv) hd]:
//   q <- q / sqrt(mean(q^2 over all nh hd columns) + eps) * wq,   k likewise over its nkv hd columns with wk;
//   columns (2i, 2i + 1), i < rot_dim / 2, of every head become (u cos a - v sin a, v cos a + u sin a) with
//   a = position * inv_freq[i]  (angles, sines and cosines in float32; the other columns pass unchanged);
//   q goes to q_out [T, nh hd] in the activation dtype, the rotated k into the key tiles, and the values' tiles
//   receive either the k projection as it left the product (values tied to the keys) or nothing.
// The heads may leave wider than they came (hd_out >= hd): the columns beyond hd are zeros in q_out and in both
// tiles, so that head sizes which the attention kernels do not take run as the next size they do take (zeros add
// nothing to a score, and a value's zero columns meet zero columns of the output projection).
// The tiles' element order is the attention kernels' (cache_layout.h).  One workgroup a token.
#include "common.h"
#include "cache_layout.h"

using namespace atoma;

template <typename TQ, typename TC>
__global__ void __launch_bounds__(256)
qk_norm_rope_kernel(const float* __restrict__ qk, int ld, const int32_t* __restrict__ positions,
                    const float* __restrict__ inv_freq, int rot_dim, const float* __restrict__ wq,
                    const float* __restrict__ wk, float eps, TQ* __restrict__ q_out, int ldq, TC* __restrict__ kcache,
                    TC* __restrict__ vcache, const int32_t* __restrict__ slot_mapping, int page_size, int nh, int nkv,
                    int hd, int hd_out) {
  __shared__ float scratch[4];
  __shared__ float cs[128], sn[128];
  const int t = blockIdx.x;
  const float* row = qk + (size_t)t * ld;
  const int nq = nh * hd, nk = nkv * hd;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < nq; i += 256) sq += row[i] * row[i];
  for (int i = threadIdx.x; i < nk; i += 256) sk += row[nq + i] * row[nq + i];
  sq = block_sum<4>(sq, scratch);
  sk = block_sum<4>(sk, scratch);
  const float iq = 1.0f / sqrtf(sq / (float)nq + eps), ik = 1.0f / sqrtf(sk / (float)nk + eps);
  const float p = (float)positions[t];
  for (int i = threadIdx.x; i < rot_dim / 2; i += 256) {
    float s, c;
    sincosf(p * inv_freq[i], &s, &c);
    cs[i] = c, sn[i] = s;
  }
  __syncthreads();
  // a thread takes a pair of neighbouring columns
  for (int pr = threadIdx.x; pr < nq / 2; pr += 256) {
    const int col = 2 * pr, head = col / hd, d = col % hd;
    float u = row[col] * iq * wq[col], v = row[col + 1] * iq * wq[col + 1];
    if (d < rot_dim) {
      const float c = cs[d >> 1], s = sn[d >> 1];
      const float u2 = u * c - v * s;
      v = v * c + u * s;
      u = u2;
    }
    q_out[(size_t)t * ldq + head * hd_out + d] = from_f32<TQ>(u);
    q_out[(size_t)t * ldq + head * hd_out + d + 1] = from_f32<TQ>(v);
  }
  const int pad = hd_out - hd;
  for (int i = threadIdx.x; i < nh * pad; i += 256)
    q_out[(size_t)t * ldq + (i / pad) * hd_out + hd + i % pad] = from_f32<TQ>(0.f);
  if (kcache == nullptr) return;
  const int slot = slot_mapping[t];
  const int page = slot / page_size, off = slot % page_size;
  for (int pr = threadIdx.x; pr < nk / 2; pr += 256) {
    const int col = 2 * pr, head = col / hd, d = col % hd;
    const float r0 = row[nq + col], r1 = row[nq + col + 1];
    float u = r0 * ik * wk[col], v = r1 * ik * wk[col + 1];
    if (d < rot_dim) {
      const float c = cs[d >> 1], s = sn[d >> 1];
      const float u2 = u * c - v * s;
      v = v * c + u * s;
      u = u2;
    }
    const size_t tile = ((size_t)page * nkv + head) * page_size * hd_out;
    TC* kt = kcache + tile;
    kt[key_offset(off, d, page_size)] = from_f32<TC>(u);
    kt[key_offset(off, d + 1, page_size)] = from_f32<TC>(v);
    if (vcache != nullptr) {
      TC* vt = vcache + tile;
      vt[value_offset(d, off, hd_out, page_size)] = from_f32<TC>(r0);
      vt[value_offset(d + 1, off, hd_out, page_size)] = from_f32<TC>(r1);
    }
  }
  for (int i = threadIdx.x; i < nkv * pad; i += 256) {
    const int head = i / pad, d = hd + i % pad;
    const size_t tile = ((size_t)page * nkv + head) * page_size * hd_out;
    kcache[tile + key_offset(off, d, page_size)] = from_f32<TC>(0.f);
    if (vcache != nullptr) vcache[tile + value_offset(d, off, hd_out, page_size)] = from_f32<TC>(0.f);
  }
}

extern "C" int atoma_qk_norm_rope(const float* qk, int ld, const int32_t* positions, const float* inv_freq, int rot_dim,
                                  const float* wq, const float* wk, float eps, void* q_out, int ldq, int q_dtype,
                                  void* kcache, void* vcache, int cache_dtype, const int32_t* slot_mapping,
                                  int page_size, int n_tokens, int nh, int nkv, int hd, int hd_out,
                                  hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (hd <= 0 || hd % 2 || rot_dim < 0 || rot_dim % 2 || rot_dim > hd || rot_dim > 256 || nh <= 0 || nkv <= 0 ||
      page_size <= 0 || ld < (nh + nkv) * hd || hd_out < hd || ldq < nh * hd_out)
    return ATOMA_ERR_SHAPE;
  dim3 grid(n_tokens), block(256);
#define ATOMA_QKN(TQ, TC)                                                                                          \
  hipLaunchKernelGGL((qk_norm_rope_kernel<TQ, TC>), grid, block, 0, stream, qk, ld, positions, inv_freq, rot_dim, \
                     wq, wk, eps, (TQ*)q_out, ldq, (TC*)kcache, (TC*)vcache, slot_mapping, page_size, nh, nkv, hd,    \
                     hd_out)
  if (q_dtype == kF32 && cache_dtype == kF32) ATOMA_QKN(float, float);
  else if (q_dtype == kBF16 && cache_dtype == kBF16) ATOMA_QKN(bf16_t, bf16_t);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_QKN
  ATOMA_LAUNCH_CHECK();
  return 0;
}
