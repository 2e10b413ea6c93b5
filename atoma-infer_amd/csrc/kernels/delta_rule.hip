// The gated delta rule: a recurrent mixer whose state is one float32 matrix S [dim, vdim] per head and request.
//
// Per token and head (q, k of size dim, unit length; v of size vdim; beta a scalar; g a decay per key channel):
//   S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q          (the read-out sees the token's write)
// Everything here is float32.  Four kernels:
//   delta_prepare      per token: short causal convolution over time and SiLU of the q, k, v projections (the taps - 1
//                      inputs before an entry's first token come from the request's state), q and k to unit length per
//                      head (q also times dim^-1/2), beta = sigmoid(b), g = exp(-exp(A_log) softplus(a + dt_bias));
//   delta_conv_state   per request: the last taps - 1 inputs of the convolution, for the request's next step;
//   delta_scan         per (request, head, 16 columns of S): the recurrence over the entry's tokens in order, S read from
//                      the request's state slot before and written back after.  A column of S lives in the registers
//                      of 16 neighbouring lanes (dim / 16 rows each, rounded up), so a token costs a lane a few dozen
//                      multiply-adds and one four-step exchange among those lanes; the tokens' inputs pass LDS in
//                      blocks, fetched a block ahead;
//   delta_out          per token and head: o / sqrt(mean(o^2) + eps) * w * sigmoid(gate), in the activation dtype.
// The order of every sum depends on the sizes alone, so a token's result does not depend on how the request was cut
// into steps or on what else the step holds.
//
// State of a request (float32, one row of the state tensor):  [taps - 1][conv channels]  then  [heads][vdim][dim].
#include "common.h"

using namespace atoma;

struct DeltaShape {
  int heads, kv_heads, dim, vdim, taps;
  int ldp;                 // row stride of the projections
  int off_q, off_k, off_v, off_b;   // first columns of the q, k, v and b projections in a row
};

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// conv channels: q (kv_heads * dim), then k (the same), then v (heads * vdim); taps_w [channels, taps] in that order
__global__ void __launch_bounds__(256)
delta_prepare_kernel(const float* __restrict__ proj, DeltaShape sh, const int32_t* __restrict__ token_seq,
                     const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                     const float* __restrict__ state, size_t state_stride, const float* __restrict__ taps_w,
                     const float* __restrict__ dt_pre, int ld_dt, const float* __restrict__ dt_bias,
                     const float* __restrict__ a_log, float* __restrict__ qn, float* __restrict__ kn,
                     float* __restrict__ vn, float* __restrict__ beta, float* __restrict__ decay,
                     float* __restrict__ kq) {
  extern __shared__ float act[];       // the token's channels after convolution and SiLU
  const int t = blockIdx.x;
  const int e = token_seq[t];
  const int n = t - q_start[e];        // the token's index inside its entry
  const int nqk = sh.kv_heads * sh.dim, nv = sh.heads * sh.vdim, channels = 2 * nqk + nv;
  if (blockIdx.y == 1) {
    // the token's second workgroup: the gates of the recurrence, which need nothing of the convolution
    for (int h = threadIdx.x; h < sh.heads; h += 256)
      beta[(size_t)t * sh.heads + h] = sigmoidf_(proj[(size_t)t * sh.ldp + sh.off_b + h]);
    const int nd = sh.heads * sh.dim;
    for (int c = threadIdx.x; c < nd; c += 256) {
      const float rate = expf(a_log[c / sh.dim]);
      decay[(size_t)t * nd + c] = expf(-rate * softplusf_(dt_pre[(size_t)t * ld_dt + c] + dt_bias[c]));
    }
    return;
  }
  const float* conv_state = state + (size_t)state_slots[e] * state_stride;
  // (unrolled so that the loads of several channels and taps are in flight together)
#pragma unroll 4
  for (int c = threadIdx.x; c < channels; c += 256) {
    const int col = c < nqk ? sh.off_q + c : c < 2 * nqk ? sh.off_k + (c - nqk) : sh.off_v + (c - 2 * nqk);
    float y = 0.f;
#pragma unroll 4
    for (int j = 0; j < sh.taps; ++j) {
      const int s = n - (sh.taps - 1) + j;      // index inside the entry of the input under tap j
      const float x = s >= 0 ? proj[(size_t)(t - (sh.taps - 1) + j) * sh.ldp + col]
                             : conv_state[(size_t)(sh.taps - 1 + s) * channels + c];
      y = fmaf(taps_w[(size_t)c * sh.taps + j], x, y);
    }
    act[c] = y * sigmoidf_(y);
  }
  __syncthreads();
  // unit length per head: a wave a head
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float q_scale = 1.0f / sqrtf((float)sh.dim);
  for (int hh = wave; hh < 2 * sh.kv_heads; hh += 4) {
    float* x = act + (size_t)hh * sh.dim;
    float ss = 0.f;
    for (int i = lane; i < sh.dim; i += 64) ss += x[i] * x[i];
    ss = wave_sum(ss);
    const bool is_q = hh < sh.kv_heads;
    const float inv = (is_q ? q_scale : 1.0f) / sqrtf(ss + 1e-6f);
    float* dst = (is_q ? qn : kn) + (size_t)t * nqk + (size_t)(is_q ? hh : hh - sh.kv_heads) * sh.dim;
    for (int i = lane; i < sh.dim; i += 64) dst[i] = act[(size_t)hh * sh.dim + i] = x[i] * inv;
  }
  __syncthreads();
  // k . q of every q/k head, which the recurrence's read-out needs once a token
  for (int hh = wave; hh < sh.kv_heads; hh += 4) {
    float d = 0.f;
    for (int i = lane; i < sh.dim; i += 64) d = fmaf(act[(size_t)hh * sh.dim + i], act[(size_t)(sh.kv_heads + hh) * sh.dim + i], d);
    d = wave_sum(d);
    if (lane == 0) kq[(size_t)t * sh.kv_heads + hh] = d;
  }
  for (int c = threadIdx.x; c < nv; c += 256) vn[(size_t)t * nv + c] = act[2 * nqk + c];
}

// one thread a (entry, channel): the state's rows in ascending order, so that a row is read before it is overwritten
__global__ void __launch_bounds__(256)
delta_conv_state_kernel(const float* __restrict__ proj, DeltaShape sh, const int32_t* __restrict__ q_start,
                        const int32_t* __restrict__ state_slots, float* __restrict__ state, size_t state_stride) {
  const int e = blockIdx.y;
  const int nqk = sh.kv_heads * sh.dim, nv = sh.heads * sh.vdim, channels = 2 * nqk + nv;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= channels) return;
  const int first = q_start[e], count = q_start[e + 1] - first;
  const int col = c < nqk ? sh.off_q + c : c < 2 * nqk ? sh.off_k + (c - nqk) : sh.off_v + (c - 2 * nqk);
  float* st = state + (size_t)state_slots[e] * state_stride;
  const int keep = sh.taps - 1;
  for (int r = 0; r < keep; ++r) {
    const int s = count - keep + r;     // index inside the entry of the input that row r holds afterwards
    st[(size_t)r * channels + c] = s >= 0 ? proj[(size_t)(first + s) * sh.ldp + col] : st[(size_t)(r + count) * channels + c];
  }
}

// Sum over the 16 lanes of a DPP row; every lane gets the same sum (the pairs of each step add the same two numbers).
__device__ __forceinline__ float row16_sum(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xf, 0xf, false));    // lanes i ^ 1
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xf, 0xf, false));    // lanes i ^ 2
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xf, 0xf, false));   // the other quad of 8
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xf, 0xf, false));   // the other half of 16
  return x;
}

// R: rows of S a lane holds.  16 lanes (a DPP row) share a column of S, so dim <= 16 R; a wave holds 4 columns, a
// workgroup of four waves 16.  The tokens' q, k, decay (for the head), v (for the 16 columns), beta and k . q pass
// LDS in blocks of TB tokens: the next block is fetched from memory while this one is worked on, so the walk over the
// tokens waits for LDS only.
template <int R>
__global__ void __launch_bounds__(256)
delta_scan_kernel(const float* __restrict__ qn, const float* __restrict__ kn, const float* __restrict__ vn,
                  const float* __restrict__ beta, const float* __restrict__ decay, const float* __restrict__ kq,
                  DeltaShape sh, const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                  float* __restrict__ state, size_t state_stride, size_t s_offset, float* __restrict__ o) {
  constexpr int DP = 16 * R;                   // dim rounded up; rows beyond dim hold zeros
  constexpr int TB = R <= 8 ? 16 : 8;          // tokens a block
  constexpr int PER = TB * DP / 256;           // elements of q (k, decay) a thread fetches a block
  __shared__ float sq[2][TB][DP], sk[2][TB][DP], sg[2][TB][DP];
  __shared__ float sv[2][TB][16], sb[2][TB], skq[2][TB];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int part = lane & 15;
  const int col_local = wave * 4 + (lane >> 4);
  const int col = blockIdx.x * 16 + col_local;
  const int h = blockIdx.y, e = blockIdx.z;
  const int kv = h / (sh.heads / sh.kv_heads);
  const int dim = sh.dim, vdim = sh.vdim;
  const bool col_ok = col < vdim;
  const int i0 = part * R;
  const int first = q_start[e], count = q_start[e + 1] - first;
  float* sp = state + (size_t)state_slots[e] * state_stride + s_offset +
              ((size_t)h * vdim + (col_ok ? col : 0)) * dim + i0;
  float s[R];
#pragma unroll
  for (int r = 0; r < R; ++r) s[r] = (col_ok && i0 + r < dim) ? sp[r] : 0.f;

  const int nqk = sh.kv_heads * dim, nd = sh.heads * dim, nv = sh.heads * vdim;
  float pq[PER], pk[PER], pg[PER], pv = 0.f, pb = 0.f, pkq = 0.f;
  // block b's share of this thread: element idx = tid + j * 256 of [TB][DP]; v: thread tid of [TB][16]; beta, k . q: tid < TB
  auto fetch = [&](int b) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = tid + j * 256, tok = idx / DP, i = idx % DP;
      const int n = b * TB + tok;
      const bool ok = n < count && i < dim;
      const size_t t = (size_t)(first + n);
      pq[j] = ok ? qn[t * nqk + (size_t)kv * dim + i] : 0.f;
      pk[j] = ok ? kn[t * nqk + (size_t)kv * dim + i] : 0.f;
      pg[j] = ok ? decay[t * nd + (size_t)h * dim + i] : 0.f;
    }
    if (tid < TB * 16) {
      const int tok = tid >> 4, c = blockIdx.x * 16 + (tid & 15);
      const int n = b * TB + tok;
      pv = (n < count && c < vdim) ? vn[(size_t)(first + n) * nv + (size_t)h * vdim + c] : 0.f;
    }
    if (tid < TB) {
      const bool ok = b * TB + tid < count;
      pb = ok ? beta[(size_t)(first + b * TB + tid) * sh.heads + h] : 0.f;
      pkq = ok ? kq[(size_t)(first + b * TB + tid) * sh.kv_heads + kv] : 0.f;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = tid + j * 256, tok = idx / DP, i = idx % DP;
      sq[buf][tok][i] = pq[j];
      sk[buf][tok][i] = pk[j];
      sg[buf][tok][i] = pg[j];
    }
    if (tid < TB * 16) sv[buf][tid >> 4][tid & 15] = pv;
    if (tid < TB) sb[buf][tid] = pb, skq[buf][tid] = pkq;
  };
  const int blocks = (count + TB - 1) / TB;
  if (blocks > 0) {
    fetch(0);
    stash(0);
  }
  __syncthreads();
  for (int b = 0; b < blocks; ++b) {
    const int buf = b & 1;
    if (b + 1 < blocks) fetch(b + 1);
    const int n_tok = min(TB, count - b * TB);
#pragma unroll 2
    for (int tok = 0; tok < n_tok; ++tok) {
      float d1 = 0.f, d2 = 0.f;
      float kr[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        kr[r] = sk[buf][tok][i0 + r];
        s[r] *= sg[buf][tok][i0 + r];
        d1 = fmaf(s[r], kr[r], d1);
        d2 = fmaf(s[r], sq[buf][tok][i0 + r], d2);
      }
      d1 = row16_sum(d1);
      d2 = row16_sum(d2);
      const float u = sb[buf][tok] * (sv[buf][tok][col_local] - d1);
      // o = S_new^T q with S_new = diag(g) S + k u^T
      if (part == 0 && col_ok)
        o[(size_t)(first + b * TB + tok) * nv + (size_t)h * vdim + col] = fmaf(u, skq[buf][tok], d2);
#pragma unroll
      for (int r = 0; r < R; ++r) s[r] = fmaf(kr[r], u, s[r]);
    }
    if (b + 1 < blocks) stash(buf ^ 1);
    __syncthreads();
  }
  if (col_ok) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (i0 + r < dim) sp[r] = s[r];
  }
}

template <typename TO>
__global__ void __launch_bounds__(256)
delta_out_kernel(const float* __restrict__ o, const float* __restrict__ gate_pre, int ld_gate,
                 const float* __restrict__ w, float eps, TO* __restrict__ out, int heads, int vdim) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int h = wave; h < heads; h += 4) {
    const size_t base = ((size_t)t * heads + h) * vdim;
    float ss = 0.f;
    for (int j = lane; j < vdim; j += 64) ss += o[base + j] * o[base + j];
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
    for (int j = lane; j < vdim; j += 64)
      out[base + j] = from_f32<TO>(o[base + j] * inv * w[j] *
                                   sigmoidf_(gate_pre[(size_t)t * ld_gate + (size_t)h * vdim + j]));
  }
}

// The second half of a low-rank map for few tokens: out[t, n] = sum_k x[t, k] * w[n, k], K small (the inner size of
// the map), float32 sums in ascending order of k.  A thread an output; the token's K inputs wait in LDS.  With many
// tokens the general product is the better kernel (it reads a tile of w once for 64 tokens).
template <typename TW>
__global__ void __launch_bounds__(256)
lowrank_up_kernel(const float* __restrict__ x, int ldx, const TW* __restrict__ w, float* __restrict__ out, int ldo,
                  int N, int K) {
  extern __shared__ float xs[];
  const int t = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
  for (int k = threadIdx.x; k < K; k += 256) xs[k] = x[(size_t)t * ldx + k];
  __syncthreads();
  if (n >= N) return;
  const TW* wr = w + (size_t)n * K;
  float acc = 0.f;
#pragma unroll 8
  for (int k = 0; k < K; ++k) acc = fmaf(xs[k], to_f32(wr[k]), acc);
  out[(size_t)t * ldo + n] = acc;
}

extern "C" int atoma_lowrank_up(const float* x, int ldx, const void* w, int w_dtype, float* out, int ldo, int n_tokens,
                                int N, int K, hipStream_t stream) {
  if (n_tokens <= 0 || N <= 0) return 0;
  if (K <= 0 || K > 8192 || ldx < K || ldo < N || n_tokens > 65535) return ATOMA_ERR_SHAPE;
  dim3 grid((N + 255) / 256, n_tokens), block(256);
  if (w_dtype == kBF16)
    hipLaunchKernelGGL((lowrank_up_kernel<bf16_t>), grid, block, K * sizeof(float), stream, x, ldx, (const bf16_t*)w,
                       out, ldo, N, K);
  else if (w_dtype == kF32)
    hipLaunchKernelGGL((lowrank_up_kernel<float>), grid, block, K * sizeof(float), stream, x, ldx, (const float*)w, out,
                       ldo, N, K);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

static bool shape_ok(const DeltaShape& sh) {
  return sh.heads > 0 && sh.kv_heads > 0 && sh.heads % sh.kv_heads == 0 && sh.dim > 0 && sh.dim <= 256 && sh.vdim > 0 &&
         sh.taps >= 1 && sh.taps <= 64 && sh.ldp > 0;
}

extern "C" int atoma_delta_prepare(const float* proj, int ldp, int off_q, int off_k, int off_v, int off_b, int heads,
                                   int kv_heads, int dim, int vdim, int taps, const int32_t* token_seq,
                                   const int32_t* q_start, const int32_t* state_slots, float* state,
                                   size_t state_stride, const float* taps_w, const float* dt_pre, int ld_dt,
                                   const float* dt_bias,
                                   const float* a_log, float* qn, float* kn, float* vn, float* beta, float* decay,
                                   float* kq, int n_tokens, int n_entries, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  DeltaShape sh{heads, kv_heads, dim, vdim, taps, ldp, off_q, off_k, off_v, off_b};
  if (!shape_ok(sh) || n_entries <= 0 || n_entries > 65535) return ATOMA_ERR_SHAPE;
  // (a token has two workgroups: convolution, SiLU and unit lengths; beta and decay)
  const int channels = 2 * kv_heads * dim + heads * vdim;
  if ((size_t)channels * sizeof(float) > 60 * 1024) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(delta_prepare_kernel, dim3(n_tokens, 2), dim3(256), channels * sizeof(float), stream, proj, sh,
                     token_seq, q_start, state_slots, state, state_stride, taps_w, dt_pre, ld_dt, dt_bias, a_log, qn, kn, vn,
                     beta, decay, kq);
  ATOMA_LAUNCH_CHECK();
  if (taps > 1) {
    hipLaunchKernelGGL(delta_conv_state_kernel, dim3((channels + 255) / 256, n_entries), dim3(256), 0, stream, proj, sh,
                       q_start, state_slots, state, state_stride);
    ATOMA_LAUNCH_CHECK();
  }
  return 0;
}

extern "C" int atoma_delta_scan(const float* qn, const float* kn, const float* vn, const float* beta,
                                const float* decay, const float* kq, int heads, int kv_heads, int dim, int vdim, int taps,
                                const int32_t* q_start, const int32_t* state_slots, float* state, size_t state_stride,
                                int n_entries, float* o, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  DeltaShape sh{heads, kv_heads, dim, vdim, taps, 1, 0, 0, 0, 0};
  if (!shape_ok(sh) || n_entries > 65535 || heads > 65535) return ATOMA_ERR_SHAPE;
  const size_t s_offset = (size_t)(taps - 1) * (2 * kv_heads * dim + heads * vdim);
  dim3 grid((vdim + 15) / 16, heads, n_entries), block(256);
#define ATOMA_SCAN(R_)                                                                                            \
  hipLaunchKernelGGL((delta_scan_kernel<R_>), grid, block, 0, stream, qn, kn, vn, beta, decay, kq, sh, q_start,   \
                     state_slots, state, state_stride, s_offset, o)
  if (dim <= 16) ATOMA_SCAN(1);
  else if (dim <= 32) ATOMA_SCAN(2);
  else if (dim <= 64) ATOMA_SCAN(4);
  else if (dim <= 128) ATOMA_SCAN(8);
  else ATOMA_SCAN(16);
#undef ATOMA_SCAN
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_delta_out(const float* o, const float* gate_pre, int ld_gate, const float* w, float eps, void* out,
                               int out_dtype, int n_tokens, int heads, int vdim, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (heads <= 0 || vdim <= 0 || ld_gate < heads * vdim) return ATOMA_ERR_SHAPE;
  if (out_dtype == kF32)
    hipLaunchKernelGGL((delta_out_kernel<float>), dim3(n_tokens), dim3(256), 0, stream, o, gate_pre, ld_gate, w,
                       eps, (float*)out, heads, vdim);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL((delta_out_kernel<bf16_t>), dim3(n_tokens), dim3(256), 0, stream, o, gate_pre, ld_gate, w,
                       eps, (bf16_t*)out, heads, vdim);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}
