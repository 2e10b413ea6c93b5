// A selective state-space recurrence with one scalar decay per head (the Mamba-2 form): per head and request a
// float32 matrix S [n, vdim] that every token decays, writes and reads,
//
//   S <- a S + dt B x^T;   y = S^T C + D x,        a = exp(-exp(A_log) dt),  dt = softplus(dt_raw + dt_bias),
//
// with x (vdim per head), B and C (n per group of heads) the token's projections after a short causal convolution over
// time (with bias) and SiLU.  Everything here is float32.  Four kernels:
//   ssd_prepare      per token: the convolution (the taps - 1 inputs before an entry's first token come from the
//                    request's state), bias and SiLU of the x, B, C channels; dt and the decay of every head;
//   ssd_conv_state   per request: the last taps - 1 inputs of the convolution, for the request's next step;
//   ssd_scan         per (request, head, 16 columns of S): the recurrence over the entry's tokens in order, S read from
//                    the request's state slot before and written back after.  A column of S lives in the registers of
//                    16 neighbouring lanes (n / 16 rows each, rounded up); the tokens' inputs pass LDS in blocks;
//   ssd_scores,      the same recurrence for entries of many tokens (prompts and their portions), 64 tokens at a time on
//   ssd_chunk        the matrix cores in float32 (v_mfma_f32_16x16x4_f32), see below;
//   ssd_out          per token and norm group: y * silu(z), divided by the root mean square of its group, times the
//                    weight, in the activation dtype.
// The order of every sum depends on the sizes alone, so a token's result does not depend on how the request was cut
// into steps or on what else the step holds.
//
// State of a request (float32, one row of the state tensor):  [taps - 1][conv channels]  then  [heads][vdim][n].
#include "common.h"

using namespace atoma;

struct SsdShape {
  int heads, groups, vdim, n, taps;
  int ldp;                          // row stride of the projections
  int off_z, off_x, off_dt;         // first columns of z, of the convolved channels (x, B, C) and of dt in a row
};

__device__ __forceinline__ float ssd_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float ssd_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// conv channels: x (heads * vdim), then B (groups * n), then C (the same), as they lie in a row of the projections
__global__ void __launch_bounds__(256)
ssd_prepare_kernel(const float* __restrict__ proj, SsdShape sh, const int32_t* __restrict__ token_seq,
                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                   const float* __restrict__ state, size_t state_stride, const float* __restrict__ taps_w,
                   const float* __restrict__ conv_bias, const float* __restrict__ dt_bias,
                   const float* __restrict__ a_log, float* __restrict__ xbc, float* __restrict__ dt,
                   float* __restrict__ decay) {
  const int t = blockIdx.x;
  const int e = token_seq[t];
  const int i = t - q_start[e];        // the token's index inside its entry
  const int channels = sh.heads * sh.vdim + 2 * sh.groups * sh.n;
  if (blockIdx.y == gridDim.y - 1) {
    // the token's last workgroup: step sizes and decays, which need nothing of the convolution
    for (int h = threadIdx.x; h < sh.heads; h += 256) {
      const float d = ssd_softplus(proj[(size_t)t * sh.ldp + sh.off_dt + h] + dt_bias[h]);
      dt[(size_t)t * sh.heads + h] = d;
      decay[(size_t)t * sh.heads + h] = expf(-expf(a_log[h]) * d);
    }
    return;
  }
  const float* conv_state = state + (size_t)state_slots[e] * state_stride;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  float y = conv_bias[c];
  for (int j = 0; j < sh.taps; ++j) {
    const int s = i - (sh.taps - 1) + j;      // index inside the entry of the input under tap j
    const float x = s >= 0 ? proj[(size_t)(t - (sh.taps - 1) + j) * sh.ldp + sh.off_x + c]
                           : conv_state[(size_t)(sh.taps - 1 + s) * channels + c];
    y = fmaf(taps_w[(size_t)c * sh.taps + j], x, y);
  }
  xbc[(size_t)t * channels + c] = y * ssd_sigmoid(y);
}

// one thread a (entry, channel): the state's rows in ascending order, so that a row is read before it is overwritten
__global__ void __launch_bounds__(256)
ssd_conv_state_kernel(const float* __restrict__ proj, SsdShape sh, const int32_t* __restrict__ q_start,
                      const int32_t* __restrict__ state_slots, float* __restrict__ state, size_t state_stride) {
  const int e = blockIdx.y;
  const int channels = sh.heads * sh.vdim + 2 * sh.groups * sh.n;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= channels) return;
  const int first = q_start[e], count = q_start[e + 1] - first;
  float* st = state + (size_t)state_slots[e] * state_stride;
  const int keep = sh.taps - 1;
  for (int r = 0; r < keep; ++r) {
    const int s = count - keep + r;     // index inside the entry of the input that row r holds afterwards
    st[(size_t)r * channels + c] = s >= 0 ? proj[(size_t)(first + s) * sh.ldp + sh.off_x + c]
                                          : st[(size_t)(r + count) * channels + c];
  }
}

constexpr int kScanTokens = 16;      // tokens whose inputs wait in LDS at a time
constexpr int kScanCols = 16;        // columns of S a workgroup owns

// Sum over 16 neighbouring lanes; every lane gets the same sum (the pairs of each step add the same two numbers).
__device__ __forceinline__ float lanes16_sum(float x) {
  x += __shfl_xor(x, 1, 64);
  x += __shfl_xor(x, 2, 64);
  x += __shfl_xor(x, 4, 64);
  x += __shfl_xor(x, 8, 64);
  return x;
}

// R: rows of S a lane holds; lane l of a column owns rows l, l + 16, l + 32, ...
template <int R>
__global__ void __launch_bounds__(256)
ssd_scan_kernel(const float* __restrict__ xbc, const float* __restrict__ dt, const float* __restrict__ decay,
                const float* __restrict__ d_skip, SsdShape sh, const int32_t* __restrict__ q_start,
                const int32_t* __restrict__ state_slots, float* __restrict__ state, size_t state_stride,
                float* __restrict__ y, int below) {
  __shared__ float sb[kScanTokens][16 * R], sc[kScanTokens][16 * R];
  __shared__ float sx[kScanTokens][kScanCols], sdt[kScanTokens], sa[kScanTokens];
  const int e = blockIdx.z, h = blockIdx.y, v0 = blockIdx.x * kScanCols;
  const int first = q_start[e], count = q_start[e + 1] - first;
  if (count <= 0 || count >= below) return;      // (entries of `below` tokens or more are the chunk kernel's)
  const int col = threadIdx.x >> 4, l = threadIdx.x & 15;
  const int v = v0 + col;
  const bool live = v < sh.vdim;
  const int inner = sh.heads * sh.vdim, gn = sh.groups * sh.n, channels = inner + 2 * gn;
  const int g = h / (sh.heads / sh.groups);
  float* s_ptr = state + (size_t)state_slots[e] * state_stride + (size_t)(sh.taps - 1) * channels +
                 ((size_t)h * sh.vdim + (live ? v : 0)) * sh.n;
  float s[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = l + 16 * r;
    s[r] = (live && row < sh.n) ? s_ptr[row] : 0.f;
  }
  const float dh = d_skip[h];
  for (int t0 = 0; t0 < count; t0 += kScanTokens) {
    const int nt = count - t0 < kScanTokens ? count - t0 : kScanTokens;
    __syncthreads();
    for (int idx = threadIdx.x; idx < nt * 16 * R; idx += 256) {
      const int tt = idx / (16 * R), row = idx % (16 * R);
      const size_t base = (size_t)(first + t0 + tt) * channels + inner + (size_t)g * sh.n;
      sb[tt][row] = row < sh.n ? xbc[base + row] : 0.f;
      sc[tt][row] = row < sh.n ? xbc[base + gn + row] : 0.f;
    }
    for (int idx = threadIdx.x; idx < nt * kScanCols; idx += 256) {
      const int tt = idx / kScanCols, cc = idx % kScanCols;
      sx[tt][cc] = v0 + cc < sh.vdim ? xbc[(size_t)(first + t0 + tt) * channels + (size_t)h * sh.vdim + v0 + cc] : 0.f;
    }
    if (threadIdx.x < nt) {
      sdt[threadIdx.x] = dt[(size_t)(first + t0 + threadIdx.x) * sh.heads + h];
      sa[threadIdx.x] = decay[(size_t)(first + t0 + threadIdx.x) * sh.heads + h];
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float a = sa[tt], xv = sx[tt][col], w = sdt[tt] * xv;
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        s[r] = fmaf(a, s[r], w * sb[tt][l + 16 * r]);
        acc = fmaf(s[r], sc[tt][l + 16 * r], acc);
      }
      acc = lanes16_sum(acc);
      if (l == 0 && live) y[(size_t)(first + t0 + tt) * inner + (size_t)h * sh.vdim + v] = acc + dh * xv;
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int row = l + 16 * r;
      if (row < sh.n) s_ptr[row] = s[r];
    }
  }
}

// The recurrence 64 tokens at a time.  With c_t the sum of the log decays of the chunk's tokens up to t (inclusive),
//   y_t = sum_{s <= t} exp(c_t - c_s) dt_s (C_t . B_s) x_s  +  exp(c_t) S_0^T C_t  +  D x_t,
//   S_64 = exp(c_63) S_0 + sum_s exp(c_63 - c_s) dt_s B_s x_s^T,
// every exponent at most zero.  The products C_t . B_s are the same for all heads of a group and all columns of S: a
// first kernel (ssd_scores) makes them once per (chunk, group).  Then a workgroup owns (entry, head, 16 columns of S)
// and walks the entry's chunks in order; per chunk its four waves make M[t][s] = (C_t . B_s) exp(c_t - c_s) dt_s for
// s <= t (ten tiles of 16 x 16 shared out among them, into LDS), then each takes 16 tokens of
// y = M X + diag(exp(c)) C S, then each its share of the rows of S.
// All products are float32 MFMAs of 16 x 16 x 4 (result D[4 (l / 16) + i][l % 16] in lane l).  The sum over k of a
// block of 16 is taken in the order that lets a lane fetch its four values with one 16-byte load from LDS: in the
// block's MFMA j, lane l gives A[l % 16][4 (l / 16) + j] and B[4 (l / 16) + j][l % 16]; tiles whose k runs along their
// rows in memory (x and S) are kept transposed in LDS for it.  The next chunk's B, C, x and dt are asked for while this
// one is worked on.  An entry's result depends on its own length and sizes alone.
constexpr int kChunk = 64;
constexpr int kChunkLdt = kChunk + 4;      // row stride of the tiles whose rows are 64 tokens long (M, x transposed)
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

__host__ __device__ constexpr int chunk_lds_floats(int nb) {
  return 2 * kChunk * (16 * nb + 4) + kChunk * kChunkLdt + 16 * kChunkLdt + 16 * (16 * nb + 4) + 4 * kChunk;
}

__device__ __forceinline__ f32x4 lds4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }

// VEC: B and C rows are fetched and put into LDS 16 bytes at a time (state size, channel counts and the first column
// of the group's B all multiples of 4)
template <int NB, bool VEC>      // NB: blocks of 16 rows of S (the state size rounded up)
__global__ void __launch_bounds__(256)
ssd_chunk_kernel(const float* __restrict__ xbc, const float* __restrict__ dt, const float* __restrict__ a_log,
                 const float* __restrict__ d_skip, SsdShape sh, const int32_t* __restrict__ q_start,
                 const int32_t* __restrict__ state_slots, float* __restrict__ state, size_t state_stride,
                 float* __restrict__ y, int at_least, const float* __restrict__ scores, int max_chunks) {
  constexpr int NP = 16 * NB, LDN = NP + 4;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* Bs = lds;                         // [kChunk][LDN]   B of the chunk's tokens
  float* Cs = Bs + kChunk * LDN;           // [kChunk][LDN]   C
  float* Ms = Cs + kChunk * LDN;           // [kChunk][kChunkLdt]   M[t][s]
  float* Xt = Ms + kChunk * kChunkLdt;     // [16][kChunkLdt]  x transposed: [column][token]
  float* St = Xt + 16 * kChunkLdt;         // [16][LDN]        S transposed: [column][row], as the state keeps it
  float* cum = St + 16 * LDN;              // [kChunk] log decays summed up to each token
  float* dts = cum + kChunk;               // [kChunk]
  float* wts = dts + kChunk;               // [kChunk] exp(c_last - c_s) dt_s
  float* ect = wts + kChunk;               // [kChunk] exp(c_t)
  const int e = blockIdx.z, h = blockIdx.y, v0 = blockIdx.x * 16;
  const int first = q_start[e], count = q_start[e + 1] - first;
  if (count < at_least) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int inner = sh.heads * sh.vdim, gn = sh.groups * sh.n, channels = inner + 2 * gn;
  const int g = h / (sh.heads / sh.groups);
  const int vlive = min(16, sh.vdim - v0);
  float* s_ptr = state + (size_t)state_slots[e] * state_stride + (size_t)(sh.taps - 1) * channels +
                 ((size_t)h * sh.vdim + v0) * sh.n;
  for (int idx = tid; idx < NP * 16; idx += 256) {
    const int v = idx / NP, n = idx % NP;
    St[v * LDN + n] = (v < vlive && n < sh.n) ? s_ptr[(size_t)v * sh.n + n] : 0.f;
  }
  const float rate = expf(a_log[h]), dh = d_skip[h];
  // A chunk's B, C, x and dt are asked for while the chunk before is worked on, and wait in registers meanwhile.
  constexpr int PER = kChunk * NP / 256;        // elements of a [64][NP] tile a thread moves
  float rb[PER], rc[PER], rx[4], rdt = 0.f;
  f32x4 mt[3];       // the wave's tiles of C . B of the chunk, as the scores kernel left them
  auto fetch = [&](int t0) {
    const int nt = min(kChunk, count - t0);
    const size_t tok0 = (size_t)(first + t0);
    const float* sc = scores + (((size_t)e * max_chunks + t0 / kChunk) * sh.groups + g) * (10 * 256);
#pragma unroll
    for (int m = 0; m < 3; ++m)      // tile wave + 4 m is the wave's m-th
      if (wave + 4 * m < 10) mt[m] = *reinterpret_cast<const f32x4*>(sc + ((wave + 4 * m) * 64 + lane) * 4);
    if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < PER / 4; ++i) {
        const int idx = tid + i * 256, tt = idx / (NP / 4), n = (idx % (NP / 4)) * 4;
        const bool in = tt < nt && n < sh.n;
        const size_t base = (tok0 + tt) * channels + inner + (size_t)g * sh.n + n;
        const f32x4 zero = f32x4{0.f, 0.f, 0.f, 0.f};
        const f32x4 b4 = in ? *reinterpret_cast<const f32x4*>(xbc + base) : zero;
        const f32x4 c4 = in ? *reinterpret_cast<const f32x4*>(xbc + base + gn) : zero;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          rb[4 * i + q] = b4[q];
          rc[4 * i + q] = c4[q];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int idx = tid + i * 256, tt = idx / NP, n = idx % NP;
        const bool in = tt < nt && n < sh.n;
        const size_t base = (tok0 + tt) * channels + inner + (size_t)g * sh.n + n;
        rb[i] = in ? xbc[base] : 0.f;
        rc[i] = in ? xbc[base + gn] : 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256, tt = idx >> 4, v = idx & 15;
      rx[i] = (tt < nt && v < vlive) ? xbc[(tok0 + tt) * channels + (size_t)h * sh.vdim + v0 + v] : 0.f;
    }
    if (tid < kChunk) rdt = tid < nt ? dt[(tok0 + tid) * sh.heads + h] : 0.f;
  };
  fetch(0);
  for (int t0 = 0; t0 < count; t0 += kChunk) {
    const int nt = min(kChunk, count - t0);
    const size_t tok0 = (size_t)(first + t0);
    __syncthreads();       // the chunk before is done with every tile
    if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < PER / 4; ++i) {
        const int idx = tid + i * 256, tt = idx / (NP / 4), n = (idx % (NP / 4)) * 4;
        *reinterpret_cast<f32x4*>(Bs + tt * LDN + n) = f32x4{rb[4 * i], rb[4 * i + 1], rb[4 * i + 2], rb[4 * i + 3]};
        *reinterpret_cast<f32x4*>(Cs + tt * LDN + n) = f32x4{rc[4 * i], rc[4 * i + 1], rc[4 * i + 2], rc[4 * i + 3]};
      }
    } else {
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int idx = tid + i * 256, tt = idx / NP, n = idx % NP;
        Bs[tt * LDN + n] = rb[i];
        Cs[tt * LDN + n] = rc[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      Xt[(idx & 15) * kChunkLdt + (idx >> 4)] = rx[i];
    }
    if (tid < kChunk) dts[tid] = rdt;
    __syncthreads();
    if (wave == 0) {
      // inclusive sums of the log decays over the 64 lanes
      float c = -rate * dts[lane];
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const float up = __shfl_up(c, o, 64);
        if (lane >= o) c += up;
      }
      cum[lane] = c;
      const float last = __shfl(c, 63, 64);
      wts[lane] = expf(last - c) * dts[lane];
      ect[lane] = expf(c);
    }
    // (the chunk after this one is fetched further down, when this chunk's tiles of scores have been used)
    __syncthreads();       // the sums of the log decays are there
#pragma unroll
    for (int j = 0; j < 10; ++j) {
      const int tb = j >= 6 ? 3 : j >= 3 ? 2 : j >= 1 ? 1 : 0, sb = j - tb * (tb + 1) / 2;
      if ((j & 3) == wave) {
        const f32x4 acc = mt[j >> 2];
        const int s = sb * 16 + r16;
        const float cs = cum[s], ds = dts[s];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int t = tb * 16 + 4 * kg + i;
          Ms[t * kChunkLdt + s] = s <= t ? acc[i] * expf(cum[t] - cs) * ds : 0.f;
        }
      }
    }
    if (t0 + kChunk < count) fetch(t0 + kChunk);
    __syncthreads();
    // y of the wave's 16 tokens
    if (wave * 16 < nt) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
      const int tb = wave;
      const float* mp = Ms + (tb * 16 + r16) * kChunkLdt + 4 * kg;
      const float* xp = Xt + r16 * kChunkLdt + 4 * kg;
      for (int k = 0; k < (tb + 1) * 16; k += 16) {
        const f32x4 a4 = lds4(mp + k), b4 = lds4(xp + k);
#pragma unroll
        for (int q = 0; q < 4; ++q) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[q], b4[q], acc, 0, 0, 0);
      }
      const float et = ect[tb * 16 + r16];
      const float* cp = Cs + (tb * 16 + r16) * LDN + 4 * kg;
      const float* sp = St + r16 * LDN + 4 * kg;
#pragma unroll
      for (int k = 0; k < NP; k += 16) {
        const f32x4 a4 = lds4(cp + k), b4 = lds4(sp + k);
#pragma unroll
        for (int q = 0; q < 4; ++q) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(et * a4[q], b4[q], acc, 0, 0, 0);
      }
      if (r16 < vlive) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int t = tb * 16 + 4 * kg + i;
          if (t < nt) y[(tok0 + t) * inner + (size_t)h * sh.vdim + v0 + r16] = acc[i] + dh * Xt[r16 * kChunkLdt + t];
        }
      }
    }
    __syncthreads();       // every wave has read S
    {
      const float keep = ect[kChunk - 1];
      for (int nb = wave; nb < NB; nb += 4) {
        // lane: rows nb * 16 + 4 (l / 16) .. + 3 of S, column l % 16: four neighbours of the transposed tile
        float* sp = St + r16 * LDN + nb * 16 + 4 * kg;
        f32x4 acc = lds4(sp);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] *= keep;
        const float* bp = Bs + (4 * kg) * LDN + nb * 16 + r16;
        const float* xp = Xt + r16 * kChunkLdt + 4 * kg;
#pragma unroll
        for (int k = 0; k < kChunk; k += 16) {
          const f32x4 w4 = lds4(wts + k + 4 * kg), b4 = lds4(xp + k);
#pragma unroll
          for (int q = 0; q < 4; ++q)
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(bp[(k + q) * LDN] * w4[q], b4[q], acc, 0, 0, 0);
        }
        *reinterpret_cast<f32x4*>(sp) = acc;
      }
    }
  }
  __syncthreads();
  for (int idx = tid; idx < NP * 16; idx += 256) {
    const int v = idx / NP, n = idx % NP;
    if (v < vlive && n < sh.n) s_ptr[(size_t)v * sh.n + n] = St[v * LDN + n];
  }
}

// C_t . B_s of every chunk of 64 tokens, once per group of heads: the ten 16 x 16 tiles on and below the diagonal, each
// as its 64 lanes' four numbers (lane l: rows 4 (l / 16) .. + 3, column l % 16 of the tile), [entry][chunk][group][10][64][4].
template <int NB>
__global__ void __launch_bounds__(256)
ssd_scores_kernel(const float* __restrict__ xbc, SsdShape sh, const int32_t* __restrict__ q_start, int at_least,
                  float* __restrict__ scores, int max_chunks) {
  constexpr int NP = 16 * NB, LDN = NP + 4;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* Bs = lds;
  float* Cs = Bs + kChunk * LDN;
  const int e = blockIdx.z, g = blockIdx.y, t0 = blockIdx.x * kChunk;
  const int first = q_start[e], count = q_start[e + 1] - first;
  if (count < at_least || t0 >= count) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int inner = sh.heads * sh.vdim, gn = sh.groups * sh.n, channels = inner + 2 * gn;
  const int nt = min(kChunk, count - t0);
  for (int idx = tid; idx < kChunk * NP; idx += 256) {
    const int tt = idx / NP, n = idx % NP;
    const bool in = tt < nt && n < sh.n;
    const size_t base = ((size_t)(first + t0) + tt) * channels + inner + (size_t)g * sh.n + n;
    Bs[tt * LDN + n] = in ? xbc[base] : 0.f;
    Cs[tt * LDN + n] = in ? xbc[base + gn] : 0.f;
  }
  __syncthreads();
  float* out = scores + (((size_t)e * max_chunks + blockIdx.x) * sh.groups + g) * (10 * 256);
#pragma unroll
  for (int j = 0; j < 10; ++j) {
    const int tb = j >= 6 ? 3 : j >= 3 ? 2 : j >= 1 ? 1 : 0, sb = j - tb * (tb + 1) / 2;
    if ((j & 3) == wave) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
      const float* cp = Cs + (tb * 16 + r16) * LDN + 4 * kg;
      const float* bp = Bs + (sb * 16 + r16) * LDN + 4 * kg;
#pragma unroll
      for (int k = 0; k < NP; k += 16) {
        const f32x4 a4 = lds4(cp + k), b4 = lds4(bp + k);
#pragma unroll
        for (int q = 0; q < 4; ++q) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[q], b4[q], acc, 0, 0, 0);
      }
      *reinterpret_cast<f32x4*>(out + (j * 64 + lane) * 4) = acc;
    }
  }
}

// one workgroup per (token, norm group); parts of up to 4,096 columns wait in registers between the two passes
template <typename TO, int PER>
__global__ void __launch_bounds__(256)
ssd_out_kernel(const float* __restrict__ y, const float* __restrict__ proj, int ldp, int off_z,
               const float* __restrict__ w, float eps, int inner, int part, TO* __restrict__ out) {
  __shared__ float scratch[4];
  const int t = blockIdx.x, p0 = blockIdx.y * part;
  const float* zp = proj + (size_t)t * ldp + off_z + p0;
  const float* yp = y + (size_t)t * inner + p0;
  float ss = 0.f;
  if constexpr (PER > 0) {
    constexpr int P = PER > 0 ? PER : 1;
    float u[P], yv[P], zv[P];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * 256;
      yv[j] = i < part ? yp[i] : 0.f;
      zv[j] = i < part ? zp[i] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      u[j] = yv[j] * (zv[j] * ssd_sigmoid(zv[j]));
      ss = fmaf(u[j], u[j], ss);
    }
    ss = block_sum<4>(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)part + eps);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * 256;
      if (i < part) out[(size_t)t * inner + p0 + i] = from_f32<TO>(u[j] * inv * w[p0 + i]);
    }
    return;
  }
  for (int i = threadIdx.x; i < part; i += 256) {
    const float z = zp[i];
    const float u = yp[i] * (z * ssd_sigmoid(z));
    ss = fmaf(u, u, ss);
  }
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)part + eps);
  for (int i = threadIdx.x; i < part; i += 256) {
    const float z = zp[i];
    const float u = yp[i] * (z * ssd_sigmoid(z));
    out[(size_t)t * inner + p0 + i] = from_f32<TO>(u * inv * w[p0 + i]);
  }
}

static bool shape_ok(const SsdShape& sh) {
  return sh.heads > 0 && sh.groups > 0 && sh.heads % sh.groups == 0 && sh.vdim > 0 && sh.n > 0 && sh.n <= 256 &&
         sh.taps >= 1 && sh.taps <= 64 && sh.ldp > 0 && sh.off_z >= 0 && sh.off_x >= 0 && sh.off_dt >= 0;
}

extern "C" int atoma_ssd_prepare(const float* proj, int ldp, int off_z, int off_x, int off_dt, int heads, int groups,
                                 int vdim, int n, int taps, const int32_t* token_seq, const int32_t* q_start,
                                 const int32_t* state_slots, const float* state, size_t state_stride,
                                 const float* taps_w, const float* conv_bias, const float* dt_bias,
                                 const float* a_log, float* xbc, float* dt, float* decay, int n_tokens,
                                 hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  SsdShape sh{heads, groups, vdim, n, taps, ldp, off_z, off_x, off_dt};
  if (!shape_ok(sh)) return ATOMA_ERR_SHAPE;
  const int channels = heads * vdim + 2 * groups * n;
  const int blocks = (channels + 255) / 256 + 1;
  if (blocks > 65535) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(ssd_prepare_kernel, dim3(n_tokens, blocks), dim3(256), 0, stream, proj, sh, token_seq, q_start,
                     state_slots, state, state_stride, taps_w, conv_bias, dt_bias, a_log, xbc, dt, decay);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_ssd_conv_state(const float* proj, int ldp, int off_x, int heads, int groups, int vdim, int n,
                                    int taps, const int32_t* q_start, const int32_t* state_slots, float* state,
                                    size_t state_stride, int n_entries, hipStream_t stream) {
  if (n_entries <= 0 || taps <= 1) return 0;
  SsdShape sh{heads, groups, vdim, n, taps, ldp, 0, off_x, 0};
  if (!shape_ok(sh) || n_entries > 65535) return ATOMA_ERR_SHAPE;
  const int channels = heads * vdim + 2 * groups * n;
  hipLaunchKernelGGL(ssd_conv_state_kernel, dim3((channels + 255) / 256, n_entries), dim3(256), 0, stream, proj, sh,
                     q_start, state_slots, state, state_stride);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_ssd_scan(const float* xbc, const float* dt, const float* decay, const float* d_skip, int heads,
                              int groups, int vdim, int n, int taps, const int32_t* q_start,
                              const int32_t* state_slots, float* state, size_t state_stride, float* y,
                              int n_entries, int below, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  SsdShape sh{heads, groups, vdim, n, taps, 1, 0, 0, 0};
  if (!shape_ok(sh) || n_entries > 65535 || heads > 65535) return ATOMA_ERR_SHAPE;
  dim3 grid((vdim + kScanCols - 1) / kScanCols, heads, n_entries), block(256);
  const int rows = (n + 15) / 16;
#define ATOMA_SCAN(R)                                                                                              \
  hipLaunchKernelGGL((ssd_scan_kernel<R>), grid, block, 0, stream, xbc, dt, decay, d_skip, sh, q_start, state_slots, \
                     state, state_stride, y, below)
  if (rows <= 1) ATOMA_SCAN(1);
  else if (rows <= 2) ATOMA_SCAN(2);
  else if (rows <= 3) ATOMA_SCAN(3);
  else if (rows <= 4) ATOMA_SCAN(4);
  else if (rows <= 6) ATOMA_SCAN(6);
  else if (rows <= 8) ATOMA_SCAN(8);
  else if (rows <= 12) ATOMA_SCAN(12);
  else ATOMA_SCAN(16);
#undef ATOMA_SCAN
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// The largest state size the chunk kernel takes (its tiles of B and C must fit the CU's LDS beside the rest).
extern "C" int atoma_ssd_chunk_max_state() { return 128; }

template <int NB, bool VEC>
static int launch_chunk(dim3 grid, hipStream_t stream, const float* xbc, const float* dt, const float* a_log,
                        const float* d_skip, const SsdShape& sh, const int32_t* q_start, const int32_t* state_slots,
                        float* state, size_t state_stride, float* y, int at_least, float* scores, int max_chunks) {
  const size_t bytes = (size_t)chunk_lds_floats(NB) * sizeof(float);
  const size_t sbytes = (size_t)2 * kChunk * (16 * NB + 4) * sizeof(float);
  static bool asked = false;      // (per instantiation) more than the default 64 KB of LDS
  if (!asked) {
    if (bytes > 64 * 1024) {
      hipError_t err = hipFuncSetAttribute((const void*)ssd_chunk_kernel<NB, VEC>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
      if (err != hipSuccess) return (int)err;
    }
    if (sbytes > 64 * 1024) {
      hipError_t err = hipFuncSetAttribute((const void*)ssd_scores_kernel<NB>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)sbytes);
      if (err != hipSuccess) return (int)err;
    }
    asked = true;
  }
  hipLaunchKernelGGL((ssd_scores_kernel<NB>), dim3(max_chunks, sh.groups, grid.z), dim3(256), sbytes, stream, xbc, sh,
                     q_start, at_least, scores, max_chunks);
  hipLaunchKernelGGL((ssd_chunk_kernel<NB, VEC>), grid, dim3(256), bytes, stream, xbc, dt, a_log, d_skip, sh, q_start,
                     state_slots, state, state_stride, y, at_least, scores, max_chunks);
  return 0;
}

// Floats of scratch that atoma_ssd_chunk needs for entries of up to `max_chunks` chunks of 64 tokens.
extern "C" size_t atoma_ssd_chunk_scratch_floats(int n_entries, int max_chunks, int groups) {
  return (size_t)n_entries * max_chunks * groups * 10 * 256;
}

// entries of at least `at_least` tokens; the others are left to atoma_ssd_scan(below = at_least).  `max_chunks`: chunks
// of 64 tokens of the longest entry; `scores`: scratch of atoma_ssd_chunk_scratch_floats floats.
extern "C" int atoma_ssd_chunk(const float* xbc, const float* dt, const float* a_log, const float* d_skip, int heads,
                               int groups, int vdim, int n, int taps, const int32_t* q_start,
                               const int32_t* state_slots, float* state, size_t state_stride, float* y,
                               int n_entries, int at_least, float* scores, int max_chunks, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  SsdShape sh{heads, groups, vdim, n, taps, 1, 0, 0, 0};
  if (!shape_ok(sh) || n > 128 || n_entries > 65535 || heads > 65535 || groups > 65535 || at_least < 1 ||
      max_chunks < 1 || scores == nullptr)
    return ATOMA_ERR_SHAPE;
  dim3 grid((vdim + 15) / 16, heads, n_entries);
  int rc;
  // (a state size that is a multiple of 4 is then also a whole number of 16-byte pieces of its NB blocks' row)
  const bool vec = n % 4 == 0 && (heads * vdim) % 4 == 0 && ((uintptr_t)xbc & 15) == 0;
#define ATOMA_CHUNK(NB_)                                                                                            \
  rc = vec ? launch_chunk<NB_, true>(grid, stream, xbc, dt, a_log, d_skip, sh, q_start, state_slots, state,        \
                                     state_stride, y, at_least, scores, max_chunks)                               \
           : launch_chunk<NB_, false>(grid, stream, xbc, dt, a_log, d_skip, sh, q_start, state_slots, state,       \
                                      state_stride, y, at_least, scores, max_chunks)
  switch ((n + 15) / 16) {
    case 1: ATOMA_CHUNK(1); break;
    case 2: ATOMA_CHUNK(2); break;
    case 3: ATOMA_CHUNK(3); break;
    case 4: ATOMA_CHUNK(4); break;
    case 5: ATOMA_CHUNK(5); break;
    case 6: ATOMA_CHUNK(6); break;
    case 7: ATOMA_CHUNK(7); break;
    default: ATOMA_CHUNK(8); break;
  }
#undef ATOMA_CHUNK
  if (rc != 0) return rc;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_ssd_out(const float* y, const float* proj, int ldp, int off_z, const float* w, float eps,
                             int inner, int norm_groups, void* out, int out_dtype, int n_tokens, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (inner <= 0 || norm_groups <= 0 || inner % norm_groups || norm_groups > 65535 || ldp < inner) return ATOMA_ERR_SHAPE;
  const int part = inner / norm_groups;
  dim3 grid(n_tokens, norm_groups), block(256);
#define ATOMA_SSD_OUT(TO, PER)                                                                                    \
  hipLaunchKernelGGL((ssd_out_kernel<TO, PER>), grid, block, 0, stream, y, proj, ldp, off_z, w, eps, inner, part, \
                     (TO*)out)
#define ATOMA_SSD_OUT_BY_PART(TO)                 \
  do {                                            \
    if (part <= 1024) ATOMA_SSD_OUT(TO, 4);       \
    else if (part <= 4096) ATOMA_SSD_OUT(TO, 16); \
    else ATOMA_SSD_OUT(TO, 0);                    \
  } while (0)
  if (out_dtype == kF32) ATOMA_SSD_OUT_BY_PART(float);
  else if (out_dtype == kBF16) ATOMA_SSD_OUT_BY_PART(bf16_t);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_SSD_OUT_BY_PART
#undef ATOMA_SSD_OUT
  ATOMA_LAUNCH_CHECK();
  return 0;
}
