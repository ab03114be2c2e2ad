// Attention over one small cached vector per token: the kernels around the paged attention kernels.
//
// A token's keys and values of every head are products of one latent vector c (rank numbers), so the cache holds c
// alone and the heads' key and value maps move to the query's side:
//
//   score_h(i, j) = (W_uk,h c_j) . q_h,i = c_j . (W_uk,h^T q_h,i),       out_h,i = W_uv,h (sum_j p_ij c_j),
//
// which is attention with one shared key/value head of `rank` columns whose values are its keys.
//   latent_prepare   per token: c = rmsnorm(down projection) * w into the cache (as key and as value: the two tiles
//                    differ in the order of their elements only), the heads' gates sigmoid(g) in float32, and q in
//                    the activation dtype;
//   head_linear      per head a product of its own: out[t, h, :] = W[h] x[t, h, :], optionally times a scalar per
//                    (token, head) or per (token, output column), float32 sums in an order that depends on the sizes
//                    alone.
#include "common.h"
#include "cache_layout.h"

using namespace atoma;

// proj [T, ldp] float32: q (heads * dim columns from off_q), the down projection (rank from off_c), gates (heads from
// off_g).  Cache tiles hold rank_p >= rank columns a token; the added ones are zero.
template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const float* __restrict__ proj, int ldp, int off_q, int off_c, int off_g, int nq, int rank,
                      int rank_p, int heads, const float* __restrict__ w_norm, float eps,
                      TC* __restrict__ kcache, TC* __restrict__ vcache, const int32_t* __restrict__ slot_mapping,
                      int page_size, TA* __restrict__ q_out, float* __restrict__ gate) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const float* row = proj + (size_t)t * ldp;
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += 256) ss = fmaf(row[off_c + i], row[off_c + i], ss);
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  const int slot = slot_mapping[t];
  if (slot >= 0) {
    const int page = slot / page_size, off = slot % page_size;
    TC* ktile = kcache + (size_t)page * page_size * rank_p;
    TC* vtile = vcache + (size_t)page * page_size * rank_p;
    for (int i = threadIdx.x; i < rank_p; i += 256) {
      const TC c = from_f32<TC>(i < rank ? row[off_c + i] * inv * w_norm[i] : 0.f);
      ktile[key_offset(off, i, page_size)] = c;
      vtile[value_offset(i, off, rank_p, page_size)] = c;
    }
  }
  for (int i = threadIdx.x; i < nq; i += 256) q_out[(size_t)t * nq + i] = from_f32<TA>(row[off_q + i]);
  for (int h = threadIdx.x; h < heads; h += 256) gate[(size_t)t * heads + h] = 1.0f / (1.0f + expf(-row[off_g + h]));
}

// out[t, h * N + n] = (sum_k x[t, h * K + k] * w[(h * N + n) * K + k]) * (gate ? gate[t * H + h] : 1)
// A workgroup: 16 tokens x 64 outputs of one head; K in chunks of 32 through LDS.
template <typename TA, typename TW, typename TO>
__global__ void __launch_bounds__(256)
head_linear_kernel(const TA* __restrict__ x, int ldx, const TW* __restrict__ w, TO* __restrict__ out, int ldo,
                   const float* __restrict__ gate, int gate_cols, int T, int H, int K, int N) {
  __shared__ float xs[16][33], ws[64][33];
  const int h = blockIdx.z, n0 = blockIdx.x * 64, t0 = blockIdx.y * 16;
  const int nl = threadIdx.x & 63, rg = threadIdx.x >> 6;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    __syncthreads();
    for (int idx = threadIdx.x; idx < 16 * 32; idx += 256) {
      const int r = idx >> 5, kk = idx & 31;
      xs[r][kk] = (t0 + r < T && k0 + kk < K) ? to_f32(x[(size_t)(t0 + r) * ldx + (size_t)h * K + k0 + kk]) : 0.f;
    }
    for (int idx = threadIdx.x; idx < 64 * 32; idx += 256) {
      const int r = idx >> 5, kk = idx & 31;
      ws[r][kk] = (n0 + r < N && k0 + kk < K) ? to_f32(w[((size_t)h * N + n0 + r) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 32; ++kk) {
      const float wv = ws[nl][kk];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(xs[rg + 4 * i][kk], wv, acc[i]);
    }
  }
  if (n0 + nl >= N) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + rg + 4 * i;
    if (t < T) {
      const float s = !gate ? 1.0f : gate_cols ? gate[((size_t)t * H + h) * N + n0 + nl] : gate[(size_t)t * H + h];
      out[(size_t)t * ldo + (size_t)h * N + n0 + nl] = from_f32<TO>(acc[i] * s);
    }
  }
}

// The same on the matrix cores for bfloat16 operands (v_mfma_f32_16x16x32_bf16, float32 sums): a workgroup takes 64
// tokens x 16 NS outputs of one head, a wave 16 of the tokens against all of those outputs, so that a token's row is
// fetched by one wave only and what the waves fetch in common is the head's weight, which is small and stays in the
// caches.  Both operands' fragments come straight from memory (K is a head's width: a few steps), four steps of 32
// columns asked for at a time.  K a multiple of 8; a last step shorter than 32 columns is filled with zeros.  The
// MFMA's result holds, per lane, token (lane % 16) and outputs (lane / 16) * 4 .. + 3.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

template <typename TO, int NS>
__global__ void __launch_bounds__(256)
head_linear_mfma_kernel(const uint16_t* __restrict__ x, int ldx, const uint16_t* __restrict__ w, TO* __restrict__ out,
                        int ldo, const float* __restrict__ gate, int gate_cols, int T, int H, int K, int N) {
  const int h = blockIdx.z, n0 = blockIdx.x * (16 * NS);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int tb = blockIdx.y * 64 + wave * 16;              // the wave's 16 tokens
  if (tb >= T) return;
  int t = tb + r16;
  if (t > T - 1) t = T - 1;                                // clamped rows are computed and never stored
  const uint16_t* xp = x + (size_t)t * ldx + (size_t)h * K + kg * 8;
  const uint16_t* wp[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    int n = n0 + s * 16 + r16;
    if (n > N - 1) n = N - 1;
    wp[s] = w + ((size_t)h * N + n) * K + kg * 8;
  }
  f32x4 acc[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) acc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < K; k0 += 64) {
    bf16x8 xf[2], wf[2][NS];
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int k = k0 + 32 * st;
      const bool in = k + kg * 8 < K;
      xf[st] = in ? *reinterpret_cast<const bf16x8*>(xp + k) : zero;
#pragma unroll
      for (int s = 0; s < NS; ++s) wf[st][s] = in ? *reinterpret_cast<const bf16x8*>(wp[s] + k) : zero;
    }
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      if (k0 + 32 * st < K) {
#pragma unroll
        for (int s = 0; s < NS; ++s) acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[st][s], xf[st], acc[s], 0, 0, 0);
      }
    }
  }
  t = tb + r16;
  if (t >= T) return;
  const float g = gate && !gate_cols ? gate[(size_t)t * H + h] : 1.0f;
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int nb = n0 + s * 16 + kg * 4;
    TO* dst = out + (size_t)t * ldo + (size_t)h * N + nb;
    const float* gc = gate + ((size_t)t * H + h) * N + nb;      // (read only with a gate per column)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (nb + i < N) dst[i] = from_f32<TO>(acc[s][i] * (gate && gate_cols ? gc[i] : g));
  }
}

// The same for float32 rows of at most 16 tokens (the small products a decode step has): a wave an output column,
// its lanes share the columns of K (coalesced reads of the weight's row), one sum per token, added over the lanes.
template <typename TW>
__global__ void __launch_bounds__(256)
head_gemv_kernel(const float* __restrict__ x, int ldx, const TW* __restrict__ w, float* __restrict__ out, int ldo, int T,
                 int H, int K, int N) {
  const int lane = threadIdx.x & 63;
  const long col = (long)blockIdx.x * 4 + (threadIdx.x >> 6);      // h * N + n
  if (col >= (long)H * N) return;
  const int h = (int)(col / N);
  const TW* wr = w + (size_t)col * K;
  float acc[16];
#pragma unroll
  for (int t = 0; t < 16; ++t) acc[t] = 0.f;
  for (int k = lane; k < K; k += 64) {
    const float wv = to_f32(wr[k]);
#pragma unroll
    for (int t = 0; t < 16; ++t)
      if (t < T) acc[t] = fmaf(x[(size_t)t * ldx + (size_t)h * K + k], wv, acc[t]);
  }
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    if (t < T) {
      const float v = wave_sum(acc[t]);
      if (lane == 0) out[(size_t)t * ldo + col] = v;
    }
  }
}

extern "C" int atoma_latent_prepare(const float* proj, int ldp, int off_q, int off_c, int off_g, int nq, int rank,
                                    int rank_p, int heads, const float* w_norm, float eps, void* kcache, void* vcache,
                                    int cache_dtype, const int32_t* slot_mapping, int page_size, void* q_out,
                                    int act_dtype, float* gate, int n_tokens, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (rank <= 0 || rank_p < rank || heads <= 0 || nq <= 0 || page_size <= 0 || ldp <= 0) return ATOMA_ERR_SHAPE;
  dim3 grid(n_tokens), block(256);
#define ATOMA_LATENT(TA, TC)                                                                                      \
  hipLaunchKernelGGL((latent_prepare_kernel<TA, TC>), grid, block, 0, stream, proj, ldp, off_q, off_c, off_g, nq, \
                     rank, rank_p, heads, w_norm, eps, (TC*)kcache, (TC*)vcache, slot_mapping, page_size,         \
                     (TA*)q_out, gate)
  if (act_dtype == kF32 && cache_dtype == kF32) ATOMA_LATENT(float, float);
  else if (act_dtype == kBF16 && cache_dtype == kBF16) ATOMA_LATENT(bf16_t, bf16_t);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_LATENT
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_head_linear(const void* x, int x_dtype, int ldx, const void* w, int w_dtype, void* out,
                                 int out_dtype, int ldo, const float* gate, int gate_cols, int T, int H, int K, int N,
                                 hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || K <= 0 || N <= 0 || ldx < H * K || ldo < H * N || H > 65535 || (T + 15) / 16 > 65535) return ATOMA_ERR_SHAPE;
  if (x_dtype == kBF16 && w_dtype == kBF16 && K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x & 15) == 0 &&
      ((uintptr_t)w & 15) == 0 && (T + 63) / 64 <= 65535) {
    const bool wide = N > 64;                  // eight blocks of 16 outputs a wave, else four
    dim3 mgrid((N + (wide ? 127 : 63)) / (wide ? 128 : 64), (T + 63) / 64, H);
#define ATOMA_HLM(TO, NS)                                                                                          \
  hipLaunchKernelGGL((head_linear_mfma_kernel<TO, NS>), mgrid, dim3(256), 0, stream, (const uint16_t*)x, ldx,      \
                     (const uint16_t*)w, (TO*)out, ldo, gate, gate_cols, T, H, K, N)
    if (out_dtype == kBF16) {
      if (wide) ATOMA_HLM(bf16_t, 8);
      else ATOMA_HLM(bf16_t, 4);
    } else if (out_dtype == kF32) {
      if (wide) ATOMA_HLM(float, 8);
      else ATOMA_HLM(float, 4);
    } else {
      return ATOMA_ERR_DTYPE;
    }
#undef ATOMA_HLM
    ATOMA_LAUNCH_CHECK();
    return 0;
  }
  if (T <= 16 && gate == nullptr && x_dtype == kF32 && out_dtype == kF32 && (long)H * N <= 4L * 2147483647L) {
    const unsigned blocks = (unsigned)(((long)H * N + 3) / 4);
    if (w_dtype == kF32)
      hipLaunchKernelGGL((head_gemv_kernel<float>), dim3(blocks), dim3(256), 0, stream, (const float*)x, ldx,
                         (const float*)w, (float*)out, ldo, T, H, K, N);
    else if (w_dtype == kBF16)
      hipLaunchKernelGGL((head_gemv_kernel<bf16_t>), dim3(blocks), dim3(256), 0, stream, (const float*)x, ldx,
                         (const bf16_t*)w, (float*)out, ldo, T, H, K, N);
    else
      return ATOMA_ERR_DTYPE;
    ATOMA_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid((N + 63) / 64, (T + 15) / 16, H), block(256);
#define ATOMA_HL(TA, TW, TO)                                                                                  \
  hipLaunchKernelGGL((head_linear_kernel<TA, TW, TO>), grid, block, 0, stream, (const TA*)x, ldx, (const TW*)w, \
                     (TO*)out, ldo, gate, gate_cols, T, H, K, N)
  if (x_dtype == kF32 && w_dtype == kF32 && out_dtype == kF32) ATOMA_HL(float, float, float);
  else if (x_dtype == kF32 && w_dtype == kBF16 && out_dtype == kF32) ATOMA_HL(float, bf16_t, float);
  else if (x_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kBF16) ATOMA_HL(bf16_t, bf16_t, bf16_t);
  else if (x_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kF32) ATOMA_HL(bf16_t, bf16_t, float);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_HL
  ATOMA_LAUNCH_CHECK();
  return 0;
}
