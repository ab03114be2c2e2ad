// Differential attention: every head has two score maps over one set of values, and its output is the difference of
// the two attentions, normed and gated.
//
// Both maps of a head run through the framework's attention kernels as two query heads of one wide head size HDO:
// a key/value head keeps [k1 | k2 | zeros] as its key and [v | zeros] as its value, and the query of map m is its
// `dim` columns at column m * dim with zeros elsewhere, so that q' . k' = q_m . k_m and the values are kept once.
//
//   diff_prepare   per token, from the fused projection [q | k | v | g] (float32 or the activation dtype):
//                  the first rot_dim columns of every map of q and k turned in pairs (c, c + rot_dim / 2) by
//                  a = position * inv_freq[c] (position, angle, sine and cosine in float32); the queries to
//                  q_out [T, 2 heads, HDO]; keys and values into their cache tiles (cache_layout.h); sigmoid of the
//                  heads' gates to gate [T, heads] in float32.  A call that reads another call's cache passes no
//                  tiles and its projection holds [q | g] only.
//   diff_combine   per (token, head): o = a1 - lam a2 over the first vdim columns of the two maps' outputs,
//                  o / sqrt(mean(o^2) + eps) * post * gate, in float32, to y [T, heads * vdim].
#include "common.h"
#include "cache_layout.h"

using namespace atoma;

// one output column of a map: `src` points at the map's dim columns of the projection
template <typename TP>
__device__ __forceinline__ float turned(const TP* src, int d, int rot_dim, const float* cs, const float* sn) {
  const float x = to_f32(src[d]);
  if (d >= rot_dim) return x;
  const int half = rot_dim >> 1;
  if (d < half) return x * cs[d] - to_f32(src[d + half]) * sn[d];
  return x * cs[d - half] + to_f32(src[d - half]) * sn[d - half];
}

template <typename TP, typename TQ, typename TC>
__global__ void __launch_bounds__(256)
diff_prepare_kernel(const TP* __restrict__ proj, int ld, const int32_t* __restrict__ positions,
                    const float* __restrict__ inv_freq, int rot_dim, TQ* __restrict__ q_out, int ldq,
                    TC* __restrict__ kcache, TC* __restrict__ vcache, const int32_t* __restrict__ slot_mapping,
                    int page_size, float* __restrict__ gate, int heads, int kv_heads, int dim, int vdim, int hdo,
                    int off_k, int off_v, int off_g) {
  __shared__ float cs[128], sn[128];
  const int t = blockIdx.x;
  const TP* row = proj + (size_t)t * ld;
  const float p = (float)positions[t];
  for (int i = threadIdx.x; i < rot_dim / 2; i += 256) {
    float s, c;
    sincosf(p * inv_freq[i], &s, &c);
    cs[i] = c, sn[i] = s;
  }
  __syncthreads();
  // a token's columns are dealt over the gridDim.y workgroups that share it (steps of few tokens)
  const int first = blockIdx.y * 256 + threadIdx.x, step = gridDim.y * 256;
  // queries: head j = 2 * head + map, its dim columns at column map * dim of HDO
  const int nq = 2 * heads * hdo;
  for (int i = first; i < nq; i += step) {
    const int j = i / hdo, c = i - j * hdo;
    const int d = c - (j & 1) * dim;
    float v = 0.f;
    if (d >= 0 && d < dim) v = turned(row + (size_t)j * dim, d, rot_dim, cs, sn);
    q_out[(size_t)t * ldq + i] = from_f32<TQ>(v);
  }
  for (int h = first; h < heads; h += step)
    gate[(size_t)t * heads + h] = 1.0f / (1.0f + expf(-to_f32(row[off_g + h])));
  if (kcache == nullptr) return;
  const int slot = slot_mapping[t];
  const int page = slot / page_size, off = slot % page_size;
  const int nk = kv_heads * hdo;
  for (int i = first; i < nk; i += step) {
    const int g = i / hdo, c = i - g * hdo;
    const size_t tile = ((size_t)page * kv_heads + g) * page_size * hdo;
    float k = 0.f;
    if (c < 2 * dim) {
      const int m = c / dim, d = c - m * dim;
      k = turned(row + off_k + (size_t)(2 * g + m) * dim, d, rot_dim, cs, sn);
    }
    kcache[tile + key_offset(off, c, page_size)] = from_f32<TC>(k);
    const float v = c < vdim ? to_f32(row[off_v + g * vdim + c]) : 0.f;
    vcache[tile + value_offset(c, off, hdo, page_size)] = from_f32<TC>(v);
  }
}

// one wave a (token, head)
template <typename TA, typename TO>
__global__ void __launch_bounds__(256)
diff_combine_kernel(const TA* __restrict__ att, int lda, const float* __restrict__ gate, TO* __restrict__ y, int ldy,
                    int n_pairs, int heads, int vdim, int hdo, float lam, float eps, float post) {
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (pair >= n_pairs) return;
  const int t = pair / heads, h = pair - t * heads;
  const TA* a1 = att + (size_t)t * lda + (size_t)(2 * h) * hdo;
  const TA* a2 = a1 + hdo;
  constexpr int PER = 4;      // vdim <= 256
  float o[PER];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int c = lane + j * 64;
    o[j] = c < vdim ? to_f32(a1[c]) - lam * to_f32(a2[c]) : 0.f;
    ss += o[j] * o[j];
  }
  ss = wave_sum(ss);
  const float f = post * gate[pair] / sqrtf(ss / (float)vdim + eps);
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int c = lane + j * 64;
    if (c < vdim) y[(size_t)t * ldy + h * vdim + c] = from_f32<TO>(o[j] * f);
  }
}

extern "C" int atoma_diff_prepare(const void* proj, int proj_dtype, int ld, const int32_t* positions,
                                  const float* inv_freq, int rot_dim, void* q_out, int ldq, int q_dtype, void* kcache,
                                  void* vcache, int cache_dtype, const int32_t* slot_mapping, int page_size,
                                  float* gate, int n_tokens, int heads, int kv_heads, int dim, int vdim, int hdo,
                                  int off_k, int off_v, int off_g, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || dim <= 0 || vdim <= 0 || hdo < 2 * dim || hdo < vdim || rot_dim < 0 ||
      rot_dim % 2 || rot_dim > dim || rot_dim > 256 || page_size <= 0 || ldq < 2 * heads * hdo || ld < off_g + heads ||
      (kcache != nullptr && (vcache == nullptr || slot_mapping == nullptr)))
    return ATOMA_ERR_SHAPE;
  // steps of few tokens: several workgroups a token, so that about a thousand of them share the step's columns
  const int per_token = (2 * heads * hdo + 255) / 256;
  int parts = 1024 / n_tokens;
  parts = parts < 1 ? 1 : parts > per_token ? per_token : parts > 16 ? 16 : parts;
  dim3 grid(n_tokens, parts), block(256);
#define ATOMA_DP(TP, TQ, TC)                                                                                        \
  hipLaunchKernelGGL((diff_prepare_kernel<TP, TQ, TC>), grid, block, 0, stream, (const TP*)proj, ld, positions,     \
                     inv_freq, rot_dim, (TQ*)q_out, ldq, (TC*)kcache, (TC*)vcache, slot_mapping, page_size, gate,   \
                     heads, kv_heads, dim, vdim, hdo, off_k, off_v, off_g)
  if (kcache == nullptr) cache_dtype = q_dtype;
  if (proj_dtype == kF32 && q_dtype == kF32 && cache_dtype == kF32) ATOMA_DP(float, float, float);
  else if (proj_dtype == kF32 && q_dtype == kBF16 && cache_dtype == kBF16) ATOMA_DP(float, bf16_t, bf16_t);
  else if (proj_dtype == kBF16 && q_dtype == kBF16 && cache_dtype == kBF16) ATOMA_DP(bf16_t, bf16_t, bf16_t);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_DP
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_diff_combine(const void* att, int att_dtype, int lda, const float* gate, void* y, int y_dtype,
                                  int ldy, int n_tokens, int heads, int vdim, int hdo, float lam, float eps, float post,
                                  hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (heads <= 0 || vdim <= 0 || vdim > 256 || hdo < vdim || lda < 2 * heads * hdo || ldy < heads * vdim)
    return ATOMA_ERR_SHAPE;
  const int n_pairs = n_tokens * heads;
  dim3 grid((n_pairs + 3) / 4), block(256);
#define ATOMA_DC(TA, TO)                                                                                            \
  hipLaunchKernelGGL((diff_combine_kernel<TA, TO>), grid, block, 0, stream, (const TA*)att, lda, gate, (TO*)y, ldy, \
                     n_pairs, heads, vdim, hdo, lam, eps, post)
  if (att_dtype == kF32 && y_dtype == kF32) ATOMA_DC(float, float);
  else if (att_dtype == kBF16 && y_dtype == kBF16) ATOMA_DC(bf16_t, bf16_t);
  else if (att_dtype == kF32 && y_dtype == kBF16) ATOMA_DC(float, bf16_t);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_DC
  ATOMA_LAUNCH_CHECK();
  return 0;
}
