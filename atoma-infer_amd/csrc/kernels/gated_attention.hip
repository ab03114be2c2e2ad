// The kernels between the projections and the paged attention kernels for two gated kinds of attention.
//
// Rotation: the first `rot` columns of a head are turned by angle position * freq[i] (float32, no table), pair i being
// columns (2i, 2i + 1) (`interleaved`) or (i, i + rot / 2) (half-split); (u, v) -> mag (u cos - v sin, v cos + u sin).
//
//   tied_rope_prepare    attention whose values are its keys as projected: from the float32 result of one product
//                        [q | k | g] a token's q and k get their biases, k (with bias, not rotated) goes into the
//                        value tiles, q and k are rotated, q leaves in the activation dtype and k goes into the key
//                        tiles; sigmoid(g) leaves in float32, one number per output column.  Heads may leave wider
//                        than they came (zeros beyond), for head sizes the attention kernels do not take.
//   latent_rope_prepare  attention over one latent vector per token with a rotated key part shared by all heads:
//                        from [dq | dkv | g], cq = rmsnorm(dq) wq in the activation dtype; c = rmsnorm(dkv[:rank]) wc
//                        and the rotated last `rd` columns of dkv form the cached key [c | k_rot | 0], the cached
//                        value is [c | 0]; sigmoid(g) in float32.
//   latent_q_rope        the queries behind their second projection: the last `rd` columns of every head rotated,
//                        all columns to the activation dtype.
//   gate_mul             y[t, h, j] = att[t, h, j] * gate[t, h, j] for the first vd of a head's hd_out columns.
// One workgroup a token.  The tiles' element order is the attention kernels' (cache_layout.h).
#include "common.h"
#include "cache_layout.h"

using namespace atoma;

// the rotated value of column d (< rot) of a head whose columns are x[0 .. rot), given cos and sin tables of the pairs
__device__ __forceinline__ float turned(const float* __restrict__ x, int d, int rot, int interleaved,
                                        const float* __restrict__ cs, const float* __restrict__ sn) {
  int i, partner;
  bool first;
  if (interleaved) {
    i = d >> 1, first = !(d & 1), partner = d ^ 1;
  } else {
    const int half = rot >> 1;
    first = d < half, i = first ? d : d - half, partner = first ? d + half : d - half;
  }
  return first ? x[d] * cs[i] - x[partner] * sn[i] : x[d] * cs[i] + x[partner] * sn[i];
}

__device__ __forceinline__ void angles(int position, const float* __restrict__ freq, int rot, float mag, float* cs,
                                       float* sn) {
  const float p = (float)position;
  for (int i = threadIdx.x; i < rot / 2; i += 256) {
    float s, c;
    sincosf(p * freq[i], &s, &c);
    cs[i] = c * mag, sn[i] = s * mag;
  }
}

template <typename TQ, typename TC>
__global__ void __launch_bounds__(256)
tied_rope_prepare_kernel(const float* __restrict__ proj, int ld, int off_q, int off_k, int off_g,
                         const float* __restrict__ bq, const float* __restrict__ bk,
                         const int32_t* __restrict__ positions, const float* __restrict__ freq, int rot,
                         int interleaved, float mag, TQ* __restrict__ q_out, TC* __restrict__ kcache,
                         TC* __restrict__ vcache, const int32_t* __restrict__ slot_mapping, int page_size,
                         float* __restrict__ gate, int nh, int nkv, int hd, int hd_out) {
  extern __shared__ float row[];      // q and k of the token with their biases: (nh + nkv) hd
  __shared__ float cs[128], sn[128];
  const int t = blockIdx.x;
  const float* p = proj + (size_t)t * ld;
  const int nq = nh * hd, nk = nkv * hd;
#pragma unroll 8
  for (int i = threadIdx.x; i < nq; i += 256) row[i] = p[off_q + i] + (bq ? bq[i] : 0.f);
#pragma unroll 4
  for (int i = threadIdx.x; i < nk; i += 256) row[nq + i] = p[off_k + i] + (bk ? bk[i] : 0.f);
  angles(positions[t], freq, rot, mag, cs, sn);
  __syncthreads();
  for (int i = threadIdx.x; i < nh * hd_out; i += 256) {
    const int h = i / hd_out, d = i % hd_out;
    const float* x = row + h * hd;
    const float v = d >= hd ? 0.f : d < rot ? turned(x, d, rot, interleaved, cs, sn) : x[d];
    q_out[(size_t)t * nh * hd_out + i] = from_f32<TQ>(v);
  }
#pragma unroll 8
  for (int i = threadIdx.x; i < nq; i += 256) gate[(size_t)t * nq + i] = 1.0f / (1.0f + expf(-p[off_g + i]));
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const int page = slot / page_size, off = slot % page_size;
  for (int i = threadIdx.x; i < nkv * hd_out; i += 256) {
    const int h = i / hd_out, d = i % hd_out;
    const float* x = row + nq + h * hd;
    const float kv = d >= hd ? 0.f : d < rot ? turned(x, d, rot, interleaved, cs, sn) : x[d];
    const size_t tile = ((size_t)page * nkv + h) * page_size * hd_out;
    kcache[tile + key_offset(off, d, page_size)] = from_f32<TC>(kv);
    vcache[tile + value_offset(d, off, hd_out, page_size)] = from_f32<TC>(d >= hd ? 0.f : x[d]);
  }
}

template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
latent_rope_prepare_kernel(const float* __restrict__ proj, int ld, int off_dq, int off_c, int off_g, int q_rank,
                           int rank, int rd, int rank_p, int n_gate, const float* __restrict__ wq,
                           const float* __restrict__ wc, float eps, const int32_t* __restrict__ positions,
                           const float* __restrict__ freq, int rot, TA* __restrict__ cq, TC* __restrict__ kcache,
                           TC* __restrict__ vcache, const int32_t* __restrict__ slot_mapping, int page_size,
                           float* __restrict__ gate) {
  __shared__ float scratch[4];
  __shared__ float cs[128], sn[128];
  const int t = blockIdx.x;
  const float* p = proj + (size_t)t * ld;
  float sq = 0.f, sc = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += 256) sq = fmaf(p[off_dq + i], p[off_dq + i], sq);
  for (int i = threadIdx.x; i < rank; i += 256) sc = fmaf(p[off_c + i], p[off_c + i], sc);
  sq = block_sum<4>(sq, scratch);
  sc = block_sum<4>(sc, scratch);
  const float iq = 1.0f / sqrtf(sq / (float)q_rank + eps), ic = 1.0f / sqrtf(sc / (float)rank + eps);
  angles(positions[t], freq, rot, 1.0f, cs, sn);
  __syncthreads();
  for (int i = threadIdx.x; i < q_rank; i += 256) cq[(size_t)t * q_rank + i] = from_f32<TA>(p[off_dq + i] * iq * wq[i]);
#pragma unroll 8
  for (int i = threadIdx.x; i < n_gate; i += 256) gate[(size_t)t * n_gate + i] = 1.0f / (1.0f + expf(-p[off_g + i]));
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const int page = slot / page_size, off = slot % page_size;
  TC* kt = kcache + (size_t)page * page_size * rank_p;
  TC* vt = vcache + (size_t)page * page_size * rank_p;
  const float* kr = p + off_c + rank;      // the key part that is rotated
  for (int i = threadIdx.x; i < rank_p; i += 256) {
    float kv = 0.f, vv = 0.f;
    if (i < rank) {
      kv = vv = p[off_c + i] * ic * wc[i];
    } else if (i < rank + rd) {
      const int d = i - rank;
      kv = d < rot ? turned(kr, d, rot, 1, cs, sn) : kr[d];
    }
    kt[key_offset(off, i, page_size)] = from_f32<TC>(kv);
    vt[value_offset(i, off, rank_p, page_size)] = from_f32<TC>(vv);
  }
}

// q float32 [T, heads (dim + rd)] -> the activation dtype, the last rd columns of every head rotated in pairs
template <typename TA>
__global__ void __launch_bounds__(256)
latent_q_rope_kernel(const float* __restrict__ q, int ld, const int32_t* __restrict__ positions,
                     const float* __restrict__ freq, int rot, TA* __restrict__ out, int heads, int dim, int rd) {
  __shared__ float cs[128], sn[128];
  const int t = blockIdx.x;
  angles(positions[t], freq, rot, 1.0f, cs, sn);
  __syncthreads();
  const int hw = dim + rd;
  const float* p = q + (size_t)t * ld;
  for (int i = threadIdx.x; i < heads * hw; i += 256) {
    const int h = i / hw, d = i % hw;
    float v = p[i];
    if (d >= dim && d - dim < rot) v = turned(p + h * hw + dim, d - dim, rot, 1, cs, sn);
    out[(size_t)t * heads * hw + i] = from_f32<TA>(v);
  }
}

template <typename TA>
__global__ void __launch_bounds__(256)
gate_mul_kernel(const TA* __restrict__ att, const float* __restrict__ gate, TA* __restrict__ y, int heads, int vd,
                int hd_out) {
  const size_t t = blockIdx.x;
#pragma unroll 8
  for (int i = threadIdx.x; i < heads * vd; i += 256) {
    const int h = i / vd, j = i % vd;
    y[t * heads * vd + i] = from_f32<TA>(to_f32(att[t * heads * hd_out + h * hd_out + j]) * gate[t * heads * vd + i]);
  }
}

extern "C" int atoma_tied_rope_prepare(const float* proj, int ld, int off_q, int off_k, int off_g, const float* bq,
                                       const float* bk, const int32_t* positions, const float* freq, int rot,
                                       int interleaved, float mag, void* q_out, int q_dtype, void* kcache,
                                       void* vcache, int cache_dtype, const int32_t* slot_mapping, int page_size,
                                       float* gate, int n_tokens, int nh, int nkv, int hd, int hd_out,
                                       hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (nh <= 0 || nkv <= 0 || hd <= 0 || hd_out < hd || rot < 0 || rot % 2 || rot > hd || rot > 256 || page_size <= 0 ||
      off_q < 0 || off_k < 0 || off_g < 0 || ld < off_q + nh * hd || ld < off_k + nkv * hd || ld < off_g + nh * hd ||
      (size_t)(nh + nkv) * hd * 4 > 96 * 1024)
    return ATOMA_ERR_SHAPE;
  const size_t lds = (size_t)(nh + nkv) * hd * sizeof(float);
#define ATOMA_TRP(TQ, TC)                                                                                          \
  do {                                                                                                             \
    if (lds > 32 * 1024)                                                                                           \
      (void)hipFuncSetAttribute((const void*)tied_rope_prepare_kernel<TQ, TC>,                                     \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                             \
    hipLaunchKernelGGL((tied_rope_prepare_kernel<TQ, TC>), dim3(n_tokens), dim3(256), lds, stream, proj, ld, off_q, \
                       off_k, off_g, bq, bk, positions, freq, rot, interleaved, mag, (TQ*)q_out, (TC*)kcache,      \
                       (TC*)vcache, slot_mapping, page_size, gate, nh, nkv, hd, hd_out);                           \
  } while (0)
  if (q_dtype == kF32 && cache_dtype == kF32) ATOMA_TRP(float, float);
  else if (q_dtype == kBF16 && cache_dtype == kBF16) ATOMA_TRP(bf16_t, bf16_t);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_TRP
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_latent_rope_prepare(const float* proj, int ld, int off_dq, int off_c, int off_g, int q_rank,
                                         int rank, int rd, int rank_p, int n_gate, const float* wq, const float* wc,
                                         float eps, const int32_t* positions, const float* freq, int rot, void* cq,
                                         int act_dtype, void* kcache, void* vcache, int cache_dtype,
                                         const int32_t* slot_mapping, int page_size, float* gate, int n_tokens,
                                         hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (q_rank <= 0 || rank <= 0 || rd < 0 || rank_p < rank + rd || n_gate <= 0 || rot < 0 || rot % 2 || rot > rd ||
      rot > 256 || page_size <= 0 || off_dq < 0 || off_c < 0 || off_g < 0 || ld < off_dq + q_rank ||
      ld < off_c + rank + rd || ld < off_g + n_gate)
    return ATOMA_ERR_SHAPE;
#define ATOMA_LRP(TA, TC)                                                                                            \
  hipLaunchKernelGGL((latent_rope_prepare_kernel<TA, TC>), dim3(n_tokens), dim3(256), 0, stream, proj, ld, off_dq,   \
                     off_c, off_g, q_rank, rank, rd, rank_p, n_gate, wq, wc, eps, positions, freq, rot, (TA*)cq,     \
                     (TC*)kcache, (TC*)vcache, slot_mapping, page_size, gate)
  if (act_dtype == kF32 && cache_dtype == kF32) ATOMA_LRP(float, float);
  else if (act_dtype == kBF16 && cache_dtype == kBF16) ATOMA_LRP(bf16_t, bf16_t);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_LRP
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_latent_q_rope(const float* q, int ld, const int32_t* positions, const float* freq, int rot,
                                   void* out, int out_dtype, int n_tokens, int heads, int dim, int rd,
                                   hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (heads <= 0 || dim < 0 || rd < 0 || dim + rd <= 0 || rot < 0 || rot % 2 || rot > rd || rot > 256 ||
      ld < heads * (dim + rd))
    return ATOMA_ERR_SHAPE;
  if (out_dtype == kF32)
    hipLaunchKernelGGL((latent_q_rope_kernel<float>), dim3(n_tokens), dim3(256), 0, stream, q, ld, positions, freq,
                       rot, (float*)out, heads, dim, rd);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL((latent_q_rope_kernel<bf16_t>), dim3(n_tokens), dim3(256), 0, stream, q, ld, positions, freq,
                       rot, (bf16_t*)out, heads, dim, rd);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_gate_mul(const void* att, const float* gate, void* y, int dtype, int n_tokens, int heads, int vd,
                              int hd_out, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (heads <= 0 || vd <= 0 || hd_out < vd) return ATOMA_ERR_SHAPE;
  if (dtype == kF32)
    hipLaunchKernelGGL((gate_mul_kernel<float>), dim3(n_tokens), dim3(256), 0, stream, (const float*)att, gate,
                       (float*)y, heads, vd, hd_out);
  else if (dtype == kBF16)
    hipLaunchKernelGGL((gate_mul_kernel<bf16_t>), dim3(n_tokens), dim3(256), 0, stream, (const bf16_t*)att, gate,
                       (bf16_t*)y, heads, vd, hd_out);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}
