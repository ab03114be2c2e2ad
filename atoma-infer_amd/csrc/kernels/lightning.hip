// Linear attention with one fixed decay per head (the lightning form): per head, with q, k [dim] and v [vdim] the
// SiLU of a token's projections,
//
//   S <- decay_h S + k v^T,        o = S^T q,
//
// S [dim, vdim] float32 per request and head, read from the request's state row before an entry's first token and
// written back after its last, so that prompts, portions and decoded tokens are one code path and a request may be
// cut anywhere.  The heads' outputs of a token are RMS-normed together, weighted, gated by sigmoid(g) and leave in the
// activation dtype.
//
//   lightning_scan   a workgroup owns (entry, head, 16 columns of S) and walks the entry's tokens in order; a column
//                    of S lies in the registers of 16 neighbouring lanes (dim / 16 rows each), the lanes' shares of
//                    S^T q are added with four shuffles; q, k, v of 16 tokens at a time pass LDS, SiLU applied on
//                    the way in.
//   lightning_out    one workgroup a token: norm over all heads' outputs, weight, gate.
// State row layout: [heads][vdim][dim] (a column of S contiguous).
#include "common.h"

using namespace atoma;

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }

constexpr int kLtTokens = 16;      // tokens staged in LDS at a time
constexpr int kLtMaxRows = 16;     // rows of S a lane holds: dim <= 256

__global__ void __launch_bounds__(256)
lightning_scan_kernel(const float* __restrict__ proj, int ld, int off_q, int off_k, int off_v,
                      const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                      float* __restrict__ state, const float* __restrict__ decay, float* __restrict__ o, int heads,
                      int dim, int vdim) {
  extern __shared__ float lds[];      // q [16][dim], k [16][dim], v [16][16]
  float* qs = lds;
  float* ks = lds + kLtTokens * dim;
  float* vs = ks + kLtTokens * dim;
  const int e = blockIdx.y;
  const int vblocks = (vdim + 15) / 16;
  const int h = blockIdx.x / vblocks, vb = blockIdx.x % vblocks;
  const int t0 = q_start[e], t1 = q_start[e + 1];
  if (t1 <= t0) return;
  const int col = threadIdx.x >> 4, part = threadIdx.x & 15;      // column of the block, share of its rows
  const int j = vb * 16 + col;
  const bool live = j < vdim;
  const int rows = (dim + 15) / 16;
  float* srow = state + ((size_t)state_slots[e] * heads + h) * (size_t)vdim * dim + (size_t)(live ? j : 0) * dim;
  float s[kLtMaxRows];
#pragma unroll
  for (int i = 0; i < kLtMaxRows; ++i) {
    const int r = part + 16 * i;
    s[i] = (live && i < rows && r < dim) ? srow[r] : 0.f;
  }
  const float dec = decay[h];
  for (int tb = t0; tb < t1; tb += kLtTokens) {
    const int n = t1 - tb < kLtTokens ? t1 - tb : kLtTokens;
    __syncthreads();
    for (int idx = threadIdx.x; idx < n * dim; idx += 256) {
      const int tt = idx / dim, r = idx % dim;
      const float* row = proj + (size_t)(tb + tt) * ld;
      qs[tt * dim + r] = silu_f(row[off_q + h * dim + r]);
      ks[tt * dim + r] = silu_f(row[off_k + h * dim + r]);
    }
    for (int idx = threadIdx.x; idx < n * 16; idx += 256) {
      const int tt = idx >> 4, c = idx & 15;
      vs[idx] = vb * 16 + c < vdim ? silu_f(proj[(size_t)(tb + tt) * ld + off_v + h * vdim + vb * 16 + c]) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float v = vs[tt * 16 + col];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < kLtMaxRows; ++i) {
        if (i < rows) {
          const int r = part + 16 * i;
          const float kq = r < dim ? ks[tt * dim + r] : 0.f, qq = r < dim ? qs[tt * dim + r] : 0.f;
          s[i] = fmaf(dec, s[i], kq * v);
          acc = fmaf(s[i], qq, acc);
        }
      }
      acc += __shfl_xor(acc, 1, 64);
      acc += __shfl_xor(acc, 2, 64);
      acc += __shfl_xor(acc, 4, 64);
      acc += __shfl_xor(acc, 8, 64);
      if (part == 0 && live) o[(size_t)(tb + tt) * heads * vdim + h * vdim + j] = acc;
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < kLtMaxRows; ++i) {
      const int r = part + 16 * i;
      if (i < rows && r < dim) srow[r] = s[i];
    }
  }
}

template <typename TO>
__global__ void __launch_bounds__(256)
lightning_out_kernel(const float* __restrict__ o, const float* __restrict__ proj, int ld, int off_g,
                     const float* __restrict__ w, float eps, TO* __restrict__ y, int n) {
  __shared__ float scratch[4];
  const size_t t = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += 256) ss = fmaf(o[t * n + c], o[t * n + c], ss);
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += 256) {
    const float g = 1.0f / (1.0f + expf(-proj[t * ld + off_g + c]));
    y[t * n + c] = from_f32<TO>(o[t * n + c] * inv * w[c] * g);
  }
}

extern "C" int atoma_lightning_scan(const float* proj, int ld, int off_q, int off_k, int off_v, const int32_t* q_start,
                                    const int32_t* state_slots, float* state, const float* decay, float* o,
                                    int n_entries, int heads, int dim, int vdim, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (heads <= 0 || dim <= 0 || dim > 16 * kLtMaxRows || vdim <= 0 || n_entries > 65535 || off_q < 0 || off_k < 0 ||
      off_v < 0 || ld < off_q + heads * dim || ld < off_k + heads * dim || ld < off_v + heads * vdim)
    return ATOMA_ERR_SHAPE;
  const size_t lds = (size_t)(2 * kLtTokens * dim + kLtTokens * 16) * sizeof(float);
  dim3 grid(heads * ((vdim + 15) / 16), n_entries);
  hipLaunchKernelGGL(lightning_scan_kernel, grid, dim3(256), lds, stream, proj, ld, off_q, off_k, off_v, q_start,
                     state_slots, state, decay, o, heads, dim, vdim);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_lightning_out(const float* o, const float* proj, int ld, int off_g, const float* w, float eps,
                                   void* y, int y_dtype, int n_tokens, int n, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (n <= 0 || off_g < 0 || ld < off_g + n) return ATOMA_ERR_SHAPE;
  if (y_dtype == kF32)
    hipLaunchKernelGGL((lightning_out_kernel<float>), dim3(n_tokens), dim3(256), 0, stream, o, proj, ld, off_g, w, eps,
                       (float*)y, n);
  else if (y_dtype == kBF16)
    hipLaunchKernelGGL((lightning_out_kernel<bf16_t>), dim3(n_tokens), dim3(256), 0, stream, o, proj, ld, off_g, w,
                       eps, (bf16_t*)y, n);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}
