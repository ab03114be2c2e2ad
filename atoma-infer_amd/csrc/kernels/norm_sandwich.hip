// A sublayer's output normed before it joins the residual stream, fused with the sum and with the norm that reads
// the stream next:
//
//   d     = sum_i scale_i * (sum over planes of delta_i)          (up to two terms: mixers that run side by side)
//   resid += d / sqrt(mean(d^2) + eps) * w_post                   (float32, in place)
//   out   = resid / sqrt(mean(resid^2) + eps) * w_next            (optional, in the activation dtype)
//
// Without w_post the sum joins the stream as it is, resid += d: blocks whose sublayers read one norm and add their
// outputs side by side.
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
  float inv = 1.0f;
  if (w_post != nullptr) {
    ss = block_sum<4>(ss, scratch);
    inv = 1.0f / sqrtf(ss / (float)width + eps_post);
  }
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float x = resid[base + i] + (w_post != nullptr ? row[i] * inv * w_post[i] : row[i]);
    resid[base + i] = x;
    row[i] = x;
    ss2 += x * x;
  }
  if (out == nullptr) return;
  ss2 = block_sum<4>(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
  for (int i = threadIdx.x; i < width; i += 256) out[base + i] = from_f32<TO>(row[i] * inv2 * w_next[i]);
}

// The same for rows whose width is a multiple of 4, at most 1024 * MAXJ columns, with 16-byte aligned operands: a
// thread keeps its columns in registers through all three passes, and the loads of a pass (up to four planes of a term
// at a time) are issued together.
struct f4 {
  float v[4];
};

__device__ __forceinline__ f4 load4(const float* p) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  return f4{{x.x, x.y, x.z, x.w}};
}

__device__ __forceinline__ f4 load4(const bf16_t* p) {
  const uint2 x = *reinterpret_cast<const uint2*>(p);
  return f4{{bf16_bits_to_f32((uint16_t)(x.x & 0xffff)), bf16_bits_to_f32((uint16_t)(x.x >> 16)),
             bf16_bits_to_f32((uint16_t)(x.y & 0xffff)), bf16_bits_to_f32((uint16_t)(x.y >> 16))}};
}

__device__ __forceinline__ void store4(float* p, const f4& x) {
  *reinterpret_cast<float4*>(p) = make_float4(x.v[0], x.v[1], x.v[2], x.v[3]);
}

__device__ __forceinline__ void store4(bf16_t* p, const f4& x) {
  uint2 o;
  o.x = (uint32_t)f32_to_bf16_bits(x.v[0]) | ((uint32_t)f32_to_bf16_bits(x.v[1]) << 16);
  o.y = (uint32_t)f32_to_bf16_bits(x.v[2]) | ((uint32_t)f32_to_bf16_bits(x.v[3]) << 16);
  *reinterpret_cast<uint2*>(p) = o;
}

template <typename TD, int MAXJ>
__device__ __forceinline__ void add_term(f4 (&d)[MAXJ], const Term& t, size_t base, int n4) {
  const TD* p0 = (const TD*)t.data + base;
  f4 sum[MAXJ];
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) sum[j] = f4{{0.f, 0.f, 0.f, 0.f}};
  for (int s0 = 0; s0 < t.planes; s0 += 4) {
    f4 x[4][MAXJ];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int s = s0 + q < t.planes ? s0 + q : t.planes - 1;
#pragma unroll
      for (int j = 0; j < MAXJ; ++j) {
        const int c = threadIdx.x + j * 256;
        if (c < n4) x[q][j] = load4(p0 + s * t.plane_stride + 4 * c);
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (s0 + q < t.planes)
#pragma unroll
        for (int j = 0; j < MAXJ; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) sum[j].v[i] += x[q][j].v[i];
  }
#pragma unroll
  for (int j = 0; j < MAXJ; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) d[j].v[i] += sum[j].v[i] * t.scale;
}

template <typename TO, int MAXJ>
__global__ void __launch_bounds__(256)
add_normed_vec_kernel(float* __restrict__ resid, Term a, Term b, int n_terms, const float* __restrict__ w_post,
                      const float* __restrict__ w_next, TO* __restrict__ out, int width, float eps_post,
                      float eps_next) {
  __shared__ float scratch[4];
  const size_t base = (size_t)blockIdx.x * width;
  const int n4 = width >> 2;
  f4 d[MAXJ], x[MAXJ];
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) {
    d[j] = f4{{0.f, 0.f, 0.f, 0.f}};
    const int c = threadIdx.x + j * 256;
    if (c < n4) x[j] = load4(resid + base + 4 * c);
  }
  if (a.dtype == kF32) add_term<float, MAXJ>(d, a, base, n4);
  else add_term<bf16_t, MAXJ>(d, a, base, n4);
  if (n_terms > 1) {
    if (b.dtype == kF32) add_term<float, MAXJ>(d, b, base, n4);
    else add_term<bf16_t, MAXJ>(d, b, base, n4);
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < MAXJ; ++j)
    if (threadIdx.x + j * 256 < n4)
#pragma unroll
      for (int i = 0; i < 4; ++i) ss += d[j].v[i] * d[j].v[i];
  float inv = 1.0f;
  if (w_post != nullptr) {
    ss = block_sum<4>(ss, scratch);
    inv = 1.0f / sqrtf(ss / (float)width + eps_post);
  }
  float ss2 = 0.f;
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) {
    const int c = threadIdx.x + j * 256;
    if (c < n4) {
      const f4 wp = w_post != nullptr ? load4(w_post + 4 * c) : f4{{1.f, 1.f, 1.f, 1.f}};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        x[j].v[i] += w_post != nullptr ? d[j].v[i] * inv * wp.v[i] : d[j].v[i];
        ss2 += x[j].v[i] * x[j].v[i];
      }
      store4(resid + base + 4 * c, x[j]);
    }
  }
  if (out == nullptr) return;
  ss2 = block_sum<4>(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) {
    const int c = threadIdx.x + j * 256;
    if (c < n4) {
      const f4 wn = load4(w_next + 4 * c);
      f4 y;
#pragma unroll
      for (int i = 0; i < 4; ++i) y.v[i] = x[j].v[i] * inv2 * wn.v[i];
      store4(out + base + 4 * c, y);
    }
  }
}

template <typename TO>
static void launch_vec(dim3 grid, hipStream_t stream, float* resid, const Term& a, const Term& b, int n_terms,
                       const float* w_post, const float* w_next, void* out, int width, float eps_post, float eps_next) {
  const dim3 block(256);
  if (width <= 2048)
    hipLaunchKernelGGL((add_normed_vec_kernel<TO, 2>), grid, block, 0, stream, resid, a, b, n_terms, w_post, w_next,
                       (TO*)out, width, eps_post, eps_next);
  else if (width <= 4096)
    hipLaunchKernelGGL((add_normed_vec_kernel<TO, 4>), grid, block, 0, stream, resid, a, b, n_terms, w_post, w_next,
                       (TO*)out, width, eps_post, eps_next);
  else
    hipLaunchKernelGGL((add_normed_vec_kernel<TO, 8>), grid, block, 0, stream, resid, a, b, n_terms, w_post, w_next,
                       (TO*)out, width, eps_post, eps_next);
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
  auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  const bool vec = width % 4 == 0 && width <= 8192 && aligned(resid) && aligned(d0) && aligned(d1) && aligned(w_post) &&
                   aligned(w_next) && aligned(out) && stride0 % 4 == 0 && (d1 == nullptr || stride1 % 4 == 0);
  if (vec && (out == nullptr || out_dtype == kF32))
    launch_vec<float>(grid, stream, resid, a, b, n_terms, w_post, w_next, out, width, eps_post, eps_next);
  else if (vec && out_dtype == kBF16)
    launch_vec<bf16_t>(grid, stream, resid, a, b, n_terms, w_post, w_next, out, width, eps_post, eps_next);
  else if (out == nullptr || out_dtype == kF32)
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

// The same sum behind a sublayer, for designs whose layers read a weighted average of all earlier layers' results
// instead of the last one:
//
//   X      = resid + d / sqrt(mean(d^2) + eps) * w_post          the layer's result, kept as results[n - 1]
//   resid  = sum_(j < n) dw[j] * results[j]                       (float32, j ascending; results[0]: the embedding's rows)
//   out    = resid / sqrt(mean(resid^2) + eps) * w_next           (optional)
//
// results is [layers + 1, T, width] float32 and lives for one step.  One workgroup a row, the row in LDS between the
// passes.
template <typename TO>
__global__ void __launch_bounds__(256)
depth_average_kernel(float* __restrict__ resid, Term a, Term b, int n_terms, const float* __restrict__ w_post,
                     float* __restrict__ results, size_t result_stride, int n, const float* __restrict__ dw,
                     const float* __restrict__ w_next, TO* __restrict__ out, int width, float eps_post,
                     float eps_next) {
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
  float inv = 1.0f;
  if (w_post != nullptr) {
    ss = block_sum<4>(ss, scratch);
    inv = 1.0f / sqrtf(ss / (float)width + eps_post);
  }
  const float last = dw[n - 1];
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float x = resid[base + i] + (w_post != nullptr ? row[i] * inv * w_post[i] : row[i]);
    results[(size_t)(n - 1) * result_stride + base + i] = x;
    float y = 0.f;
    for (int j = 0; j < n - 1; ++j) y += dw[j] * results[(size_t)j * result_stride + base + i];
    y += last * x;
    resid[base + i] = y;
    row[i] = y;
    ss2 += y * y;
  }
  if (out == nullptr) return;
  ss2 = block_sum<4>(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
  for (int i = threadIdx.x; i < width; i += 256) out[base + i] = from_f32<TO>(row[i] * inv2 * w_next[i]);
}

// The same for rows whose width is a multiple of 4 (at most 1024 * MAXJ columns, 16-byte aligned operands): a thread
// keeps its columns in registers; the earlier results are fetched four at a time, together with the stream's rows
// and the sublayer's planes, before the first sum over the row, so a step of few rows waits for memory once.
template <typename TO, int MAXJ>
__global__ void __launch_bounds__(256)
depth_average_vec_kernel(float* __restrict__ resid, Term a, Term b, int n_terms, const float* __restrict__ w_post,
                         const float* __restrict__ earlier, float* __restrict__ kept, size_t result_stride, int n,
                         const float* __restrict__ dw, const float* __restrict__ w_next, TO* __restrict__ out,
                         int width, float eps_post, float eps_next) {
  __shared__ float scratch[4];
  const size_t base = (size_t)blockIdx.x * width;
  const int n4 = width >> 2;
  f4 d[MAXJ], x[MAXJ], acc[MAXJ];
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) {
    d[j] = f4{{0.f, 0.f, 0.f, 0.f}};
    acc[j] = f4{{0.f, 0.f, 0.f, 0.f}};
    const int c = threadIdx.x + j * 256;
    if (c < n4) x[j] = load4(resid + base + 4 * c);
  }
  // sum_(j < n - 1) dw[j] * results[j], j ascending
  for (int s0 = 0; s0 < n - 1; s0 += 4) {
    f4 r[4][MAXJ];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int s = s0 + q < n - 1 ? s0 + q : n - 2;
#pragma unroll
      for (int j = 0; j < MAXJ; ++j) {
        const int c = threadIdx.x + j * 256;
        if (c < n4) r[q][j] = load4(earlier + (size_t)s * result_stride + base + 4 * c);
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (s0 + q < n - 1) {
        const float w = dw[s0 + q];
#pragma unroll
        for (int j = 0; j < MAXJ; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[j].v[i] += w * r[q][j].v[i];
      }
  }
  if (a.dtype == kF32) add_term<float, MAXJ>(d, a, base, n4);
  else add_term<bf16_t, MAXJ>(d, a, base, n4);
  if (n_terms > 1) {
    if (b.dtype == kF32) add_term<float, MAXJ>(d, b, base, n4);
    else add_term<bf16_t, MAXJ>(d, b, base, n4);
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < MAXJ; ++j)
    if (threadIdx.x + j * 256 < n4)
#pragma unroll
      for (int i = 0; i < 4; ++i) ss += d[j].v[i] * d[j].v[i];
  float inv = 1.0f;
  if (w_post != nullptr) {
    ss = block_sum<4>(ss, scratch);
    inv = 1.0f / sqrtf(ss / (float)width + eps_post);
  }
  const float last = dw[n - 1];
  float ss2 = 0.f;
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) {
    const int c = threadIdx.x + j * 256;
    if (c < n4) {
      const f4 wp = w_post != nullptr ? load4(w_post + 4 * c) : f4{{1.f, 1.f, 1.f, 1.f}};
#pragma unroll
      for (int i = 0; i < 4; ++i) x[j].v[i] += w_post != nullptr ? d[j].v[i] * inv * wp.v[i] : d[j].v[i];
      store4(kept + base + 4 * c, x[j]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        x[j].v[i] = acc[j].v[i] + last * x[j].v[i];
        ss2 += x[j].v[i] * x[j].v[i];
      }
      store4(resid + base + 4 * c, x[j]);
    }
  }
  if (out == nullptr) return;
  ss2 = block_sum<4>(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) {
    const int c = threadIdx.x + j * 256;
    if (c < n4) {
      const f4 wn = load4(w_next + 4 * c);
      f4 y;
#pragma unroll
      for (int i = 0; i < 4; ++i) y.v[i] = x[j].v[i] * inv2 * wn.v[i];
      store4(out + base + 4 * c, y);
    }
  }
}

template <typename TO>
static void launch_depth_vec(dim3 grid, hipStream_t stream, float* resid, const Term& a, const Term& b, int n_terms,
                             const float* w_post, float* results, size_t result_stride, int n, const float* dw,
                             const float* w_next, void* out, int width, float eps_post, float eps_next) {
  const dim3 block(256);
  float* kept = results + (size_t)(n - 1) * result_stride;
  if (width <= 2048)
    hipLaunchKernelGGL((depth_average_vec_kernel<TO, 2>), grid, block, 0, stream, resid, a, b, n_terms, w_post, results,
                       kept, result_stride, n, dw, w_next, (TO*)out, width, eps_post, eps_next);
  else if (width <= 4096)
    hipLaunchKernelGGL((depth_average_vec_kernel<TO, 4>), grid, block, 0, stream, resid, a, b, n_terms, w_post, results,
                       kept, result_stride, n, dw, w_next, (TO*)out, width, eps_post, eps_next);
  else
    hipLaunchKernelGGL((depth_average_vec_kernel<TO, 8>), grid, block, 0, stream, resid, a, b, n_terms, w_post, results,
                       kept, result_stride, n, dw, w_next, (TO*)out, width, eps_post, eps_next);
}

extern "C" int atoma_depth_average(float* resid, const void* d0, int dtype0, int planes0, size_t stride0, float scale0,
                                   const void* d1, int dtype1, int planes1, size_t stride1, float scale1,
                                   const float* w_post, float eps_post, float* results, size_t result_stride, int n,
                                   const float* dw, const float* w_next, float eps_next, void* out, int out_dtype,
                                   int n_rows, int width, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || width > 16384 || d0 == nullptr || planes0 <= 0 || (d1 != nullptr && planes1 <= 0) || n < 1 ||
      results == nullptr || dw == nullptr || result_stride < (size_t)n_rows * width)
    return ATOMA_ERR_SHAPE;
  if ((dtype0 != kF32 && dtype0 != kBF16) || (d1 != nullptr && dtype1 != kF32 && dtype1 != kBF16)) return ATOMA_ERR_DTYPE;
  Term a{d0, dtype0, planes0, stride0, scale0}, b{d1, dtype1, planes1, stride1, scale1};
  const int n_terms = d1 != nullptr ? 2 : 1;
  const size_t lds = (size_t)width * sizeof(float);
  dim3 grid(n_rows), block(256);
  auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  const bool vec = width % 4 == 0 && width <= 8192 && aligned(resid) && aligned(d0) && aligned(d1) && aligned(w_post) &&
                   aligned(w_next) && aligned(out) && aligned(results) && result_stride % 4 == 0 && stride0 % 4 == 0 &&
                   (d1 == nullptr || stride1 % 4 == 0);
  if (vec && (out == nullptr || out_dtype == kF32))
    launch_depth_vec<float>(grid, stream, resid, a, b, n_terms, w_post, results, result_stride, n, dw, w_next, out,
                            width, eps_post, eps_next);
  else if (vec && out_dtype == kBF16)
    launch_depth_vec<bf16_t>(grid, stream, resid, a, b, n_terms, w_post, results, result_stride, n, dw, w_next, out,
                             width, eps_post, eps_next);
  else if (out == nullptr || out_dtype == kF32)
    hipLaunchKernelGGL((depth_average_kernel<float>), grid, block, lds, stream, resid, a, b, n_terms, w_post, results,
                       result_stride, n, dw, w_next, (float*)out, width, eps_post, eps_next);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL((depth_average_kernel<bf16_t>), grid, block, lds, stream, resid, a, b, n_terms, w_post, results,
                       result_stride, n, dw, w_next, (bf16_t*)out, width, eps_post, eps_next);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// Rows of the stream set anew: resid[t] = y[t] + bias (float32), for a map of the whole stream that replaces it
// (the entry of a pass over looped layers).  The second kernel packs the rows of two float32 streams side by side in
// the activation dtype, [a | b], as such a map's input.
__global__ void __launch_bounds__(256)
set_rows_kernel(float* __restrict__ resid, const float* __restrict__ y, const float* __restrict__ bias, int width) {
  const size_t base = (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += 256) resid[base + i] = y[base + i] + bias[i];
}

template <typename TO>
__global__ void __launch_bounds__(256)
pack_pair_kernel(const float* __restrict__ a, const float* __restrict__ b, TO* __restrict__ out, int width) {
  const size_t base = (size_t)blockIdx.x * width;
  TO* o = out + 2 * base;
  for (int i = threadIdx.x; i < width; i += 256) {
    o[i] = from_f32<TO>(a[base + i]);
    o[width + i] = from_f32<TO>(b[base + i]);
  }
}

extern "C" int atoma_set_rows(float* resid, const float* y, const float* bias, int n_rows, int width,
                              hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(set_rows_kernel, dim3(n_rows), dim3(256), 0, stream, resid, y, bias, width);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_pack_pair(const float* a, const float* b, void* out, int out_dtype, int n_rows, int width,
                               hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0) return ATOMA_ERR_SHAPE;
  if (out_dtype == kF32)
    hipLaunchKernelGGL((pack_pair_kernel<float>), dim3(n_rows), dim3(256), 0, stream, a, b, (float*)out, width);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL((pack_pair_kernel<bf16_t>), dim3(n_rows), dim3(256), 0, stream, a, b, (bf16_t*)out, width);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}
