// A residual stream kept in several copies (hyper-connections), the embedding that starts it, and the sum of two
// normed branches.
//
// The stream is float32 [S, T, W]: S copies x_1 .. x_S of every token's row.  Around a sublayer with the weights
// in [S], mix [S, S] (indexed [from, to]) and out [S]:
//
//   u   = sum_s in[s] x_s                       the sublayer's input, before its norm
//   x_t <- sum_s mix[s, t] x_s + out[t] y       all copies at once from the old ones, y the sublayer's output
//
//   stream_step     one workgroup a row: the update with the output y of the sublayer before (optional), then the
//                   read u for the sublayer behind with its RMS norm (optional), in one pass over the row: the new
//                   copies never travel to memory and back between the two.  With `rows` only those rows are read
//                   (and nothing is written back): the last read of a step, for the rows whose logits are wanted.
//                   S = 1 with mix = out = in = 1 is the plain pre-norm residual.
//   bigram_embed    x = table[token] * scale + pairs[(prev * mul_prev + token * mul_cur) mod buckets], the row
//                   `buckets` of `pairs` for a request's first token, written to every copy.  The token before an
//                   entry's first is the request's state (one int32), which the entry's last token replaces.
//   normed_branches y = scale * (a / rms(a) * wa + b / rms(b) * wb), each branch with its own statistics.
// All arithmetic is float32; a sum's order depends on the column alone.
#include "common.h"

using namespace atoma;

constexpr int kMaxStreams = 8;

struct StreamWeights {
  float mix[kMaxStreams * kMaxStreams];
  float out[kMaxStreams];
  float in[kMaxStreams];
};

// V values of neighbouring columns at a time (V = 4: 16-byte loads of the copies, for rows of a multiple of 4 columns)
template <int V> struct Vals {
  float v[V];
};
template <int V> __device__ __forceinline__ Vals<V> load_vals(const float* p) {
  Vals<V> r;
  if constexpr (V == 4) {
    const float4 q = *reinterpret_cast<const float4*>(p);
    r.v[0] = q.x, r.v[1] = q.y, r.v[2] = q.z, r.v[3] = q.w;
  } else {
    r.v[0] = *p;
  }
  return r;
}
template <int V> __device__ __forceinline__ Vals<V> load_vals(const bf16_t* p) {
  Vals<V> r;
  if constexpr (V == 4) {
    const uint2 q = *reinterpret_cast<const uint2*>(p);
    r.v[0] = bf16_bits_to_f32(q.x & 0xffff), r.v[1] = bf16_bits_to_f32(q.x >> 16);
    r.v[2] = bf16_bits_to_f32(q.y & 0xffff), r.v[3] = bf16_bits_to_f32(q.y >> 16);
  } else {
    r.v[0] = to_f32(*p);
  }
  return r;
}
template <int V> __device__ __forceinline__ void store_vals(float* p, const Vals<V>& a) {
  if constexpr (V == 4) *reinterpret_cast<float4*>(p) = make_float4(a.v[0], a.v[1], a.v[2], a.v[3]);
  else *p = a.v[0];
}
template <int V> __device__ __forceinline__ void store_vals(bf16_t* p, const Vals<V>& a) {
  if constexpr (V == 4) {
    *reinterpret_cast<uint2*>(p) = make_uint2(f32_to_bf16_bits(a.v[0]) | ((uint32_t)f32_to_bf16_bits(a.v[1]) << 16),
                                              f32_to_bf16_bits(a.v[2]) | ((uint32_t)f32_to_bf16_bits(a.v[3]) << 16));
  } else {
    *p = from_f32<bf16_t>(a.v[0]);
  }
}

template <typename TY, typename TO, int SM, int V>
__global__ void __launch_bounds__(256)
stream_step_kernel(float* __restrict__ x, size_t copy_stride, int W, int S, const TY* __restrict__ y, int planes,
                   size_t plane_stride, const float* __restrict__ mix, const float* __restrict__ outw,
                   const float* __restrict__ inw, const float* __restrict__ norm_w, float eps, TO* __restrict__ h,
                   const int32_t* __restrict__ rows, int write_back) {
  extern __shared__ float urow[];
  __shared__ float scratch[4];
  __shared__ StreamWeights sw;
  const int r = blockIdx.x;
  const int t = rows ? rows[r] : r;
  if (threadIdx.x < S * S) sw.mix[threadIdx.x] = y ? mix[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    sw.out[threadIdx.x] = y ? outw[threadIdx.x] : 0.f;
    sw.in[threadIdx.x] = inw ? inw[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float ss = 0.f;
  // (loops over the copies have the constant bound SM >= S, so that the copies' values stay in registers)
  for (int c = threadIdx.x * V; c < W; c += 256 * V) {
    Vals<V> old[SM], cur[SM];
#pragma unroll
    for (int s = 0; s < SM; ++s) {
      if (s < S) old[s] = load_vals<V>(x + s * copy_stride + (size_t)t * W + c);
      else
#pragma unroll
        for (int e = 0; e < V; ++e) old[s].v[e] = 0.f;
    }
    if (y) {
      Vals<V> yv;
#pragma unroll
      for (int e = 0; e < V; ++e) yv.v[e] = 0.f;
      for (int p = 0; p < planes; ++p) {
        const Vals<V> a = load_vals<V>(y + p * plane_stride + (size_t)t * W + c);
#pragma unroll
        for (int e = 0; e < V; ++e) yv.v[e] += a.v[e];
      }
#pragma unroll
      for (int to = 0; to < SM; ++to) {
#pragma unroll
        for (int e = 0; e < V; ++e) {
          float v = 0.f;
#pragma unroll
          for (int s = 0; s < SM; ++s)
            if (s < S && to < S) v = fmaf(sw.mix[s * S + to], old[s].v[e], v);
          cur[to].v[e] = to < S ? fmaf(sw.out[to], yv.v[e], v) : 0.f;
        }
      }
      if (write_back) {
#pragma unroll
        for (int s = 0; s < SM; ++s)
          if (s < S) store_vals<V>(x + s * copy_stride + (size_t)t * W + c, cur[s]);
      }
    } else {
#pragma unroll
      for (int s = 0; s < SM; ++s) cur[s] = old[s];
    }
    if (h) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < SM; ++s)
          if (s < S) u = fmaf(sw.in[s], cur[s].v[e], u);
        urow[c + e] = u;
        ss = fmaf(u, u, ss);
      }
    }
  }
  if (!h) return;
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x * V; c < W; c += 256 * V) {
    Vals<V> o;
#pragma unroll
    for (int e = 0; e < V; ++e) o.v[e] = urow[c + e] * inv * norm_w[c + e];
    store_vals<V>(h + (size_t)r * W + c, o);
  }
}

extern "C" int atoma_stream_step(float* x, int T, int W, int S, const void* y, int y_dtype, int planes,
                                 size_t plane_stride, const float* mix, const float* outw, const float* inw,
                                 const float* norm_w, float eps, void* h, int h_dtype, const int32_t* rows, int n_rows,
                                 int write_back, hipStream_t stream) {
  const int n = rows ? n_rows : T;
  if (n <= 0) return 0;
  if (W <= 0 || S <= 0 || S > kMaxStreams || (size_t)W * 4 > 150 * 1024 || (y && (!mix || !outw || planes <= 0)) ||
      (h && (!inw || !norm_w)))
    return ATOMA_ERR_SHAPE;
  const size_t copy_stride = (size_t)T * W, lds = h ? (size_t)W * 4 : 0;
#define ATOMA_SS_V(TY, TO, SM, V)                                                                                 \
  do {                                                                                                            \
    if (lds > 48 * 1024)                                                                                          \
      (void)hipFuncSetAttribute((const void*)stream_step_kernel<TY, TO, SM, V>,                                   \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                            \
    hipLaunchKernelGGL((stream_step_kernel<TY, TO, SM, V>), dim3(n), dim3(256), lds, stream, x, copy_stride, W, S, \
                       (const TY*)y, planes, plane_stride, mix, outw, inw, norm_w, eps, (TO*)h, rows, write_back); \
  } while (0)
#define ATOMA_SS_N(TY, TO, SM)           \
  do {                                   \
    if (vec) ATOMA_SS_V(TY, TO, SM, 4);  \
    else ATOMA_SS_V(TY, TO, SM, 1);      \
  } while (0)
#define ATOMA_SS(TY, TO)                   \
  do {                                     \
    if (S == 1) ATOMA_SS_N(TY, TO, 1);     \
    else if (S == 2) ATOMA_SS_N(TY, TO, 2); \
    else if (S <= 4) ATOMA_SS_N(TY, TO, 4); \
    else ATOMA_SS_N(TY, TO, 8);            \
  } while (0)
  // rows of a multiple of 4 columns in tensors that torch allocated (aligned) take 16 bytes of a copy at a time
  const bool vec = W % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)y & 15) == 0 && ((uintptr_t)h & 15) == 0 &&
                   ((uintptr_t)norm_w & 15) == 0;
  const bool yb = y && y_dtype == kBF16, hb = h && h_dtype == kBF16;
  if (y && y_dtype != kF32 && y_dtype != kBF16) return ATOMA_ERR_DTYPE;
  if (h && h_dtype != kF32 && h_dtype != kBF16) return ATOMA_ERR_DTYPE;
  if (yb && hb) ATOMA_SS(bf16_t, bf16_t);
  else if (yb) ATOMA_SS(bf16_t, float);
  else if (hb) ATOMA_SS(float, bf16_t);
  else ATOMA_SS(float, float);
#undef ATOMA_SS
#undef ATOMA_SS_N
#undef ATOMA_SS_V
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// One workgroup a token.  The thread group of an entry's FIRST token reads the request's previous token from `state`
// and (thread 0) stores the entry's LAST token there afterwards: one group reads and writes a state row, in that order.
template <typename TE>
__global__ void __launch_bounds__(256)
bigram_embed_kernel(const int32_t* __restrict__ tokens, const int32_t* __restrict__ positions,
                    const int32_t* __restrict__ token_seq, const int32_t* __restrict__ q_start,
                    const int32_t* __restrict__ state_slots, int32_t* __restrict__ state, const TE* __restrict__ table,
                    int vocab, const TE* __restrict__ pairs, int buckets, long long mul_prev, long long mul_cur,
                    float scale, float* __restrict__ x, size_t copy_stride, int S, int W) {
  const int t = blockIdx.x;
  const int tok = tokens[t];
  const int before = t > 0 ? tokens[t - 1] : 0;      // (asked for beside the rest; used inside an entry only)
  const int e = token_seq[t];
  const int pos = positions[t];
  const int first = q_start[e], last = q_start[e + 1] - 1;
  int prev = before;
  if (pairs && t == first) {
    int32_t* st = state + state_slots[e];
    const int32_t latest = tokens[last];
    prev = *st;
    __syncthreads();      // every thread has read the row before one of them replaces it
    if (threadIdx.x == 0) *st = latest;
  }
  const bool ok = tok >= 0 && tok < vocab;
  long long row = buckets;
  if (pairs && pos > 0) {
    row = ((long long)prev * mul_prev + (long long)tok * mul_cur) % (long long)buckets;
    if (row < 0) row += buckets;
  }
#pragma unroll 4
  for (int c = threadIdx.x; c < W; c += 256) {
    float v = __builtin_nanf("");
    if (ok) {
      v = to_f32(table[(size_t)tok * W + c]) * scale;
      if (pairs) v += to_f32(pairs[(size_t)row * W + c]);
    }
    for (int s = 0; s < S; ++s) x[s * copy_stride + (size_t)t * W + c] = v;
  }
}

extern "C" int atoma_bigram_embed(const int32_t* tokens, const int32_t* positions, const int32_t* token_seq,
                                  const int32_t* q_start, const int32_t* state_slots, int32_t* state,
                                  const void* table, int table_dtype, int vocab, const void* pairs, int buckets,
                                  long long mul_prev, long long mul_cur, float scale, float* x, int T, int S, int W,
                                  hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || S <= 0 || vocab <= 0 || (pairs && (buckets <= 0 || !state))) return ATOMA_ERR_SHAPE;
  const size_t copy_stride = (size_t)T * W;
  if (table_dtype == kF32)
    hipLaunchKernelGGL((bigram_embed_kernel<float>), dim3(T), dim3(256), 0, stream, tokens, positions, token_seq,
                       q_start, state_slots, state, (const float*)table, vocab, (const float*)pairs, buckets, mul_prev,
                       mul_cur, scale, x, copy_stride, S, W);
  else if (table_dtype == kBF16)
    hipLaunchKernelGGL((bigram_embed_kernel<bf16_t>), dim3(T), dim3(256), 0, stream, tokens, positions, token_seq,
                       q_start, state_slots, state, (const bf16_t*)table, vocab, (const bf16_t*)pairs, buckets,
                       mul_prev, mul_cur, scale, x, copy_stride, S, W);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// a [planes_a, T, W] and b [planes_b, T, W] (planes summed first), bias_a / bias_b optional rows added before the
// statistics; one workgroup a row, the row's two sums kept in LDS between the passes
template <typename TA, typename TB>
__global__ void __launch_bounds__(256)
normed_branches_kernel(const TA* __restrict__ a, int planes_a, const TB* __restrict__ b, int planes_b,
                       size_t plane_stride, const float* __restrict__ bias_a, const float* __restrict__ bias_b,
                       const float* __restrict__ wa, const float* __restrict__ wb, float eps, float scale,
                       float* __restrict__ y, int W) {
  extern __shared__ float rowbuf[];      // [2][W]
  __shared__ float scratch[4];
  const size_t t = blockIdx.x;
  float sa = 0.f, sb = 0.f;
#pragma unroll 4
  for (int c = threadIdx.x; c < W; c += 256) {
    float va = bias_a ? bias_a[c] : 0.f, vb = bias_b ? bias_b[c] : 0.f;
    for (int p = 0; p < planes_a; ++p) va += to_f32(a[p * plane_stride + t * W + c]);
    for (int p = 0; p < planes_b; ++p) vb += to_f32(b[p * plane_stride + t * W + c]);
    rowbuf[c] = va, rowbuf[W + c] = vb;
    sa = fmaf(va, va, sa), sb = fmaf(vb, vb, sb);
  }
  sa = block_sum<4>(sa, scratch);
  sb = block_sum<4>(sb, scratch);
  const float ia = 1.0f / sqrtf(sa / (float)W + eps), ib = 1.0f / sqrtf(sb / (float)W + eps);
#pragma unroll 4
  for (int c = threadIdx.x; c < W; c += 256)
    y[t * W + c] = scale * (rowbuf[c] * ia * wa[c] + rowbuf[W + c] * ib * wb[c]);
}

extern "C" int atoma_normed_branches(const void* a, int a_dtype, int planes_a, const void* b, int b_dtype, int planes_b,
                                     const float* bias_a, const float* bias_b, const float* wa, const float* wb,
                                     float eps, float scale, float* y, int T, int W, hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || planes_a <= 0 || planes_b <= 0 || (size_t)W * 8 > 150 * 1024) return ATOMA_ERR_SHAPE;
  const size_t plane_stride = (size_t)T * W, lds = (size_t)W * 8;
#define ATOMA_NB(TA, TB)                                                                                           \
  do {                                                                                                             \
    if (lds > 48 * 1024)                                                                                           \
      (void)hipFuncSetAttribute((const void*)normed_branches_kernel<TA, TB>,                                       \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                             \
    hipLaunchKernelGGL((normed_branches_kernel<TA, TB>), dim3(T), dim3(256), lds, stream, (const TA*)a, planes_a,  \
                       (const TB*)b, planes_b, plane_stride, bias_a, bias_b, wa, wb, eps, scale, y, W);            \
  } while (0)
  if (a_dtype == kF32 && b_dtype == kF32) ATOMA_NB(float, float);
  else if (a_dtype == kBF16 && b_dtype == kBF16) ATOMA_NB(bf16_t, bf16_t);
  else if (a_dtype == kF32 && b_dtype == kBF16) ATOMA_NB(float, bf16_t);
  else if (a_dtype == kBF16 && b_dtype == kF32) ATOMA_NB(bf16_t, float);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_NB
  ATOMA_LAUNCH_CHECK();
  return 0;
}
