// A gated linear recurrence per channel behind a short causal convolution (the real-gated linear recurrent unit of
// Griffin's recurrent block).  From one fused projection [y | x] of a token, with biases:
//
//   g = gelu_tanh(y + by),   xin = x + bx,   u = sum_j conv[c][j] xin(t - (taps - 1 - j)) + conv_b   (no activation)
//   r = sigmoid(Ra u + ba),  i = sigmoid(Ri u + bi)        Ra, Ri block-diagonal (made by a per-block product)
//   a = exp(-8 r softplus(lam)),   S <- a S + sqrt(1 - a^2) i u,   out = S g
//
// Everything behind the projection is float32.  A request's state row is [taps - 1][width] inputs of the convolution
// (the latest last, biases included) followed by S [width]; zero at admission, which is "zeros before the start".
//
//   rglru_conv        a thread a (token, channel): u and g.  Inputs before the entry's first token come from the state row.
//   rglru_conv_state  a thread a (entry, channel): the state's inputs for the next step.
//   rglru_scan        a thread a (entry, channel): the entry's tokens in order.
//   long entries      S_t = a_t S_(t-1) + b_t is linear in S: rglru_stretch gives every (stretch of tokens, channel)
//                     its pair (prod a, the stretch run from zero), rglru_carry walks an entry's stretches from the
//                     state row and leaves S before each, rglru_apply runs every stretch again from there.
#include "common.h"

using namespace atoma;

__device__ __forceinline__ float sigm(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

__global__ void __launch_bounds__(256)
rglru_conv_kernel(const float* __restrict__ proj, int ld, int off_y, int off_x, const float* __restrict__ by,
                  const float* __restrict__ bx, const float* __restrict__ conv, const float* __restrict__ conv_b,
                  const int32_t* __restrict__ token_seq, const int32_t* __restrict__ q_start,
                  const int32_t* __restrict__ state_slots, const float* __restrict__ state, size_t state_stride,
                  float* __restrict__ u, float* __restrict__ g, int width, int taps) {
  const int t = blockIdx.x;
  const int e = token_seq[t];
  const int i = t - q_start[e];                       // tokens of this entry before t
  const float* tail = state + (size_t)state_slots[e] * state_stride;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c < width) {
    float acc = conv_b[c];
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      float xin;
      if (back <= i) xin = proj[(size_t)(t - back) * ld + off_x + c] + bx[c];
      else xin = tail[(size_t)(taps - 1 + i - back) * width + c];
      acc = fmaf(conv[(size_t)c * taps + j], xin, acc);
    }
    u[(size_t)t * width + c] = acc;
    g[(size_t)t * width + c] = gelu_tanh_f(proj[(size_t)t * ld + off_y + c] + by[c]);
  }
}

__global__ void __launch_bounds__(256)
rglru_conv_state_kernel(const float* __restrict__ proj, int ld, int off_x, const float* __restrict__ bx,
                        const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                        float* __restrict__ state, size_t state_stride, int width, int taps) {
  const int e = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int t0 = q_start[e], n = q_start[e + 1] - t0;
  if (n <= 0) return;
  float* tail = state + (size_t)state_slots[e] * state_stride;
  // row k of the new tail is element n + k of (old tail, then the entry's inputs); rows are written in rising order
  // and each reads a row behind itself, so no row is read after it was replaced
  for (int k = 0; k < taps - 1; ++k) {
    const int m = n + k;
    tail[(size_t)k * width + c] = m < taps - 1 ? tail[(size_t)m * width + c]
                                               : proj[(size_t)(t0 + m - (taps - 1)) * ld + off_x + c] + bx[c];
  }
}

struct Step {
  float a, b;
};

// gates [T, ldg]: for block blk of bs channels, [r | i] before their biases at columns blk * 2 bs
__device__ __forceinline__ Step step_of(const float* __restrict__ gates, int ldg, const float* __restrict__ u, int t,
                                        int c, int width, int bs, float bra, float bri, float sp) {
  const int blk = c / bs, k = c % bs;
  const float* gr = gates + (size_t)t * ldg + (size_t)blk * 2 * bs;
  const float r = sigm(gr[k] + bra), i = sigm(gr[bs + k] + bri);
  // 1 - a^2 = -expm1(2 log a): exact also where a is close to one
  const float la = -8.0f * r * sp;
  const float a = expf(la);
  return Step{a, sqrtf(-expm1f(2.0f * la)) * i * u[(size_t)t * width + c]};
}

template <typename TO>
__global__ void __launch_bounds__(256)
rglru_scan_kernel(const float* __restrict__ gates, int ldg, const float* __restrict__ u, const float* __restrict__ g,
                  const float* __restrict__ ba, const float* __restrict__ bi, const float* __restrict__ sp,
                  const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                  float* __restrict__ state, size_t state_stride, size_t off_s, TO* __restrict__ out, int width,
                  int bs) {
  const int e = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int t0 = q_start[e], t1 = q_start[e + 1];
  if (t1 <= t0) return;
  float* srow = state + (size_t)state_slots[e] * state_stride + off_s;
  float s = srow[c];
  const float bra = ba[c], bri = bi[c], spc = sp[c];
  for (int t = t0; t < t1; ++t) {
    const Step st = step_of(gates, ldg, u, t, c, width, bs, bra, bri, spc);
    s = fmaf(st.a, s, st.b);
    out[(size_t)t * width + c] = from_f32<TO>(s * g[(size_t)t * width + c]);
  }
  srow[c] = s;
}

// stretches [n][3] = (entry, first token, end), an entry's stretches in order and side by side
__global__ void __launch_bounds__(256)
rglru_stretch_kernel(const float* __restrict__ gates, int ldg, const float* __restrict__ u,
                     const float* __restrict__ ba, const float* __restrict__ bi, const float* __restrict__ sp,
                     const int32_t* __restrict__ stretches, float* __restrict__ ab, int width, int bs) {
  const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int t0 = stretches[3 * r + 1], t1 = stretches[3 * r + 2];
  const float bra = ba[c], bri = bi[c], spc = sp[c];
  float a = 1.0f, b = 0.f;
  for (int t = t0; t < t1; ++t) {
    const Step st = step_of(gates, ldg, u, t, c, width, bs, bra, bri, spc);
    a *= st.a;
    b = fmaf(st.a, b, st.b);
  }
  ab[((size_t)r * 2) * width + c] = a;
  ab[((size_t)r * 2 + 1) * width + c] = b;
}

__global__ void __launch_bounds__(256)
rglru_carry_kernel(float* __restrict__ ab, const int32_t* __restrict__ first_stretch,
                   const int32_t* __restrict__ state_slots, float* __restrict__ state, size_t state_stride,
                   size_t off_s, int width) {
  const int e = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int r0 = first_stretch[e], r1 = first_stretch[e + 1];
  if (r1 <= r0) return;
  float* srow = state + (size_t)state_slots[e] * state_stride + off_s;
  float s = srow[c];
  for (int r = r0; r < r1; ++r) {
    const float a = ab[((size_t)r * 2) * width + c], b = ab[((size_t)r * 2 + 1) * width + c];
    ab[((size_t)r * 2) * width + c] = s;      // S before the stretch
    s = fmaf(a, s, b);
  }
  srow[c] = s;
}

template <typename TO>
__global__ void __launch_bounds__(256)
rglru_apply_kernel(const float* __restrict__ gates, int ldg, const float* __restrict__ u, const float* __restrict__ g,
                   const float* __restrict__ ba, const float* __restrict__ bi, const float* __restrict__ sp,
                   const int32_t* __restrict__ stretches, const float* __restrict__ ab, TO* __restrict__ out,
                   int width, int bs) {
  const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int t0 = stretches[3 * r + 1], t1 = stretches[3 * r + 2];
  const float bra = ba[c], bri = bi[c], spc = sp[c];
  float s = ab[((size_t)r * 2) * width + c];
  for (int t = t0; t < t1; ++t) {
    const Step st = step_of(gates, ldg, u, t, c, width, bs, bra, bri, spc);
    s = fmaf(st.a, s, st.b);
    out[(size_t)t * width + c] = from_f32<TO>(s * g[(size_t)t * width + c]);
  }
}

extern "C" int atoma_rglru_conv(const float* proj, int ld, int off_y, int off_x, const float* by, const float* bx,
                                const float* conv, const float* conv_b, const int32_t* token_seq,
                                const int32_t* q_start, const int32_t* state_slots, float* state, float* u, float* g,
                                int n_tokens, int n_entries, int width, int taps, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (width <= 0 || taps <= 0 || taps > 64 || off_y < 0 || off_x < 0 || ld < off_y + width || ld < off_x + width ||
      n_entries <= 0 || n_entries > 65535)
    return ATOMA_ERR_SHAPE;
  const size_t stride = (size_t)taps * width;      // taps - 1 rows of inputs, then S
  if ((width + 255) / 256 > 65535) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(rglru_conv_kernel, dim3(n_tokens, (width + 255) / 256), dim3(256), 0, stream, proj, ld, off_y, off_x, by, bx, conv,
                     conv_b, token_seq, q_start, state_slots, state, stride, u, g, width, taps);
  if (taps > 1)
    hipLaunchKernelGGL(rglru_conv_state_kernel, dim3((width + 255) / 256, n_entries), dim3(256), 0, stream, proj, ld,
                       off_x, bx, q_start, state_slots, state, stride, width, taps);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// stretches == nullptr: the plain walk.  ab: float32 [n_stretches][2][width] scratch.
extern "C" int atoma_rglru_scan(const float* gates, int ldg, const float* u, const float* g, const float* ba,
                                const float* bi, const float* sp, const int32_t* q_start, const int32_t* state_slots,
                                float* state, const int32_t* stretches, int n_stretches, const int32_t* first_stretch,
                                float* ab, void* out, int out_dtype, int n_entries, int width, int blocks, int taps,
                                hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (width <= 0 || blocks <= 0 || width % blocks || ldg < 2 * width || taps <= 0 || n_entries > 65535 ||
      n_stretches > 65535)
    return ATOMA_ERR_SHAPE;
  if (out_dtype != kF32 && out_dtype != kBF16) return ATOMA_ERR_DTYPE;
  const int bs = width / blocks;
  const size_t stride = (size_t)taps * width, off_s = (size_t)(taps - 1) * width;
  const dim3 block(256), per_entry((width + 255) / 256, n_entries);
  if (stretches == nullptr || n_stretches <= 0) {
    if (out_dtype == kF32)
      hipLaunchKernelGGL((rglru_scan_kernel<float>), per_entry, block, 0, stream, gates, ldg, u, g, ba, bi, sp, q_start,
                         state_slots, state, stride, off_s, (float*)out, width, bs);
    else
      hipLaunchKernelGGL((rglru_scan_kernel<bf16_t>), per_entry, block, 0, stream, gates, ldg, u, g, ba, bi, sp,
                         q_start, state_slots, state, stride, off_s, (bf16_t*)out, width, bs);
    ATOMA_LAUNCH_CHECK();
    return 0;
  }
  const dim3 per_stretch((width + 255) / 256, n_stretches);
  hipLaunchKernelGGL(rglru_stretch_kernel, per_stretch, block, 0, stream, gates, ldg, u, ba, bi, sp, stretches, ab,
                     width, bs);
  hipLaunchKernelGGL(rglru_carry_kernel, per_entry, block, 0, stream, ab, first_stretch, state_slots, state, stride,
                     off_s, width);
  if (out_dtype == kF32)
    hipLaunchKernelGGL((rglru_apply_kernel<float>), per_stretch, block, 0, stream, gates, ldg, u, g, ba, bi, sp,
                       stretches, ab, (float*)out, width, bs);
  else
    hipLaunchKernelGGL((rglru_apply_kernel<bf16_t>), per_stretch, block, 0, stream, gates, ldg, u, g, ba, bi, sp,
                       stretches, ab, (bf16_t*)out, width, bs);
  ATOMA_LAUNCH_CHECK();
  return 0;
}
