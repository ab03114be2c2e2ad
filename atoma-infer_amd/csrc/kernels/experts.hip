// Feed-forward layers that route every token to a few of many experts.
//
//   route_topk    per token: scores = sigmoid(router logits), or their softmax over all experts, in float32; the `top`
//                 experts with the largest score + correction[expert] (no correction: the score alone; the lower
//                 index wins a tie) with their weights, score * scale (the correction chooses, it does not weigh):
//                 a (token, choice) pair is a "slot", numbered token * top + choice;
//   route_group   one workgroup: slots ordered by expert (perm), where each expert's slots start (offsets), and the
//                 list of row tiles (expert, first place in perm) that the products below walk.  Which place a slot
//                 gets inside its expert's range is not fixed; no result depends on it, since every row of a product
//                 is computed by itself;
//   expert_gemm   C[row(slot)] = (scale[slot] * A[src(slot)]) . W[expert]^T for all slots, tile by tile: true float32
//                 multiply-adds over float32 or bfloat16 operands, K in ascending order, so a row's result does not
//                 depend on the batch around it.  src is the slot's token (first product: the token's input, times its
//                 score) or the slot itself (second product); the second product writes choice c of token t to row
//                 c * T + t, so that the choices of a token lie in planes which the next norm adds in order.
//                 act = 2 squares what is positive of a result and drops the rest (experts without a gate: relu^2);
//                 out_scale[slot] multiplies a result (experts whose weight applies to their output).
#include "common.h"

using namespace atoma;

constexpr int kTileM = 64, kTileN = 64, kStepK = 16;

__global__ void __launch_bounds__(256)
route_topk_kernel(const float* __restrict__ logits, int ld, int experts, int top, int32_t* __restrict__ ids,
                  float* __restrict__ weights, int n_tokens, int softmax, const float* __restrict__ correction,
                  float scale) {
  // a wave a token; lane l holds experts l, l + 64, ...
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= n_tokens) return;
  constexpr int PER = 16;      // experts <= 1024
  // sc: what chooses (score, plus the correction where there is one); wt: what weighs (the score alone)
  float sc[PER], wt[PER];
  if (softmax) {
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + j * 64;
      wt[j] = e < experts ? logits[(size_t)t * ld + e] : -INFINITY;
      mx = fmaxf(mx, wt[j]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      wt[j] = lane + j * 64 < experts ? expf(wt[j] - mx) : 0.f;
      sum += wt[j];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int j = 0; j < PER; ++j) wt[j] /= sum;
  } else {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + j * 64;
      wt[j] = e < experts ? 1.0f / (1.0f + expf(-logits[(size_t)t * ld + e])) : 0.f;
    }
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + j * 64;
    sc[j] = e < experts ? (correction != nullptr ? wt[j] + correction[e] : wt[j]) : -INFINITY;
  }
  for (int c = 0; c < top; ++c) {
    float best = -INFINITY, bw = 0.f;
    int arg = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (sc[j] > best) best = sc[j], bw = wt[j], arg = lane + j * 64;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const float ow = __shfl_xor(bw, off, 64);
      const int oa = __shfl_xor(arg, off, 64);
      if (ob > best || (ob == best && oa < arg)) best = ob, bw = ow, arg = oa;
    }
    if (arg >= experts) arg = c, bw = 0.f;     // logits that are no numbers: still an expert of the layer
    if (lane == 0) {
      ids[(size_t)t * top + c] = arg;
      weights[(size_t)t * top + c] = bw * scale;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (lane + j * 64 == arg) sc[j] = -INFINITY;
  }
}

__global__ void __launch_bounds__(1024)
route_group_kernel(const int32_t* __restrict__ ids, int n_slots, int experts, int32_t* __restrict__ perm,
                   int32_t* __restrict__ offsets, int32_t* __restrict__ tiles, int max_tiles, int tile_m) {
  __shared__ int32_t counts[1024];
  __shared__ int32_t cursor[1024];
  for (int e = threadIdx.x; e < experts; e += 1024) counts[e] = 0;
  __syncthreads();
  for (int s = threadIdx.x; s < n_slots; s += 1024) atomicAdd(&counts[ids[s]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, n = 0;
    for (int e = 0; e < experts; ++e) {
      offsets[e] = at;
      cursor[e] = at;
      for (int r = 0; r < counts[e]; r += tile_m) {
        tiles[2 * n] = e;
        tiles[2 * n + 1] = at + r;
        ++n;
      }
      at += counts[e];
    }
    offsets[experts] = at;
    for (; n < max_tiles; ++n) tiles[2 * n] = -1, tiles[2 * n + 1] = 0;
  }
  __syncthreads();
  for (int s = threadIdx.x; s < n_slots; s += 1024) perm[atomicAdd(&cursor[ids[s]], 1)] = s;
}

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
expert_gemm_kernel(const TA* __restrict__ a, int lda, int a_div, const float* __restrict__ scale,
                   const TW* __restrict__ w, TC* __restrict__ c, int ldc, int N, int K,
                   const int32_t* __restrict__ perm, const int32_t* __restrict__ offsets,
                   const int32_t* __restrict__ tiles, int top, int plane_rows, int act,
                   const float* __restrict__ out_scale) {
  __shared__ float as[kStepK][kTileM + 4];
  __shared__ float ws[kStepK][kTileN + 4];
  __shared__ int32_t slot_of[kTileM];
  const int e = tiles[2 * blockIdx.y];
  if (e < 0) return;
  const int row0 = tiles[2 * blockIdx.y + 1], row_end = offsets[e + 1];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int n0 = blockIdx.x * kTileN;
  if (tid < kTileM) slot_of[tid] = row0 + tid < row_end ? perm[row0 + tid] : -1;
  __syncthreads();
  const TW* we = w + (size_t)e * N * K;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += kStepK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int el = tid + i * 256;
      const int r = el >> 4, kk = el & 15, k = k0 + kk;
      const int slot = slot_of[r];
      float av = 0.f;
      if (slot >= 0 && k < K) {
        av = to_f32(a[(size_t)(slot / a_div) * lda + k]);
        if (scale) av *= scale[slot];
      }
      as[kk][r] = av;
      ws[kk][r] = (n0 + r < N && k < K) ? to_f32(we[(size_t)(n0 + r) * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kStepK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int slot = slot_of[ty * 4 + i];
    if (slot < 0) continue;
    const size_t row = plane_rows > 0 ? (size_t)(slot % top) * plane_rows + slot / top : (size_t)slot;
    const float os = out_scale != nullptr ? out_scale[slot] : 1.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      float v = acc[i][j];
      if (act == 2) v = v > 0.f ? v * v : 0.f;
      if (n < N) c[row * ldc + n] = from_f32<TC>(v * os);
    }
  }
}

// ---- bfloat16 on the matrix cores -------------------------------------------------------------------------------
//
//   gather_scale      xs[place] = bfloat16(score[slot] * x[token of slot]) for every place of perm: the inputs of the
//                     first product, ordered by expert, so that a tile's rows are contiguous;
//   expert_gemm_mfma  a workgroup takes a tile of up to 64 places of one expert against 128 rows of that expert's
//                     weight, v_mfma_f32_16x16x32_bf16 with float32 sums: the weight's fragments come straight from
//                     global memory (an element is used by one wave only), the tile of activations passes LDS, 64
//                     columns of K at a time, and is shared by the four waves; both are asked for a step ahead.  Tiles
//                     hold 64 places, or 128 where the experts have many (prompts).  With few places an expert (decode
//                     steps) the blocks of 16 places without a live one are skipped and the product streams the
//                     weight once.  SWIGLU: the weight's rows come in blocks of 16 gate rows followed by the 16 up
//                     rows of the same outputs, a lane then holds a gate value and its up value, and silu(gate) * up
//                     leaves as bfloat16 [places, ff]; else the float32 result goes to the plane and row of the
//                     place's slot (choice c of token t: row c * T + t).
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__global__ void __launch_bounds__(256)
gather_scale_kernel(const uint16_t* __restrict__ x, int ldx, const float* __restrict__ score,
                    const int32_t* __restrict__ perm, uint16_t* __restrict__ xs, int K, int top) {
  const int place = blockIdx.x, slot = perm[place];
  const float sc = score != nullptr ? score[slot] : 1.0f;      // (no scores: the inputs as they are)
  const uint16_t* src = x + (size_t)(slot / top) * ldx;
  for (int k = threadIdx.x; k < K; k += 256) xs[(size_t)place * K + k] = f32_to_bf16_bits(bf16_bits_to_f32(src[k]) * sc);
}


// NS: blocks of 16 rows of the weight a wave takes.  KSUB: pieces of 32 columns of K a step (2, or 4 for tiles of 64
// places: a decode step's tile holds a place or two, the product streams the weight, and what it needs is many bytes
// in flight a step).
// ACT: 0 the float32 result (times out_scale[slot] where given) by place or by slot; 1 silu(gate) * up over interleaved
// rows, bfloat16 [places, N / 2]; 2 relu^2 of the result, bfloat16 [places, N].
template <int ACT, int TM, int NS, int KSUB>
__global__ void __launch_bounds__(256)
expert_gemm_mfma_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ w, void* __restrict__ c, int ldc,
                        int N, int K, const int32_t* __restrict__ perm, const int32_t* __restrict__ offsets,
                        const int32_t* __restrict__ tiles, int top, int plane_rows,
                        const float* __restrict__ out_scale) {
  constexpr bool SWIGLU = ACT == 1;
  constexpr int MS = TM / 16;          // blocks of 16 places a tile
  constexpr int KSTEP = 32 * KSUB;     // columns of K a step
  constexpr int kLdsRow = KSTEP + 8;   // bfloat16 elements a row of the activations' tile takes in LDS (padded)
  constexpr int SEGS = KSTEP / 8;      // 16-byte pieces a row of the tile
  constexpr int AP = TM * SEGS / 256;  // ... and a thread moves a step
  __shared__ __attribute__((aligned(16))) uint16_t at[TM * kLdsRow];
  const int e = tiles[2 * blockIdx.y];
  if (e < 0) return;
  const int row0 = tiles[2 * blockIdx.y + 1];
  const int rows = min(TM, offsets[e + 1] - row0);
  const int msub = (rows + 15) >> 4;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int n_base = blockIdx.x * (64 * NS) + wave * (16 * NS);
  // (a wave whose columns lie beyond N still joins the barriers below; its rows are clamped and never stored)
  const uint16_t* we = w + (size_t)e * N * K;
  const uint16_t* wp[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    int n = n_base + s * 16 + r16;
    if (n > N - 1) n = N - 1;
    wp[s] = we + (size_t)n * K + kg * 8;
  }
  f32x4 acc[NS][MS];
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int m = 0; m < MS; ++m) acc[s][m] = f32x4{0.f, 0.f, 0.f, 0.f};

  // The operands of a step are asked for a step ahead: the weight's fragments wait in registers, the activations' pieces
  // too, until the tile of the step before has been read and they may go to LDS.
  bf16x8 wf[KSUB][NS], wn[KSUB][NS];
  uint4 ar[AP];
  auto fetch = [&](int k0, bf16x8 (&dst)[KSUB][NS]) {
#pragma unroll
    for (int kk = 0; kk < KSUB; ++kk)
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        // (K is a multiple of 32: the last step may be short)
        if (k0 + kk * 32 < K) dst[kk][s] = *reinterpret_cast<const bf16x8*>(wp[s] + k0 + kk * 32);
        else dst[kk][s] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
#pragma unroll
    for (int i = 0; i < AP; ++i) {
      const int idx = tid + i * 256, r = idx / SEGS, seg = idx % SEGS;
      ar[i] = make_uint4(0, 0, 0, 0);
      if (r < rows && k0 + seg * 8 < K) ar[i] = *reinterpret_cast<const uint4*>(a + (size_t)(row0 + r) * K + k0 + seg * 8);
    }
  };
  fetch(0, wf);
  for (int k0 = 0; k0 < K; k0 += KSTEP) {
    __syncthreads();          // the tile of the step before has been read
#pragma unroll
    for (int i = 0; i < AP; ++i) {
      const int idx = tid + i * 256, r = idx / SEGS, seg = idx % SEGS;
      if (r < msub * 16) *reinterpret_cast<uint4*>(at + r * kLdsRow + seg * 8) = ar[i];
    }
    __syncthreads();
    if (k0 + KSTEP < K) fetch(k0 + KSTEP, wn);
#pragma unroll
    for (int kk = 0; kk < KSUB; ++kk) {
#pragma unroll
      for (int m = 0; m < MS; ++m) {
        if (m < msub) {
          const bf16x8 af = *reinterpret_cast<const bf16x8*>(at + (m * 16 + r16) * kLdsRow + kk * 32 + kg * 8);
#pragma unroll
          for (int s = 0; s < NS; ++s)
            acc[s][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[kk][s], af, acc[s][m], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int kk = 0; kk < KSUB; ++kk)
#pragma unroll
      for (int s = 0; s < NS; ++s) wf[kk][s] = wn[kk][s];
  }
  // lane: place m * 16 + r16 of the tile, columns kg * 4 .. + 3 of each of its NS blocks of 16 rows of the weight
#pragma unroll
  for (int m = 0; m < MS; ++m) {
    const int r = m * 16 + r16;
    if (m >= msub || r >= rows) continue;
    const int place = row0 + r;
    if constexpr (SWIGLU) {
#pragma unroll
      for (int s = 0; s < NS; s += 2) {        // blocks come in pairs: 16 gate rows, then their 16 up rows
        const int n0 = (n_base + s * 16) / 2 + kg * 4;      // outputs: one for every pair of a gate row and an up row
        uint16_t* dst = (uint16_t*)c + (size_t)place * ldc + n0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (n_base + s * 16 + 16 + kg * 4 + i < N) {
            const float g = acc[s][m][i];
            dst[i] = f32_to_bf16_bits(g / (1.0f + expf(-g)) * acc[s + 1][m][i]);
          }
        }
      }
    } else if constexpr (ACT == 2) {
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const int n0 = n_base + s * 16 + kg * 4;
        uint16_t* dst = (uint16_t*)c + (size_t)place * ldc + n0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float v = acc[s][m][i];
          if (n0 + i < N) dst[i] = f32_to_bf16_bits(v > 0.f ? v * v : 0.f);
        }
      }
    } else {
      const int slot = perm[place];
      const size_t row = plane_rows > 0 ? (size_t)(slot % top) * plane_rows + slot / top : (size_t)place;
      const float os = out_scale != nullptr ? out_scale[slot] : 1.0f;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const int n0 = n_base + s * 16 + kg * 4;
        float* dst = (float*)c + row * ldc + n0;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n0 + i < N) dst[i] = acc[s][m][i] * os;
      }
    }
  }
}

// out[t, i] = relu(u[t, i])^2 * sigmoid(u[t, off_gate]) for an expert that every token uses: its first product's
// result u [T, ld] holds the ff columns of the expert and, at off_gate, the token's gate (off_gate < 0: no gate).
template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
relu2_gate_kernel(const TI* __restrict__ u, int ld, TO* __restrict__ out, int ff, int off_gate) {
  const size_t t = blockIdx.x;
  const float g = off_gate >= 0 ? 1.0f / (1.0f + expf(-to_f32(u[t * ld + off_gate]))) : 1.0f;
  for (int i = threadIdx.x; i < ff; i += 256) {
    const float v = to_f32(u[t * ld + i]);
    out[t * ff + i] = from_f32<TO>(v > 0.f ? v * v * g : 0.f);
  }
}

extern "C" int atoma_relu2_gate(const void* u, int u_dtype, int ld, void* out, int out_dtype, int n_tokens, int ff,
                                int off_gate, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (ff <= 0 || ld < ff || off_gate >= ld) return ATOMA_ERR_SHAPE;
  dim3 grid(n_tokens), block(256);
  if (u_dtype == kF32 && out_dtype == kF32)
    hipLaunchKernelGGL((relu2_gate_kernel<float, float>), grid, block, 0, stream, (const float*)u, ld, (float*)out, ff,
                       off_gate);
  else if (u_dtype == kF32 && out_dtype == kBF16)
    hipLaunchKernelGGL((relu2_gate_kernel<float, bf16_t>), grid, block, 0, stream, (const float*)u, ld, (bf16_t*)out,
                       ff, off_gate);
  else if (u_dtype == kBF16 && out_dtype == kBF16)
    hipLaunchKernelGGL((relu2_gate_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (const bf16_t*)u, ld, (bf16_t*)out,
                       ff, off_gate);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_gather_scale(const void* x, int ldx, const float* score, const int32_t* perm, void* xs, int K,
                                  int top, int n_slots, hipStream_t stream) {
  if (n_slots <= 0) return 0;
  if (K <= 0 || ldx < K || top <= 0) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(gather_scale_kernel, dim3(n_slots), dim3(256), 0, stream, (const uint16_t*)x, ldx, score, perm,
                     (uint16_t*)xs, K, top);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// a [places, K] bfloat16 in the order of perm; w [experts, N, K] bfloat16.  act 1: c bfloat16 [places, N / 2] (ldc),
// the rows of w in blocks of 16 gate rows and their 16 up rows; act 2: c bfloat16 [places, N], relu^2; act 0: c
// float32, by place or (plane_rows > 0) by slot, times out_scale[slot] where given
extern "C" int atoma_expert_gemm_mfma(const void* a, const void* w, void* c, int ldc, int N, int K, const int32_t* perm,
                                      const int32_t* offsets, const int32_t* tiles, int max_tiles, int top,
                                      int plane_rows, int act, int tile_m, const float* out_scale,
                                      hipStream_t stream) {
  if (max_tiles <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 32 || N % 32 || (tile_m != 64 && tile_m != 128) || top <= 0 || max_tiles > 65535 || ((uintptr_t)a & 15) || ((uintptr_t)w & 15) ||
      act < 0 || act > 2 || ldc < (act == 1 ? N / 2 : N) || (act != 0 && (plane_rows > 0 || out_scale != nullptr)))
    return ATOMA_ERR_SHAPE;
  const int ns = 2;      // (four blocks a wave measured slower for tiles of 128 places: 467 against 336 us)
  dim3 grid((N + 64 * ns - 1) / (64 * ns), max_tiles), block(256);
#define ATOMA_EGM(SW, TM_, NS_, KSUB_)                                                                           \
  hipLaunchKernelGGL((expert_gemm_mfma_kernel<SW, TM_, NS_, KSUB_>), grid, block, 0, stream, (const uint16_t*)a, \
                     (const uint16_t*)w, c, ldc, N, K, perm, offsets, tiles, top, plane_rows, out_scale)
  if (act == 1 && tile_m == 64) ATOMA_EGM(1, 64, 2, 4);
  else if (act == 1) ATOMA_EGM(1, 128, 2, 2);
  else if (act == 2 && tile_m == 64) ATOMA_EGM(2, 64, 2, 4);
  else if (act == 2) ATOMA_EGM(2, 128, 2, 2);
  else if (tile_m == 64) ATOMA_EGM(0, 64, 2, 4);
  else ATOMA_EGM(0, 128, 2, 2);
#undef ATOMA_EGM
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_route_topk(const float* logits, int ld, int experts, int top, int32_t* ids, float* weights,
                                int n_tokens, int softmax, const float* correction, float scale, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (experts <= 0 || experts > 1024 || top <= 0 || top > experts || ld < experts) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(route_topk_kernel, dim3((n_tokens + 3) / 4), dim3(256), 0, stream, logits, ld, experts, top, ids,
                     weights, n_tokens, softmax, correction, scale);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// the most row tiles of tile_m places that n_slots slots of `experts` experts can need
extern "C" int atoma_route_max_tiles(int n_slots, int experts, int tile_m) {
  const int full = n_slots / tile_m + experts;
  return full < n_slots ? full : (n_slots > 0 ? n_slots : 1);
}

extern "C" int atoma_route_group(const int32_t* ids, int n_slots, int experts, int32_t* perm, int32_t* offsets,
                                 int32_t* tiles, int max_tiles, int tile_m, hipStream_t stream) {
  if (n_slots <= 0) return 0;
  if (experts <= 0 || experts > 1024 || (tile_m != 64 && tile_m != 128) ||
      max_tiles < atoma_route_max_tiles(n_slots, experts, tile_m))
    return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(route_group_kernel, dim3(1), dim3(1024), 0, stream, ids, n_slots, experts, perm, offsets, tiles,
                     max_tiles, tile_m);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_expert_gemm(const void* a, int a_dtype, int lda, int a_div, const float* scale, const void* w,
                                 int w_dtype, void* c, int c_dtype, int ldc, int N, int K, const int32_t* perm,
                                 const int32_t* offsets, const int32_t* tiles, int max_tiles, int top, int plane_rows,
                                 int act, const float* out_scale, hipStream_t stream) {
  if (max_tiles <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N || a_div <= 0 || top <= 0 || max_tiles > 65535 || (act != 0 && act != 2))
    return ATOMA_ERR_SHAPE;
  dim3 grid((N + kTileN - 1) / kTileN, max_tiles), block(256);
#define ATOMA_EG(TA, TW, TC)                                                                                       \
  hipLaunchKernelGGL((expert_gemm_kernel<TA, TW, TC>), grid, block, 0, stream, (const TA*)a, lda, a_div, scale,     \
                     (const TW*)w, (TC*)c, ldc, N, K, perm, offsets, tiles, top, plane_rows, act, out_scale)
  if (a_dtype == kF32 && w_dtype == kF32 && c_dtype == kF32) ATOMA_EG(float, float, float);
  else if (a_dtype == kF32 && w_dtype == kBF16 && c_dtype == kF32) ATOMA_EG(float, bf16_t, float);
  else if (a_dtype == kBF16 && w_dtype == kBF16 && c_dtype == kF32) ATOMA_EG(bf16_t, bf16_t, float);
  else if (a_dtype == kBF16 && w_dtype == kBF16 && c_dtype == kBF16) ATOMA_EG(bf16_t, bf16_t, bf16_t);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_EG
  ATOMA_LAUNCH_CHECK();
  return 0;
}
