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
//   lightning_chunk  entries of many tokens on the matrix cores, 64 tokens at a time (its own text below).
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
                      int dim, int vdim, int below) {
  extern __shared__ float lds[];      // q [16][dim], k [16][dim], v [16][16], the state's tile [16][dim]
  float* qs = lds;
  float* ks = lds + kLtTokens * dim;
  float* vs = ks + kLtTokens * dim;
  const int e = blockIdx.y;
  const int vblocks = (vdim + 15) / 16;
  const int h = blockIdx.x / vblocks, vb = blockIdx.x % vblocks;
  const int t0 = q_start[e], t1 = q_start[e + 1];
  if (t1 <= t0 || (below > 0 && t1 - t0 >= below)) return;      // (longer entries are the chunked kernel's)
  const int col = threadIdx.x >> 4, part = threadIdx.x & 15;      // column of the block, share of its rows
  const int j = vb * 16 + col;
  const bool live = j < vdim;
  const int rows = (dim + 15) / 16;
  // The workgroup's columns of S are one stretch of memory (a column's rows are contiguous, and so are neighbouring
  // columns): it is copied through LDS, 16 bytes a lane, so that the loads and stores of the state, which are most of
  // what a decoded token moves, are whole cache lines; the lanes then pick their rows (part, part + 16, ...) from LDS.
  float* stile = state + ((size_t)state_slots[e] * heads + h) * (size_t)vdim * dim + (size_t)vb * 16 * dim;
  const int cols_live = vdim - vb * 16 < 16 ? vdim - vb * 16 : 16;
  const int tile_n = cols_live * dim;
  float* sbuf = vs + kLtTokens * 16;                     // [16][dim]
  const bool vec = (dim & 3) == 0 && (((uintptr_t)stile) & 15) == 0;
  if (vec) {
    for (int i = threadIdx.x * 4; i < tile_n; i += 1024)
      *reinterpret_cast<float4*>(sbuf + i) = *reinterpret_cast<const float4*>(stile + i);
  } else {
    for (int i = threadIdx.x; i < tile_n; i += 256) sbuf[i] = stile[i];
  }
  __syncthreads();
  float s[kLtMaxRows];
#pragma unroll
  for (int i = 0; i < kLtMaxRows; ++i) {
    const int r = part + 16 * i;
    s[i] = (live && i < rows && r < dim) ? sbuf[col * dim + r] : 0.f;
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
  __syncthreads();
  if (live) {
#pragma unroll
    for (int i = 0; i < kLtMaxRows; ++i) {
      const int r = part + 16 * i;
      if (i < rows && r < dim) sbuf[col * dim + r] = s[i];
    }
  }
  __syncthreads();
  if (vec) {
    for (int i = threadIdx.x * 4; i < tile_n; i += 1024)
      *reinterpret_cast<float4*>(stile + i) = *reinterpret_cast<const float4*>(sbuf + i);
  } else {
    for (int i = threadIdx.x; i < tile_n; i += 256) stile[i] = sbuf[i];
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Entries of many tokens, 64 tokens at a time on the matrix cores (v_mfma_f32_16x16x32_bf16, float32 sums).  With S0
// the state before a chunk of n tokens and i, j the places inside it,
//
//   o_i = lambda^(i+1) S0^T q_i + sum_(j <= i) lambda^(i-j) (q_i . k_j) v_j,
//   S_n = lambda^n S0 + sum_j lambda^(n-1-j) k_j v_j^T;
//
// every exponent is at least zero, so nothing overflows and no inverse of a decay is needed.  q, k, v enter as
// bfloat16 (they are activations of projections); whatever is float32 by nature and has to be an operand of a matrix
// instruction (the state, the weighted scores, the weighted keys) is split into two bfloat16 terms hi + lo, which
// keeps 16 bits of mantissa, and all sums are float32.  The state itself stays in float32 registers across the chunks.
// A workgroup owns (entry, head, 32 columns of S); its four waves share the chunk's operands through LDS:
//   Q, K [64][dim] row-major; Kt = weighted K transposed [dim][64] (hi, lo); Vt = V transposed [32][64];
//   P = weighted scores [64][64] (hi, lo); St = S transposed [32][dim] (hi, lo).
// Rows are padded by 16 bytes so that the 16 rows a fragment load touches fall into different banks.
// The matrix instruction as used here: D[m][n] += sum_k A[m][k] B[n][k]; a lane hands in A[m = lane % 16][8 values of
// k from (lane / 16) * 8] and B[n = lane % 16][the same k], and holds D[m = (lane / 16) * 4 + r][n = lane % 16].
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kChunk = 64, kPad = 8, kCols = 32;

// (the chunked kernel's conversions are the hardware's round-to-nearest-even ones, and its SiLU uses the fast
// exponential and reciprocal: its results are rounded to bfloat16 at once)
__device__ __forceinline__ uint16_t bf16_of(float x) {
  const __bf16 b = static_cast<__bf16>(x);
  return __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ float silu_fast(float x) { return x * __frcp_rn(1.0f + __expf(-x)); }
__device__ __forceinline__ uint16_t hi_of(float x) { return bf16_of(x); }
__device__ __forceinline__ uint16_t lo_of(float x, uint16_t hi) { return bf16_of(x - bf16_bits_to_f32(hi)); }
__device__ __forceinline__ float pow_int(float l2, int n) { return n == 0 ? 1.0f : exp2f(l2 * (float)n); }
__device__ __forceinline__ bf16x8 frag(const uint16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

template <int DIM>
__global__ void __launch_bounds__(256)
lightning_chunk_kernel(const float* __restrict__ proj, int ld, int off_q, int off_k, int off_v,
                       const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                       float* __restrict__ state, const float* __restrict__ decay, float* __restrict__ o, int heads,
                       int vdim, int at_least) {
  constexpr int QS = DIM + kPad, TS = kChunk + kPad;      // row strides in elements
  constexpr int CT = DIM / 16;                            // 16-column tiles of S^T's columns (key channels)
  constexpr int TPW = (CT + 3) / 4;                       // ... of which a wave owns this many
  extern __shared__ uint16_t sm[];
  uint16_t* Qs = sm;                                      // [64][QS]
  uint16_t* Ks = Qs + kChunk * QS;                        // [64][QS]
  uint16_t* Kth = Ks + kChunk * QS;                       // [DIM][TS]
  uint16_t* Ktl = Kth + DIM * TS;
  uint16_t* Vt = Ktl + DIM * TS;                          // [32][TS]
  uint16_t* Ph = Vt + kCols * TS;                         // [64][TS]
  uint16_t* Pl = Ph + kChunk * TS;
  uint16_t* Sh = Pl + kChunk * TS;                        // [32][QS]
  uint16_t* Sl = Sh + kCols * QS;
  const int e = blockIdx.y;
  const int vblocks = (vdim + kCols - 1) / kCols;
  const int h = blockIdx.x / vblocks, v0 = (blockIdx.x % vblocks) * kCols;
  const int t0 = q_start[e], t1 = q_start[e + 1];
  if (t1 - t0 < at_least || t1 <= t0) return;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, r16 = lane & 15, kg = lane >> 4;
  const float dec = decay[h], l2 = log2f(dec);
  float* srow = state + ((size_t)state_slots[e] * heads + h) * (size_t)vdim * DIM;
  // the wave's share of S^T [v][c]: tiles (vt, ct), a lane holds c = ct * 16 + r16 and v = vt * 16 + 4 kg + r
  f32x4 sacc[TPW][2];
#pragma unroll
  for (int x = 0; x < TPW; ++x) {
    const int ct = w * TPW + x;
#pragma unroll
    for (int vt = 0; vt < 2; ++vt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int v = v0 + vt * 16 + 4 * kg + r, c = ct * 16 + r16;
        const float sv = (ct < CT && v < vdim) ? srow[(size_t)v * DIM + c] : 0.f;
        sacc[x][vt][r] = sv;
        if (ct < CT) {
          const uint16_t hh = hi_of(sv);
          Sh[(vt * 16 + 4 * kg + r) * QS + c] = hh;
          Sl[(vt * 16 + 4 * kg + r) * QS + c] = lo_of(sv, hh);
        }
      }
  }
  // A chunk's q, k, v are asked for a chunk ahead and wait in registers: 4 neighbouring columns of q and of k per
  // load, DIM / 16 loads of each a thread, and 8 values of v.
  constexpr int NQ = DIM / 16, NV = kChunk * kCols / 256, RT = DIM / 4;      // RT: threads a row of q
  float4 rq[NQ], rk[NQ];
  float rv[NV];
  auto ask = [&](int tb, int n) {
#pragma unroll
    for (int it = 0; it < NQ; ++it) {
      const int idx = threadIdx.x + 256 * it, j = idx / RT, c = (idx % RT) * 4;
      const float* row = proj + (size_t)(tb + (j < n ? j : n - 1)) * ld + h * DIM + c;
      rq[it] = *reinterpret_cast<const float4*>(row + off_q);
      rk[it] = *reinterpret_cast<const float4*>(row + off_k);
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = threadIdx.x + 256 * it, j = idx / kCols, v = idx % kCols;
      rv[it] = v0 + v < vdim ? proj[(size_t)(tb + (j < n ? j : n - 1)) * ld + off_v + h * vdim + v0 + v] : 0.f;
    }
  };
  ask(t0, t1 - t0 < kChunk ? t1 - t0 : kChunk);
  for (int tb = t0; tb < t1; tb += kChunk) {
    const int n = t1 - tb < kChunk ? t1 - tb : kChunk;
    __syncthreads();      // the chunk before is done with the operands, and S^T of its end is in LDS
    // q, k: SiLU, bfloat16; the weighted keys transposed.  v transposed.  Tokens beyond n are zeros.
#pragma unroll
    for (int it = 0; it < NQ; ++it) {
      const int idx = threadIdx.x + 256 * it, j = idx / RT, c = (idx % RT) * 4;
      const float qa[4] = {rq[it].x, rq[it].y, rq[it].z, rq[it].w}, ka[4] = {rk[it].x, rk[it].y, rk[it].z, rk[it].w};
      const float wj = j < n ? pow_int(l2, n - 1 - j) : 0.f;
      uint16_t qb[4], kb[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        qb[x] = bf16_of(j < n ? silu_fast(qa[x]) : 0.f);
        kb[x] = bf16_of(j < n ? silu_fast(ka[x]) : 0.f);
        const float kw = bf16_bits_to_f32(kb[x]) * wj;
        const uint16_t hh = hi_of(kw);
        Kth[(c + x) * TS + j] = hh;
        Ktl[(c + x) * TS + j] = lo_of(kw, hh);
      }
      *reinterpret_cast<uint2*>(Qs + j * QS + c) = make_uint2(qb[0] | ((uint32_t)qb[1] << 16), qb[2] | ((uint32_t)qb[3] << 16));
      *reinterpret_cast<uint2*>(Ks + j * QS + c) = make_uint2(kb[0] | ((uint32_t)kb[1] << 16), kb[2] | ((uint32_t)kb[3] << 16));
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = threadIdx.x + 256 * it, j = idx / kCols, v = idx % kCols;
      Vt[v * TS + j] = bf16_of((j < n && v0 + v < vdim) ? silu_fast(rv[it]) : 0.f);
    }
    if (tb + kChunk < t1) ask(tb + kChunk, t1 - tb - kChunk < kChunk ? t1 - tb - kChunk : kChunk);
    __syncthreads();
    // weighted scores of the wave's 16 tokens i against the keys j <= i: D[j][i] with A = K, B = Q
    const int i_in = w * 16 + r16;                       // the token this lane holds in every tile below
    for (int jt = 0; jt < 4; ++jt) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      if (jt <= w) {
#pragma unroll
        for (int ks = 0; ks < DIM / 32; ++ks)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(frag(Ks + (jt * 16 + r16) * QS + ks * 32 + kg * 8),
                                                        frag(Qs + (w * 16 + r16) * QS + ks * 32 + kg * 8), acc, 0, 0, 0);
      }
      uint16_t ph[4], pl[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = jt * 16 + 4 * kg + r;
        const float pv = (jt <= w && j <= i_in) ? acc[r] * pow_int(l2, i_in - j) : 0.f;
        ph[r] = hi_of(pv);
        pl[r] = lo_of(pv, ph[r]);
      }
      *reinterpret_cast<uint2*>(Ph + i_in * TS + jt * 16 + 4 * kg) =
          make_uint2(ph[0] | ((uint32_t)ph[1] << 16), ph[2] | ((uint32_t)ph[3] << 16));
      *reinterpret_cast<uint2*>(Pl + i_in * TS + jt * 16 + 4 * kg) =
          make_uint2(pl[0] | ((uint32_t)pl[1] << 16), pl[2] | ((uint32_t)pl[3] << 16));
    }
    // what the state before the chunk gives: D[v][i] with A = S^T, B = Q, times lambda^(i + 1)
    f32x4 oacc[2];
#pragma unroll
    for (int vt = 0; vt < 2; ++vt) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DIM / 32; ++ks) {
        const bf16x8 qf = frag(Qs + (w * 16 + r16) * QS + ks * 32 + kg * 8);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(frag(Sh + (vt * 16 + r16) * QS + ks * 32 + kg * 8), qf, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(frag(Sl + (vt * 16 + r16) * QS + ks * 32 + kg * 8), qf, acc, 0, 0, 0);
      }
      const float f = pow_int(l2, i_in + 1);
#pragma unroll
      for (int r = 0; r < 4; ++r) oacc[vt][r] = acc[r] * f;
    }
    __syncthreads();      // the scores are in LDS, and every wave has read S^T
    // the chunk's own tokens: D[v][i] += sum_j V^T[v][j] P[i][j]
#pragma unroll
    for (int vt = 0; vt < 2; ++vt) {
      for (int s = 0; s < 2; ++s) {
        if (2 * s > w) continue;                         // keys behind the wave's tokens
        const bf16x8 vf = frag(Vt + (vt * 16 + r16) * TS + s * 32 + kg * 8);
        oacc[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, frag(Ph + (w * 16 + r16) * TS + s * 32 + kg * 8), oacc[vt], 0, 0, 0);
        oacc[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, frag(Pl + (w * 16 + r16) * TS + s * 32 + kg * 8), oacc[vt], 0, 0, 0);
      }
      if (i_in < n) {
        float* dst = o + (size_t)(tb + i_in) * heads * vdim + h * vdim + v0 + vt * 16 + 4 * kg;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (v0 + vt * 16 + 4 * kg + r < vdim) dst[r] = oacc[vt][r];
      }
    }
    // the state behind the chunk: S^T[v][c] = lambda^n S^T[v][c] + sum_j V^T[v][j] Kt[c][j]
    const float fn = pow_int(l2, n);
#pragma unroll
    for (int x = 0; x < TPW; ++x) {
      const int ct = w * TPW + x;
      if (ct >= CT) continue;
#pragma unroll
      for (int vt = 0; vt < 2; ++vt) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const bf16x8 vf = frag(Vt + (vt * 16 + r16) * TS + s * 32 + kg * 8);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, frag(Kth + (ct * 16 + r16) * TS + s * 32 + kg * 8), acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, frag(Ktl + (ct * 16 + r16) * TS + s * 32 + kg * 8), acc, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float sv = fmaf(fn, sacc[x][vt][r], acc[r]);
          sacc[x][vt][r] = sv;
          const uint16_t hh = hi_of(sv);
          Sh[(vt * 16 + 4 * kg + r) * QS + ct * 16 + r16] = hh;
          Sl[(vt * 16 + 4 * kg + r) * QS + ct * 16 + r16] = lo_of(sv, hh);
        }
      }
    }
  }
#pragma unroll
  for (int x = 0; x < TPW; ++x) {
    const int ct = w * TPW + x;
    if (ct >= CT) continue;
#pragma unroll
    for (int vt = 0; vt < 2; ++vt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int v = v0 + vt * 16 + 4 * kg + r;
        if (v < vdim) srow[(size_t)v * DIM + ct * 16 + r16] = sacc[x][vt][r];
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
  // (unrolled: a thread's loads of a row are in flight together, which is what a step of few tokens waits for)
#pragma unroll 8
  for (int c = threadIdx.x; c < n; c += 256) ss = fmaf(o[t * n + c], o[t * n + c], ss);
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
#pragma unroll 8
  for (int c = threadIdx.x; c < n; c += 256) {
    const float g = 1.0f / (1.0f + expf(-proj[t * ld + off_g + c]));
    y[t * n + c] = from_f32<TO>(o[t * n + c] * inv * w[c] * g);
  }
}

static size_t chunk_lds(int dim) {
  const size_t qs = dim + kPad, ts = kChunk + kPad;
  return 2 * (2 * kChunk * qs + 2 * (size_t)dim * ts + kCols * ts + 2 * kChunk * ts + 2 * kCols * qs) / 2;
}

// chunked != 0: entries of at least `chunked` tokens run on the matrix cores (key sizes 32, 64, 96, 128 and decays
// above zero only; the caller checks), the shorter ones token by token; 0: every entry token by token.  run_scan == 0:
// the caller knows that no entry is shorter than `chunked` tokens, and the walk token by token is not launched.
extern "C" int atoma_lightning_scan(const float* proj, int ld, int off_q, int off_k, int off_v, const int32_t* q_start,
                                    const int32_t* state_slots, float* state, const float* decay, float* o,
                                    int n_entries, int heads, int dim, int vdim, int chunked, int run_scan,
                                    hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (heads <= 0 || dim <= 0 || dim > 16 * kLtMaxRows || vdim <= 0 || n_entries > 65535 || off_q < 0 || off_k < 0 ||
      off_v < 0 || ld < off_q + heads * dim || ld < off_k + heads * dim || ld < off_v + heads * vdim || chunked < 0 ||
      (chunked && (dim % 32 || dim > 128)))
    return ATOMA_ERR_SHAPE;
  const size_t lds = (size_t)(2 * kLtTokens * dim + kLtTokens * 16 + 16 * dim) * sizeof(float);
  dim3 grid(heads * ((vdim + 15) / 16), n_entries);
  if (run_scan || !chunked)
    hipLaunchKernelGGL(lightning_scan_kernel, grid, dim3(256), lds, stream, proj, ld, off_q, off_k, off_v, q_start,
                       state_slots, state, decay, o, heads, dim, vdim, chunked);
  if (chunked) {
    const size_t clds = chunk_lds(dim) * sizeof(uint16_t);
    dim3 cgrid(heads * ((vdim + kCols - 1) / kCols), n_entries);
#define ATOMA_LC(D)                                                                                                  \
  do {                                                                                                               \
    (void)hipFuncSetAttribute((const void*)lightning_chunk_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize,    \
                              (int)clds);                                                                            \
    hipLaunchKernelGGL((lightning_chunk_kernel<D>), cgrid, dim3(256), clds, stream, proj, ld, off_q, off_k, off_v,   \
                       q_start, state_slots, state, decay, o, heads, vdim, chunked);                                 \
  } while (0)
    if (dim == 32) ATOMA_LC(32);
    else if (dim == 64) ATOMA_LC(64);
    else if (dim == 96) ATOMA_LC(96);
    else ATOMA_LC(128);
#undef ATOMA_LC
  }
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
