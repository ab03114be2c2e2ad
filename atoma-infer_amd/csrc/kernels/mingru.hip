// A gated recurrence whose gates read the current token only (the minGRU form): per channel
//
//   z = sigmoid(pz + bz),   u = px + bx,   c = u + 1/2 (u >= 0) or sigmoid(u) (u < 0),
//   S <- (1 - z) S + z c,   y = S * silu(pg),
//
// with pz, px, pg the token's columns of one fused projection.  Gates, candidate and S are float32; a request's S is a
// row of the state tensor, read before an entry's first token and written after its last, so that prompts, portions
// and decoded tokens are one code path and a request may be cut anywhere.
//
//   mingru_scan     a thread a (entry, channel): the entry's tokens in order, four tokens' inputs asked for at a time.
//                   Decoded tokens and short portions.
//   long entries    S_t = a_t S_(t-1) + b_t (a = 1 - z, b = z c) is linear in S, so a stretch of tokens acts on S as
//                   (A, B) = (prod a, the stretch run from zero).  mingru_stretch gives every (stretch, channel) its
//                   pair; mingru_carry walks an entry's stretches in order, S_in of each stretch written out;
//                   mingru_apply runs every stretch again from its S_in and writes y.  The tokens are read twice and
//                   the work is spread over (tokens / stretch) x channels threads where the plain walk has only one
//                   thread a channel.
#include "common.h"

using namespace atoma;

struct Gates {
  float a, b;
};

__device__ __forceinline__ float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ Gates gates_of(float pz, float px) {
  const float z = sigmoidf(pz);
  const float c = px >= 0.f ? px + 0.5f : sigmoidf(px);
  return Gates{1.0f - z, z * c};
}

template <typename TO>
__global__ void __launch_bounds__(256)
mingru_scan_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ bz, const float* __restrict__ bx,
                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                   float* __restrict__ state, TO* __restrict__ y, int ldy, int width, int off_x, int off_g) {
  const int e = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int t0 = q_start[e], t1 = q_start[e + 1];
  if (t1 <= t0) return;
  float* srow = state + (size_t)state_slots[e] * width;
  float s = srow[c];
  const float bzc = bz[c], bxc = bx[c];
  for (int t = t0; t < t1; t += 4) {
    float pz[4], px[4], pg[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int tt = t + j < t1 ? t + j : t1 - 1;
      const float* row = proj + (size_t)tt * ld;
      pz[j] = row[c], px[j] = row[off_x + c], pg[j] = row[off_g + c];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (t + j < t1) {
        const Gates g = gates_of(pz[j] + bzc, px[j] + bxc);
        s = g.a * s + g.b;
        y[(size_t)(t + j) * ldy + c] = from_f32<TO>(s * pg[j] * sigmoidf(pg[j]));
      }
    }
  }
  srow[c] = s;
}

// stretch r of the step covers the tokens [r * len, (r + 1) * len) cut to its entry: the host lists (entry, first
// token, end) per stretch in `stretches` [n][3], an entry's stretches in order and side by side
__global__ void __launch_bounds__(256)
mingru_stretch_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ bz,
                      const float* __restrict__ bx, const int32_t* __restrict__ stretches, float* __restrict__ ab,
                      int width, int off_x) {
  const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int t0 = stretches[3 * r + 1], t1 = stretches[3 * r + 2];
  const float bzc = bz[c], bxc = bx[c];
  float a = 1.0f, b = 0.f;
  for (int t = t0; t < t1; t += 4) {
    float pz[4], px[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int tt = t + j < t1 ? t + j : t1 - 1;
      const float* row = proj + (size_t)tt * ld;
      pz[j] = row[c], px[j] = row[off_x + c];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (t + j < t1) {
        const Gates g = gates_of(pz[j] + bzc, px[j] + bxc);
        a *= g.a;
        b = g.a * b + g.b;
      }
    }
  }
  ab[((size_t)r * 2) * width + c] = a;
  ab[((size_t)r * 2 + 1) * width + c] = b;
}

// a thread a (entry, channel): S before each of the entry's stretches replaces the stretch's A, the state row takes
// S behind the last
__global__ void __launch_bounds__(256)
mingru_carry_kernel(float* __restrict__ ab, const int32_t* __restrict__ first_stretch,
                    const int32_t* __restrict__ state_slots, float* __restrict__ state, int width) {
  const int e = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int r0 = first_stretch[e], r1 = first_stretch[e + 1];
  if (r1 <= r0) return;
  float* srow = state + (size_t)state_slots[e] * width;
  float s = srow[c];
  for (int r = r0; r < r1; ++r) {
    const float a = ab[((size_t)r * 2) * width + c], b = ab[((size_t)r * 2 + 1) * width + c];
    ab[((size_t)r * 2) * width + c] = s;
    s = a * s + b;
  }
  srow[c] = s;
}

template <typename TO>
__global__ void __launch_bounds__(256)
mingru_apply_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ bz, const float* __restrict__ bx,
                    const int32_t* __restrict__ stretches, const float* __restrict__ ab, TO* __restrict__ y, int ldy,
                    int width, int off_x, int off_g) {
  const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int t0 = stretches[3 * r + 1], t1 = stretches[3 * r + 2];
  const float bzc = bz[c], bxc = bx[c];
  float s = ab[((size_t)r * 2) * width + c];
  for (int t = t0; t < t1; t += 4) {
    float pz[4], px[4], pg[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int tt = t + j < t1 ? t + j : t1 - 1;
      const float* row = proj + (size_t)tt * ld;
      pz[j] = row[c], px[j] = row[off_x + c], pg[j] = row[off_g + c];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (t + j < t1) {
        const Gates g = gates_of(pz[j] + bzc, px[j] + bxc);
        s = g.a * s + g.b;
        y[(size_t)(t + j) * ldy + c] = from_f32<TO>(s * pg[j] * sigmoidf(pg[j]));
      }
    }
  }
}

static bool sizes_ok(int ld, int ldy, int width, int off_x, int off_g) {
  return width > 0 && off_x >= width && off_g >= off_x + width && ld >= off_g + width && ldy >= width;
}

extern "C" int atoma_mingru_scan(const float* proj, int ld, const float* bz, const float* bx, const int32_t* q_start,
                                 const int32_t* state_slots, float* state, void* y, int y_dtype, int ldy,
                                 int n_entries, int width, int off_x, int off_g, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (!sizes_ok(ld, ldy, width, off_x, off_g) || n_entries > 65535) return ATOMA_ERR_SHAPE;
  dim3 grid((width + 255) / 256, n_entries), block(256);
  if (y_dtype == kF32)
    hipLaunchKernelGGL((mingru_scan_kernel<float>), grid, block, 0, stream, proj, ld, bz, bx, q_start, state_slots,
                       state, (float*)y, ldy, width, off_x, off_g);
  else if (y_dtype == kBF16)
    hipLaunchKernelGGL((mingru_scan_kernel<bf16_t>), grid, block, 0, stream, proj, ld, bz, bx, q_start, state_slots,
                       state, (bf16_t*)y, ldy, width, off_x, off_g);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// stretches [n_stretches][3] and first_stretch [n_entries + 1] on the device; ab: float32 [n_stretches][2][width]
extern "C" int atoma_mingru_stretched(const float* proj, int ld, const float* bz, const float* bx,
                                      const int32_t* stretches, int n_stretches, const int32_t* first_stretch,
                                      const int32_t* state_slots, float* state, float* ab, void* y, int y_dtype,
                                      int ldy, int n_entries, int width, int off_x, int off_g, hipStream_t stream) {
  if (n_entries <= 0 || n_stretches <= 0) return 0;
  if (!sizes_ok(ld, ldy, width, off_x, off_g) || n_entries > 65535 || n_stretches > 65535) return ATOMA_ERR_SHAPE;
  if (y_dtype != kF32 && y_dtype != kBF16) return ATOMA_ERR_DTYPE;
  const dim3 block(256), per_stretch((width + 255) / 256, n_stretches), per_entry((width + 255) / 256, n_entries);
  hipLaunchKernelGGL(mingru_stretch_kernel, per_stretch, block, 0, stream, proj, ld, bz, bx, stretches, ab, width,
                     off_x);
  hipLaunchKernelGGL(mingru_carry_kernel, per_entry, block, 0, stream, ab, first_stretch, state_slots, state, width);
  if (y_dtype == kF32)
    hipLaunchKernelGGL((mingru_apply_kernel<float>), per_stretch, block, 0, stream, proj, ld, bz, bx, stretches, ab,
                       (float*)y, ldy, width, off_x, off_g);
  else
    hipLaunchKernelGGL((mingru_apply_kernel<bf16_t>), per_stretch, block, 0, stream, proj, ld, bz, bx, stretches, ab,
                       (bf16_t*)y, ldy, width, off_x, off_g);
  ATOMA_LAUNCH_CHECK();
  return 0;
}
