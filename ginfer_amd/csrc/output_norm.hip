// A norm on a sublayer's OUTPUT with a factor per channel behind it, fused with the residual add and, where the caller
// wants it, with the norm that the NEXT sublayer reads through:
//   residual[t] += s * g * y[t] / sqrt(mean(y[t]^2) + eps)                  g, s: one number per channel (s may be absent)
//   next[t]      = g2 * residual[t] / sqrt(mean(residual[t]^2) + eps2)      (optional; in the compute dtype)
// The row stays in registers between the two (up to ON_THREADS * ON_PER elements; longer rows are read again).
// All arithmetic in 32-bit; a row's sums are taken in an order that depends on its length alone.
#include "common.h"
#include "ginfer_amd.h"

#define ON_THREADS 256
#define ON_PER 16            // elements a thread keeps: rows of up to 4,096 stay in registers

template <typename Y, typename C>
__global__ __launch_bounds__(ON_THREADS) void output_norm_add_kernel(float* __restrict__ residual, const Y* __restrict__ y,
                                                                      const float* __restrict__ gain,
                                                                      const float* __restrict__ scale, float eps,
                                                                      const float* __restrict__ next_gain, float next_eps,
                                                                      C* __restrict__ next, int hidden) {
  __shared__ float scratch[ON_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  const Y* row = y + t * hidden;
  float* res = residual + t * hidden;
  const bool kept = hidden <= ON_THREADS * ON_PER;
  float v[ON_PER];
  float ss = 0.f;
  if (kept) {
#pragma unroll
    for (int j = 0; j < ON_PER; ++j) {
      const int i = threadIdx.x + j * ON_THREADS;
      v[j] = i < hidden ? Num<Y>::ld(row + i) : 0.f;
      ss += v[j] * v[j];
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += ON_THREADS) {
      const float a = Num<Y>::ld(row + i);
      ss += a * a;
    }
  }
  ss = block_sum<ON_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)hidden + eps);
  float ss2 = 0.f;
  if (kept) {
#pragma unroll
    for (int j = 0; j < ON_PER; ++j) {
      const int i = threadIdx.x + j * ON_THREADS;
      if (i < hidden) {
        float a = v[j] / rms * gain[i];
        if (scale) a *= scale[i];
        v[j] = res[i] + a;
        res[i] = v[j];
        ss2 += v[j] * v[j];
      }
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += ON_THREADS) {
      float a = Num<Y>::ld(row + i) / rms * gain[i];
      if (scale) a *= scale[i];
      const float h = res[i] + a;
      res[i] = h;
      ss2 += h * h;
    }
  }
  if (next == nullptr) return;
  ss2 = block_sum<ON_THREADS / WAVE>(ss2, scratch);
  const float rms2 = sqrtf(ss2 / (float)hidden + next_eps);
  C* out = next + t * hidden;
  if (kept) {
#pragma unroll
    for (int j = 0; j < ON_PER; ++j) {
      const int i = threadIdx.x + j * ON_THREADS;
      if (i < hidden) Num<C>::st(out + i, v[j] / rms2 * next_gain[i]);
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += ON_THREADS) Num<C>::st(out + i, res[i] / rms2 * next_gain[i]);   // this thread's own stores
  }
}

extern "C" int ga_output_norm_add(void* residual, const void* y, const void* gain, const void* scale, float eps,
                                  const void* next_gain, float next_eps, void* next, int tokens, int hidden, int y_bf16,
                                  int next_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 0 || !gain) return -1;
  if (next && !next_gain) return -2;
  dim3 grid(tokens), block(ON_THREADS);
#define GO(Y, C) hipLaunchKernelGGL((output_norm_add_kernel<Y, C>), grid, block, 0, stream, (float*)residual, (const Y*)y, \
                                    (const float*)gain, (const float*)scale, eps, (const float*)next_gain, next_eps,       \
                                    (C*)next, hidden)
  if (y_bf16) { if (next_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float); }
  else { if (next_bf16) GO(float, bf16_t); else GO(float, float); }
#undef GO
  return GA_CHECK_LAUNCH();
}
