// RMS norm whose gain is ONE number for all coordinates, in the two places a model uses it:
//   rows:   out[r] = g * x[rows[r]] / sqrt(mean(x^2) + eps)             (the norm before the output head)
//   add:    residual[t] += g * y[t] / sqrt(mean(y[t]^2) + eps)          (a norm on a sublayer's OUTPUT: the
//           sublayer's result is normalised and then added to the 32-bit residual stream), optionally with a copy
//           of the new residual row in the compute dtype, which is what the next matrix product reads.
// All arithmetic in 32-bit; the sum over a row is taken in an order that depends on the row's length alone.
#include "common.h"
#include "ginfer_amd.h"

#define SN_THREADS 256

template <typename T, typename G>
__global__ __launch_bounds__(SN_THREADS) void scalar_rmsnorm_rows_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                                          const G* __restrict__ gain,
                                                                          const int32_t* __restrict__ rows, int hidden,
                                                                          float eps) {
  __shared__ float scratch[SN_THREADS / WAVE];
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? (int64_t)rows[r] : r;
  const float* row = x + t * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += SN_THREADS) ss += row[i] * row[i];
  ss = block_sum<SN_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)hidden + eps), g = Num<G>::ld(gain);
  for (int i = threadIdx.x; i < hidden; i += SN_THREADS) Num<T>::st(out + r * hidden + i, row[i] / rms * g);
}

// Y: the sublayer's output (compute dtype); C: the dtype of the copy
template <typename Y, typename G, typename C>
__global__ __launch_bounds__(SN_THREADS) void add_scalar_rmsnorm_kernel(float* __restrict__ residual, const Y* __restrict__ y,
                                                                         const G* __restrict__ gain, C* __restrict__ copy,
                                                                         int hidden, float eps) {
  __shared__ float scratch[SN_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  const Y* row = y + t * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += SN_THREADS) {
    const float v = Num<Y>::ld(row + i);
    ss += v * v;
  }
  ss = block_sum<SN_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)hidden + eps), g = Num<G>::ld(gain);
  for (int i = threadIdx.x; i < hidden; i += SN_THREADS) {
    const float h = residual[t * hidden + i] + Num<Y>::ld(row + i) / rms * g;
    residual[t * hidden + i] = h;
    if (copy) Num<C>::st(copy + t * hidden + i, h);
  }
}

extern "C" int ga_scalar_rmsnorm_rows(void* out, const void* x, const void* gain, const void* rows, int num_rows,
                                      int hidden, float eps, int out_bf16, int gain_bf16, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  if (hidden <= 0) return -1;
  dim3 grid(num_rows), block(SN_THREADS);
#define GO(T, G) hipLaunchKernelGGL((scalar_rmsnorm_rows_kernel<T, G>), grid, block, 0, stream, (T*)out, (const float*)x, \
                                    (const G*)gain, (const int32_t*)rows, hidden, eps)
  if (out_bf16) { if (gain_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float); }
  else { if (gain_bf16) GO(float, bf16_t); else GO(float, float); }
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_add_scalar_rmsnorm(void* residual, const void* y, const void* gain, void* copy, int tokens, int hidden,
                                     float eps, int y_bf16, int gain_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 0) return -1;
  dim3 grid(tokens), block(SN_THREADS);
  // the copy, where one is wanted, is in the dtype of y
#define GO(Y, G) hipLaunchKernelGGL((add_scalar_rmsnorm_kernel<Y, G, Y>), grid, block, 0, stream, (float*)residual, \
                                    (const Y*)y, (const G*)gain, (Y*)copy, hidden, eps)
  if (y_bf16) { if (gain_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float); }
  else { if (gain_bf16) GO(float, bf16_t); else GO(float, float); }
#undef GO
  return GA_CHECK_LAUNCH();
}
