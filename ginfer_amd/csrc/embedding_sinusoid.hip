// Token embedding plus a sinusoidal position vector, then a norm with one gain:
//   e[2i] = table[id][2i] + sin(p * freq[i]),  e[2i+1] = table[id][2i+1] + cos(p * freq[i]),
//   out = g * e / sqrt(mean(e^2) + eps)
// The angle is a 32-bit product of the position and a 32-bit frequency (the table comes from the host); sine and
// cosine are the accurate ones (full range reduction).  Output: the 32-bit residual stream.
#include "common.h"
#include "ginfer_amd.h"

#define ES_THREADS 256

template <typename T, typename G>
__global__ __launch_bounds__(ES_THREADS) void embedding_sinusoid_norm_kernel(float* __restrict__ out, const T* __restrict__ table,
                                                                              const int32_t* __restrict__ ids,
                                                                              const int32_t* __restrict__ positions,
                                                                              const float* __restrict__ freq,
                                                                              const G* __restrict__ gain, int hidden, float eps,
                                                                              int normed) {
  __shared__ float scratch[ES_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  const T* row = table + (int64_t)ids[t] * hidden;
  const float p = (float)positions[t];
  float* o = out + t * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += ES_THREADS) {
    const float a = p * freq[i >> 1];
    const float e = Num<T>::ld(row + i) + ((i & 1) ? cosf(a) : sinf(a));
    o[i] = e;
    ss += e * e;
  }
  if (!normed) return;
  ss = block_sum<ES_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)hidden + eps), g = Num<G>::ld(gain);
  for (int i = threadIdx.x; i < hidden; i += ES_THREADS) o[i] = o[i] / rms * g;     // a thread reads what it wrote itself
}

extern "C" int ga_embedding_sinusoid_norm(void* out, const void* table, const void* ids, const void* positions,
                                          const void* freq, const void* gain, int tokens, int hidden, float eps,
                                          int table_bf16, int gain_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 0) return -1;
  dim3 grid(tokens), block(ES_THREADS);
  const int normed = gain != nullptr;
#define GO(T, G) hipLaunchKernelGGL((embedding_sinusoid_norm_kernel<T, G>), grid, block, 0, stream, (float*)out, \
                                    (const T*)table, (const int32_t*)ids, (const int32_t*)positions, (const float*)freq, \
                                    (const G*)gain, hidden, eps, normed)
  if (table_bf16) { if (gain_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float); }
  else { if (gain_bf16) GO(float, bf16_t); else GO(float, float); }
#undef GO
  return GA_CHECK_LAUNCH();
}
