// Routing of tokens to experts, and the gated activation of many experts side by side.
//   route:   from router scores z [T, E] (32-bit) the `top` largest of every row (the lowest index among equals), their
//            weights = softmax over the chosen scores alone; written as lists (ids, weights [T, top]) and as a row of E
//            weights with zeros at the experts not chosen.
//   weighted gated activation:  act[t, c] = w(t, c) * silu(gate[t, c]) * up[t, c] over the columns of all experts laid
//            side by side (expert e owns columns [e * ff, (e + 1) * ff)); columns behind the experts' (a shared expert that
//            every token uses) have the weight 1.  The product with the stacked down matrices then IS the weighted sum
//            of the chosen experts' outputs: the others enter with exact zeros.
#include "common.h"
#include "ginfer_amd.h"

#define ROUTE_MAX_EXPERTS 256
#define ROUTE_THREADS 64

// one wavefront per token; experts dealt to lanes, ROUTE_MAX_EXPERTS / 64 each
__global__ __launch_bounds__(ROUTE_THREADS) void route_topk_kernel(const float* __restrict__ scores, int32_t* __restrict__ ids,
                                                                   float* __restrict__ weights, float* __restrict__ dense,
                                                                   int experts, int top) {
  constexpr int PER = ROUTE_MAX_EXPERTS / ROUTE_THREADS;
  __shared__ float chosen_s[ROUTE_MAX_EXPERTS];
  __shared__ int32_t chosen_i[ROUTE_MAX_EXPERTS];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  float z[PER];
  bool taken[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + j * ROUTE_THREADS;
    z[j] = e < experts ? scores[t * experts + e] : -INFINITY;
    // a score that is no number (the rows that pad a recorded step may hold anything) counts as the smallest: with
    // it no comparison below would hold, the lanes would come to different winners, each strike out its own, and the
    // next round would find no expert left
    if (!(z[j] == z[j])) z[j] = -INFINITY;
    taken[j] = e >= experts;
  }
  for (int k = 0; k < top; ++k) {
    // this lane's best that is still free, then the best over the lanes; equal scores go to the lowest index
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + j * ROUTE_THREADS;
      if (!taken[j] && (at == 0x7fffffff || z[j] > best)) { best = z[j]; at = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, WAVE);
      const int oa = __shfl_xor(at, o, WAVE);
      if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (lane + j * ROUTE_THREADS == at) taken[j] = true;
    if (lane == 0) { chosen_s[k] = best; chosen_i[k] = at < experts ? at : 0; }   // top <= experts: one is always left
  }
  __syncthreads();
  // softmax over the chosen scores; chosen_s[0] is the largest
  const float top_score = chosen_s[0];
  float total = 0.f;
  for (int k = 0; k < top; ++k) total += expf(chosen_s[k] - top_score);
  for (int e = lane; e < experts; e += ROUTE_THREADS) dense[t * experts + e] = 0.f;
  __syncthreads();
  for (int k = lane; k < top; k += ROUTE_THREADS) {
    const float w = expf(chosen_s[k] - top_score) / total;
    ids[t * top + k] = chosen_i[k];
    weights[t * top + k] = w;
    dense[t * experts + chosen_i[k]] = w;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void weighted_silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gate_up,
                                                                const float* __restrict__ dense, int64_t total, int width,
                                                                int experts, int ff) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / width;
  const int c = (int)(i - t * width);
  const int e = c / ff;
  const float w = e < experts ? dense[t * experts + e] : 1.f;
  float r = 0.f;
  if (w != 0.f) {                              // an expert that the token does not use: an exact zero, whatever it holds
    const float g = Num<T>::ld(gate_up + t * 2 * width + c), u = Num<T>::ld(gate_up + t * 2 * width + width + c);
    r = w * (g / (1.f + expf(-g)) * u);
  }
  Num<T>::st(out + i, r);
}

extern "C" int ga_route_topk(void* ids, void* weights, void* dense, const void* scores, int tokens, int experts, int top,
                             hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (experts <= 0 || experts > ROUTE_MAX_EXPERTS || top <= 0 || top > experts) return -1;
  hipLaunchKernelGGL(route_topk_kernel, dim3(tokens), dim3(ROUTE_THREADS), 0, stream, (const float*)scores, (int32_t*)ids,
                     (float*)weights, (float*)dense, experts, top);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_weighted_silu_mul(void* out, const void* gate_up, const void* dense, int tokens, int width, int experts,
                                    int ff, int is_bf16, hipStream_t stream) {
  if (tokens <= 0 || width <= 0) return 0;
  if (experts < 0 || ff <= 0 || (int64_t)experts * ff > width) return -1;
  const int64_t total = (int64_t)tokens * width;
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (is_bf16)
    hipLaunchKernelGGL(weighted_silu_mul_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, (const bf16_t*)gate_up,
                       (const float*)dense, total, width, experts, ff);
  else
    hipLaunchKernelGGL(weighted_silu_mul_kernel<float>, grid, block, 0, stream, (float*)out, (const float*)gate_up,
                       (const float*)dense, total, width, experts, ff);
  return GA_CHECK_LAUNCH();
}
