// A norm on a sublayer's OUTPUT with a factor per channel behind it, fused with the residual add and, where the caller
// wants it, with the norm that the NEXT sublayer reads through:
//   residual[t] += s * g * y[t] / sqrt(mean(y[t]^2) + eps)                  g, s: one number per channel (s may be absent)
//   (y may come as the 32-bit partial sums [parts, tokens, hidden] of a product whose K was split: added in order first)
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
                                                                      C* __restrict__ next, int hidden, int parts,
                                                                      int64_t part_stride) {
  __shared__ float scratch[ON_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  const Y* row = y + t * hidden;
  float* res = residual + t * hidden;
  const bool kept = hidden <= ON_THREADS * ON_PER;
  // y may be the partial sums of a product whose K was split (parts > 1, 32-bit): they are added in order
  auto value = [&](int i) {
    float a = Num<Y>::ld(row + i);
    for (int p = 1; p < parts; ++p) a += Num<Y>::ld(row + p * part_stride + i);
    return a;
  };
  float v[ON_PER];
  float ss = 0.f;
  if (kept) {
#pragma unroll
    for (int j = 0; j < ON_PER; ++j) {
      const int i = threadIdx.x + j * ON_THREADS;
      v[j] = i < hidden ? value(i) : 0.f;
      ss += v[j] * v[j];
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += ON_THREADS) {
      const float a = value(i);
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
      float a = value(i) / rms * gain[i];
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

// The same on rows of up to ON_THREADS * 16 elements whose length is a multiple of four: 16-byte accesses (8 bytes for
// bfloat16), every operand of a thread asked for before the first sum, four elements side by side.
template <typename T> struct Four;
template <> struct Four<float> {
  static __device__ __forceinline__ float4 ld(const float* p) { return *reinterpret_cast<const float4*>(p); }
  static __device__ __forceinline__ void st(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct Four<bf16_t> {
  static __device__ __forceinline__ float4 ld(const bf16_t* p) {
    union { uint2 u; bf16_t e[4]; } a;
    a.u = *reinterpret_cast<const uint2*>(p);
    return float4{bf16_to_f32(a.e[0]), bf16_to_f32(a.e[1]), bf16_to_f32(a.e[2]), bf16_to_f32(a.e[3])};
  }
  static __device__ __forceinline__ void st(bf16_t* p, float4 v) {
    union { uint2 u; bf16_t e[4]; } a;
    a.e[0] = f32_to_bf16(v.x); a.e[1] = f32_to_bf16(v.y); a.e[2] = f32_to_bf16(v.z); a.e[3] = f32_to_bf16(v.w);
    *reinterpret_cast<uint2*>(p) = a.u;
  }
};

#define ON_CHUNKS 4          // chunks of four elements a thread keeps

template <typename Y, typename C>
__global__ __launch_bounds__(ON_THREADS) void output_norm_add_vec_kernel(float* __restrict__ residual, const Y* __restrict__ y,
                                                                          const float* __restrict__ gain,
                                                                          const float* __restrict__ scale, float eps,
                                                                          const float* __restrict__ next_gain, float next_eps,
                                                                          C* __restrict__ next, int hidden, int parts,
                                                                          int64_t part_stride) {
  __shared__ float scratch[ON_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  const Y* row = y + t * hidden;
  float* res = residual + t * hidden;
  const int chunks = hidden / 4;
  float4 v[ON_CHUNKS], r[ON_CHUNKS], g[ON_CHUNKS], s[ON_CHUNKS], n[ON_CHUNKS];
  const float4 zero = float4{0.f, 0.f, 0.f, 0.f}, one = float4{1.f, 1.f, 1.f, 1.f};
#pragma unroll
  for (int j = 0; j < ON_CHUNKS; ++j) {
    const int i = threadIdx.x + j * ON_THREADS;
    const bool in = i < chunks;
    v[j] = in ? Four<Y>::ld(row + 4 * i) : zero;
    for (int p = 1; p < parts; ++p) {              // partial sums of a product whose K was split: added in order
      if (in) {
        const float4 more = Four<Y>::ld(row + p * part_stride + 4 * i);
        v[j].x += more.x; v[j].y += more.y; v[j].z += more.z; v[j].w += more.w;
      }
    }
    r[j] = in ? Four<float>::ld(res + 4 * i) : zero;
    g[j] = in ? Four<float>::ld(gain + 4 * i) : zero;
    s[j] = (in && scale) ? Four<float>::ld(scale + 4 * i) : one;
    n[j] = (in && next) ? Four<float>::ld(next_gain + 4 * i) : zero;
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < ON_CHUNKS; ++j) ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
  ss = block_sum<ON_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)hidden + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int j = 0; j < ON_CHUNKS; ++j) {
    const int i = threadIdx.x + j * ON_THREADS;
    r[j].x += v[j].x / rms * g[j].x * s[j].x;
    r[j].y += v[j].y / rms * g[j].y * s[j].y;
    r[j].z += v[j].z / rms * g[j].z * s[j].z;
    r[j].w += v[j].w / rms * g[j].w * s[j].w;
    if (i < chunks) {
      Four<float>::st(res + 4 * i, r[j]);
      ss2 += r[j].x * r[j].x + r[j].y * r[j].y + r[j].z * r[j].z + r[j].w * r[j].w;
    }
  }
  if (next == nullptr) return;
  ss2 = block_sum<ON_THREADS / WAVE>(ss2, scratch);
  const float rms2 = sqrtf(ss2 / (float)hidden + next_eps);
  C* out = next + t * hidden;
#pragma unroll
  for (int j = 0; j < ON_CHUNKS; ++j) {
    const int i = threadIdx.x + j * ON_THREADS;
    if (i < chunks)
      Four<C>::st(out + 4 * i, float4{r[j].x / rms2 * n[j].x, r[j].y / rms2 * n[j].y, r[j].z / rms2 * n[j].z, r[j].w / rms2 * n[j].w});
  }
}

extern "C" int ga_output_norm_add(void* residual, const void* y, const void* gain, const void* scale, float eps,
                                  const void* next_gain, float next_eps, void* next, int tokens, int hidden, int y_bf16,
                                  int next_bf16, int parts, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 0 || !gain) return -1;
  if (next && !next_gain) return -2;
  if (parts < 1 || (parts > 1 && y_bf16)) return -3;       // parts: 32-bit [parts, tokens, hidden]
  const int64_t part_stride = (int64_t)tokens * hidden;
  dim3 grid(tokens), block(ON_THREADS);
  const uintptr_t all = (uintptr_t)residual | (uintptr_t)y | (uintptr_t)gain | (uintptr_t)scale | (uintptr_t)next_gain | (uintptr_t)next;
  const bool vec = hidden % 4 == 0 && hidden <= 4 * ON_CHUNKS * ON_THREADS && all % 16 == 0;
#define GO(Y, C)                                                                                                          \
  do {                                                                                                                    \
    if (vec)                                                                                                              \
      hipLaunchKernelGGL((output_norm_add_vec_kernel<Y, C>), grid, block, 0, stream, (float*)residual, (const Y*)y,       \
                         (const float*)gain, (const float*)scale, eps, (const float*)next_gain, next_eps, (C*)next,       \
                         hidden, parts, part_stride);                                                                     \
    else                                                                                                                  \
      hipLaunchKernelGGL((output_norm_add_kernel<Y, C>), grid, block, 0, stream, (float*)residual, (const Y*)y,           \
                         (const float*)gain, (const float*)scale, eps, (const float*)next_gain, next_eps, (C*)next,       \
                         hidden, parts, part_stride);                                                                     \
  } while (0)
  if (y_bf16) { if (next_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float); }
  else { if (next_bf16) GO(float, bf16_t); else GO(float, float); }
#undef GO
  return GA_CHECK_LAUNCH();
}
