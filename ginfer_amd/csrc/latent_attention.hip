// Attention over a cached LATENT: per token only c (kv_rank numbers) is kept, in pages; a head's keys and values are
// linear maps of c (k = Wuk c, v = Wuv c), so with the query carried into the latent space (qa = Wuk^T q) a head's score
// is qa . c and its output Wuv (sum_j p_j c_j): every head attends to the same rows c, which serve as keys and as values.
//   s_j = scale * qa . c_j  for positions j with 0 <= i - j < window (window 0: all earlier positions)
//   p_j = exp(s_j) / (exp(sink) + sum_j exp(s_j))        the sink is a learned number per head with no key and no value
//   out = gate * sum_j p_j c_j                            gate: a number per token and head (or none)
// Scores, weights and sums are 32-bit.  Keys are taken in tiles that start at absolute multiples of the tile length and
// every sum has a fixed order, so a token's result does not depend on how its request was cut into steps.
//
// latent_prepare: the two RMS norms (each with a weight per coordinate) on the down-projections, the sigmoid of the
// gate logits, and the write of c into its page.
#include "common.h"
#include "ginfer_amd.h"

#define LA_MAX_HEADS_PER_WG 8
#define LA_PAD 4
#define LA_MAX_RANK 512

// ---------------------------------------------------------------------------------------------------- prepare
// proj float [T, q_rank + kv_rank + heads]: (down-projection of the queries | of keys and values | gate logits)
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(T* __restrict__ cq, T* __restrict__ c_pages, float* __restrict__ gate,
                                                             const float* __restrict__ proj, int64_t proj_stride,
                                                             const float* __restrict__ wq, const float* __restrict__ wkv,
                                                             const int64_t* __restrict__ slot_mapping, int q_rank, int kv_rank,
                                                             int heads, float eps, int write_c) {
  __shared__ float scratch[4];
  const int64_t t = blockIdx.x;
  const float* p = proj + t * proj_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += 256) ss += p[i] * p[i];
  ss = block_sum<4>(ss, scratch);
  float rms = sqrtf(ss / (float)q_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += 256) Num<T>::st(cq + t * q_rank + i, p[i] / rms * wq[i]);
  const int64_t slot = slot_mapping[t];
  if (write_c && slot >= 0) {                       // uniform over the workgroup
    p += q_rank;
    ss = 0.f;
    for (int i = threadIdx.x; i < kv_rank; i += 256) ss += p[i] * p[i];
    ss = block_sum<4>(ss, scratch);
    rms = sqrtf(ss / (float)kv_rank + eps);
    for (int i = threadIdx.x; i < kv_rank; i += 256) Num<T>::st(c_pages + slot * kv_rank + i, p[i] / rms * wkv[i]);
    p -= q_rank;
  }
  if (gate)
    for (int i = threadIdx.x; i < heads; i += 256) gate[t * heads + i] = 1.0f / (1.0f + expf(-p[q_rank + kv_rank + i]));
}

// ---------------------------------------------------------------------------------------------------- attention
// One workgroup per token and up to 8 heads (a wavefront each).  A tile of TK keys (rows of c, widened to 32-bit) goes
// through LDS once for all heads.  Scores: a lane takes key lane % TK and a share lane / TK of the rank, the shares meet
// by lane exchanges; outputs: a lane takes the coordinates lane, lane + 64, ... and adds the tile's keys in order.
template <typename T, int TK>
__global__ void latent_attention_kernel(T* __restrict__ out, int64_t out_t, int64_t out_h, const float* __restrict__ qa,
                                        int64_t qa_t, int64_t qa_h, const T* __restrict__ c_pages,
                                        const int32_t* __restrict__ block_table, int table_width,
                                        const int32_t* __restrict__ token_entry, const int32_t* __restrict__ positions,
                                        const float* __restrict__ sink, const float* __restrict__ gate, int heads, int rank,
                                        int page_size, int window, float scale, int heads_per_wg) {
  extern __shared__ float lds[];
  constexpr int G = WAVE / TK;                       // shares of the rank per key
  constexpr int RL = LA_MAX_RANK / WAVE;             // output coordinates per lane, at most
  const int stride = rank + LA_PAD;
  float* tile = lds;                                 // [TK][rank + pad]
  float* pw = tile + TK * stride;                    // [waves][TK]
  float* qw = pw + heads_per_wg * TK;                // [waves][rank]
  const int t = blockIdx.x, w = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int h = blockIdx.y * heads_per_wg + w;
  const bool head_ok = h < heads;
  const int e = token_entry[t], pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int32_t* bt = block_table + (int64_t)e * table_width;
  if (head_ok)
    for (int r = lane; r < rank; r += WAVE) qw[w * rank + r] = qa[(int64_t)t * qa_t + (int64_t)h * qa_h + r];
  const int key = lane % TK, g = lane / TK;
  const int share = (rank + G - 1) / G;
  const int r0 = g * share, r1 = min(rank, r0 + share);
  float m = -INFINITY, l = 0.f, acc[RL];
#pragma unroll
  for (int x = 0; x < RL; ++x) acc[x] = 0.f;
  const int nthreads = blockDim.x;
  for (int k0 = (lo / TK) * TK; k0 <= pos; k0 += TK) {
    __syncthreads();                                 // the tile before is used up (and qw is written)
    if ((rank & 7) == 0) {
      const int chunks = rank >> 3;
      for (int item = threadIdx.x; item < TK * chunks; item += nthreads) {
        const int kk = item / chunks, r = (item - kk * chunks) << 3;
        const int kp = k0 + kk;
        float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (kp >= lo && kp <= pos) {
          const int page = bt[kp / page_size];
          const T* src = c_pages + ((int64_t)page * page_size + kp % page_size) * rank + r;
#pragma unroll
          for (int x = 0; x < 8; ++x) v[x] = Num<T>::ld(src + x);
        }
        float* dst = tile + kk * stride + r;
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
      }
    } else {
      for (int item = threadIdx.x; item < TK * rank; item += nthreads) {
        const int kk = item / rank, r = item - kk * rank;
        const int kp = k0 + kk;
        float v = 0.f;
        if (kp >= lo && kp <= pos) {
          const int page = bt[kp / page_size];
          v = Num<T>::ld(c_pages + ((int64_t)page * page_size + kp % page_size) * rank + r);
        }
        tile[kk * stride + r] = v;
      }
    }
    __syncthreads();
    float alpha = 1.f;
    if (head_ok) {
      const float* crow = tile + key * stride;
      const float* q = qw + w * rank;
      float dot = 0.f;
      for (int r = r0; r < r1; ++r) dot += q[r] * crow[r];
#pragma unroll
      for (int off = TK; off < WAVE; off <<= 1) dot += __shfl_xor(dot, off, WAVE);
      const int kp = k0 + key;
      const bool valid = kp >= lo && kp <= pos;
      const float sc = valid ? dot * scale : -INFINITY;
      const float m_new = fmaxf(m, wave_max(sc));
      const float p = valid ? expf(sc - m_new) : 0.f;
      alpha = expf(m - m_new);
      l = l * alpha + wave_sum(g == 0 ? p : 0.f);
      m = m_new;
      if (g == 0) pw[w * TK + key] = p;
    }
    __syncthreads();
    if (head_ok) {
      const float* pk = pw + w * TK;
      const int kend = min(TK, pos - k0 + 1), kbeg = max(0, lo - k0);
#pragma unroll
      for (int x = 0; x < RL; ++x) {
        const int r = lane + x * WAVE;
        if (r < rank) {
          float a = acc[x] * alpha;
          for (int kk = kbeg; kk < kend; ++kk) a += pk[kk] * tile[kk * stride + r];
          acc[x] = a;
        }
      }
    }
  }
  if (!head_ok) return;
  float top = m, den = l, keep = 1.f;
  if (sink) {
    const float s = sink[h];
    top = fmaxf(m, s);
    keep = expf(m - top);
    den = l * keep + expf(s - top);
  }
  const float f = keep / den * (gate ? gate[(int64_t)t * heads + h] : 1.f);
#pragma unroll
  for (int x = 0; x < RL; ++x) {
    const int r = lane + x * WAVE;
    if (r < rank) Num<T>::st(out + (int64_t)t * out_t + (int64_t)h * out_h + r, acc[x] * f);
  }
}

static int la_tile_keys(int rank) { return rank <= 128 ? 64 : (rank <= 256 ? 32 : 16); }

extern "C" int ga_latent_attention_max_rank() { return LA_MAX_RANK; }

extern "C" int ga_latent_prepare(void* cq, void* c_pages, void* gate, const void* proj, int64_t proj_stride, const void* wq,
                                 const void* wkv, const void* slot_mapping, int tokens, int q_rank, int kv_rank, int heads,
                                 float eps, int write_c, int is_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (q_rank <= 0 || kv_rank <= 0 || heads <= 0) return -1;
  dim3 grid(tokens), block(256);
  if (is_bf16)
    hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)cq, (bf16_t*)c_pages, (float*)gate,
                       (const float*)proj, proj_stride, (const float*)wq, (const float*)wkv, (const int64_t*)slot_mapping,
                       q_rank, kv_rank, heads, eps, write_c);
  else
    hipLaunchKernelGGL(latent_prepare_kernel<float>, grid, block, 0, stream, (float*)cq, (float*)c_pages, (float*)gate,
                       (const float*)proj, proj_stride, (const float*)wq, (const float*)wkv, (const int64_t*)slot_mapping,
                       q_rank, kv_rank, heads, eps, write_c);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_latent_attention(void* out, int64_t out_t, int64_t out_h, const void* qa, int64_t qa_t, int64_t qa_h,
                                   const void* c_pages, const void* block_table, int table_width, const void* token_entry,
                                   const void* positions, const void* sink, const void* gate, int tokens, int heads, int rank,
                                   int page_size, int window, float scale, int is_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads <= 0 || rank <= 0 || rank > LA_MAX_RANK || page_size <= 0 || table_width <= 0 || window < 0) return -1;
  const int hpw = heads < LA_MAX_HEADS_PER_WG ? heads : LA_MAX_HEADS_PER_WG;
  const int tk = la_tile_keys(rank);
  const size_t bytes = ((size_t)tk * (rank + LA_PAD) + (size_t)hpw * (tk + rank)) * sizeof(float);
  if (bytes > 64 * 1024) return -2;
  dim3 grid(tokens, (heads + hpw - 1) / hpw), block(WAVE * hpw);
#define GO(T, TK) hipLaunchKernelGGL((latent_attention_kernel<T, TK>), grid, block, bytes, stream, (T*)out, out_t, out_h,     \
                                     (const float*)qa, qa_t, qa_h, (const T*)c_pages, (const int32_t*)block_table,          \
                                     table_width, (const int32_t*)token_entry, (const int32_t*)positions,                   \
                                     (const float*)sink, (const float*)gate, heads, rank, page_size, window, scale, hpw)
  if (is_bf16) { if (tk == 64) GO(bf16_t, 64); else if (tk == 32) GO(bf16_t, 32); else GO(bf16_t, 16); }
  else { if (tk == 64) GO(float, 64); else if (tk == 32) GO(float, 32); else GO(float, 16); }
#undef GO
  return GA_CHECK_LAUNCH();
}
