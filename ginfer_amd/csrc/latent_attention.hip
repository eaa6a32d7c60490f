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
__global__ __launch_bounds__(256) void latent_prepare_kernel(T* __restrict__ cq, T* __restrict__ c_pages, T* __restrict__ ct_pages,
                                                             int page_size, float* __restrict__ gate,
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
    int64_t page, off;
    slot_page(slot, page_size, page, off);
    for (int i = threadIdx.x; i < kv_rank; i += 256) {
      const float v = p[i] / rms * wkv[i];
      Num<T>::st(c_pages + slot * kv_rank + i, v);
      // the second copy, transposed inside the page ([rank][slot]), which the matrix-core kernel reads as values
      if (ct_pages) Num<T>::st(ct_pages + (page * kv_rank + i) * page_size + off, v);
    }
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

extern "C" int ga_latent_prepare(void* cq, void* c_pages, void* ct_pages, int page_size, void* gate, const void* proj,
                                 int64_t proj_stride, const void* wq, const void* wkv, const void* slot_mapping, int tokens,
                                 int q_rank, int kv_rank, int heads, float eps, int write_c, int is_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (q_rank <= 0 || kv_rank <= 0 || heads <= 0 || page_size <= 0) return -1;
  dim3 grid(tokens), block(256);
  if (is_bf16)
    hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)cq, (bf16_t*)c_pages, (bf16_t*)ct_pages,
                       page_size, (float*)gate,
                       (const float*)proj, proj_stride, (const float*)wq, (const float*)wkv, (const int64_t*)slot_mapping,
                       q_rank, kv_rank, heads, eps, write_c);
  else
    hipLaunchKernelGGL(latent_prepare_kernel<float>, grid, block, 0, stream, (float*)cq, (float*)c_pages, (float*)ct_pages,
                       page_size, (float*)gate,
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

// ---------------------------------------------------------------------------------------------------- matrix cores
// bfloat16 on v_mfma_f32_16x16x32_bf16 (D[m][n] += sum_k A[m][k] B[n][k]; lane l supplies row l % 16 and k-slots
// (l / 16) * 8 .. + 7 of both operands and receives D[(l / 16) * 4 + i][l % 16]).  The 16 columns n of a wavefront are 16
// (token, head) pairs that attend to the same request:
//   MODE 0  16 neighbouring tokens of the step for one head (prompt portions); a workgroup's 4 wavefronts take HPW heads each.
//           Where the 16 tokens belong to several requests they are worked off request by request, the others masked.
//   MODE 1  16 heads of one single token (decoding); the token's keys may be dealt to several workgroups, whose partial
//           results a second kernel merges.
//   S^T = C QA^T   A = 16 latent rows x 32 coordinates, one 16-byte load per lane from the page [slot][rank]; row m of
//                  product t holds key 8 (m / 4) + 4 t + m % 4 of the tile of 32, so a lane ends up with the scores of the 8
//                  consecutive keys 8 (l / 16) .. + 7 of its column, which is the k-slot layout of operand B for P:
//   O^T += C^T P^T A = 16 coordinates x 8 consecutive keys from the page's transposed copy [rank][slot], one 16-byte load.
// Softmax in 32-bit, per column, over tiles of 32 keys at absolute multiples of 32.  No LDS: the wavefronts of a workgroup
// read the same lines of the vector cache.  RP: the rank rounded up (64, 128, 256, 512); coordinates beyond the rank are zeros.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 lm_zero8() {
  const uint4 z = make_uint4(0u, 0u, 0u, 0u);
  return __builtin_bit_cast(bf16x8, z);
}
__device__ __forceinline__ bf16x8 lm_load8(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ __forceinline__ bf16x8 lm_pack8(const float* v) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f32_to_bf16(v[2 * i]) | ((uint32_t)f32_to_bf16(v[2 * i + 1]) << 16);
  return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
}
__device__ __forceinline__ int lm_wave_min(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, WAVE));
  return v;
}
__device__ __forceinline__ int lm_wave_max(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, WAVE));
  return v;
}

// The walk over the tiles [tile_lo, tile_hi] (multiples of 32) for NS sets of 16 columns that share the request's pages.
// qb: the columns' queries as B operands; lo_c / pos_c: the column's first and last visible key (pos_c < lo_c: the column
// sees nothing); keys outside [lo_min, hi_max] are not loaded.  Leaves the running maximum, the lane's part of the sum of
// weights and the unnormalised O^T in m_run, l_run, acc.
template <int RP, int NS>
__device__ __forceinline__ void lm_walk(f32x4 (&acc)[NS][RP / 16], float (&m_run)[NS], float (&l_run)[NS],
                                        const bf16x8 (&qb)[NS][RP / 32], const bf16_t* __restrict__ c_pages,
                                        const bf16_t* __restrict__ ct_pages, const int32_t* __restrict__ bt, int rank,
                                        int ps_shift, int lo_c, int pos_c, int lo_min, int hi_max, int tile_lo, int tile_hi,
                                        float scale, int c, int g) {
  const int ps = 1 << ps_shift, ps_mask = ps - 1;
  for (int k0 = tile_lo; k0 <= tile_hi; k0 += 32) {
    f32x4 s[NS][2];
#pragma unroll
    for (int k = 0; k < NS; ++k) s[k][0] = s[k][1] = f32x4{0.f, 0.f, 0.f, 0.f};
    const bf16_t* rowp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int kp = k0 + 8 * (c >> 2) + 4 * t + (c & 3);
      rowp[t] = nullptr;
      if (kp >= lo_min && kp <= hi_max) rowp[t] = c_pages + ((int64_t)bt[kp >> ps_shift] * ps + (kp & ps_mask)) * rank + 8 * g;
    }
    // operands are asked for a batch at a time and multiplied after: a load that stands right before its product would
    // make every product wait for the whole way to memory (measured: 30 us a tile; with batches under 2)
    constexpr int SB = (RP / 32 < 8) ? RP / 32 : 8;     // 32-coordinate blocks per batch (two operands each)
#pragma unroll
    for (int kb = 0; kb < RP / 32; kb += SB) {
      bf16x8 a[SB][2];
#pragma unroll
      for (int u = 0; u < SB; ++u)
#pragma unroll
        for (int t = 0; t < 2; ++t)
          a[u][t] = (rowp[t] != nullptr && 32 * (kb + u) + 8 * g < rank) ? lm_load8(rowp[t] + 32 * (kb + u)) : lm_zero8();
#pragma unroll
      for (int u = 0; u < SB; ++u)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int k = 0; k < NS; ++k) s[k][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][t], qb[k][kb + u], s[k][t], 0, 0, 0);
    }
    bf16x8 pb[NS];
    bool rescale = false;
    float alpha[NS];
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      float sc[8], mt = -INFINITY;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int kp = k0 + 8 * g + j;
        const bool valid = kp >= lo_c && kp <= pos_c;
        sc[j] = valid ? s[k][j >> 2][j & 3] * scale : -INFINITY;
        mt = fmaxf(mt, sc[j]);
      }
      mt = fmaxf(mt, __shfl_xor(mt, 16, WAVE));
      mt = fmaxf(mt, __shfl_xor(mt, 32, WAVE));
      const float m_new = fmaxf(m_run[k], mt);
      const float ref = (m_new == -INFINITY) ? 0.f : m_new;       // a column that has seen no key yet
      float sum = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        sc[j] = (sc[j] == -INFINITY) ? 0.f : expf(sc[j] - ref);
        sum += sc[j];
      }
      alpha[k] = expf(m_run[k] - ref);
      l_run[k] = l_run[k] * alpha[k] + sum;
      m_run[k] = m_new;
      pb[k] = lm_pack8(sc);
      rescale = rescale || alpha[k] != 1.f;
    }
    if (__any(rescale)) {
#pragma unroll
      for (int k = 0; k < NS; ++k)
#pragma unroll
        for (int rt = 0; rt < RP / 16; ++rt) acc[k][rt] *= alpha[k];
    }
    const int gs = k0 + 8 * g;                          // the lane's 8 consecutive keys, inside one page
    const bf16_t* colp = nullptr;
    if (gs <= hi_max && gs + 7 >= lo_min)
      colp = ct_pages + (int64_t)bt[gs >> ps_shift] * ps * rank + (gs & ps_mask);
    constexpr int PB = (RP / 16 < 16) ? RP / 16 : 16;   // 16-coordinate blocks per batch
#pragma unroll
    for (int rb = 0; rb < RP / 16; rb += PB) {
      bf16x8 a[PB];
#pragma unroll
      for (int u = 0; u < PB; ++u) {
        const int r = 16 * (rb + u) + c;
        a[u] = (colp != nullptr && r < rank) ? lm_load8(colp + (int64_t)r * ps) : lm_zero8();
      }
#pragma unroll
      for (int u = 0; u < PB; ++u)
#pragma unroll
        for (int k = 0; k < NS; ++k) acc[k][rb + u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], pb[k], acc[k][rb + u], 0, 0, 0);
    }
  }
}

template <int RP>
__device__ __forceinline__ void lm_load_query(bf16x8 (&qb)[RP / 32], const float* __restrict__ q, int rank, int g, bool ok) {
#pragma unroll
  for (int ks = 0; ks < RP / 32; ++ks) {
    const int r = 32 * ks + 8 * g;
    if (ok && r < rank) {
      float v[8];
      const float4 a = *reinterpret_cast<const float4*>(q + r), b = *reinterpret_cast<const float4*>(q + r + 4);
      v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
      qb[ks] = lm_pack8(v);
    } else {
      qb[ks] = lm_zero8();
    }
  }
}

// the column's share of the result: weights over (sum + exp(sink)), times the gate
__device__ __forceinline__ float lm_finish(float m, float l, const float* sink, const float* gate, int t, int h, int heads) {
  float top = m, keep = 1.f, den = l;
  if (sink) {
    const float s = sink[h];
    top = fmaxf(m, s);
    keep = expf(m - top);
    den = l * keep + expf(s - top);
  }
  return keep / den * (gate ? gate[(int64_t)t * heads + h] : 1.f);
}

template <int RP>
__device__ __forceinline__ void lm_store(bf16_t* __restrict__ o, const f32x4 (&acc)[RP / 16], float f, int rank, int g) {
#pragma unroll
  for (int rt = 0; rt < RP / 16; ++rt) {
    const int r = 16 * rt + 4 * g;
    if (r < rank) {
      const uint32_t lo = (uint32_t)f32_to_bf16(acc[rt][0] * f) | ((uint32_t)f32_to_bf16(acc[rt][1] * f) << 16);
      const uint32_t hi = (uint32_t)f32_to_bf16(acc[rt][2] * f) | ((uint32_t)f32_to_bf16(acc[rt][3] * f) << 16);
      *reinterpret_cast<uint2*>(o + r) = make_uint2(lo, hi);
    }
  }
}

// MODE 0: grid (ceil(tokens / 16), ceil(heads / (4 HPW))), 256 threads
template <int RP, int HPW>
__global__ __launch_bounds__(256) void latent_attention_rows_kernel(
    bf16_t* __restrict__ out, int64_t out_t, int64_t out_h, const float* __restrict__ qa, int64_t qa_t, int64_t qa_h,
    const bf16_t* __restrict__ c_pages, const bf16_t* __restrict__ ct_pages, const int32_t* __restrict__ block_table,
    int table_width, const int32_t* __restrict__ token_entry, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ cu, const float* __restrict__ sink, const float* __restrict__ gate, int tokens, int heads,
    int rank, int ps_shift, int window, float scale, int skip_singles) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;
  const int h0 = (blockIdx.y * 4 + wave) * HPW;
  if (h0 >= heads) return;                              // the whole wavefront; nothing below meets other wavefronts
  const int t = blockIdx.x * 16 + c;
  const bool col_ok = t < tokens;
  const int e_c = col_ok ? token_entry[t] : -1, pos_c = col_ok ? positions[t] : 0;
  const int single = (col_ok && skip_singles && cu[e_c + 1] - cu[e_c] == 1) ? 1 : 0;
  const int lo_c = (window > 0 && pos_c - window + 1 > 0) ? pos_c - window + 1 : 0;
  bf16x8 qb[HPW][RP / 32];
#pragma unroll
  for (int k = 0; k < HPW; ++k)
    lm_load_query<RP>(qb[k], qa + (int64_t)(h0 + k) * qa_h + (int64_t)t * qa_t, rank, g, col_ok && h0 + k < heads);
  int seg = 0;
  while (seg < 16) {
    const int e = __shfl(e_c, seg, WAVE);               // the same for every lane
    if (e < 0) break;                                   // columns beyond the step's tokens
    const bool mine = e_c == e && c >= seg;             // a request's tokens lie side by side
    const int n = __popcll(__ballot(mine) & 0xffffull);
    const int skip = __shfl(single, seg, WAVE);
    if (!skip) {
      const int lo_min = lm_wave_min(mine ? lo_c : 0x7fffffff), hi_max = lm_wave_max(mine ? pos_c : -1);
      f32x4 acc[HPW][RP / 16];
      float m_run[HPW], l_run[HPW];
#pragma unroll
      for (int k = 0; k < HPW; ++k) {
        m_run[k] = -INFINITY;
        l_run[k] = 0.f;
#pragma unroll
        for (int rt = 0; rt < RP / 16; ++rt) acc[k][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
      lm_walk<RP, HPW>(acc, m_run, l_run, qb, c_pages, ct_pages, block_table + (int64_t)e * table_width, rank, ps_shift,
                       mine ? lo_c : 1, mine ? pos_c : 0, lo_min, hi_max, (lo_min >> 5) << 5, hi_max, scale, c, g);
#pragma unroll
      for (int k = 0; k < HPW; ++k) {
        float l = l_run[k];
        l += __shfl_xor(l, 16, WAVE);
        l += __shfl_xor(l, 32, WAVE);
        if (mine && h0 + k < heads) {
          const float f = lm_finish(m_run[k], l, sink, gate, t, h0 + k, heads);
          lm_store<RP>(out + (int64_t)(h0 + k) * out_h + (int64_t)t * out_t, acc[k], f, rank, g);
        }
      }
    }
    seg += n;
  }
}

// MODE 1: grid (single tokens, ceil(ceil(heads / 16) / 4), splits), 256 threads; info: int32 x 4 per token = (row of the
// step, position, entry, -).  splits == 1: the result goes to out; else the split's unnormalised O (ws_o: [token][head]
// [split][RP] floats) and (maximum, sum) (ws_ml) for the merge kernel.
template <int RP>
__global__ __launch_bounds__(256) void latent_attention_heads_kernel(
    bf16_t* __restrict__ out, int64_t out_t, int64_t out_h, float* __restrict__ ws_o, float* __restrict__ ws_ml,
    const float* __restrict__ qa, int64_t qa_t, int64_t qa_h, const bf16_t* __restrict__ c_pages,
    const bf16_t* __restrict__ ct_pages, const int32_t* __restrict__ block_table, int table_width,
    const int32_t* __restrict__ info, const float* __restrict__ sink, const float* __restrict__ gate, int heads, int rank,
    int ps_shift, int window, float scale, int splits, int tiles_per_split) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;
  const int h = (blockIdx.y * 4 + wave) * 16 + c;
  if ((blockIdx.y * 4 + wave) * 16 >= heads) return;
  const int n = blockIdx.x, t = info[4 * n], pos = info[4 * n + 1], e = info[4 * n + 2], z = blockIdx.z;
  const bool head_ok = h < heads;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  bf16x8 qb[1][RP / 32];
  lm_load_query<RP>(qb[0], qa + (int64_t)h * qa_h + (int64_t)t * qa_t, rank, g, head_ok);
  f32x4 acc[1][RP / 16];
  float m_run[1] = {-INFINITY}, l_run[1] = {0.f};
#pragma unroll
  for (int rt = 0; rt < RP / 16; ++rt) acc[0][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int first = ((lo >> 5) + z * tiles_per_split) << 5;
  int last = first + 32 * (tiles_per_split - 1);
  if (last > pos || splits == 1) last = pos;            // the walk takes every tile that starts at or before `last`
  lm_walk<RP, 1>(acc, m_run, l_run, qb, c_pages, ct_pages, block_table + (int64_t)e * table_width, rank, ps_shift,
                 head_ok ? lo : 1, head_ok ? pos : 0, lo, pos, first, last, scale, c, g);
  float l = l_run[0];
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  if (!head_ok) return;
  if (splits == 1) {
    lm_store<RP>(out + (int64_t)h * out_h + (int64_t)t * out_t, acc[0], lm_finish(m_run[0], l, sink, gate, t, h, heads), rank, g);
    return;
  }
  const int64_t slot = ((int64_t)n * heads + h) * splits + z;
  if (g == 0) {
    ws_ml[2 * slot] = m_run[0];
    ws_ml[2 * slot + 1] = l;
  }
#pragma unroll
  for (int rt = 0; rt < RP / 16; ++rt)
    *reinterpret_cast<float4*>(ws_o + slot * RP + 16 * rt + 4 * g) = make_float4(acc[0][rt][0], acc[0][rt][1], acc[0][rt][2], acc[0][rt][3]);
}

// merges the splits of a single token's heads: grid (tokens, heads), 64 threads; at most 64 splits.  Lane z works out
// split z's weight once; every lane then adds its coordinates over the splits, four loads under way at a time.
__global__ __launch_bounds__(64) void latent_attention_merge_kernel(bf16_t* __restrict__ out, int64_t out_t, int64_t out_h,
                                                                    const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                                                                    const int32_t* __restrict__ info, const float* __restrict__ sink,
                                                                    const float* __restrict__ gate, int heads, int rank, int rp,
                                                                    int splits) {
  const int n = blockIdx.x, h = blockIdx.y, t = info[4 * n], lane = threadIdx.x;
  const int64_t base = ((int64_t)n * heads + h) * splits;
  const float m = lane < splits ? ws_ml[2 * (base + lane)] : -INFINITY;
  const float l = lane < splits ? ws_ml[2 * (base + lane) + 1] : 0.f;
  const float top = fmaxf(wave_max(m), sink ? sink[h] : -INFINITY);
  const float wz = (m == -INFINITY) ? 0.f : expf(m - top);
  const float den = wave_sum(wz * l) + (sink ? expf(sink[h] - top) : 0.f);
  const float f = (gate ? gate[(int64_t)t * heads + h] : 1.f) / den;
  for (int r0 = 0; r0 < rank; r0 += 64) {
    const int r = r0 + lane;
    const bool ok = r < rank;
    float o = 0.f;
    int z = 0;
    for (; z + 4 <= splits; z += 4) {
      float v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = ok ? ws_o[(base + z + u) * rp + r] : 0.f;
#pragma unroll
      for (int u = 0; u < 4; ++u) o += __shfl(wz, z + u, WAVE) * v[u];
    }
    for (; z < splits; ++z) o += __shfl(wz, z, WAVE) * (ok ? ws_o[(base + z) * rp + r] : 0.f);
    if (ok) out[(int64_t)h * out_h + (int64_t)t * out_t + r] = f32_to_bf16(o * f);
  }
}

// heads per wavefront in the kernel for portions: as many as the registers hold beside the queries (two at a padded rank
// of 512 spill: 2.2 -> 3.7 ms for 2,048 tokens of 28 heads on MI355X)
static int lm_padded_rank(int rank) { return rank <= 64 ? 64 : rank <= 128 ? 128 : rank <= 256 ? 256 : 512; }

extern "C" int ga_latent_attention_mfma_padded_rank(int rank) { return lm_padded_rank(rank); }

// Prompt portions (and, unless skip_singles, every token) on the matrix cores.  bfloat16; rank a multiple of 8 up to 512;
// page_size a power of two >= 8; qa rows 16-byte aligned.
extern "C" int ga_latent_attention_rows(void* out, int64_t out_t, int64_t out_h, const void* qa, int64_t qa_t, int64_t qa_h,
                                        const void* c_pages, const void* ct_pages, const void* block_table, int table_width,
                                        const void* token_entry, const void* positions, const void* cu, const void* sink,
                                        const void* gate, int tokens, int heads, int rank, int page_size, int window,
                                        float scale, int skip_singles, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads <= 0 || rank <= 0 || rank > 512 || rank % 8 || page_size < 8 || (page_size & (page_size - 1)) || table_width <= 0 ||
      window < 0 || qa_t % 4 || qa_h % 4 || out_t % 4 || out_h % 4 || ((uintptr_t)qa & 15) || ((uintptr_t)out & 7))
    return -1;
  const int ps_shift = __builtin_ctz(page_size), rp = lm_padded_rank(rank);
#define GO(RP, HPW)                                                                                                          \
  {                                                                                                                          \
    dim3 grid((tokens + 15) / 16, (heads + 4 * HPW - 1) / (4 * HPW)), block(256);                                            \
    if (grid.y > 65535) return -2;                                                                                           \
    hipLaunchKernelGGL((latent_attention_rows_kernel<RP, HPW>), grid, block, 0, stream, (bf16_t*)out, out_t, out_h,          \
                       (const float*)qa, qa_t, qa_h, (const bf16_t*)c_pages, (const bf16_t*)ct_pages,                        \
                       (const int32_t*)block_table, table_width, (const int32_t*)token_entry, (const int32_t*)positions,     \
                       (const int32_t*)cu, (const float*)sink, (const float*)gate, tokens, heads, rank, ps_shift, window,    \
                       scale, skip_singles);                                                                                 \
  }
  if (rp == 64) GO(64, 4) else if (rp == 128) GO(128, 4) else if (rp == 256) GO(256, 2) else GO(512, 1)
#undef GO
  return GA_CHECK_LAUNCH();
}

// Single tokens on the matrix cores; info int32 [n][4].  splits > 1: ws_o n * heads * splits * padded rank floats, ws_ml
// n * heads * splits * 2 floats; every token's keys are dealt to `splits` workgroups of tiles_per_split tiles of 32 each
// (splits * tiles_per_split must cover the longest walk: the window, or the longest context, in tiles, plus one).
extern "C" int ga_latent_attention_heads(void* out, int64_t out_t, int64_t out_h, void* ws_o, void* ws_ml, const void* qa,
                                         int64_t qa_t, int64_t qa_h, const void* c_pages, const void* ct_pages,
                                         const void* block_table, int table_width, const void* info, int n, const void* sink,
                                         const void* gate, int heads, int rank, int page_size, int window, float scale,
                                         int splits, int tiles_per_split, hipStream_t stream) {
  if (n <= 0) return 0;
  if (heads <= 0 || rank <= 0 || rank > 512 || rank % 8 || page_size < 8 || (page_size & (page_size - 1)) || table_width <= 0 ||
      window < 0 || qa_t % 4 || qa_h % 4 || out_t % 4 || out_h % 4 || ((uintptr_t)qa & 15) || ((uintptr_t)out & 7) ||
      splits < 1 || splits > 64 || tiles_per_split < 1 || (splits > 1 && (ws_o == nullptr || ws_ml == nullptr)))
    return -1;
  const int ps_shift = __builtin_ctz(page_size), rp = lm_padded_rank(rank);
  const int sets = (heads + 15) / 16;
  dim3 grid(n, (sets + 3) / 4, splits), block(256);
#define GO(RP)                                                                                                               \
  hipLaunchKernelGGL(latent_attention_heads_kernel<RP>, grid, block, 0, stream, (bf16_t*)out, out_t, out_h, (float*)ws_o,    \
                     (float*)ws_ml, (const float*)qa, qa_t, qa_h, (const bf16_t*)c_pages, (const bf16_t*)ct_pages,           \
                     (const int32_t*)block_table, table_width, (const int32_t*)info, (const float*)sink,                     \
                     (const float*)gate, heads, rank, ps_shift, window, scale, splits, tiles_per_split)
  if (rp == 64) GO(64); else if (rp == 128) GO(128); else if (rp == 256) GO(256); else GO(512);
#undef GO
  int rc = GA_CHECK_LAUNCH();
  if (rc != 0 || splits == 1) return rc;
  if (heads > 65535) return -2;
  hipLaunchKernelGGL(latent_attention_merge_kernel, dim3(n, heads), dim3(64), 0, stream, (bf16_t*)out, out_t, out_h,
                     (const float*)ws_o, (const float*)ws_ml, (const int32_t*)info, (const float*)sink, (const float*)gate,
                     heads, rank, rp, splits);
  return GA_CHECK_LAUNCH();
}
