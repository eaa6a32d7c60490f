// Linear attention whose forget gate also decides what is written (HGRN2), as a recurrence over per-request state:
//   q = silu(pq),  f = lower + (1 - lower) * sigmoid(pf + bias),  v = pv           (pq | pf | pv: one projection, 32-bit)
//   per head:  S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T   (S is [dim, vdim]; f acts on the rows, which belong to q),
//              o_t = S_t^T q_t
// The state is 32-bit, [slot][head][dim][vdim]; a request whose q_start is 0 starts from zeros.  Gates, state and the
// output sum are 32-bit.  A workgroup owns one (entry, head, block of 16 value columns) and walks the entry's tokens in
// order, 16 at a time: the tile's q, f and v go through LDS with their activations applied, every thread keeps the
// state of one column and every 16th row in registers, and the rows' partial outputs are added in a fixed order.  So a
// token's result does not depend on how the request's tokens were cut into steps, nor on what else is in the batch.
// A second kernel norms each head's output over its value columns (RMS, with a weight per column).
#include "common.h"
#include "ginfer_amd.h"

#define GR_THREADS 256
#define GR_COLS 16        // value columns of a workgroup
#define GR_SLICES 16      // a column's rows are dealt to this many threads
#define GR_TILE 16        // tokens per trip through LDS

__device__ __forceinline__ float gr_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

template <int R>          // rows of the state per thread: dim <= 16 * R
__global__ __launch_bounds__(GR_THREADS) void hgrn2_scan_kernel(float* __restrict__ out, const float* __restrict__ proj,
                                                                 int64_t proj_stride, const float* __restrict__ f_bias,
                                                                 const float* __restrict__ lower, float* __restrict__ state,
                                                                 const int64_t* __restrict__ slots, const int32_t* __restrict__ cu,
                                                                 const int32_t* __restrict__ q_start, int heads, int dim, int vdim) {
  constexpr int DP = GR_SLICES * R;
  __shared__ float qs[GR_TILE][DP], fs[GR_TILE][DP], vs[GR_TILE][GR_COLS];
  __shared__ float partial[GR_TILE][GR_SLICES][GR_COLS];
  const int e = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * GR_COLS;
  const int first = cu[e], n = cu[e + 1] - first;
  if (n <= 0) return;
  const int j = threadIdx.x % GR_COLS, s = threadIdx.x / GR_COLS;
  const bool col_ok = v0 + j < vdim;
  float* st = state + ((slots[e] * heads + h) * (int64_t)dim) * vdim + v0 + j;
  float S[R];
  const bool fresh = q_start[e] == 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = s + GR_SLICES * r;
    S[r] = (!fresh && col_ok && i < dim) ? st[(int64_t)i * vdim] : 0.f;
  }
  const int hd = heads * dim;
  for (int t0 = 0; t0 < n; t0 += GR_TILE) {
    const int nt = min(GR_TILE, n - t0);
    __syncthreads();                                   // the tile before is read out
    for (int idx = threadIdx.x; idx < GR_TILE * DP; idx += GR_THREADS) {
      const int tt = idx / DP, i = idx % DP;
      float q = 0.f, f = 0.f;
      if (tt < nt && i < dim) {
        const float* p = proj + (int64_t)(first + t0 + tt) * proj_stride + h * dim + i;
        const float pq = p[0];
        q = pq * gr_sigmoid(pq);
        const float lo = lower[h * dim + i];
        f = lo + (1.0f - lo) * gr_sigmoid(p[hd] + f_bias[h * dim + i]);
      }
      qs[tt][i] = q;
      fs[tt][i] = f;
    }
    {
      const int tt = threadIdx.x / GR_COLS, jj = threadIdx.x % GR_COLS;      // GR_TILE * GR_COLS == GR_THREADS
      vs[tt][jj] = (tt < nt && v0 + jj < vdim)
                       ? proj[(int64_t)(first + t0 + tt) * proj_stride + 2 * hd + h * vdim + v0 + jj] : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float v = vs[tt][j];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int i = s + GR_SLICES * r;
        const float f = fs[tt][i];
        S[r] = f * S[r] + (1.0f - f) * v;
        acc += S[r] * qs[tt][i];
      }
      partial[tt][s][j] = acc;
    }
    __syncthreads();
    {
      const int tt = threadIdx.x / GR_COLS, jj = threadIdx.x % GR_COLS;
      if (tt < nt && v0 + jj < vdim) {
        float o = 0.f;
#pragma unroll
        for (int k = 0; k < GR_SLICES; ++k) o += partial[tt][k][jj];
        out[((int64_t)(first + t0 + tt) * heads + h) * vdim + v0 + jj] = o;
      }
    }
  }
  if (col_ok) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = s + GR_SLICES * r;
      if (i < dim) st[(int64_t)i * vdim] = S[r];
    }
  }
}

// out[t, h, :] = x[t, h, :] / sqrt(mean(x[t, h, :]^2) + eps) * weight[:], one wavefront per (token, head)
template <typename T>
__global__ __launch_bounds__(GR_THREADS) void headwise_rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                                       const float* __restrict__ weight, int64_t rows, int vdim,
                                                                       float eps) {
  const int64_t row = (int64_t)blockIdx.x * (GR_THREADS / WAVE) + threadIdx.x / WAVE;
  if (row >= rows) return;
  const int lane = threadIdx.x % WAVE;
  const float* p = x + row * vdim;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += WAVE) ss += p[i] * p[i];
  ss = wave_sum(ss);
  const float rms = sqrtf(ss / (float)vdim + eps);
  for (int i = lane; i < vdim; i += WAVE) Num<T>::st(out + row * vdim + i, p[i] / rms * weight[i]);
}

extern "C" int ga_hgrn2_scan(void* out, const void* proj, int64_t proj_stride, const void* f_bias, const void* lower,
                             void* state, const void* slots, const void* cu, const void* q_start, int entries, int heads,
                             int dim, int vdim, hipStream_t stream) {
  if (entries <= 0) return 0;
  if (heads <= 0 || dim <= 0 || vdim <= 0 || dim > 16 * GR_SLICES) return -1;
  if (heads > 65535 || (vdim + GR_COLS - 1) / GR_COLS > 65535) return -2;
  dim3 grid(entries, heads, (vdim + GR_COLS - 1) / GR_COLS), block(GR_THREADS);
  const int rows = (dim + GR_SLICES - 1) / GR_SLICES;
#define GO(R) hipLaunchKernelGGL(hgrn2_scan_kernel<R>, grid, block, 0, stream, (float*)out, (const float*)proj, proj_stride, \
                                 (const float*)f_bias, (const float*)lower, (float*)state, (const int64_t*)slots,           \
                                 (const int32_t*)cu, (const int32_t*)q_start, heads, dim, vdim)
  if (rows <= 1) GO(1);
  else if (rows <= 2) GO(2);
  else if (rows <= 3) GO(3);
  else if (rows <= 4) GO(4);
  else if (rows <= 6) GO(6);
  else if (rows <= 8) GO(8);
  else if (rows <= 12) GO(12);
  else GO(16);
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_headwise_rmsnorm(void* out, const void* x, const void* weight, int64_t rows, int vdim, float eps,
                                   int out_bf16, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vdim <= 0) return -1;
  const int per = GR_THREADS / WAVE;
  dim3 grid((unsigned)((rows + per - 1) / per)), block(GR_THREADS);
  if (out_bf16)
    hipLaunchKernelGGL(headwise_rmsnorm_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, (const float*)x,
                       (const float*)weight, rows, vdim, eps);
  else
    hipLaunchKernelGGL(headwise_rmsnorm_kernel<float>, grid, block, 0, stream, (float*)out, (const float*)x,
                       (const float*)weight, rows, vdim, eps);
  return GA_CHECK_LAUNCH();
}
