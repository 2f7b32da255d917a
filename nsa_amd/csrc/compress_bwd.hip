// Backward of the KV block compression (reference: nsa/compression_kv.py:62-171, 220-266 for the
// functional compressor; the Conv1d compressor of :292-312 differentiates through autograd there).
//   out[n][h][o] = b[o] + sum_{j,i} x[n*stride + j][h][i] * W[j*dim + i][o]
//   dx[t][h][i]  = sum over windows n that contain t, j = t - n*stride:  sum_o d_out[n][h][o] * W[j*dim+i][o]
//   dW[j*dim+i][o] = sum_{n,h} x[n*stride + j][h][i] * d_out[n][h][o],   db[o] = sum_{n,h} d_out[n][h][o]
// mean pooling is W = eye/block per j: dx[t] = (1/block) * sum of d_out over the windows containing t.
//
// dx (weighted): tokens with the same phase r = t mod stride meet the same weight slices
// j = r, r + stride, ..., so a wavefront takes one phase and 32 consecutive window starts m (tokens
// r + stride*m) and accumulates dx^T = sum_q W_{r+q*stride} d_out[m-q]^T with the weight slice as
// the A operand (rows i, 8 consecutive o per lane) and d_out rows as the B operand, both straight
// from global memory (the weights are L2 resident).  Every dx row is written exactly once.
// dW: contraction over the (window, head) rows, so both operands are read with the transposing
// fragment load from row-major LDS tiles; one workgroup per (j, 256-row chunk), fp32 atomics.
#include "tiles.h"

namespace nsa {

__device__ __forceinline__ int upper_seq_of(const int32_t* __restrict__ cu, int batch, int r) {
  int lo = 0, hi = batch;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= r) lo = mid; else hi = mid;
  }
  return lo;
}

// ---- dx, mean pooling: one thread per (token, 8 channels of the heads*dim row)
template <typename T>
__global__ void __launch_bounds__(256)
compress_mean_bwd_kernel(const T* __restrict__ d_out, T* __restrict__ dx, const int32_t* __restrict__ cu_seq,
                         const int32_t* __restrict__ cu_out, int batch, int total, int row_elems, int block,
                         int stride) {
  const int ppr = row_elems / 8;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const int t = (int)(idx / ppr), piece = (int)(idx % ppr);
  if (t >= total) return;
  const int b = upper_seq_of(cu_seq, batch, t);
  const int tl = t - cu_seq[b];
  const int nc = cu_out[b + 1] - cu_out[b];
  const int n_lo = tl >= block ? (tl - block) / stride + 1 : 0;
  const int n_hi = min(nc - 1, tl / stride);
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  for (int n = n_lo; n <= n_hi; ++n) {
    const vec8_t<T> v = load8(d_out + (long)(cu_out[b] + n) * row_elems + piece * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += (float)v[i];
  }
  const float inv = 1.0f / (float)block;
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] *= inv;
  store8(dx + (long)t * row_elems + piece * 8, pack8<T>(acc));
}

// ---- dx, weighted
template <typename T, int DIM>
__global__ void __launch_bounds__(256)
compress_dx_kernel(const T* __restrict__ w_lin, const T* __restrict__ d_out, T* __restrict__ dx,
                   const int32_t* __restrict__ cu_seq, const int32_t* __restrict__ cu_out, int batch, int heads,
                   int block, int stride) {
  constexpr int NG = 2;
  const int lane = threadIdx.x & 63;
  const int n = lane & 15, g = lane >> 4;
  const int phase = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (phase >= stride) return;
  // super tile: NG*16 window starts = NG*16*stride tokens of one sequence
  int tile = blockIdx.x, b = 0, start = 0, len = 0;
  bool found = false;
  for (int prev = cu_seq[0]; b < batch; ++b) {
    const int next = cu_seq[b + 1];
    len = next - prev;
    const int nt = (len + NG * 16 * stride - 1) / (NG * 16 * stride);
    if (tile < nt) { start = prev; found = true; break; }
    tile -= nt;
    prev = next;
  }
  if (!found) return;
  const int h = blockIdx.z;
  const int nc = cu_out[b + 1] - cu_out[b];
  const long obase = cu_out[b];
  const int m0 = tile * NG * 16;
  f32x4_t acc[NG][DIM / 16];
#pragma unroll
  for (int j = 0; j < NG; ++j)
#pragma unroll
    for (int t = 0; t < DIM / 16; ++t) acc[j][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int q = 0; phase + q * stride < block; ++q) {
    const int j = phase + q * stride;
    vec8_t<T> bf[NG][DIM / 32];
#pragma unroll
    for (int gi = 0; gi < NG; ++gi) {
      const int win = m0 + gi * 16 + n - q;                    // window whose element j is this lane's token
      const bool ok = win >= 0 && win < nc;
      const T* src = d_out + ((obase + (ok ? win : 0)) * heads + h) * DIM + 8 * g;
#pragma unroll
      for (int kk = 0; kk < DIM / 32; ++kk) bf[gi][kk] = ok ? load8(src + 32 * kk) : zero8<T>();
    }
#pragma unroll
    for (int t = 0; t < DIM / 16; ++t) {
      const T* wrow = w_lin + ((long)j * DIM + 16 * t + n) * DIM + 8 * g;
#pragma unroll
      for (int kk = 0; kk < DIM / 32; ++kk) {
        const vec8_t<T> wa = load8(wrow + 32 * kk);
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) acc[gi][t] = mma16(wa, bf[gi][kk], acc[gi][t]);
      }
    }
  }
#pragma unroll
  for (int gi = 0; gi < NG; ++gi) {
    const int tl = phase + (m0 + gi * 16 + n) * stride;
    if (tl < len) {
      T* dst = dx + (((long)start + tl) * heads + h) * DIM + 4 * g;
#pragma unroll
      for (int t = 0; t < DIM / 16; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[16 * t + i] = (T)acc[gi][t][i];
    }
  }
}

// ---- dW: one workgroup per (j, chunk of kDwRows (window, head) rows)
constexpr int kDwRows = 256;

template <typename T, int DIM>
__global__ void __launch_bounds__(256)
compress_dw_kernel(const T* __restrict__ x, const T* __restrict__ d_out, float* __restrict__ dw,
                   const int32_t* __restrict__ cu_seq, const int32_t* __restrict__ cu_out, int batch, int heads,
                   int stride) {
  constexpr int LD = DIM + 8, TI = (DIM / 16 + 3) / 4, TO = DIM / 16;
  __shared__ __attribute__((aligned(16))) T xs[32 * LD];
  __shared__ __attribute__((aligned(16))) T ds[32 * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int j = blockIdx.y;
  const long rows = (long)cu_out[batch] * heads;
  const long r_begin = (long)blockIdx.x * kDwRows;
  if (r_begin >= rows) return;
  f32x4_t acc[TI][TO];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int t = 0; t < TO; ++t) acc[a][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int step = 0; step < kDwRows / 32; ++step) {
    const long r0 = r_begin + step * 32;
    if (r0 >= rows) break;                                            // uniform over the workgroup
    for (int p = tid; p < 32 * (DIM / 8); p += 256) {
      const int r = p / (DIM / 8), pc = p % (DIM / 8);
      const long row = r0 + r;
      vec8_t<T> xv = zero8<T>(), dv = zero8<T>();
      if (row < rows) {
        const int win = (int)(row / heads), h = (int)(row % heads);
        const int b = upper_seq_of(cu_out, batch, win);
        const long tok = (long)cu_seq[b] + (long)(win - cu_out[b]) * stride + j;
        xv = load8(x + (tok * heads + h) * DIM + pc * 8);
        dv = load8(d_out + row * DIM + pc * 8);
      }
      store8(xs + r * LD + pc * 8, xv);
      store8(ds + r * LD + pc * 8, dv);
    }
    __syncthreads();
    vec8_t<T> bfr[TO];
#pragma unroll
    for (int t = 0; t < TO; ++t) bfr[t] = load8_tr(ds + 16 * t, LD, lane);
#pragma unroll
    for (int a = 0; a < TI; ++a) {
      const int ti = wave + 4 * a;
      if (ti < DIM / 16) {
        const vec8_t<T> af = load8_tr(xs + 16 * ti, LD, lane);
#pragma unroll
        for (int t = 0; t < TO; ++t) acc[a][t] = mma16(af, bfr[t], acc[a][t]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int a = 0; a < TI; ++a) {
    const int ti = wave + 4 * a;
    if (ti < DIM / 16) {
#pragma unroll
      for (int t = 0; t < TO; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          unsafeAtomicAdd(dw + ((long)j * DIM + 16 * ti + 4 * g + i) * DIM + 16 * t + n, acc[a][t][i]);
    }
  }
}

// db[o] += sum over a chunk of rows of d_out[row][o]
template <typename T>
__global__ void __launch_bounds__(256)
compress_db_kernel(const T* __restrict__ d_out, float* __restrict__ db, const int32_t* __restrict__ cu_out, int batch,
                   int heads, int dim) {
  const long rows = (long)cu_out[batch] * heads;
  const long r_begin = (long)blockIdx.x * 256;
  const int c = threadIdx.x;
  if (c >= dim || r_begin >= rows) return;
  float acc = 0.f;
  const long r_end = min(rows, r_begin + 256);
  for (long r = r_begin; r < r_end; ++r) acc += (float)d_out[r * dim + c];
  unsafeAtomicAdd(db + c, acc);
}

__global__ void __launch_bounds__(256)
compress_zero_kernel(float* __restrict__ p, long n) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

template <typename T>
static int launch_compress_bwd_t(const CompressBwdArgs& a, hipStream_t st) {
  const T* d_out = reinterpret_cast<const T*>(a.d_out);
  T* dx = reinterpret_cast<T*>(a.dx);
  if (a.w_lin == nullptr) {
    const long threads = (long)a.total * (a.heads * a.dim / 8);
    hipLaunchKernelGGL(compress_mean_bwd_kernel<T>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, d_out,
                       dx, a.cu_seq, a.cu_out, a.batch, a.total, a.heads * a.dim, a.block, a.stride);
    return 0;
  }
  const T* w = reinterpret_cast<const T*>(a.w_lin);
  const T* x = reinterpret_cast<const T*>(a.x);
  const dim3 gx(a.total / (32 * a.stride) + a.batch, (a.stride + 3) / 4, a.heads);
  const long wn = (long)a.block * a.dim * a.dim;
  if (a.dw != nullptr)
    hipLaunchKernelGGL(compress_zero_kernel, dim3((unsigned)((wn + 255) / 256)), dim3(256), 0, st, a.dw, wn);
  if (a.dbias != nullptr) hipLaunchKernelGGL(compress_zero_kernel, dim3(1), dim3(256), 0, st, a.dbias, (long)a.dim);
  const int chunks = (int)(((long)a.out_rows_bound * a.heads + kDwRows - 1) / kDwRows);
  if (a.dbias != nullptr && chunks > 0)
    hipLaunchKernelGGL(compress_db_kernel<T>, dim3(chunks), dim3(256), 0, st, d_out, a.dbias, a.cu_out, a.batch,
                       a.heads, a.dim);
#define NSA_CBWD(D)                                                                                            \
  hipLaunchKernelGGL((compress_dx_kernel<T, D>), gx, dim3(256), 0, st, w, d_out, dx, a.cu_seq, a.cu_out,       \
                     a.batch, a.heads, a.block, a.stride);                                                     \
  if (a.dw != nullptr && chunks > 0)                                                                           \
    hipLaunchKernelGGL((compress_dw_kernel<T, D>), dim3(chunks, a.block), dim3(256), 0, st, x, d_out, a.dw,    \
                       a.cu_seq, a.cu_out, a.batch, a.heads, a.stride)
  switch (a.dim) {
    case 32: NSA_CBWD(32); break;
    case 64: NSA_CBWD(64); break;
    case 128: NSA_CBWD(128); break;
    case 192: NSA_CBWD(192); break;
    default: return -2;
  }
#undef NSA_CBWD
  return 0;
}

int launch_compress_bwd(const CompressBwdArgs& a, hipStream_t st) {
  if (a.dtype == 2) return launch_compress_bwd_t<f16_t>(a, st);
  return a.dtype == 0 ? launch_compress_bwd_t<bf16_t>(a, st) : launch_compress_bwd_t<float>(a, st);
}

}  // namespace nsa
