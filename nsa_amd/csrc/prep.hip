// KV block compression and the key-contiguous ("transposed") copy the attention kernels read V from.
//
// compress (mean-pool): pure HBM streaming. One thread owns 8 contiguous channels of one output
//   row; consecutive threads cover one full [heads*dim] token row, so every load instruction of a
//   wavefront reads whole contiguous token rows. Each input row is needed by block/stride output
//   rows; the second use hits L2. Algorithmic bytes: rows_in*heads*dim*sizeof(T) read +
//   rows_out*heads*dim*sizeof(T) written.
// compress (weighted): out[n][o] = b[o] + sum_{j,i} x[n*stride+j][i] * Wt[o][j*dim+i] as an MFMA
//   GEMM with the [dim_out x block*dim] weight (L2 resident) as the A operand, split over the taps j
//   between the wavefronts of a workgroup and summed in LDS.
// transpose: out[h][d][col] = x[row(col)][h][d], 64-column tiles through LDS.
#include "common.h"
#include "kernels.h"

namespace nsa {

int set_smem(const void* fn, size_t bytes);

__device__ __forceinline__ int upper_seq(const int32_t* __restrict__ cu, int batch, int r) {
  // largest b in [0,batch) with cu[b] <= r   (cu non-decreasing, cu[0] <= r assumed)
  int lo = 0, hi = batch;  // invariant: cu[lo] <= r, answer in [lo, hi)
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= r) lo = mid; else hi = mid;
  }
  return lo;
}

// One or two tensors over the same token axis (K and V of a layer) in one launch: blockIdx.y picks the tensor.
#ifndef NSA_MEAN_U
#define NSA_MEAN_U 32
#endif
struct MeanOperand {
  const void* x;
  void* out;
  int dim;
};

// U rows of the window are requested before the first is added: the kernel is a pure stream whose time is the
// memory latency times the number of dependent rounds, so a 32-row window is one round (bf16) or two (fp32).
template <typename T>
__global__ void __launch_bounds__(256)
compress_mean_kernel(const MeanOperand s0, const MeanOperand s1, const int32_t* __restrict__ cu_seq,
                     const int32_t* __restrict__ cu_out, int batch, int heads, int block, int stride) {
  constexpr int U = NSA_MEAN_U / (int)(sizeof(T) / 2);
  const MeanOperand s = blockIdx.y == 0 ? s0 : s1;
  const int row_elems = heads * s.dim;
  const int ppr = row_elems / 8;  // 8-element pieces per token row
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const int r = (int)(idx / ppr);
  const int piece = (int)(idx % ppr);
  if (r >= cu_out[batch]) return;
  const int b = upper_seq(cu_out, batch, r);
  const int n = r - cu_out[b];
  const T* src = reinterpret_cast<const T*>(s.x) + ((long)cu_seq[b] + (long)n * stride) * row_elems + piece * 8;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  for (int j0 = 0; j0 < block; j0 += U) {
    vec8_t<T> v[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (j0 + u < block) v[u] = load8(src + (long)(j0 + u) * row_elems);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (j0 + u < block) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] += (float)v[u][i];
      }
  }
  const float inv = 1.0f / (float)block;
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] *= inv;
  store8(reinterpret_cast<T*>(s.out) + (long)r * row_elems + piece * 8, pack8<T>(acc));
}

// The same for windows of two strides (block == 2 * stride, stride <= 16: the usual 32 / 16), reading every token
// row about once instead of twice.  A wavefront is 8 stride groups x 8 pieces (64 channels): lane (s, p) sums the
// `stride` rows of group s -- the first half of output row r0 + s -- and takes the second half from lane (s + 1, p),
// which has just summed exactly those rows as the first half of the next output row.  Lane group 7 only helps
// (its output row belongs to the next wavefront); a lane whose neighbour is past the end or in another sequence
// sums its second half itself.
template <typename T>
__global__ void __launch_bounds__(256)
compress_mean_halves_kernel(const MeanOperand s0, const MeanOperand s1, const int32_t* __restrict__ cu_seq,
                            const int32_t* __restrict__ cu_out, int batch, int heads, int stride) {
  constexpr int U = 16;
  const MeanOperand sp = blockIdx.y == 0 ? s0 : s1;
  const int row_elems = heads * sp.dim;
  const int cblocks = row_elems / 64;
  const int lane = threadIdx.x & 63, s = lane >> 3, p = lane & 7;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);       // (run of 7 output rows, 64-channel block)
  const int total_out = cu_out[batch];
  const long r0 = (item / cblocks) * 7;
  if (r0 >= total_out) return;
  const int col = (int)(item % cblocks) * 64 + p * 8;
  const long r = r0 + s;
  const bool valid = r < total_out;
  int b = -1;
  const T* src = reinterpret_cast<const T*>(sp.x);
  if (valid) {
    b = upper_seq(cu_out, batch, (int)r);
    src += ((long)cu_seq[b] + (r - cu_out[b]) * stride) * row_elems + col;
  }
  auto half_sum = [&](const T* base, float (&acc)[8]) {
    vec8_t<T> v[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (u < stride) v[u] = load8(base + (long)u * row_elems);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (u < stride) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] += (float)v[u][i];
      }
  };
  float g1[8], g2[8];
  if (valid) half_sum(src, g1);
  else {
#pragma unroll
    for (int i = 0; i < 8; ++i) g1[i] = 0.f;
  }
  const int b_next = __shfl_down(b, 8);
#pragma unroll
  for (int i = 0; i < 8; ++i) g2[i] = __shfl_down(g1[i], 8);
  if (!valid || s == 7) return;
  if (b_next != b) half_sum(src + (long)stride * row_elems, g2);     // b_next is -1 past the end
  const float inv = 0.5f / (float)stride;
  float o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = (g1[i] + g2[i]) * inv;
  store8(reinterpret_cast<T*>(sp.out) + r * row_elems + col, pack8<T>(o));
}

// One workgroup per (32 output rows, head).  The block's taps are dealt to the 4 wavefronts (split-K):
// each multiplies its taps' weight slices (A operand, straight from L2) with the rows' inputs (B operand,
// two 16-row groups per weight fragment) and adds its [32 x DIM] partial sum into an fp32 LDS tile, from
// which whole rows are written with the bias.  4 x the wavefronts of a one-wavefront-per-tile layout:
// the GEMM is small (Nc x l*D x D) and otherwise leaves most SIMDs idle, waiting on L2 latency.
template <typename T, int DIM>
__global__ void __launch_bounds__(256)
compress_weighted_kernel(const T* __restrict__ x, const T* __restrict__ wt, const T* __restrict__ bias,
                         T* __restrict__ out, const int32_t* __restrict__ cu_seq,
                         const int32_t* __restrict__ cu_out, int batch, int heads, int block, int stride) {
  constexpr int NG = 2, LD = DIM + 4;
  __shared__ float tile[NG * 16 * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int total_out = cu_out[batch];
  const int r0 = blockIdx.x * NG * 16, h = blockIdx.y;
  if (r0 >= total_out) return;
  for (int e = tid; e < NG * 16 * LD; e += 256) tile[e] = 0.f;
  const T* xrow[NG];
#pragma unroll
  for (int gi = 0; gi < NG; ++gi) {
    const int rc = min(r0 + gi * 16 + n, total_out - 1);
    const int b = upper_seq(cu_out, batch, rc);
    xrow[gi] = x + (((long)cu_seq[b] + (long)(rc - cu_out[b]) * stride) * heads + h) * DIM + 8 * g;
  }
  f32x4_t acc[NG][DIM / 16];
#pragma unroll
  for (int gi = 0; gi < NG; ++gi)
#pragma unroll
    for (int t = 0; t < DIM / 16; ++t) acc[gi][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int K = block * DIM;
  __syncthreads();
  for (int j = wave; j < block; j += 4) {
    vec8_t<T> xb[NG][DIM / 32];
#pragma unroll
    for (int gi = 0; gi < NG; ++gi)
#pragma unroll
      for (int kk = 0; kk < DIM / 32; ++kk) xb[gi][kk] = load8(xrow[gi] + (long)j * heads * DIM + 32 * kk);
#pragma unroll
    for (int t = 0; t < DIM / 16; ++t) {
      const T* wrow = wt + (long)(t * 16 + n) * K + j * DIM + 8 * g;
#pragma unroll
      for (int kk = 0; kk < DIM / 32; ++kk) {
        const vec8_t<T> wa = load8(wrow + 32 * kk);
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) acc[gi][t] = mma16(wa, xb[gi][kk], acc[gi][t]);
      }
    }
  }
#pragma unroll
  for (int gi = 0; gi < NG; ++gi)
#pragma unroll
    for (int t = 0; t < DIM / 16; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) atomicAdd(&tile[(gi * 16 + n) * LD + 16 * t + 4 * g + i], acc[gi][t][i]);
  __syncthreads();
  for (int p = tid; p < NG * 16 * (DIM / 8); p += 256) {
    const int r = p / (DIM / 8), pc = p % (DIM / 8);
    if (r0 + r >= total_out) continue;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[e] = tile[r * LD + pc * 8 + e];
      if (bias != nullptr) v[e] += (float)bias[pc * 8 + e];
    }
    store8(out + ((long)(r0 + r) * heads + h) * DIM + pc * 8, pack8<T>(v));
  }
}

// The learned compressor as a tiled GEMM (16-bit types): out[row][:] = sum_j x[token(row) + j][:] W_j + bias, i.e.
// [rows x block*DIM] x [block*DIM x DIM] per head with rows that overlap in memory (row r of sequence b starts at
// token cu_seq[b] + r*stride).  One workgroup owns 64 output rows of one head and ALL DIM output channels; the
// reduction runs in steps of 64 (one 64-channel slice of one tap, two matrix-instruction depths).  A step's operands
// -- 2 x 4 x fragments and 2 x DIM / 16 weight fragments of 1 KB -- go from global memory straight into LDS
// (global_load_lds: every lane names the 16 bytes of its place in the fragment, so the tile arrives in fragment
// order and the reads are conflict-free) through a ring of kGemmRing step buffers, kGemmRing - 1 steps ahead: the
// GEMM is small (one workgroup per CU), so nothing but the loads in flight hides the memory latency.  One barrier
// per step.  The four wavefronts split the output channels; each weight fragment read from LDS feeds four matrix
// instructions (the four 16-row groups), each x fragment DIM / 64.  K and V of a layer go in ONE launch
// (blockIdx.z picks the tensor).  A 64-row tile takes in block * DIM * 2 * (64 + DIM) bytes for
// 2 * 64 * DIM * block * DIM flops; measured, a workgroup receives about 14 bytes per clock with either step depth
// (32 or 64) and either ring length (8 or 4), which is what bounds the kernel, not the matrix instructions.
constexpr int kGemmRing = 4;

__device__ __forceinline__ void gemm_wait_loads(int n) {      // at most n vector-memory loads of this wavefront outstanding
  switch (n) {
#define NSA_WAIT_CASE(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    NSA_WAIT_CASE(4) NSA_WAIT_CASE(8) NSA_WAIT_CASE(12) NSA_WAIT_CASE(16) NSA_WAIT_CASE(20) NSA_WAIT_CASE(24)
    NSA_WAIT_CASE(2) NSA_WAIT_CASE(6) NSA_WAIT_CASE(10) NSA_WAIT_CASE(14) NSA_WAIT_CASE(18)
    NSA_WAIT_CASE(3) NSA_WAIT_CASE(9) NSA_WAIT_CASE(15)
#undef NSA_WAIT_CASE
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}

template <typename T>
__device__ __forceinline__ void gemm_global_to_lds16(const T* src, const T* lds) {
  const unsigned dst = (unsigned)(uintptr_t)((__attribute__((address_space(3))) const char*)lds);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(src), "s"(dst) : "memory");
}

template <typename T, int DIM>
__device__ __forceinline__ void compress_gemm_body(const T* __restrict__ x, const T* __restrict__ wt,
                                                   const T* __restrict__ bias, T* __restrict__ out,
                                                   const int32_t* __restrict__ cu_seq,
                                                   const int32_t* __restrict__ cu_out, int batch, int heads, int block,
                                                   int stride, unsigned char* smem) {
  constexpr int TM = 64, NCT = DIM / 64;               // 16-channel tiles per wavefront
  constexpr int SLOT = 2 * (4 + DIM / 16) * 512;       // elements of one 64-deep step's operands in LDS
  constexpr int LPS = 2 * (1 + NCT);                   // loads per step and wavefront
  static_assert(DIM % 64 == 0, "the output channels are dealt to four wavefronts in 16-channel tiles");
  T* ring = reinterpret_cast<T*>(smem);                // [kGemmRing][2 halves][x fragments 0..3 | weight fragments]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int total_out = cu_out[batch];
  const int m0 = blockIdx.x * TM, h = blockIdx.y;
  if (m0 >= total_out) return;
  const int K = block * DIM;
  // wavefront w brings x fragment w (rows m0 + 16 w ..) and the weight fragments of its own channel tiles; the two
  // 32-deep halves of a step are requested back to back: together a lane group reads whole 128-byte lines
  const T* xsrc;
  {
    const int rc = min(m0 + wave * 16 + (lane & 15), total_out - 1);
    const int b = upper_seq(cu_out, batch, rc);
    xsrc = x + (((long)cu_seq[b] + (long)(rc - cu_out[b]) * stride) * heads + h) * DIM + 8 * (lane >> 4);
  }
  const T* wsrc = wt + (long)(wave * NCT * 16 + (lane & 15)) * K + 8 * (lane >> 4);
  f32x4_t acc[4][NCT];
#pragma unroll
  for (int rg = 0; rg < 4; ++rg)
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) acc[rg][ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int steps = block * (DIM / 64);
  auto issue = [&](int s) {
    const int j = s / (DIM / 64), kk = s % (DIM / 64);
    T* slot = ring + (s % kGemmRing) * SLOT;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
      gemm_global_to_lds16(xsrc + (long)j * heads * DIM + 64 * kk + 32 * hf, slot + hf * (SLOT / 2) + wave * 512);
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
        gemm_global_to_lds16(wsrc + (long)ct * 16 * K + 64 * s + 32 * hf,
                             slot + hf * (SLOT / 2) + (4 + wave * NCT + ct) * 512);
  };
  for (int s = 0; s < kGemmRing - 1 && s < steps; ++s) issue(s);
  for (int s = 0; s < steps; ++s) {
    // steps s + 1 .. min(s + kGemmRing - 2, steps - 1) may still be in flight; step s must have landed
    gemm_wait_loads(LPS * (min(s + kGemmRing - 2, steps - 1) - s));
    __syncthreads();                                   // everybody's part of step s is in; step s - 1 is consumed
    if (s + kGemmRing - 1 < steps) issue(s + kGemmRing - 1);
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const T* xb = ring + (s % kGemmRing) * SLOT + hf * (SLOT / 2) + lane * 8;
      const T* wb = xb + (4 + wave * NCT) * 512;
      vec8_t<T> xf[4];
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) xf[rg] = load8(xb + rg * 512);
#pragma unroll
      for (int ct = 0; ct < NCT; ++ct) {
        const vec8_t<T> wa = load8(wb + ct * 512);
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) acc[rg][ct] = mma16(wa, xf[rg], acc[rg][ct]);   // out^T tile: rows = channels
      }
    }
  }
  __syncthreads();
  // epilogue through LDS: lane (n, g) holds channels 4g .. 4g+3 of row n; whole rows leave in 16-byte pieces
  constexpr int LD = DIM + 4;
  float* tile = reinterpret_cast<float*>(smem);        // [64][LD]  (the ring is free: last barrier passed)
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int rg = 0; rg < 4; ++rg)
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) tile[(rg * 16 + n) * LD + (wave * NCT + ct) * 16 + 4 * g + i] = acc[rg][ct][i];
  __syncthreads();
  for (int p = tid; p < TM * (DIM / 8); p += 256) {
    const int r = p / (DIM / 8), pc = p % (DIM / 8);
    if (m0 + r >= total_out) continue;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[e] = tile[r * LD + pc * 8 + e];
      if (bias != nullptr) v[e] += (float)bias[pc * 8 + e];
    }
    store8(out + ((long)(m0 + r) * heads + h) * DIM + pc * 8, pack8<T>(v));
  }
}

struct GemmOperand { const void* x; const void* wt; const void* bias; void* out; };

template <typename T> constexpr size_t compress_gemm_smem(int dmax) {
  const size_t ring = (size_t)kGemmRing * 2 * (4 + dmax / 16) * 512 * sizeof(T), epi = (size_t)64 * (dmax + 4) * 4;
  return ring > epi ? ring : epi;
}

template <typename T, int D0, int D1>
__global__ void __launch_bounds__(256)
compress_gemm_kernel(const GemmOperand s0, const GemmOperand s1, const int32_t* __restrict__ cu_seq,
                     const int32_t* __restrict__ cu_out, int batch, int heads, int block, int stride) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];      // compress_gemm_smem<T>(max(D0, D1))
  if (blockIdx.z == 0)
    compress_gemm_body<T, D0>((const T*)s0.x, (const T*)s0.wt, (const T*)s0.bias, (T*)s0.out, cu_seq, cu_out, batch, heads,
                              block, stride, smem);
  else
    compress_gemm_body<T, D1>((const T*)s1.x, (const T*)s1.wt, (const T*)s1.bias, (T*)s1.out, cu_seq, cu_out, batch, heads,
                              block, stride, smem);
}

// out[(h*dim + d) * out_cols + col], col = transposed_offset(cu[b], b) + row; every other column is 0.
template <typename T>
__global__ void __launch_bounds__(256)
transpose_kernel(const T* __restrict__ x, T* __restrict__ out, const int32_t* __restrict__ cu, int batch,
                 int dim, long row_stride, long head_stride, int out_cols) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  int* src_row = reinterpret_cast<int*>(smem_raw);           // [64]
  T* tile = reinterpret_cast<T*>(smem_raw + 64 * sizeof(int));  // [64][dim + 8]
  const int ld = dim + 8;
  const int col0 = blockIdx.x * 64;
  const int h = blockIdx.y;
  if (threadIdx.x < 64) {
    const int col = col0 + threadIdx.x;
    int row = -1;
    // largest b with transposed_offset(cu[b], b) <= col
    int lo = 0, hi = batch;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (transposed_offset(cu[mid], mid) <= col) lo = mid; else hi = mid;
    }
    const int rel = col - transposed_offset(cu[lo], lo);
    if (rel >= 0 && rel < cu[lo + 1] - cu[lo]) row = cu[lo] + rel;
    src_row[threadIdx.x] = row;
  }
  __syncthreads();
  const int pieces = dim / 8;
  for (int p = threadIdx.x; p < 64 * pieces; p += 256) {
    const int c = p / pieces, pc = p % pieces;
    const int row = src_row[c];
    vec8_t<T> v = zero8<T>();
    if (row >= 0) v = load8(x + (long)row * row_stride + (long)h * head_stride + pc * 8);
    store8(tile + c * ld + pc * 8, v);
  }
  __syncthreads();
  for (int p = threadIdx.x; p < dim * 8; p += 256) {
    const int d = p >> 3, pc = p & 7;
    vec8_t<T> v;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = tile[(pc * 8 + j) * ld + d];
    store8(out + ((long)h * dim + d) * out_cols + col0 + pc * 8, v);
  }
}

template <typename T>
static int launch_compress_t(const CompressArgs& a, hipStream_t st) {
  if (a.out_rows_bound <= 0) return 0;
  if (a.wt == nullptr) {
    const MeanOperand s0{a.x, a.out, a.dim};
    const MeanOperand s1{a.x2 ? a.x2 : a.x, a.x2 ? a.out2 : a.out, a.x2 ? a.dim2 : a.dim};
    const int dmax = a.x2 && a.dim2 > a.dim ? a.dim2 : a.dim;
    if (a.block == 2 * a.stride && a.stride <= 16 && (a.heads * s0.dim) % 64 == 0 && (a.heads * s1.dim) % 64 == 0) {
      const long items = ((long)a.out_rows_bound + 6) / 7 * (a.heads * dmax / 64);
      const dim3 grid((unsigned)((items + 3) / 4), a.x2 ? 2 : 1);
      hipLaunchKernelGGL(compress_mean_halves_kernel<T>, grid, dim3(256), 0, st, s0, s1, a.cu_seq, a.cu_out, a.batch,
                         a.heads, a.stride);
      return 0;
    }
    const long threads = (long)a.out_rows_bound * (a.heads * dmax / 8);
    const dim3 grid((unsigned)((threads + 255) / 256), a.x2 ? 2 : 1);
    hipLaunchKernelGGL(compress_mean_kernel<T>, grid, dim3(256), 0, st, s0, s1, a.cu_seq, a.cu_out, a.batch, a.heads,
                       a.block, a.stride);
    return 0;
  }
  if constexpr (sizeof(T) == 2) {
    // the tiled GEMM for head dims that split over four wavefronts; K and V of a layer in one launch
    const int d0 = a.dim, d1 = a.x2 ? a.dim2 : a.dim;
    const GemmOperand s0{a.x, a.wt, a.bias, a.out}, s1{a.x2, a.wt2, a.bias2, a.out2};
    const dim3 ggrid((a.out_rows_bound + 63) / 64, a.heads, a.x2 ? 2 : 1);
#define NSA_GEMM(DA, DB)                                                                                     \
    if (d0 == DA && d1 == DB) {                                                                              \
      const size_t smem = compress_gemm_smem<T>(DA > DB ? DA : DB);                                          \
      auto fn = compress_gemm_kernel<T, DA, DB>;                                                             \
      if (const int rc = set_smem(reinterpret_cast<const void*>(fn), smem)) return rc;                       \
      hipLaunchKernelGGL(fn, ggrid, dim3(256), smem, st, s0, s1, a.cu_seq, a.cu_out, a.batch, a.heads, a.block, \
                         a.stride);                                                                          \
      return 0;                                                                                              \
    }
    NSA_GEMM(64, 64) NSA_GEMM(128, 128) NSA_GEMM(192, 192) NSA_GEMM(192, 128)
#undef NSA_GEMM
    if (a.x2) return -7;      // no paired instance for these head dims: the caller launches the tensors one by one
  }
  const dim3 grid((a.out_rows_bound + 31) / 32, a.heads);
#define NSA_WEIGHTED(D)                                                                              \
  hipLaunchKernelGGL((compress_weighted_kernel<T, D>), grid, dim3(256), 0, st, (const T*)a.x, \
                     (const T*)a.wt, (const T*)a.bias, (T*)a.out, a.cu_seq, a.cu_out, a.batch,      \
                     a.heads, a.block, a.stride)
  switch (a.dim) {
    case 32: NSA_WEIGHTED(32); break;
    case 64: NSA_WEIGHTED(64); break;
    case 128: NSA_WEIGHTED(128); break;
    case 192: NSA_WEIGHTED(192); break;
    default: return -2;
  }
#undef NSA_WEIGHTED
  return 0;
}

int launch_compress(const CompressArgs& a, hipStream_t st) {
  if (a.dtype == 2) return launch_compress_t<f16_t>(a, st);
  return a.dtype == 0 ? launch_compress_t<bf16_t>(a, st) : launch_compress_t<float>(a, st);
}

template <typename T>
static int launch_transpose_t(const TransposeArgs& a, hipStream_t st) {
  const size_t smem = 64 * sizeof(int) + (size_t)64 * (a.dim + 8) * sizeof(T);
  hipLaunchKernelGGL(transpose_kernel<T>, dim3(a.out_cols / 64, a.heads), dim3(256), smem, st,
                     (const T*)a.x, (T*)a.out, a.cu, a.batch, a.dim, a.row_stride, a.head_stride,
                     a.out_cols);
  return 0;
}

// Gate logits out[row][o] = bias[o] + sum_i x[row][i] * w[o][i], o = 0..2 (selected, sliding,
// compressed): 16 lanes per (token, head) row, fp32 accumulation, one rounding at the end.
template <typename T>
__global__ void __launch_bounds__(256)
gate_kernel(const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ bias, T* __restrict__ out,
            long rows, int dim) {
  const int l16 = threadIdx.x & 15;
  const long row = (long)blockIdx.x * 16 + (threadIdx.x >> 4);
  float acc[3] = {0.f, 0.f, 0.f};
  if (row < rows) {
    for (int p = l16; p < dim / 8; p += 16) {
      const vec8_t<T> xv = load8(x + row * dim + 8 * p);
#pragma unroll
      for (int o = 0; o < 3; ++o) {
        const vec8_t<T> wv = load8(w + (long)o * dim + 8 * p);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[o] = fmaf((float)xv[i], (float)wv[i], acc[o]);
      }
    }
  }
#pragma unroll
  for (int o = 0; o < 3; ++o)
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) acc[o] += __shfl_xor(acc[o], off, 16);
  if (row < rows && l16 < 3) {
    const float v = l16 == 0 ? acc[0] : (l16 == 1 ? acc[1] : acc[2]);
    out[row * 3 + l16] = (T)(v + (bias != nullptr ? (float)bias[l16] : 0.f));
  }
}

int launch_gate(const void* x, const void* w, const void* bias, void* out, long rows, int dim, int dtype,
                hipStream_t st) {
  const dim3 grid((unsigned)((rows + 15) / 16));
  if (dtype == 0)
    hipLaunchKernelGGL(gate_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)x, (const bf16_t*)w,
                       (const bf16_t*)bias, (bf16_t*)out, rows, dim);
  else if (dtype == 2)
    hipLaunchKernelGGL(gate_kernel<f16_t>, grid, dim3(256), 0, st, (const f16_t*)x, (const f16_t*)w,
                       (const f16_t*)bias, (f16_t*)out, rows, dim);
  else
    hipLaunchKernelGGL(gate_kernel<float>, grid, dim3(256), 0, st, (const float*)x, (const float*)w,
                       (const float*)bias, (float*)out, rows, dim);
  return 0;
}

int launch_transpose(const TransposeArgs& a, hipStream_t st) {
  if (a.dtype == 2) return launch_transpose_t<f16_t>(a, st);
  return a.dtype == 0 ? launch_transpose_t<bf16_t>(a, st) : launch_transpose_t<float>(a, st);
}

}  // namespace nsa
