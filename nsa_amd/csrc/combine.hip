// Gated sum of the three branches as stand-alone kernels, and the backward of the gates, for the
// training path (the inference path folds the sum into the attention epilogues).
//   forward   out = act(x_slc) o_slc + act(x_swa) o_swa + act(x_cmp) o_cmp      (nsa/nsa.py:117-133)
//   backward  d_o_b = act(x_b) d_out,  d_x_b = act'(x_b) <d_out, o_b>;  on request the row sums <d_out, o_b> and
//             the gates act(x_b) are written out instead of (or next to) the scaled copies d_o_b, for attention
//             backward kernels that take d_out itself plus a per-row scale
//   gating Linear x = W q + b (nsa/nsa.py:61,117):  dq = d_x W,  dW = d_x^T q,  db = sum d_x
// All three are HBM streaming kernels: every operand is read once, 16 lanes share one (token, head) row.
#include "common.h"
#include "kernels.h"

namespace nsa {

__device__ __forceinline__ float act_of(float x, int act) { return act == 1 ? 1.0f / (1.0f + __expf(-x)) : x; }

template <typename T>
__global__ void __launch_bounds__(256)
gate_combine_fwd_kernel(const T* __restrict__ gl, const T* __restrict__ o_slc, const T* __restrict__ o_swa,
                        const T* __restrict__ o_cmp, T* __restrict__ out, long rows, int dv, int act) {
  const int ppr = dv / 8;
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  if (id >= rows * ppr) return;
  const long row = id / ppr;
  const int pc = (int)(id % ppr);
  const T* branch[3] = {o_slc, o_swa, o_cmp};
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
  for (int b = 0; b < 3; ++b) {
    if (branch[b] == nullptr) continue;
    const float g = act_of((float)gl[row * 3 + b], act);
    const vec8_t<T> o = load8(branch[b] + row * dv + pc * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = fmaf(g, (float)o[e], acc[e]);
  }
  store8(out + row * dv + pc * 8, pack8<T>(acc));
}

template <typename T>
__global__ void __launch_bounds__(256)
gate_combine_bwd_kernel(const T* __restrict__ gl, const T* __restrict__ d_out, const T* __restrict__ o_slc,
                        const T* __restrict__ o_swa, const T* __restrict__ o_cmp, T* __restrict__ d_slc,
                        T* __restrict__ d_swa, T* __restrict__ d_cmp, T* __restrict__ d_gl, float* __restrict__ stats,
                        long rows, int dv, int act) {
  const long row = ((long)blockIdx.x * 256 + threadIdx.x) >> 4;
  const int sub = threadIdx.x & 15;
  const bool live = row < rows;
  const T* branch[3] = {o_slc, o_swa, o_cmp};
  T* grad[3] = {d_slc, d_swa, d_cmp};
  float x[3], g[3], dot[3] = {0.f, 0.f, 0.f};
#pragma unroll
  for (int b = 0; b < 3; ++b) {
    x[b] = live ? (float)gl[row * 3 + b] : 0.f;
    g[b] = act_of(x[b], act);
  }
  if (live) {
    for (int c = sub * 8; c < dv; c += 128) {
      const vec8_t<T> d = load8(d_out + row * dv + c);
#pragma unroll
      for (int b = 0; b < 3; ++b) {
        if (branch[b] == nullptr) continue;
        const vec8_t<T> o = load8(branch[b] + row * dv + c);
        float s[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          dot[b] = fmaf((float)d[e], (float)o[e], dot[b]);
          s[e] = g[b] * (float)d[e];
        }
        if (grad[b] != nullptr) store8(grad[b] + row * dv + c, pack8<T>(s));
      }
    }
  }
#pragma unroll
  for (int b = 0; b < 3; ++b)
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) dot[b] += __shfl_xor(dot[b], off, 16);
  if (live && sub < 3) {
    const float dg = sub == 0 ? dot[0] : (sub == 1 ? dot[1] : dot[2]);
    const float gg = sub == 0 ? g[0] : (sub == 1 ? g[1] : g[2]);
    d_gl[row * 3 + sub] = (T)(act == 1 ? dg * gg * (1.0f - gg) : dg);
    if (stats != nullptr) {
      stats[(long)sub * rows + row] = dg;
      stats[(long)(3 + sub) * rows + row] = gg;
    }
  }
}

// rows handled by one workgroup of the Linear's backward
constexpr int kGateRows = 2048;

template <typename T, int DIM>
__global__ void __launch_bounds__(256)
gate_linear_bwd_kernel(const T* __restrict__ q, const T* __restrict__ w, const T* __restrict__ d_gl, T* __restrict__ dq,
                       float* __restrict__ dw, float* __restrict__ db, long rows) {
  constexpr int PIECES = DIM / 8, PPL = (PIECES + 15) / 16;          // 8-channel pieces per lane
  __shared__ float red[16][3 * DIM + 3];
  const int sub = threadIdx.x & 15, grp = threadIdx.x >> 4;
  float wv[PPL][3][8], aw[PPL][3][8], ab[3] = {0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < PPL; ++i) {
    const int p = sub + 16 * i;
#pragma unroll
    for (int o = 0; o < 3; ++o) {
      vec8_t<T> x = zero8<T>();
      if (p < PIECES) x = load8(w + (long)o * DIM + 8 * p);
#pragma unroll
      for (int e = 0; e < 8; ++e) { wv[i][o][e] = (float)x[e]; aw[i][o][e] = 0.f; }
    }
  }
  const long r_begin = (long)blockIdx.x * kGateRows;
  const long r_end = r_begin + kGateRows < rows ? r_begin + kGateRows : rows;
  for (long row = r_begin + grp; row < r_end; row += 16) {
    float d[3];
#pragma unroll
    for (int o = 0; o < 3; ++o) d[o] = (float)d_gl[row * 3 + o];
    if (sub == 0) { ab[0] += d[0]; ab[1] += d[1]; ab[2] += d[2]; }
#pragma unroll
    for (int i = 0; i < PPL; ++i) {
      const int p = sub + 16 * i;
      if (p < PIECES) {
        const vec8_t<T> x = load8(q + row * DIM + 8 * p);
        float out[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xe = (float)x[e];
          out[e] = d[0] * wv[i][0][e] + d[1] * wv[i][1][e] + d[2] * wv[i][2][e];
#pragma unroll
          for (int o = 0; o < 3; ++o) aw[i][o][e] = fmaf(d[o], xe, aw[i][o][e]);
        }
        store8(dq + row * DIM + 8 * p, pack8<T>(out));
      }
    }
  }
  // reduce the 16 row groups of the workgroup, then one atomic per weight element
#pragma unroll
  for (int i = 0; i < PPL; ++i) {
    const int p = sub + 16 * i;
    if (p < PIECES)
#pragma unroll
      for (int o = 0; o < 3; ++o)
#pragma unroll
        for (int e = 0; e < 8; ++e) red[grp][o * DIM + 8 * p + e] = aw[i][o][e];
  }
  if (sub == 0) { red[grp][3 * DIM] = ab[0]; red[grp][3 * DIM + 1] = ab[1]; red[grp][3 * DIM + 2] = ab[2]; }
  __syncthreads();
  for (int c = threadIdx.x; c < 3 * DIM + 3; c += 256) {
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) s += red[r][c];
    if (c < 3 * DIM) unsafeAtomicAdd(dw + c, s);
    else if (db != nullptr) unsafeAtomicAdd(db + (c - 3 * DIM), s);
  }
}

__global__ void __launch_bounds__(256)
gate_zero_kernel(float* __restrict__ a, int na, float* __restrict__ b, int nb) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < na) a[i] = 0.f;
  if (b != nullptr && i < nb) b[i] = 0.f;
}

template <typename T>
static int gate_combine_t(const GateCombineArgs& a, hipStream_t st) {
  const T* gl = reinterpret_cast<const T*>(a.gate_logits);
  if (a.d_out == nullptr) {
    const long threads = a.rows * (a.dv / 8);
    hipLaunchKernelGGL((gate_combine_fwd_kernel<T>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, gl,
                       (const T*)a.o_slc, (const T*)a.o_swa, (const T*)a.o_cmp, (T*)a.out, a.rows, a.dv, a.act);
  } else {
    hipLaunchKernelGGL((gate_combine_bwd_kernel<T>), dim3((unsigned)((a.rows * 16 + 255) / 256)), dim3(256), 0, st,
                       gl, (const T*)a.d_out, (const T*)a.o_slc, (const T*)a.o_swa, (const T*)a.o_cmp, (T*)a.d_slc,
                       (T*)a.d_swa, (T*)a.d_cmp, (T*)a.d_gate_logits, a.stats, a.rows, a.dv, a.act);
  }
  return 0;
}

int launch_gate_combine(const GateCombineArgs& a, hipStream_t st) {
  if (a.dtype == 2) return gate_combine_t<f16_t>(a, st);
  return a.dtype == 0 ? gate_combine_t<bf16_t>(a, st) : gate_combine_t<float>(a, st);
}

template <typename T>
static int gate_bwd_t(const void* q, const void* w, const void* d_gl, void* dq, float* dw, float* db, long rows,
                      int dim, hipStream_t st) {
  hipLaunchKernelGGL(gate_zero_kernel, dim3((3 * dim + 255) / 256), dim3(256), 0, st, dw, 3 * dim, db, 3);
  const dim3 grid((unsigned)((rows + kGateRows - 1) / kGateRows));
#define NSA_GATE_BWD(D)                                                                                         \
  hipLaunchKernelGGL((gate_linear_bwd_kernel<T, D>), grid, dim3(256), 0, st, (const T*)q, (const T*)w,          \
                     (const T*)d_gl, (T*)dq, dw, db, rows)
  switch (dim) {
    case 32: NSA_GATE_BWD(32); break;
    case 64: NSA_GATE_BWD(64); break;
    case 128: NSA_GATE_BWD(128); break;
    case 192: NSA_GATE_BWD(192); break;
    case 256: NSA_GATE_BWD(256); break;
    default: return -2;
  }
#undef NSA_GATE_BWD
  return 0;
}

int launch_gate_bwd(const void* q, const void* w, const void* d_gl, void* dq, float* dw, float* db, long rows,
                    int dim, int dtype, hipStream_t st) {
  if (dtype == 2) return gate_bwd_t<f16_t>(q, w, d_gl, dq, dw, db, rows, dim, st);
  return dtype == 0 ? gate_bwd_t<bf16_t>(q, w, d_gl, dq, dw, db, rows, dim, st)
                    : gate_bwd_t<float>(q, w, d_gl, dq, dw, db, rows, dim, st);
}

}  // namespace nsa
