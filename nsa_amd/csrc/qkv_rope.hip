// Boundary between the fused projection GEMM of an attention layer and the NSA kernels: one pass that
// splits the GEMM's packed output row  [ q | k | v | gate logits ]  into the contiguous tensors the
// attention kernels read, and applies the rotary position embedding to the rotary channels of q and k
// on the way (so the rotation costs no memory traffic of its own).  The reverse direction gathers the
// gradients of the four tensors back into one packed row for the GEMM's backward, with the inverse
// rotation (the transpose of a rotation is the rotation by the negative angle).
//   q [total][hq][dk], k [total][hkv][dk], v [total][hkv][dv], gates [total][hq][3]
//   rotary channels of a head: [rope_off, rope_off + rope_dim); angle of pair i = pos * inv_freq[i]
//   pairing: "half" (channel i with i + rope_dim/2) or interleaved (2i with 2i+1)
// The gate logits are ordinary output columns of the GEMM: the gating Linear of the reference module
// (nsa/nsa.py:61,117) is folded into the projection weights by the host.
// HBM streaming kernel: every element is read once and written once; thread = 8 channels.
#include "common.h"
#include "kernels.h"

namespace nsa {

__device__ __forceinline__ int position_of(const QkvRopeArgs& a, long t) {
  if (a.positions != nullptr) return a.positions[t];
  int lo = 0, hi = a.batch;                 // largest b with cu[b] <= t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a.cu_seq[mid] <= t) lo = mid; else hi = mid;
  }
  return (int)(t - a.cu_seq[lo]);
}

// most rotary pairs per head the kernel keeps angles for
constexpr int kMaxRopePairs = 128;

// grid (token, slice of 256 pieces of the token's row).  The angles depend on the token only, so the
// first rope_dim/2 threads of a workgroup compute the sines and cosines once into LDS.
template <typename T, bool PACK>
__global__ void __launch_bounds__(256)
qkv_rope_kernel(const QkvRopeArgs a) {
  __shared__ float cs[2][kMaxRopePairs];
  const int pq = a.hq * a.dk / 8, pk = a.hkv * a.dk / 8, pv = a.hkv * a.dv / 8;
  const int ng = a.gates != nullptr ? 3 * a.hq : 0;
  const int ppt = pq + pk + pv + (ng + 7) / 8;
  const long t = blockIdx.x;
  const int p = blockIdx.y * 256 + threadIdx.x;
  T* prow = reinterpret_cast<T*>(a.packed) + t * a.ld;
  // 0: nothing, 1: copy, 2: rotate; the loads are issued before the angles are worked out
  int kind = 0, r = 0;
  const T* src = nullptr;
  T* dst = nullptr;
  vec8_t<T> x = zero8<T>(), xp = zero8<T>();
  const int half = a.rope_dim / 2;
  if (p < pq + pk + pv) {
    T* split;
    int c, dim, poff;
    bool rot = a.inv_freq != nullptr;
    if (p < pq) { split = reinterpret_cast<T*>(a.q) + t * a.hq * a.dk; c = 8 * p; dim = a.dk; poff = a.q_off; }
    else if (p < pq + pk) { split = reinterpret_cast<T*>(a.k) + t * a.hkv * a.dk; c = 8 * (p - pq); dim = a.dk; poff = a.k_off; }
    else { split = reinterpret_cast<T*>(a.v) + t * a.hkv * a.dv; c = 8 * (p - pq - pk); dim = a.dv; poff = a.v_off; rot = false; }
    src = PACK ? split + c : prow + poff + c;
    dst = PACK ? prow + poff + c : split + c;
    x = load8(src);
    r = c % dim - a.rope_off;               // first rotary channel of this piece (multiple of 8)
    kind = (rot && r >= 0 && r < a.rope_dim) ? 2 : 1;
    if (kind == 2 && !a.interleaved) xp = load8(src + (r < half ? half : -half));
  } else if (p < ppt) {                     // gate logits: plain columns, any alignment
    T* g = reinterpret_cast<T*>(a.gates) + t * ng;
    const int c0 = 8 * (p - pq - pk - pv);
    for (int e = 0; e < 8 && c0 + e < ng; ++e) {
      if (PACK) prow[a.g_off + c0 + e] = g[c0 + e];
      else g[c0 + e] = prow[a.g_off + c0 + e];
    }
  }
  // slices past the q and k pieces hold nothing to rotate
  if (a.inv_freq != nullptr && blockIdx.y * 256 < pq + pk) {
    if (threadIdx.x < half) {
      const float pos = (float)position_of(a, t);
      float s, co;
      sincosf(pos * a.inv_freq[threadIdx.x], &s, &co);
      cs[0][threadIdx.x] = co;
      cs[1][threadIdx.x] = PACK ? -s : s;
    }
    __syncthreads();
  }
  if (kind == 0) return;
  if (kind == 1) {
    store8(dst, x);
    return;
  }
  float y[8];
  if (a.interleaved) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float co = cs[0][r / 2 + i], s = cs[1][r / 2 + i];
      const float x0 = (float)x[2 * i], x1 = (float)x[2 * i + 1];
      y[2 * i] = x0 * co - x1 * s;
      y[2 * i + 1] = x1 * co + x0 * s;
    }
  } else {
    const bool first = r < half;
    const int f0 = first ? r : r - half;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float co = cs[0][f0 + e], s = first ? -cs[1][f0 + e] : cs[1][f0 + e];
      y[e] = (float)x[e] * co + (float)xp[e] * s;
    }
  }
  store8(dst, pack8<T>(y));
}

template <typename T>
static int qkv_rope_t(const QkvRopeArgs& a, hipStream_t st) {
  const int ppt = (a.hq * a.dk + a.hkv * a.dk + a.hkv * a.dv) / 8 + (a.gates != nullptr ? (3 * a.hq + 7) / 8 : 0);
  const int slices = (ppt + 255) / 256;
  if (a.total > 0x7fffffffL || slices > 65535 || a.rope_dim / 2 > kMaxRopePairs) return -2;
  const dim3 grid((unsigned)a.total, (unsigned)slices);
  if (a.pack) hipLaunchKernelGGL((qkv_rope_kernel<T, true>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((qkv_rope_kernel<T, false>), grid, dim3(256), 0, st, a);
  return 0;
}

int launch_qkv_rope(const QkvRopeArgs& a, hipStream_t st) {
  if (a.dtype == 2) return qkv_rope_t<f16_t>(a, st);
  return a.dtype == 0 ? qkv_rope_t<bf16_t>(a, st) : qkv_rope_t<float>(a, st);
}

}  // namespace nsa
