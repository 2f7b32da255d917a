// MFMA tile pieces shared by the attention kernels: score / PV steps on 32-key chunks, the row
// space mapping (GQA heads of a token = consecutive rows, 16 rows = one tile column group) and
// the global -> LDS staging helpers.
#pragma once
#include "common.h"
#include "kernels.h"

namespace nsa {

// ------------------------------------------------------------------------------------------------
// tile pieces

template <typename T, int DK, int DV, int NG>
__device__ __forceinline__ void scores32(const T* __restrict__ a0p, const T* __restrict__ a1p,
                                         const RowGroup<T, DK, DV> (&grp)[NG], f32x4_t (&s0)[NG],
                                         f32x4_t (&s1)[NG]) {
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    s0[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    s1[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int kk = 0; kk < DK / 32; ++kk) {
    const vec8_t<T> a0 = load8(a0p + 32 * kk);
    const vec8_t<T> a1 = load8(a1p + 32 * kk);
#pragma unroll
    for (int j = 0; j < NG; ++j) {
      s0[j] = mma16(a0, grp[j].q[kk], s0[j]);
      s1[j] = mma16(a1, grp[j].q[kk], s1[j]);
    }
  }
}

template <typename T, int DK, int DV, int NG>
__device__ __forceinline__ void pv32(const T* __restrict__ vp, long tile_stride,
                                     RowGroup<T, DK, DV> (&grp)[NG], const vec8_t<T> (&pb)[NG],
                                     const bool (&active)[NG]) {
#pragma unroll
  for (int t = 0; t < DV / 16; ++t) {
    const vec8_t<T> av = load8(vp + t * tile_stride);
#pragma unroll
    for (int j = 0; j < NG; ++j)
      if (active[j]) grp[j].o[t] = mma16(av, pb[j], grp[j].o[t]);
  }
}

template <typename T, int DK, int DV, int NG>
__device__ __forceinline__ void pv32_all(const T* __restrict__ vp, long tile_stride,
                                         RowGroup<T, DK, DV> (&grp)[NG], const vec8_t<T> (&pb)[NG]) {
#pragma unroll
  for (int t = 0; t < DV / 16; ++t) {
    const vec8_t<T> av = load8(vp + t * tile_stride);
#pragma unroll
    for (int j = 0; j < NG; ++j) grp[j].o[t] = mma16(av, pb[j], grp[j].o[t]);
  }
}

struct RowMap {
  int tok;      // token of this lane's column (sequence local), may be >= len
  int gidx;     // head inside the GQA group, may be >= G
  bool valid;
};

__device__ __forceinline__ RowMap map_row(int t0, int group_in_tile, int n, int lgp, int G, int len) {
  const int r = group_in_tile * 16 + n;
  RowMap m;
  m.tok = t0 + (r >> lgp);
  m.gidx = r & ((1 << lgp) - 1);
  m.valid = (m.tok < len) && (m.gidx < G);
  return m;
}

template <typename T, int DK, int DV>
__device__ __forceinline__ void load_q(RowGroup<T, DK, DV>& grp, const T* __restrict__ q, long start,
                                       const RowMap& rm, int len, int hq, int h, int G, int g) {
  const int tc = rm.tok < len ? rm.tok : len - 1;
  const int gc = rm.gidx < G ? rm.gidx : G - 1;
  const T* qp = q + ((start + tc) * hq + h * G + gc) * DK + 8 * g;
#pragma unroll
  for (int kk = 0; kk < DK / 32; ++kk) grp.q[kk] = load8(qp + 32 * kk);
}

// 16-byte pieces of `rows` rows of `row_elems` elements: global (row clamp) -> LDS [rows][ld].
template <typename T>
__device__ __forceinline__ void stage_rows(T* __restrict__ dst, int ld, const T* __restrict__ src,
                                           long src_row_stride, int first_row, int last_valid_row,
                                           int rows, int row_elems) {
  const int pieces = row_elems / 8;
  for (int p = threadIdx.x; p < rows * pieces; p += blockDim.x) {
    const int r = p / pieces, pc = p % pieces;
    int sr = first_row + r;
    sr = sr > last_valid_row ? last_valid_row : sr;
    store8(dst + r * ld + pc * 8, load8(src + (long)sr * src_row_stride + pc * 8));
  }
}

template <typename T, int DV>
__device__ __forceinline__ void store_rows(T* __restrict__ out_row, const f32x4_t (&o)[DV / 16], float inv,
                                           int g) {
#pragma unroll
  for (int t = 0; t < DV / 16; ++t) {
    T* p = out_row + t * 16 + 4 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = (T)(o[t][i] * inv);
  }
}

__device__ __forceinline__ int ilog2(int x) { return 31 - __builtin_clz(x); }
__device__ __forceinline__ int next_pow2(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}


}  // namespace nsa
