// Pieces shared by the decode kernels: per-wavefront online-softmax state and the 32-key chunk of ordinary
// attention (window / selected block) with all its fragments requested together.
#pragma once
#include "tiles.h"

namespace nsa {

constexpr int kDecWaves = 8;
constexpr int kDecMaxChunks = 9;   // compressed 32-row chunks per wavefront kept in registers

// Pooled bins of a sequence with nc compressed rows (windows of k every s, padding p, ceil mode).
__host__ __device__ inline int decode_pooled_bins(int nc, int k, int s, int p) {
  const int span = nc + 2 * p - k;
  return span < 0 ? 0 : (span + s - 1) / s + 1;
}
// The one-workgroup step keeps the bins of its sequence in LDS (decode_bins_cap floats) and, for the top-n, in
// the registers of one wavefront: a quarter of the compressed rows + 4 (pooling strides of 4 and more), or half of
// them + 4 in the WIDE build (pooling stride 2).
template <bool WIDE> constexpr int kDecBinsMax = 32 * kDecWaves * kDecMaxChunks / (WIDE ? 2 : 4) + 4;
__host__ __device__ inline int decode_bins_cap(int nc_cap, bool wide) {
  return wide ? (nc_cap + 1) / 2 + 4 : (nc_cap + 3) / 4 + 4;
}
__host__ __device__ inline int decode_bins_room(int nc_cap, bool wide) {
  const int cap = decode_bins_cap(nc_cap, wide), most = wide ? kDecBinsMax<true> : kDecBinsMax<false>;
  return cap < most ? cap : most;
}

template <typename T, int DK, int DV>
struct DecState {              // online softmax state of one wavefront for one branch
  f32x4_t o[DV / 16];
  float m, l;
};

template <typename T, int DK, int DV>
__device__ __forceinline__ void dec_reset(DecState<T, DK, DV>& s) {
#pragma unroll
  for (int i = 0; i < DV / 16; ++i) s.o[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  s.m = kNegInf;
  s.l = 0.f;
}

// scores of one 32-key chunk whose K rows start at krow0 (+ key offset of this lane's fragment rows)
template <typename T, int DK>
__device__ __forceinline__ void dec_scores(const T* __restrict__ k0p, const T* __restrict__ k1p,
                                           const vec8_t<T> (&q)[DK / 32], float (&s)[8]) {
  f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int kk = 0; kk < DK / 32; ++kk) {
    s0 = mma16(load8(k0p + 32 * kk), q[kk], s0);
    s1 = mma16(load8(k1p + 32 * kk), q[kk], s1);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) { s[i] = s0[i]; s[4 + i] = s1[i]; }
}

// Fragments of one 32-key chunk of ordinary attention (window / selected block): two K tiles and
// the V^T tiles, all requested together so that a chunk costs one memory round trip.
template <typename T, int DK, int DV>
struct ChunkFrags {
  vec8_t<T> k0[DK / 32], k1[DK / 32], v[DV / 16];
};

template <typename T, int DK, int DV>
__device__ __forceinline__ void chunk_issue(ChunkFrags<T, DK, DV>& f, const T* __restrict__ kseq, long krow,
                                            const T* __restrict__ vt, long vstep, int cb, int last_row, int n,
                                            int g) {
  const T* k0p = kseq + (long)min(cb + chunk_key_of_row(0, n), last_row) * krow + 8 * g;
  const T* k1p = kseq + (long)min(cb + chunk_key_of_row(1, n), last_row) * krow + 8 * g;
#pragma unroll
  for (int kk = 0; kk < DK / 32; ++kk) { f.k0[kk] = load8(k0p + 32 * kk); f.k1[kk] = load8(k1p + 32 * kk); }
#pragma unroll
  for (int t = 0; t < DV / 16; ++t) f.v[t] = load8(vt + t * vstep + cb);
}

// keys [cb, cb+32) of the sequence, visible keys are lo..hi
template <typename T, int DK, int DV>
__device__ __forceinline__ void chunk_attend(DecState<T, DK, DV>& st, const ChunkFrags<T, DK, DV>& f,
                                             const vec8_t<T> (&q)[DK / 32], int cb, int lo, int hi, float c_attn,
                                             int g) {
  f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int kk = 0; kk < DK / 32; ++kk) {
    s0 = mma16(f.k0[kk], q[kk], s0);
    s1 = mma16(f.k1[kk], q[kk], s1);
  }
  float s[8], p[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) { s[i] = s0[i]; s[4 + i] = s1[i]; }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int key = cb + 8 * g + i;
    if (!(key >= lo && key <= hi)) s[i] = kNegInf;
  }
  float mx = s[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) mx = fmaxf(mx, s[i]);
  mx = colgroup_max(mx);
  const float m_new = fmaxf(st.m, mx);
  const float mref = m_new == kNegInf ? 0.f : m_new;
  const float alpha = fast_exp2((st.m - mref) * c_attn);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) { p[i] = fast_exp2((s[i] - mref) * c_attn); sum += p[i]; }
  st.l = st.l * alpha + sum;
  st.m = m_new;
  const vec8_t<T> pb = pack8<T>(p);
#pragma unroll
  for (int t = 0; t < DV / 16; ++t) {
    st.o[t][0] *= alpha; st.o[t][1] *= alpha; st.o[t][2] *= alpha; st.o[t][3] *= alpha;
    st.o[t] = mma16(f.v[t], pb, st.o[t]);
  }
}

}  // namespace nsa
