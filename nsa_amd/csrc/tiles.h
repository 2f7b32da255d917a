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

// ------------------------------------------------------------------------------------------------
// transposing fragment load
// tile points at element (row0, col0) of a row-major LDS tile with row pitch ld.  Lane (m = lane%16,
// g = lane/16) receives tile[8g + j][m], j = 0..7: the A operand of a product whose depth runs over
// the tile's rows.  bf16: two ds_read_b64_tr_b16, each transposing a 4 x 16 block per 16 lanes (lane
// 4a+b supplies the address of row a, columns 4b..4b+3 and receives column 4a'+b' of rows 0..3).
__device__ __forceinline__ bf16x8_t load8_tr(const bf16_t* tile, int ld, int lane) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
  typedef __attribute__((address_space(3))) bf16x4_t lds_bf16x4_t;
  const int i = lane & 15, g = lane >> 4;
  const bf16_t* p = tile + (8 * g + (i >> 2)) * ld + 4 * (i & 3);
  const bf16x4_t a = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_t*)p);
  const bf16x4_t b = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_t*)(p + 4 * ld));
  bf16x8_t r;
  r[0] = a[0]; r[1] = a[1]; r[2] = a[2]; r[3] = a[3];
  r[4] = b[0]; r[5] = b[1]; r[6] = b[2]; r[7] = b[3];
  return r;
}
// fp16: the same instruction (it moves 16-bit lanes whatever they hold)
__device__ __forceinline__ f16x8_t load8_tr(const f16_t* tile, int ld, int lane) {
  return __builtin_bit_cast(f16x8_t, load8_tr(reinterpret_cast<const bf16_t*>(tile), ld, lane));
}
__device__ __forceinline__ f32x8_t load8_tr(const float* tile, int ld, int lane) {
  const int m = lane & 15, g = lane >> 4;
  f32x8_t r;
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = tile[(8 * g + j) * ld + m];
  return r;
}

// Row of a 32-row LDS tile behind value j (0..7) of lane group g (lane / 16) wherever a 32-row tile feeds
// two products, once row-major (rows = MFMA rows, two 16-row tiles) and once transposed (rows = depth):
// group g owns rows {b, .., b+3} and {b+8, .., b+11} with b = 4 (g & 1) + 16 (g >> 1).  With rows padded by
// 32 bytes both kinds of read are free of bank conflicts: the row-major tiles are rows {0..7, 16..23} and
// {8..15, 24..31}, and each half-wavefront's transposing read touches 8 rows that differ modulo 8.
__device__ __forceinline__ int lane_row32(int g, int j) { return 4 * (g & 1) + 16 * (g >> 1) + j + 4 * (j >> 2); }
// LDS row read by MFMA row m of row-major tile `tile` (0/1) of such a 32-row tile.
__device__ __forceinline__ int tile_row32(int tile, int m) { return m + 8 * (m >> 3) + 8 * tile; }

// The transposing read for that row ownership: lane (g, m) receives tile[lane_row32(g, j)][m], j = 0..7.
__device__ __forceinline__ bf16x8_t load8_tr32(const bf16_t* tile, int ld, int lane) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
  typedef __attribute__((address_space(3))) bf16x4_t lds_bf16x4_t;
  const int i = lane & 15, g = lane >> 4;
  const bf16_t* p = tile + (4 * (g & 1) + 16 * (g >> 1) + (i >> 2)) * ld + 4 * (i & 3);
  const bf16x4_t a = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_t*)p);
  const bf16x4_t b = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_t*)(p + 8 * ld));
  bf16x8_t r;
  r[0] = a[0]; r[1] = a[1]; r[2] = a[2]; r[3] = a[3];
  r[4] = b[0]; r[5] = b[1]; r[6] = b[2]; r[7] = b[3];
  return r;
}
__device__ __forceinline__ f16x8_t load8_tr32(const f16_t* tile, int ld, int lane) {
  return __builtin_bit_cast(f16x8_t, load8_tr32(reinterpret_cast<const bf16_t*>(tile), ld, lane));
}
__device__ __forceinline__ f32x8_t load8_tr32(const float* tile, int ld, int lane) {
  const int m = lane & 15, g = lane >> 4;
  f32x8_t r;
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = tile[lane_row32(g, j) * ld + m];
  return r;
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

// Arg-max all-reduce over the 64 lanes of (score bits, tie key) packed as a signed 64-bit value:
// non-negative floats order like their bit patterns, the "taken" marker -1.0f is negative.
__device__ __forceinline__ long wave_max_i64(long key) {
  auto step = [&](int lo_other, int hi_other) {
    const long other = ((long)hi_other << 32) | (unsigned int)lo_other;
    key = other > key ? other : key;
  };
  int lo = (int)key, hi = (int)(key >> 32);
#define NSA_DPP_STEP(CTRL)                                                                       \
  lo = (int)key; hi = (int)(key >> 32);                                                          \
  step(__builtin_amdgcn_update_dpp(lo, lo, CTRL, 0xF, 0xF, false),                               \
       __builtin_amdgcn_update_dpp(hi, hi, CTRL, 0xF, 0xF, false));
  NSA_DPP_STEP(0xB1)    // quad_perm [1,0,3,2]
  NSA_DPP_STEP(0x4E)    // quad_perm [2,3,0,1]
  NSA_DPP_STEP(0x141)   // row_half_mirror
  NSA_DPP_STEP(0x140)   // row_mirror
#undef NSA_DPP_STEP
  {
    lo = (int)key; hi = (int)(key >> 32);
    const auto a = __builtin_amdgcn_permlane16_swap((unsigned)lo, (unsigned)lo, false, false);
    const auto b = __builtin_amdgcn_permlane16_swap((unsigned)hi, (unsigned)hi, false, false);
    const long k0 = ((long)(int)b[0] << 32) | a[0], k1 = ((long)(int)b[1] << 32) | a[1];
    key = k0 > k1 ? k0 : k1;
  }
  {
    lo = (int)key; hi = (int)(key >> 32);
    const auto a = __builtin_amdgcn_permlane32_swap((unsigned)lo, (unsigned)lo, false, false);
    const auto b = __builtin_amdgcn_permlane32_swap((unsigned)hi, (unsigned)hi, false, false);
    const long k0 = ((long)(int)b[0] << 32) | a[0], k1 = ((long)(int)b[1] << 32) | a[1];
    key = k0 > k1 ? k0 : k1;
  }
  return key;
}

// Top-n of row[0..ns) (non-negative scores in LDS, ns <= 64*PER) by one wavefront: every lane keeps
// its candidates b = lane + 64k in registers; each round is a local scan, one 64-lane arg-max
// (ties go to the lower index) and the winner's lane retiring its entry.  emit(r, index or -1).
template <int PER, typename Emit>
__device__ __forceinline__ void wave_topn(const volatile float* row, int ns, int top_n, int lane, Emit emit) {
  float v[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int b = lane + 64 * k;
    v[k] = b < ns ? row[b] : -1.f;
  }
  for (int r = 0; r < top_n; ++r) {
    float best = v[0];
    int bk = 0;
#pragma unroll
    for (int k = 1; k < PER; ++k)
      if (v[k] > best) { best = v[k]; bk = k; }
    const int bi = lane + 64 * bk;
    long key = ((long)__float_as_int(best) << 32) | (unsigned int)(0x7fffffff - bi);
    key = wave_max_i64(key);
    const bool found = (int)(key >> 32) >= 0;
    const int win = 0x7fffffff - (int)(unsigned int)key;
    if (found && (win & 63) == lane) {
#pragma unroll
      for (int k = 0; k < PER; ++k)
        if (k == (win >> 6)) v[k] = -1.f;
    }
    emit(r, found ? win : -1);
  }
}

// Wavefront reductions that end in a scalar register: four DPP steps inside each 16-lane row, two
// row broadcasts (lane 15 -> next row, lane 31 -> upper half), then lane 63 holds the result.
// Written as one assembly block so that every step is a single DPP-modified instruction; the
// compiler's hazard recogniser does not see inside it, so the wait states are spelled out: two
// between a VALU write and a DPP read of the same register, and after v_readlane before use.
#define NSA_WAVE_REDUCE(NAME, TYPE, OPCODE)                                                       \
  __device__ __forceinline__ TYPE NAME(TYPE x) {                                                  \
    TYPE r;                                                                                       \
    asm volatile("s_nop 1\n\t"                                                                    \
                 OPCODE " %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t" \
                 OPCODE " %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t" \
                 OPCODE " %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"     \
                 OPCODE " %1, %1, %1 row_mirror row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"          \
                 OPCODE " %1, %1, %1 row_bcast:15 row_mask:0xa bank_mask:0xf\n\ts_nop 1\n\t"        \
                 OPCODE " %1, %1, %1 row_bcast:31 row_mask:0xc bank_mask:0xf\n\ts_nop 1\n\t"        \
                 "v_readlane_b32 %0, %1, 63\n\ts_nop 3"                                            \
                 : "=s"(r), "+v"(x));                                                             \
    return r;                                                                                     \
  }
NSA_WAVE_REDUCE(wave_max_f32, float, "v_max_f32_dpp")
NSA_WAVE_REDUCE(wave_min_f32, float, "v_min_f32_dpp")
NSA_WAVE_REDUCE(wave_min_i32, int, "v_min_i32_dpp")
#undef NSA_WAVE_REDUCE

// Top-n of the PER * 64 non-negative scores a wavefront holds in registers (v[k] of lane l is bin
// l + 64k; -1 marks "no bin"), descending, ties to the lower index; emit(r, index or -1).
//
// Shortlist first: each of the 16 lane quads holds a maximum; the smallest of those, L, has at least
// 16 bins at or above it, so the 16 best bins are all >= L.  Typically fewer than a tenth of the bins
// pass; they are compacted in index order through `cand_v` / `cand_i` (128 entries each, private to
// the wavefront) to at most two per lane, and the selection rounds then cost a fraction of rounds over
// all PER bins per lane.  More than 16 picks or more than 128 candidates fall back to full rounds.
template <int PER, typename Emit>
__device__ __forceinline__ void wave_topn_shortlist(float (&v)[PER], int top_n, int lane, float* cand_v, int* cand_i,
                                                    Emit emit) {
  int total = 129;
  if (top_n <= 16) {
    float m = v[0];
#pragma unroll
    for (int k = 1; k < PER; ++k) m = fmaxf(m, v[k]);
    m = fmaxf(m, dpp_f32<0xB1>(m));
    m = fmaxf(m, dpp_f32<0x4E>(m));                       // quad maximum (-1 for a quad without bins)
    const float L = wave_min_f32(m);
    total = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const bool c = v[k] >= L && v[k] >= 0.f;
      const unsigned long long mask = __ballot(c);
      const int pos = total + (int)__builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32),
                                                             __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
      if (c && pos < 128) {
        cand_v[pos] = v[k];
        cand_i[pos] = lane + 64 * k;
      }
      total += __popcll(mask);
    }
  }
  if (total <= 128) {
    __builtin_amdgcn_wave_barrier();
    float c0 = lane < total ? cand_v[lane] : -1.f;
    float c1 = lane + 64 < total ? cand_v[lane + 64] : -1.f;
    const int i0 = cand_i[lane], i1 = cand_i[lane + 64];
    for (int r = 0; r < top_n; ++r) {
      const bool second = c1 > c0;                        // slot 0 has the lower index: it wins ties
      const float best = second ? c1 : c0;
      const int bi = second ? i1 : i0;
      const float wmax = wave_max_f32(best);
      int win = -1;
      if (wmax >= 0.f) {
        const unsigned long long tied = __ballot(best == wmax);
        if (__popcll(tied) == 1) {
          win = __builtin_amdgcn_readlane(bi, (int)__builtin_ctzll(tied));
        } else {
          win = wave_min_i32(best == wmax ? bi : 0x7fffffff);
        }
        if (bi == win) {                                  // indices are unique: exactly one lane
          if (second) c1 = -1.f; else c0 = -1.f;
        }
      }
      emit(r, win);
    }
    return;
  }
  for (int r = 0; r < top_n; ++r) {
    float best = v[0];
    int bk = 0;
#pragma unroll
    for (int k = 1; k < PER; ++k)
      if (v[k] > best) { best = v[k]; bk = k; }
    const int bi = lane + 64 * bk;
    long key = ((long)__float_as_int(best) << 32) | (unsigned int)(0x7fffffff - bi);
    key = wave_max_i64(key);
    const bool found = (int)(key >> 32) >= 0;
    const int win = 0x7fffffff - (int)(unsigned int)key;
    if (found && (win & 63) == lane) {
#pragma unroll
      for (int k = 0; k < PER; ++k)
        if (k == (win >> 6)) v[k] = -1.f;
    }
    emit(r, found ? win : -1);
  }
}

// Scheduling hint for the basic block it is placed in: alternate MF matrix instructions with VA
// vector-ALU instructions, spread evenly (one MFMA, then its share of the VALU work, ...).
template <int MF, int VA, int I = 0>
__device__ __forceinline__ void interleave_mfma_valu() {
  if constexpr (I < MF) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    constexpr int share = (VA * (I + 1)) / MF - (VA * I) / MF;
    if constexpr (share > 0) __builtin_amdgcn_sched_group_barrier(0x002, share, 0);
    interleave_mfma_valu<MF, VA, I + 1>();
  }
}

// Compressed rows a token tile needs when only the attention output is wanted: up to the last row its last token
// may attend, rounded up to 64 and at least 64 (so that every row meets the first chunk, which sets its softmax
// reference).  The rows beyond only feed the importance log-sum-exp.
__device__ __forceinline__ int cmp_visible_end(int t0, int tq, int len, int nkeys, int block, int stride, int causal) {
  if (!causal) return nkeys;
  const int t_last = min(t0 + tq, len) - 1;
  const int last = t_last >= block ? min((t_last - block) / stride, nkeys - 1) : -1;
  return min(nkeys, max(64, ((last + 1 + 63) / 64) * 64));
}

__device__ __forceinline__ int ilog2(int x) { return 31 - __builtin_clz(x); }
__device__ __forceinline__ int next_pow2(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}


}  // namespace nsa
