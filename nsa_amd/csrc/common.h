// Shared device helpers for the gfx950 NSA kernels: 16x16 MFMA tiles on 64-wide wavefronts.
//
// Fragment convention used by every attention kernel here ("transposed scores"):
//   S^T[key][row] = sum_d K[key][d] * Q[row][d]
//     A operand = K rows   : lane (m = lane%16, g = lane/16) holds K[key(m)][32*kk + 8g .. +7]
//     B operand = Q rows   : lane (n = lane%16, g)           holds Q[row n][32*kk + 8g .. +7]
//     C tile               : lane (n, g) holds S^T[key 4g+i][row n], i = 0..3
//   A 32-key chunk is two such tiles whose A rows are permuted (tile0 row m -> key 8*(m/4)+m%4,
//   tile1 -> +4) so that lane (n, g) ends up with the 8 *contiguous* keys 8g..8g+7 of the chunk.
//   Those 8 probabilities are then directly the B operand of
//   O^T[dv][row] = sum_key V^T[dv][key] * P^T[key][row]
//     A operand = V^T rows : lane (m = dv%16, g) holds V^T[dv][chunk + 8g .. +7]  (16 B contiguous)
//   so P never leaves registers and V is consumed from a key-contiguous (transposed) layout.
// fp32 inputs use the same fragments with eight v_mfma_f32_16x16x4_f32 per step.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nsa {

typedef __bf16 bf16_t;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16_t;
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x8_t __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegInf = -__builtin_huge_valf();

template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> { using type = bf16x8_t; };
template <> struct Vec8<f16_t> { using type = f16x8_t; };
template <> struct Vec8<float> { using type = f32x8_t; };
template <typename T> using vec8_t = typename Vec8<T>::type;

__device__ __forceinline__ f32x4_t mma16(bf16x8_t a, bf16x8_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4_t mma16(f16x8_t a, f16x8_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4_t mma16(f32x8_t a, f32x8_t b, f32x4_t c) {
#pragma unroll
  for (int j = 0; j < 8; ++j) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], b[j], c, 0, 0, 0);
  return c;
}

// 8 consecutive elements; p must be 16-byte aligned.
__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) {
  return *reinterpret_cast<const bf16x8_t*>(p);
}
__device__ __forceinline__ f16x8_t load8(const f16_t* p) {
  return *reinterpret_cast<const f16x8_t*>(p);
}
__device__ __forceinline__ f32x8_t load8(const float* p) {
  const f32x4_t a = *reinterpret_cast<const f32x4_t*>(p);
  const f32x4_t b = *reinterpret_cast<const f32x4_t*>(p + 4);
  f32x8_t r;
  r[0] = a[0]; r[1] = a[1]; r[2] = a[2]; r[3] = a[3];
  r[4] = b[0]; r[5] = b[1]; r[6] = b[2]; r[7] = b[3];
  return r;
}
__device__ __forceinline__ void store8(bf16_t* p, bf16x8_t v) {
  *reinterpret_cast<bf16x8_t*>(p) = v;
}
__device__ __forceinline__ void store8(f16_t* p, f16x8_t v) {
  *reinterpret_cast<f16x8_t*>(p) = v;
}
__device__ __forceinline__ void store8(float* p, f32x8_t v) {
  f32x4_t a, b;
  a[0] = v[0]; a[1] = v[1]; a[2] = v[2]; a[3] = v[3];
  b[0] = v[4]; b[1] = v[5]; b[2] = v[6]; b[3] = v[7];
  *reinterpret_cast<f32x4_t*>(p) = a;
  *reinterpret_cast<f32x4_t*>(p + 4) = b;
}

template <typename T> __device__ __forceinline__ vec8_t<T> zero8() {
  vec8_t<T> r;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = (T)0.0f;
  return r;
}
template <typename T> __device__ __forceinline__ vec8_t<T> pack8(const float (&p)[8]) {
  vec8_t<T> r;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = (T)p[i];
  return r;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Wait for every outstanding memory operation of this wavefront.  Placed after the one-time loads
// (query fragments, statistics) and before a streaming loop, it keeps the compiler from guarding
// those registers with waits inside the loop, which would also wait for the loop's own prefetches.
__device__ __forceinline__ void wait_all_loads() { __builtin_amdgcn_s_waitcnt(0); }

// A-operand row m of tile `tile` (0/1) of a 32-key chunk -> key offset inside the chunk.
__device__ __forceinline__ int chunk_key_of_row(int tile, int m) {
  return 8 * (m >> 2) + (m & 3) + 4 * tile;
}

// LDS tiles: rows are padded by 32 bytes, which spreads 16 consecutive rows (and the row sets below) over
// all banks for 16-byte reads; a padding of 16 bytes costs a second pass on most reads.
template <typename T> constexpr int kLdsRowPad = 32 / (int)sizeof(T);
// The same map for a chunk staged in LDS: lane groups 2 and 3 (m >= 8) take their two tiles in the
// opposite order, so that the 16 rows of one tile are distinct modulo 16 (no bank conflicts).  Value i
// (0..7, tile 0 first) of lane group g then belongs to key 8g + (i ^ lds_key_swap(g)).
__device__ __forceinline__ int lds_key_of_row(int tile, int m) {
  return 8 * (m >> 2) + (m & 3) + 4 * (tile ^ (m >> 3));
}
__device__ __forceinline__ int lds_key_swap(int g) { return (g >> 1) << 2; }

// All-reduce over the four lanes that share one tile column (lane%16): lanes n, n+16, n+32, n+48.
// v_permlane16_swap exchanges the odd 16-lane rows of one operand with the even rows of the other,
// v_permlane32_swap the upper half of one with the lower half of the other; fed the same value
// twice they return the two partners of every lane, so each step is one VALU swap plus one op.
__device__ __forceinline__ float colgroup_max(float x) {
  unsigned u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  x = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
  u = __float_as_uint(x);
  r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float colgroup_sum(float x) {
  unsigned u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  u = __float_as_uint(x);
  r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// Sum over the lane pairs (n, n+16) and (n+32, n+48) only.
__device__ __forceinline__ float colpair_sum(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Data-parallel-primitive move inside a 16-lane row: CTRL 0x00-0xFF = quad_perm, 0x100+n = row_shl:n
// (lane i reads lane i+n), 0x110+n = row_shr:n; lanes whose source is outside the row read 0.
template <int CTRL> __device__ __forceinline__ float dpp_f32(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}

// Column offset of sequence b inside a key-contiguous ("transposed") buffer: every sequence starts
// on a multiple of 8 elements so that 8-key fragments are 16-byte aligned.
__host__ __device__ __forceinline__ int transposed_offset(int cu_b, int b) {
  return ((cu_b + 7) & ~7) + 8 * b;
}

// Sequence / tile lookup for packed (varlen) inputs.  Tiles of `tq` tokens are numbered sequence
// after sequence; a tile index past the last one yields valid = false.  `tile` is the same for the
// whole wavefront and all 64 lanes call together.  Small batches are scanned with scalar loads; from
// 9 sequences on every lane takes one sequence of a run of 64, the run's tile counts are prefix-summed
// across the wavefront, and the hit is broadcast: batch / 64 rounds of one coalesced load instead of
// `batch` dependent scalar loads in every workgroup.
struct SeqTile {
  int b, t0, start, len;
  bool valid;
};
__device__ __forceinline__ SeqTile find_tile(const int32_t* __restrict__ cu, int batch, int tq, int tile) {
  SeqTile r;
  r.valid = false;
  r.b = 0; r.t0 = 0; r.start = 0; r.len = 0;
  if (batch <= 8) {
    int prev = cu[0];
    for (int b = 0; b < batch; ++b) {
      const int next = cu[b + 1];
      const int len = next - prev;
      const int nt = (len + tq - 1) / tq;
      if (tile < nt) {
        r.b = b; r.t0 = tile * tq; r.start = prev; r.len = len; r.valid = true;
        return r;
      }
      tile -= nt;
      prev = next;
    }
    return r;
  }
  const int lane = __lane_id();
  tile = __builtin_amdgcn_readfirstlane(tile);
  int before = 0;                                    // tiles of the sequences before this run
  for (int b0 = 0; b0 < batch; b0 += 64) {
    const int b = b0 + lane;
    const int s = b < batch ? cu[b] : 0;
    const int len = b < batch ? cu[b + 1] - s : 0;
    const int nt = (len + tq - 1) / tq;
    int incl = nt;                                   // inclusive prefix sum over the run
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    const int run = __builtin_amdgcn_readlane(incl, 63);
    if (tile < before + run) {
      const unsigned long long hit = __ballot(before + incl > tile);
      const int w = __ffsll((long long)hit) - 1;     // first sequence whose tiles reach past `tile`
      r.b = b0 + w;
      r.start = __builtin_amdgcn_readlane(s, w);
      r.len = __builtin_amdgcn_readlane(len, w);
      r.t0 = (tile - before - __builtin_amdgcn_readlane(incl - nt, w)) * tq;
      r.valid = true;
      return r;
    }
    before += run;
  }
  return r;
}

// Per-row-group state of the online softmax.  One group = 16 rows = the 16 columns of a tile.
template <typename T, int DK, int DV>
struct RowGroup {
  vec8_t<T> q[DK / 32];
  f32x4_t o[DV / 16];
  float m;  // running maximum of the raw (unscaled) visible scores of column lane%16
  float l;  // this lane's share of the running denominator
};

template <typename T, int DK, int DV>
__device__ __forceinline__ void group_reset(RowGroup<T, DK, DV>& g) {
#pragma unroll
  for (int i = 0; i < DV / 16; ++i) g.o[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  g.m = kNegInf;
  g.l = 0.f;
}

// x *= a with the result forced into the register x already lives in.  Used inside rarely taken
// branches that rescale accumulators: a plain multiply lets the compiler put the products in new
// registers, and the common not-taken path then pays one register move per accumulator.
//
// The compiler's hazard recogniser does not look inside inline assembly, so the wait states it
// would insert between a transcendental (v_exp_f32) or MFMA result and an ordinary VALU consumer
// are missing for these multiplies.  Every factor therefore has to pass through settle_factor()
// first: it is ordered after the factor's computation and holds 12 wait states, which covers the
// transcendental forwarding hazard (1) and an 8-pass MFMA write followed by a VALU read (11).
__device__ __forceinline__ void settle_factor(float& a) {
  asm volatile("s_nop 7\n\ts_nop 3" : "+v"(a));
}
__device__ __forceinline__ void settle_factor(float& a, float& b) {
  asm volatile("s_nop 7\n\ts_nop 3" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void scale_inplace(float& x, float a) {
  asm volatile("v_mul_f32 %0, %1, %0" : "+v"(x) : "v"(a));
}
__device__ __forceinline__ void scale_inplace(f32x4_t& v, float a) {
  float e0 = v[0], e1 = v[1], e2 = v[2], e3 = v[3];
  scale_inplace(e0, a); scale_inplace(e1, a); scale_inplace(e2, a); scale_inplace(e3, a);
  v[0] = e0; v[1] = e1; v[2] = e2; v[3] = e3;
}

// How far (in powers of two of the resulting probability) a score may exceed the running reference
// before the accumulators are rescaled.  The reference of an online softmax does not have to be the
// exact maximum: any value within this slack of it keeps every exponential <= 2^kMaxSlackLog2, far
// from overflow in fp32 sums and bf16 probabilities, and the final o / l is unchanged.  With 16 rows
// sharing one branch, following the exact maximum would rescale on more than half of the chunks
// (record-value statistics); with the slack it happens on the first chunk and hardly ever again.
constexpr float kMaxSlackLog2 = 8.0f;

// Move the running reference of a group up when `mx` (already reduced over the column's four
// lanes) exceeds it by more than the slack; the accumulator and denominator are rescaled then.
// c = scale * log2(e).
template <typename T, int DK, int DV>
__device__ __forceinline__ void raise_max(RowGroup<T, DK, DV>& g, float mx, float c) {
  if (__any(mx * c > fmaf(g.m, c, kMaxSlackLog2))) {       // -inf reference: any finite score moves it
    const float m_new = fmaxf(g.m, mx);
    const float mref = (m_new == kNegInf) ? 0.f : m_new;
    float alpha = fast_exp2((g.m - mref) * c);
    settle_factor(alpha);
    scale_inplace(g.l, alpha);
#pragma unroll
    for (int i = 0; i < DV / 16; ++i) scale_inplace(g.o[i], alpha);
    g.m = m_new;
  }
}

// Sum of 8 values as a balanced tree: three dependent adds instead of seven.
__device__ __forceinline__ float sum8(const float (&x)[8]) {
  return ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
}

// Online-softmax update for the 8 scores a lane holds of one 32-key chunk (masked entries are
// -inf).  Returns the unnormalised probabilities in p.
template <typename T, int DK, int DV>
__device__ __forceinline__ void softmax_update(RowGroup<T, DK, DV>& g, const float (&s)[8], float c,
                                               float (&p)[8]) {
  float mx = s[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) mx = fmaxf(mx, s[i]);
  raise_max(g, colgroup_max(mx), c);
  const float off = (g.m == kNegInf) ? 0.f : -g.m * c;
#pragma unroll
  for (int i = 0; i < 8; ++i) p[i] = fast_exp2(fmaf(s[i], c, off));
  g.l += sum8(p);
}

}  // namespace nsa
