// The three attention branches of the NSA forward path on gfx950 MFMA.
//
// Row space. For one kv head the G query heads of a token are G consecutive "rows"; G is padded
// to a power of two Gp <= 16 and 16 consecutive rows form one row group = the 16 columns of an
// MFMA tile (G = 16: one token per group, G = 4: four tokens per group).  All heads of a group
// share the K/V they read, which is what makes the GQA group the MFMA N dimension.
//
//   cmp_select_kernel  compressed attention (online softmax over the causally visible compressed
//                      rows) + block importance: softmax of the raw q.ck over ALL compressed rows,
//                      summed over the G heads, average-pooled into selection blocks, wavefront
//                      top-n.  Pass 1 streams ck / cv^T through LDS once per token tile and also
//                      accumulates the row-wise log-sum-exp of the raw scores; pass 2 recomputes the
//                      score tiles in the un-transposed orientation so that the head sum is an
//                      in-lane add plus two lane swaps, and bins exp(s - lse) in LDS.
//   swa_kernel         sliding window attention; a token tile streams the union of its windows
//                      through LDS once.
//   slc_combine_kernel selected-block attention, one wavefront per row group reading its blocks
//                      straight from global memory in fragment layout, and the gated combine of
//                      the three branches in the epilogue.
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

// ------------------------------------------------------------------------------------------------
// compressed attention + block importance + top-n

template <typename T, int DK, int DV, int NG, int CH>
__global__ void __launch_bounds__(256)
cmp_select_kernel(const CmpArgs a) {
  constexpr int KLD = DK + 8, VLD = CH + 8, ROWS = 64 * NG;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* ldsK = reinterpret_cast<T*>(smem_raw);
  T* ldsV = ldsK + CH * KLD;
  float* bins = reinterpret_cast<float*>(ldsV + DV * VLD);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv, Gp = next_pow2(G), lgp = ilog2(Gp);
  const int TQ = ROWS >> lgp;
  const SeqTile st = find_tile(a.cu_seq, a.batch, TQ, blockIdx.x);
  if (!st.valid) return;
  const int h = blockIdx.y;
  const int coff = a.cu_cmp[st.b];
  const int Nc = a.cu_cmp[st.b + 1] - coff;
  const int ctoff = transposed_offset(coff, st.b);
  int Ns = 0;
  if (Nc > 0 && Nc + 2 * a.pool_p >= a.pool_k) {
    Ns = (Nc + 2 * a.pool_p - a.pool_k + a.pool_s - 1) / a.pool_s + 1;
    if ((Ns - 1) * a.pool_s >= Nc + a.pool_p) --Ns;
  }
  Ns = min(Ns, a.max_ns);   // LDS was sized for max_ns bins per token
  const int t_last = min(st.t0 + TQ, st.len) - 1;
  const T* qb = reinterpret_cast<const T*>(a.q);
  const T* ckb = reinterpret_cast<const T*>(a.ck) + (long)coff * a.ck_row_stride + (long)h * a.ck_head_stride;
  const T* cvtb = reinterpret_cast<const T*>(a.cvt) + (long)h * DV * a.cvt_cols + ctoff;

  RowGroup<T, DK, DV> grp[NG];
  RowMap rm[NG];
  int cmaxv[NG];      // last compressed row visible to this lane's column, -1 if none
  int cmax_grp[NG];   // the same for the last token of the group (wave uniform)
  float mi[NG], li[NG];
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    const int gi = wave * NG + j;
    rm[j] = map_row(st.t0, gi, n, lgp, G, st.len);
    load_q(grp[j], qb, (long)st.start, rm[j], st.len, a.hq, h, G, g);
    group_reset(grp[j]);
    cmaxv[j] = !a.causal ? Nc - 1 : (rm[j].tok >= a.block ? (rm[j].tok - a.block) / a.stride : -1);
    const int tl = min(st.t0 + ((gi * 16 + 15) >> lgp), st.len - 1);
    cmax_grp[j] = !a.causal ? Nc - 1 : (tl >= a.block ? (tl - a.block) / a.stride : -1);
    mi[j] = kNegInf;
    li[j] = 0.f;
  }
  const int cmax_tile = !a.causal ? Nc - 1 : (t_last >= a.block ? (t_last - a.block) / a.stride : -1);
  const float c_attn = a.scale * kLog2e;

  // ---- pass 1: attention over visible rows, log-sum-exp of raw scores over all rows
  for (int c0 = 0; c0 < Nc; c0 += CH) {
    __syncthreads();
    stage_rows(ldsK, KLD, ckb, a.ck_row_stride, c0, Nc - 1, CH, DK);
    const bool need_v = c0 <= cmax_tile;
    if (need_v) stage_rows(ldsV, VLD, cvtb + c0, (long)a.cvt_cols, 0, DV - 1, DV, CH);
    __syncthreads();
#pragma unroll
    for (int sub = 0; sub < CH / 32; ++sub) {
      const int cb = c0 + 32 * sub;
      if (cb >= Nc) break;
      f32x4_t s0[NG], s1[NG];
      const T* ks = ldsK + 32 * sub * KLD + 8 * g;
      scores32<T, DK, DV, NG>(ks + chunk_key_of_row(0, n) * KLD, ks + chunk_key_of_row(1, n) * KLD, grp, s0, s1);
      vec8_t<T> pb[NG];
      bool act[NG];
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        float s[8], sm[8], p[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) { s[i] = s0[j][i]; s[4 + i] = s1[j][i]; }
        // importance statistics: every existing column, natural exponent
        float mx = kNegInf;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int c = cb + 8 * g + i;
          sm[i] = c < Nc ? s[i] : kNegInf;
          mx = fmaxf(mx, sm[i]);
        }
        mx = colgroup_max(mx);
        const float m_new = fmaxf(mi[j], mx);   // finite: column cb exists
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += fast_exp2((sm[i] - m_new) * kLog2e);
        li[j] = li[j] * fast_exp2((mi[j] - m_new) * kLog2e) + sum;
        mi[j] = m_new;
        // attention: causally visible columns only
        act[j] = cb <= cmax_grp[j];
        if (act[j]) {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int c = cb + 8 * g + i;
            sm[i] = (c <= cmaxv[j] && c < Nc) ? s[i] : kNegInf;
          }
          softmax_update(grp[j], sm, c_attn, p);
          pb[j] = pack8<T>(p);
        } else {
          pb[j] = zero8<T>();
        }
      }
      bool any = false;
#pragma unroll
      for (int j = 0; j < NG; ++j) any |= act[j];
      if (any) pv32<T, DK, DV, NG>(ldsV + n * VLD + 32 * sub + 8 * g, 16 * VLD, grp, pb, act);
    }
  }

  // ---- compressed-attention output
  T* ob = reinterpret_cast<T*>(a.o);
  float lse[NG];
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    const float lt = colgroup_sum(grp[j].l);
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    if (rm[j].valid)
      store_rows<T, DV>(ob + (((long)st.start + rm[j].tok) * a.hq + h * G + rm[j].gidx) * DV, grp[j].o, inv, g);
    const float lit = colgroup_sum(li[j]);
    lse[j] = rm[j].valid ? mi[j] + __logf(lit) : __builtin_huge_valf();   // +inf kills padded rows
  }
  if (a.indices == nullptr) return;

  // ---- pass 2: importance bins
  __syncthreads();
  for (int i = threadIdx.x; i < TQ * Ns; i += 256) bins[i] = 0.f;
  float lse_r[NG][4];   // lse of rows 4g+i (the rows this lane holds in the un-transposed tile)
#pragma unroll
  for (int j = 0; j < NG; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) lse_r[j][i] = __shfl(lse[j], 4 * g + i);

  for (int c0 = 0; c0 < Nc && Ns > 0; c0 += CH) {
    __syncthreads();
    stage_rows(ldsK, KLD, ckb, a.ck_row_stride, c0, Nc - 1, CH, DK);
    __syncthreads();
#pragma unroll
    for (int kt = 0; kt < CH / 16; ++kt) {
      const int cb = c0 + 16 * kt;
      if (cb >= Nc) break;
      f32x4_t s[NG];
#pragma unroll
      for (int j = 0; j < NG; ++j) s[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const T* kp = ldsK + (16 * kt + n) * KLD + 8 * g;
#pragma unroll
      for (int kk = 0; kk < DK / 32; ++kk) {
        const vec8_t<T> kb = load8(kp + 32 * kk);
#pragma unroll
        for (int j = 0; j < NG; ++j) s[j] = mma16(grp[j].q[kk], kb, s[j]);   // rows = heads, cols = keys
      }
      const int c = cb + n;
      // bins that contain column c: j*s - p <= c < j*s - p + k
      const int num = c + a.pool_p - a.pool_k + 1;
      const int j_lo = num <= 0 ? 0 : (num + a.pool_s - 1) / a.pool_s;
      const int j_hi = min((c + a.pool_p) / a.pool_s, Ns - 1);
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        const int gi = wave * NG + j;
        float e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = fast_exp2((s[j][i] - lse_r[j][i]) * kLog2e);
        if (lgp >= 2) {
          float v = (e[0] + e[1]) + (e[2] + e[3]);
          if (lgp >= 3) v += __shfl_xor(v, 16);
          if (lgp >= 4) v += __shfl_xor(v, 32);
          const bool adder = lgp >= 4 ? (g == 0) : (lgp == 3 ? ((g & 1) == 0) : true);
          const int tl = (gi * 16 + 4 * g) >> lgp;
          if (adder && c < Nc)
            for (int b = j_lo; b <= j_hi; ++b) atomicAdd(&bins[tl * Ns + b], v);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int tl = (gi * 16 + 4 * g + i) >> lgp;
            if (c < Nc)
              for (int b = j_lo; b <= j_hi; ++b) atomicAdd(&bins[tl * Ns + b], e[i]);
          }
        }
      }
    }
  }
  __syncthreads();

  // ---- average (divisor rule of a ceil-mode pool with padding counted) and top-n per token
  volatile float* vb = bins;
  for (int tl = wave; tl < TQ; tl += 4) {
    const int t = st.t0 + tl;
    if (t >= st.len) break;
    const long orow = ((long)st.start + t) * a.hkv + h;
    for (int b = lane; b < Ns; b += 64) {
      const int lo = b * a.pool_s - a.pool_p;
      const int div = min(lo + a.pool_k, Nc + a.pool_p) - lo;
      const float v = vb[tl * Ns + b] / (float)div;
      vb[tl * Ns + b] = v;
      if (a.pooled != nullptr) a.pooled[orow * a.pooled_stride + b] = v;
    }
    for (int r = 0; r < a.top_n; ++r) {
      float best = -1.f;
      int bi = 0x7fffffff;
      for (int b = lane; b < Ns; b += 64) {
        const float v = vb[tl * Ns + b];
        if (v > best) { best = v; bi = b; }
      }
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const float ov = __shfl_xor(best, off);
        const int oi = __shfl_xor(bi, off);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
      }
      const bool found = best >= 0.f;
      if (found && (bi & 63) == lane) vb[tl * Ns + bi] = -1.f;
      if (lane == 0) {
        const long pos = orow * a.top_n + r;
        const int val = found ? bi : -1;
        if (a.idx64) reinterpret_cast<int64_t*>(a.indices)[pos] = val;
        else reinterpret_cast<int32_t*>(a.indices)[pos] = val;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// sliding window attention

template <typename T, int DK, int DV, int NG, int CH>
__global__ void __launch_bounds__(256)
swa_kernel(const SwaArgs a) {
  constexpr int KLD = DK + 8, VLD = CH + 8, ROWS = 64 * NG;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* ldsK = reinterpret_cast<T*>(smem_raw);
  T* ldsV = ldsK + CH * KLD;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv, Gp = next_pow2(G), lgp = ilog2(Gp);
  const int TQ = ROWS >> lgp;
  const SeqTile st = find_tile(a.cu_seq, a.batch, TQ, blockIdx.x);
  if (!st.valid) return;
  const int h = blockIdx.y;
  const int W = a.window;
  const int t_last = min(st.t0 + TQ, st.len) - 1;
  const T* qb = reinterpret_cast<const T*>(a.q);
  const T* kb = reinterpret_cast<const T*>(a.k) + ((long)st.start * a.hkv + h) * DK;
  const T* vtb = reinterpret_cast<const T*>(a.vt) + (long)h * DV * a.vt_cols + transposed_offset(st.start, st.b);

  RowGroup<T, DK, DV> grp[NG];
  RowMap rm[NG];
  int g_lo[NG], g_hi[NG];   // key range any column of the group may see (wave uniform)
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    const int gi = wave * NG + j;
    rm[j] = map_row(st.t0, gi, n, lgp, G, st.len);
    load_q(grp[j], qb, (long)st.start, rm[j], st.len, a.hq, h, G, g);
    group_reset(grp[j]);
    const int tf = st.t0 + ((gi * 16) >> lgp);
    const int tl = min(st.t0 + ((gi * 16 + 15) >> lgp), st.len - 1);
    g_lo[j] = max(tf - W + 1, 0);
    g_hi[j] = tl;   // < tf when the whole group lies past the sequence end
  }
  const float c_attn = a.scale * kLog2e;
  const int k_lo = max(st.t0 - W + 1, 0);

  for (int c0 = (k_lo / CH) * CH; c0 <= t_last; c0 += CH) {
    __syncthreads();
    stage_rows(ldsK, KLD, kb, (long)a.hkv * DK, c0, st.len - 1, CH, DK);
    stage_rows(ldsV, VLD, vtb + c0, (long)a.vt_cols, 0, DV - 1, DV, CH);
    __syncthreads();
#pragma unroll
    for (int sub = 0; sub < CH / 32; ++sub) {
      const int cb = c0 + 32 * sub;
      bool act[NG];
      bool any = false;
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        act[j] = (cb <= g_hi[j]) && (cb + 31 >= g_lo[j]);
        any |= act[j];
      }
      if (!any) continue;
      f32x4_t s0[NG], s1[NG];
      const T* ks = ldsK + 32 * sub * KLD + 8 * g;
      scores32<T, DK, DV, NG>(ks + chunk_key_of_row(0, n) * KLD, ks + chunk_key_of_row(1, n) * KLD, grp, s0, s1);
      vec8_t<T> pb[NG];
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        if (act[j]) {
          float s[8], p[8];
#pragma unroll
          for (int i = 0; i < 4; ++i) { s[i] = s0[j][i]; s[4 + i] = s1[j][i]; }
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int key = cb + 8 * g + i;
            if (!(key <= rm[j].tok && key > rm[j].tok - W)) s[i] = kNegInf;
          }
          softmax_update(grp[j], s, c_attn, p);
          pb[j] = pack8<T>(p);
        } else {
          pb[j] = zero8<T>();
        }
      }
      pv32<T, DK, DV, NG>(ldsV + n * VLD + 32 * sub + 8 * g, 16 * VLD, grp, pb, act);
    }
  }

  T* ob = reinterpret_cast<T*>(a.o);
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    const float lt = colgroup_sum(grp[j].l);
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    if (rm[j].valid)
      store_rows<T, DV>(ob + (((long)st.start + rm[j].tok) * a.hq + h * G + rm[j].gidx) * DV, grp[j].o, inv, g);
  }
}

// ------------------------------------------------------------------------------------------------
// selected blocks + gated combine

__device__ __forceinline__ float gate_value(float x, int act) {
  return act == 1 ? 1.0f / (1.0f + __expf(-x)) : x;
}

template <typename T, int DK, int DV>
__global__ void __launch_bounds__(256)
slc_combine_kernel(const SlcArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv, Gp = next_pow2(G), lgp = ilog2(Gp);
  const int TQ = 64 >> lgp;
  const SeqTile st = find_tile(a.cu_seq, a.batch, TQ, blockIdx.x);
  if (!st.valid) return;
  const int h = blockIdx.y;
  const int S = a.top_n, BS = a.block_size;
  const T* qb = reinterpret_cast<const T*>(a.q);
  const T* kb = reinterpret_cast<const T*>(a.k) + ((long)st.start * a.hkv + h) * DK;
  const T* vtb = reinterpret_cast<const T*>(a.vt) + (long)h * DV * a.vt_cols + transposed_offset(st.start, st.b);
  const long krow = (long)a.hkv * DK;

  RowGroup<T, DK, DV> grp[1];
  const RowMap rm = map_row(st.t0, wave, n, lgp, G, st.len);
  load_q(grp[0], qb, (long)st.start, rm, st.len, a.hq, h, G, g);
  group_reset(grp[0]);
  const float c_attn = a.scale * kLog2e;
  const int tpg = lgp >= 4 ? 1 : (16 >> lgp);          // tokens per row group
  const int tfirst = st.t0 + ((wave * 16) >> lgp);

  for (int tk = 0; tk < tpg; ++tk) {
    const int tt = tfirst + tk;
    if (tt >= st.len) break;
    const long irow = ((long)st.start + tt) * a.hkv + h;
    int cnt = S;
    if (a.counts != nullptr) cnt = min(max(a.counts[irow], 0), S);
    long myidx = -1;
    if (lane < S) {
      myidx = a.idx64 ? reinterpret_cast<const int64_t*>(a.indices)[irow * S + lane]
                      : (long)reinterpret_cast<const int32_t*>(a.indices)[irow * S + lane];
    }
    for (int i = 0; i < cnt; ++i) {
      const long bi = __shfl(myidx, i);
      if (bi < 0 || bi > tt) continue;                   // also keeps bi * BS inside int range
      if (bi * BS > tt) continue;
      const int k0 = (int)bi * BS;
      const int k1 = min(k0 + BS - 1, tt);               // last key of the block this token may see
      for (int cb = k0; cb <= k1; cb += 32) {
        f32x4_t s0[1], s1[1];
        const int r0 = min(cb + chunk_key_of_row(0, n), st.len - 1);
        const int r1 = min(cb + chunk_key_of_row(1, n), st.len - 1);
        scores32<T, DK, DV, 1>(kb + r0 * krow + 8 * g, kb + r1 * krow + 8 * g, grp, s0, s1);
        float s[8], p[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) { s[e] = s0[0][e]; s[4 + e] = s1[0][e]; }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int key = cb + 8 * g + e;
          if (!(key <= k1 && rm.tok == tt)) s[e] = kNegInf;
        }
        softmax_update(grp[0], s, c_attn, p);
        vec8_t<T> pb[1];
        pb[0] = pack8<T>(p);
        const bool act[1] = {true};
        pv32<T, DK, DV, 1>(vtb + (long)n * a.vt_cols + cb + 8 * g, 16L * a.vt_cols, grp, pb, act);
      }
    }
  }

  if (!rm.valid) return;
  const float lt = colgroup_sum(grp[0].l);
  const float inv = lt > 0.f ? 1.0f / lt : 0.f;
  const long row = ((long)st.start + rm.tok) * a.hq + h * G + rm.gidx;
  const T* gs = reinterpret_cast<const T*>(a.g_slc);
  const T* gw = reinterpret_cast<const T*>(a.g_swa);
  const T* gc = reinterpret_cast<const T*>(a.g_cmp);
  const T* osw = reinterpret_cast<const T*>(a.o_swa);
  const T* ocm = reinterpret_cast<const T*>(a.o_cmp);
  const float w_slc = (gs ? gate_value((float)gs[row * a.gate_stride], a.gate_act) : 1.f) * inv;
  const float w_swa = (osw && gw) ? gate_value((float)gw[row * a.gate_stride], a.gate_act) : (osw ? 1.f : 0.f);
  const float w_cmp = (ocm && gc) ? gate_value((float)gc[row * a.gate_stride], a.gate_act) : (ocm ? 1.f : 0.f);
  T* orow = reinterpret_cast<T*>(a.out) + row * DV;
#pragma unroll
  for (int t = 0; t < DV / 16; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int dv = t * 16 + 4 * g + i;
      float v = grp[0].o[t][i] * w_slc;
      if (osw) v += w_swa * (float)osw[row * DV + dv];
      if (ocm) v += w_cmp * (float)ocm[row * DV + dv];
      orow[dv] = (T)v;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// launchers

template <typename T> struct Tile {
  // groups per wave and keys per LDS chunk
  static constexpr int NG = sizeof(T) == 2 ? 2 : 1;
  static constexpr int CH = sizeof(T) == 2 ? 64 : 32;
};

static int set_smem(const void* fn, size_t bytes) {
  if (bytes > 160 * 1024) return -3;
  if (bytes > 48 * 1024) {
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return -4;
  }
  return 0;
}

static int group_pow2(int G) {
  int p = 1;
  while (p < G) p <<= 1;
  return p;
}

template <typename T, int DK, int DV>
static int launch_cmp_t(const CmpArgs& a, hipStream_t st) {
  constexpr int NG = Tile<T>::NG, CH = Tile<T>::CH;
  const int Gp = group_pow2(a.hq / a.hkv);
  const int TQ = 64 * NG / Gp;
  const size_t smem = (size_t)CH * (DK + 8) * sizeof(T) + (size_t)DV * (CH + 8) * sizeof(T) +
                      (size_t)TQ * a.max_ns * sizeof(float);
  auto fn = cmp_select_kernel<T, DK, DV, NG, CH>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  const int tiles = a.total / TQ + a.batch;
  hipLaunchKernelGGL(fn, dim3(tiles, a.hkv), dim3(256), smem, st, a);
  return 0;
}

template <typename T, int DK, int DV>
static int launch_swa_t(const SwaArgs& a, hipStream_t st) {
  constexpr int NG = Tile<T>::NG, CH = Tile<T>::CH;
  const int Gp = group_pow2(a.hq / a.hkv);
  const int TQ = 64 * NG / Gp;
  const size_t smem = (size_t)CH * (DK + 8) * sizeof(T) + (size_t)DV * (CH + 8) * sizeof(T);
  auto fn = swa_kernel<T, DK, DV, NG, CH>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  const int tiles = a.total / TQ + a.batch;
  hipLaunchKernelGGL(fn, dim3(tiles, a.hkv), dim3(256), smem, st, a);
  return 0;
}

template <typename T, int DK, int DV>
static int launch_slc_t(const SlcArgs& a, hipStream_t st) {
  const int Gp = group_pow2(a.hq / a.hkv);
  const int TQ = 64 / Gp;
  const int tiles = a.total / TQ + a.batch;
  hipLaunchKernelGGL((slc_combine_kernel<T, DK, DV>), dim3(tiles, a.hkv), dim3(256), 0, st, a);
  return 0;
}

#define NSA_DISPATCH(FN, ARGS, ST)                                                    \
  do {                                                                                \
    const int key = (ARGS).dk * 1000 + (ARGS).dv;                                     \
    if ((ARGS).dtype == 0) {                                                          \
      switch (key) {                                                                  \
        case 32032: return FN<bf16_t, 32, 32>(ARGS, ST);                              \
        case 64064: return FN<bf16_t, 64, 64>(ARGS, ST);                              \
        case 128128: return FN<bf16_t, 128, 128>(ARGS, ST);                           \
        case 192128: return FN<bf16_t, 192, 128>(ARGS, ST);                           \
        default: return -2;                                                           \
      }                                                                               \
    } else {                                                                          \
      switch (key) {                                                                  \
        case 32032: return FN<float, 32, 32>(ARGS, ST);                               \
        case 64064: return FN<float, 64, 64>(ARGS, ST);                               \
        case 128128: return FN<float, 128, 128>(ARGS, ST);                            \
        case 192128: return FN<float, 192, 128>(ARGS, ST);                            \
        default: return -2;                                                           \
      }                                                                               \
    }                                                                                 \
  } while (0)

int launch_cmp_select(const CmpArgs& a, hipStream_t st) { NSA_DISPATCH(launch_cmp_t, a, st); }
int launch_swa(const SwaArgs& a, hipStream_t st) { NSA_DISPATCH(launch_swa_t, a, st); }
int launch_slc_combine(const SlcArgs& a, hipStream_t st) { NSA_DISPATCH(launch_slc_t, a, st); }

}  // namespace nsa
