// Block importance and top-n selection.
//
// For every token and kv head: p[g][c] = exp(q_g . ck_c - lse_g) over ALL compressed rows c (lse is
// the row-wise log-sum-exp the compressed-attention kernel wrote), summed over the G heads of the
// group, average-pooled into selection blocks (ceil-mode pool, padding counted in the divisor), and
// the top_n blocks by score are written in descending order.
//
// Score tiles are computed un-transposed (rows = heads, columns = compressed rows) so that a lane
// holds four heads of one column: the head sum is three adds plus two lane swaps.  One workgroup
// owns NW*NG row groups and streams ck through LDS once, double buffered; column sums are added
// into per-token bins in LDS, then each wavefront runs top_n rounds of a 64-lane arg-max per token.
#include "tiles.h"

namespace nsa {

// Any GQA group size up to 16 and any pooling window: column sums go into the bins with LDS atomics.
template <typename T, int DK, int NG, int CH, int NW>
__global__ void __launch_bounds__(NW * 64)
importance_select_kernel(const CmpArgs a) {
  constexpr int KLD = DK + kLdsRowPad<T>, ROWS = NW * NG * 16, NT = NW * 64;
  constexpr int KPIECES = CH * DK / 8;
  constexpr int KPT = (KPIECES + NT - 1) / NT;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* ldsK = reinterpret_cast<T*>(smem_raw);                       // [2][CH][KLD]
  float* bins = reinterpret_cast<float*>(ldsK + 2 * CH * KLD);    // [TQ][Ns]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv, Gp = next_pow2(G), lgp = ilog2(Gp);
  const int TQ = ROWS >> lgp;
  const SeqTile st = find_tile(a.cu_seq, a.batch, TQ, blockIdx.x);
  if (!st.valid) return;
  const int h = blockIdx.y;
  const int coff = a.cu_cmp[st.b];
  const int Nc = a.cu_cmp[st.b + 1] - coff;
  int Ns = 0;
  if (Nc > 0 && Nc + 2 * a.pool_p >= a.pool_k) {
    Ns = (Nc + 2 * a.pool_p - a.pool_k + a.pool_s - 1) / a.pool_s + 1;
    if ((Ns - 1) * a.pool_s >= Nc + a.pool_p) --Ns;
  }
  Ns = min(Ns, a.max_ns);   // LDS was sized for max_ns bins per token
  const T* ckb = reinterpret_cast<const T*>(a.ck) + (long)coff * a.ck_row_stride + (long)h * a.ck_head_stride;

  vec8_t<T> qf[NG][DK / 32];
  float lse_r[NG][4];        // lse * log2(e) of rows 4g+i of each group; +inf removes padded rows
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    const int gi = wave * NG + j;
    const RowMap rm = map_row(st.t0, gi, n, lgp, G, st.len);
    const int tc = rm.tok < st.len ? rm.tok : st.len - 1;
    const int gc = rm.gidx < G ? rm.gidx : G - 1;
    const T* qp = reinterpret_cast<const T*>(a.q) + (((long)st.start + tc) * a.hq + h * G + gc) * DK + 8 * g;
#pragma unroll
    for (int kk = 0; kk < DK / 32; ++kk) qf[j][kk] = load8(qp + 32 * kk);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const RowMap r4 = map_row(st.t0, gi, 4 * g + i, lgp, G, st.len);
      lse_r[j][i] = r4.valid ? a.lse[((long)st.start + r4.tok) * a.hq + h * G + r4.gidx] * kLog2e
                             : __builtin_huge_valf();
    }
  }

  for (int i = tid; i < TQ * Ns; i += NT) bins[i] = 0.f;
  wait_all_loads();

  vec8_t<T> kr[KPT];
  unsigned koff[KPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    const int p = tid + i * NT;
    koff[i] = (unsigned)((p / (DK / 8)) * (int)a.ck_row_stride + (p % (DK / 8)) * 8);
  }
  auto gload = [&](int c0) {
    if (c0 + CH <= Nc) {
      const unsigned base = (unsigned)c0 * (unsigned)a.ck_row_stride;
#pragma unroll
      for (int i = 0; i < KPT; ++i)
        if (KPIECES % NT == 0 || tid + i * NT < KPIECES) kr[i] = load8(ckb + (base + koff[i]));
    } else {
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        const int p = tid + i * NT;
        if (KPIECES % NT == 0 || p < KPIECES) {
          const int sr = min(c0 + p / (DK / 8), Nc - 1);
          kr[i] = load8(ckb + (long)sr * a.ck_row_stride + (p % (DK / 8)) * 8);
        }
      }
    }
  };
  auto lstore = [&](int buf) {
    T* dk = ldsK + buf * CH * KLD;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int p = tid + i * NT;
      if (KPIECES % NT == 0 || p < KPIECES) store8(dk + (p / (DK / 8)) * KLD + (p % (DK / 8)) * 8, kr[i]);
    }
  };

  const int c_end = Ns > 0 ? Nc : 0;
  if (c_end > 0) {
    gload(0);
    lstore(0);
  }
  __syncthreads();
  int buf = 0;
  for (int c0 = 0; c0 < c_end; c0 += CH) {
    const bool has_next = c0 + CH < c_end;
    if (has_next) gload(c0 + CH);
    const T* bk = ldsK + buf * CH * KLD;
#pragma unroll
    for (int kt = 0; kt < CH / 16; ++kt) {
      const int cb = c0 + 16 * kt;
      if (cb >= Nc) break;
      f32x4_t s[NG];
#pragma unroll
      for (int j = 0; j < NG; ++j) s[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const T* kp = bk + (16 * kt + n) * KLD + 8 * g;
#pragma unroll
      for (int kk = 0; kk < DK / 32; ++kk) {
        const vec8_t<T> kf = load8(kp + 32 * kk);
#pragma unroll
        for (int j = 0; j < NG; ++j) s[j] = mma16(qf[j][kk], kf, s[j]);   // rows = heads, columns = keys
      }
      const int c = cb + n;
      // bins that contain column c: b*s - p <= c < b*s - p + k
      const int num = c + a.pool_p - a.pool_k + 1;
      const int b_lo = num <= 0 ? 0 : (num + a.pool_s - 1) / a.pool_s;
      const int b_hi = min((c + a.pool_p) / a.pool_s, Ns - 1);
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        const int gi = wave * NG + j;
        float e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = fast_exp2(fmaf(s[j][i], kLog2e, -lse_r[j][i]));
        if (lgp >= 2) {
          float v = (e[0] + e[1]) + (e[2] + e[3]);
          if (lgp == 3) v = colpair_sum(v);
          if (lgp >= 4) v = colgroup_sum(v);
          const bool adder = lgp >= 4 ? (g == 0) : (lgp == 3 ? ((g & 1) == 0) : true);
          const int tl = (gi * 16 + 4 * g) >> lgp;
          if (adder && c < Nc)
            for (int b = b_lo; b <= b_hi; ++b) atomicAdd(&bins[tl * Ns + b], v);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int tl = (gi * 16 + 4 * g + i) >> lgp;
            if (c < Nc)
              for (int b = b_lo; b <= b_hi; ++b) atomicAdd(&bins[tl * Ns + b], e[i]);
          }
        }
      }
    }
    if (has_next) lstore(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
  __syncthreads();

  // average and top-n per token; each lane only ever touches the bins b == lane (mod 64)
  volatile float* vb = bins;
  for (int tl = wave; tl < TQ; tl += NW) {
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
    if (a.pooled != nullptr)
      for (int b = Ns + lane; b < a.max_ns; b += 64) a.pooled[orow * a.pooled_stride + b] = 0.f;
    auto emit = [&](int r, int val) {
      if (lane == 0) {
        const long pos = orow * a.top_n + r;
        if (a.idx64) reinterpret_cast<int64_t*>(a.indices)[pos] = val;
        else reinterpret_cast<int32_t*>(a.indices)[pos] = val;
      }
    };
    if (Ns <= 64 * 8) {
      wave_topn<8>(vb + tl * Ns, Ns, a.top_n, lane, emit);
    } else {
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
        emit(r, found ? bi : -1);
      }
    }
  }
}

// Reduce-scatter of four per-lane partial column sums over the four 16-lane rows of a wavefront:
// row g of the result holds the total of v_g.  Each step is one lane swap plus one add and needs no
// copies, because the two swapped registers hold different values that are both consumed.
__device__ __forceinline__ float row_reduce_scatter4(float v0, float v1, float v2, float v3) {
  auto rs32 = [](float a, float b) {       // lower half: a summed over rows (g, g+2); upper half: b
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
  };
  const float x = rs32(v0, v2), y = rs32(v1, v3);
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The same for two tokens whose heads share the 16 rows of a tile (rows 0-7 token A, rows 8-15 token B; v_t is the
// per-lane sum of score tile t): ra / rb receive, in lane i, the head sum of column i of token A / B.
__device__ __forceinline__ void row_reduce_scatter2x2(float v0, float v1, float v2, float v3, float& ra, float& rb) {
  auto rs16 = [](float a, float b) {       // even row g: a summed over rows (g, g+1); odd row: b
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
  };
  const float x = rs16(v0, v1), y = rs16(v2, v3);      // rows 0 / 1: tiles (0, 1) resp. (2, 3) of A; rows 2 / 3: of B
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
  ra = __uint_as_float(r[0]);
  rb = __uint_as_float(r[1]);
}

// Four tokens of up to four heads each (lane row g = token g): a 4 x 4 transpose over the lane rows, r[t] gets,
// in lane i, the head sum of column i of token t.
__device__ __forceinline__ void row_transpose4(float v0, float v1, float v2, float v3, float (&r)[4]) {
  const auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v0), __float_as_uint(v2), false, false);
  const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v1), __float_as_uint(v3), false, false);
  const auto c = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);
  const auto d = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
  r[0] = __uint_as_float(c[0]); r[1] = __uint_as_float(c[1]);
  r[2] = __uint_as_float(d[0]); r[3] = __uint_as_float(d[1]);
}

// Block importance for the common shape: GQA group of 9..16 heads (one token per row group) and
// the default pooling (windows of 5 columns every 4, no padding).  Writes the raw window sums to
// a.pooled; topn_kernel below turns them into averages and picks the blocks.
//
// A workgroup of NW wavefronts owns NW*NG tokens of one kv head and streams ck through LDS in steps
// of 64 rows, double buffered.  Per step and token a wavefront computes four 16x16 score tiles
// (rows = heads, columns = compressed rows), exponentiates, adds the four heads each lane holds and
// keeps one partial per tile; a 3-swap reduce-scatter then leaves lane i with the head sum R of
// column c0 + i.  Bin b = R[4b .. 4b+4]: the quad sum comes from two DPP adds, the fifth column from
// the next lane (wave_shl:1), so lanes 3, 7, .., 59 each store one finished bin and lane 63 carries
// its quad to the next step, where it is completed with that step's first column.  Every bin is
// written exactly once, 64 contiguous bytes per token and step, with no atomics.
// TP tokens share the 16 rows of a tile: 1 for groups of 9..16 heads, 2 for 5..8 (rows 8t .. 8t+7 = token t),
// 4 for up to 4 heads (rows 4t .. 4t+3); rows beyond the group's heads are padding (weight 0).
template <typename T, int DK, int NG, int NW, int TP>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NG <= 2 ? 4 : 2, NG <= 2 ? 4 : 2)))
importance_stream_kernel(const CmpArgs a) {
  constexpr int CH = 64, KLD = DK + kLdsRowPad<T>, NT = NW * 64, TQ = NW * NG * TP, GP = 16 / TP;
  constexpr int KPIECES = CH * DK / 8;
  constexpr int KPT = (KPIECES + NT - 1) / NT;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* ldsK = reinterpret_cast<T*>(smem_raw);                       // [2][CH][KLD]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv;
  const SeqTile st = find_tile(a.cu_seq, a.batch, TQ, blockIdx.x);
  if (!st.valid) return;
  const int h = blockIdx.y;
  const int coff = a.cu_cmp[st.b];
  const int Nc = a.cu_cmp[st.b + 1] - coff;
  // pooling windows of ps + 1 columns every ps columns; ps = 1, 2, 4 or 8 (selection blocks of 1, 2, 4, 8 strides).
  // Padding of `pad` columns (compression blocks beyond two strides): column c sits at position c + pad of the
  // padded row, the stream runs over positions 0 .. Nc + pad - 1 (lane i of a step = position x0 + i) and bin j
  // pools positions j * ps .. j * ps + ps, so the bins stay aligned with the lanes whatever the padding.
  const int ps = a.pool_s, lps = ps == 1 ? 0 : ps == 2 ? 1 : ps == 4 ? 2 : 3;
  const int pad = a.pool_p;
  const int Np = Nc + pad;                      // positions that hold a column
  int Ns = 0;
  if (Nc > 0 && Nc + 2 * pad >= ps + 1) {
    Ns = (Nc + 2 * pad - 2) / ps + 1;           // ceil((Nc + 2 pad - (ps + 1)) / ps) + 1
    if ((Ns - 1) * ps >= Np) --Ns;
  }
  Ns = min(Ns, a.max_ns);
  if (Ns == 0) return;
  // h counts sub-groups of 16 query heads; sub-group h scores against the compressed keys of kv head h / kv_rep
  const T* ckb = reinterpret_cast<const T*>(a.ck) + (long)coff * a.ck_row_stride + (long)(h / a.kv_rep) * a.ck_head_stride;

  vec8_t<T> qf[NG][DK / 32];
  float lse_r[NG][4];        // lse * log2(e) of the heads in rows 4g+i; +inf removes padded rows
  float* prow[NG][TP];       // a token's row of window sums
  int ns_tok[NG][TP];        // Ns, or 0 for a token past the end of the sequence: nothing is stored
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    const int tok0 = st.t0 + (wave * NG + j) * TP;         // first token of this row group
    {
      const int tok = tok0 + n / GP, hd = n % GP;          // row n of the tile
      const int tc = tok < st.len ? tok : st.len - 1;
      const int gc = hd < G ? hd : G - 1;
      const T* qp = reinterpret_cast<const T*>(a.q) + (((long)st.start + tc) * a.hq + h * G + gc) * DK + 8 * g;
#pragma unroll
      for (int kk = 0; kk < DK / 32; ++kk) qf[j][kk] = load8(qp + 32 * kk);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tok = tok0 + (4 * g + i) / GP, hd = (4 * g + i) % GP;
      lse_r[j][i] = (tok < st.len && hd < G) ? a.lse[((long)st.start + tok) * a.hq + h * G + hd] * kLog2e
                                             : __builtin_huge_valf();
    }
#pragma unroll
    for (int t = 0; t < TP; ++t) {
      const int tok = tok0 + t;
      const int tc = tok < st.len ? tok : st.len - 1;
      prow[j][t] = a.pooled + (((long)st.start + tc) * a.hkv + h) * a.pooled_stride;
      ns_tok[j][t] = tok < st.len ? Ns : 0;
    }
  }
  wait_all_loads();

  float pend[NG][TP];        // lane 63: the quad sum of the previous step's last bin
#pragma unroll
  for (int j = 0; j < NG; ++j)
#pragma unroll
    for (int t = 0; t < TP; ++t) pend[j][t] = 0.f;

  vec8_t<T> kr[KPT];
  unsigned koff[KPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    const int p = tid + i * NT;
    koff[i] = (unsigned)((p / (DK / 8)) * (int)a.ck_row_stride + (p % (DK / 8)) * 8);
  }
  auto gload = [&](int x0) {               // rows of the step at position x0: columns x0 - pad .. x0 - pad + CH - 1
    const int c0 = x0 - pad;
    if (c0 >= 0 && c0 + CH <= Nc) {
      const unsigned base = (unsigned)c0 * (unsigned)a.ck_row_stride;
#pragma unroll
      for (int i = 0; i < KPT; ++i)
        if (KPIECES % NT == 0 || tid + i * NT < KPIECES) kr[i] = load8(ckb + (base + koff[i]));
    } else {                                         // first step under padding, last step: clamp the row
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        const int p = tid + i * NT;
        if (KPIECES % NT == 0 || p < KPIECES) {
          const int sr = max(min(c0 + p / (DK / 8), Nc - 1), 0);
          kr[i] = load8(ckb + (long)sr * a.ck_row_stride + (p % (DK / 8)) * 8);
        }
      }
    }
  };
  auto lstore = [&](int buf) {
    T* dk = ldsK + buf * CH * KLD;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int p = tid + i * NT;
      if (KPIECES % NT == 0 || p < KPIECES) store8(dk + (p / (DK / 8)) * KLD + (p % (DK / 8)) * 8, kr[i]);
    }
  };

  gload(0);
  lstore(0);
  __syncthreads();
  const bool writer = (lane & (ps - 1)) == ps - 1;       // last lane of a window's ps own columns
  const bool carrier = lane == 63;
  // Software pipeline inside every wavefront: while the matrix unit multiplies score tile i, the
  // vector ALU exponentiates tile i-1 (kept in `sp`), one or two operations after each MFMA.
  // Without this the wavefronts of a SIMD drift into lockstep -- all multiplying, then all
  // exponentiating -- and the two units take turns instead of working at the same time.
  constexpr int NK = DK / 32, SLOTS = NK * NG, NOPS = NG * 7;
  f32x4_t sp[NG];
  float v[NG][4], e[NG][4], ea[NG], eb[NG];
#pragma unroll
  for (int j = 0; j < NG; ++j) sp[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  auto pool_store = [&](int c0) {          // window sums of the step that started at position c0
    const bool live = (unsigned)(c0 + lane - pad) < (unsigned)Nc;
    const int idx = carrier ? (c0 >> lps) - 1 : (c0 >> lps) + (lane >> lps);
#pragma unroll
    for (int j = 0; j < NG; ++j) {
      float rt[TP];                                          // lane i: column c0 + i of token t
      if constexpr (TP == 1) rt[0] = row_reduce_scatter4(v[j][0], v[j][1], v[j][2], v[j][3]);
      else if constexpr (TP == 2) row_reduce_scatter2x2(v[j][0], v[j][1], v[j][2], v[j][3], rt[0], rt[1]);
      else row_transpose4(v[j][0], v[j][1], v[j][2], v[j][3], rt);
#pragma unroll
      for (int t = 0; t < TP; ++t) {
        const float r = live ? rt[t] : 0.f;
        float quad = r;
        if (ps >= 2) quad += dpp_f32<0xB1>(r);               // quad_perm [1,0,3,2]: pairs
        if (ps >= 4) quad += dpp_f32<0x4E>(quad);            // quad_perm [2,3,0,1]: quads
        if (ps == 8) quad += __shfl_xor(quad, 4);            // eight columns
        const float nxt = dpp_f32<0x130>(r);                 // wave_shl:1 -> column c0 + i + 1 (0 in lane 63)
        const float first = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(r), 0));
        const float val = carrier ? pend[j][t] + first : quad + nxt;
        if (writer && idx >= 0 && idx < ns_tok[j][t]) prow[j][t][idx] = val;
        pend[j][t] = quad;
      }
    }
  };
  // operation `op` of the exponentiation of tile `tp` held in sp: per group 4 x (fma, exp), 3 adds
  auto exp_op = [&](int op, int tp) {
    const int r = op / NG, j = op % NG;
    // the empty asm pins the value to this point of the program: without it the optimiser sinks
    // the whole computation down to its first use, behind all the MFMAs
    if (r < 4) { e[j][r] = fast_exp2(fmaf(sp[j][r], kLog2e, -lse_r[j][r])); asm volatile("" : "+v"(e[j][r])); }
    else if (r == 4) { ea[j] = e[j][0] + e[j][1]; asm volatile("" : "+v"(ea[j])); }
    else if (r == 5) { eb[j] = e[j][2] + e[j][3]; asm volatile("" : "+v"(eb[j])); }
    else { v[j][tp] = ea[j] + eb[j]; asm volatile("" : "+v"(v[j][tp])); }
  };
  int buf = 0;
  for (int c0 = 0; c0 < Np; c0 += CH) {    // c0: position of the step's first lane
    const bool has_next = c0 + CH < Np;
    if (has_next) gload(c0 + CH);
    const T* bk = ldsK + buf * CH * KLD;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      f32x4_t sc[NG];
#pragma unroll
      for (int j = 0; j < NG; ++j) sc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const T* kp = bk + (16 * kt + n) * KLD + 8 * g;
      vec8_t<T> kf = load8(kp);
#pragma unroll
      for (int kk = 0; kk < NK; ++kk) {
        const vec8_t<T> kcur = kf;
        if (kk + 1 < NK) kf = load8(kp + 32 * (kk + 1));
#pragma unroll
        for (int j = 0; j < NG; ++j) {
          sc[j] = mma16(qf[j][kk], kcur, sc[j]);            // rows = heads, columns = keys
          const int slot = kk * NG + j;
#pragma unroll
          for (int op = slot * NOPS / SLOTS; op < (slot + 1) * NOPS / SLOTS; ++op) exp_op(op, (kt + 3) & 3);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (kt == 0 && c0 > 0) pool_store(c0 - CH);
#pragma unroll
      for (int j = 0; j < NG; ++j) sp[j] = sc[j];
    }
    if (has_next) lstore(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
#pragma unroll
  for (int op = 0; op < NOPS; ++op) exp_op(op, 3);
  pool_store(((Np - 1) >> 6) << 6);
  if (carrier) {
    const int b = ((((Np - 1) >> 6) << 6) >> lps) + (64 >> lps) - 1;   // last bin of the last step: no next column
#pragma unroll
    for (int j = 0; j < NG; ++j)
#pragma unroll
      for (int t = 0; t < TP; ++t)
        if (b < ns_tok[j][t]) prow[j][t][b] = pend[j][t];
  }
}

// One wavefront per (token, kv head): window sums -> averages (ceil-mode pool, padding counted in
// the divisor, written back over the sums, bins past the sequence's last one zeroed) and the top_n
// bins in descending order, ties to the lower index, -1 where the sequence has fewer bins.
// With kv_rep > 1 (GQA group of kv_rep * 16 heads) a.pooled holds one row of window sums per sub-group of 16
// heads, kv_rep consecutive rows per kv head: they are added up here (the importance of a block is the sum over
// all heads of the group), and the averages go to the first of them.
template <int PER>
__global__ void __launch_bounds__(256)
topn_kernel(const CmpArgs a) {
  const int lane = threadIdx.x & 63;
  const int hkv_r = a.hkv / a.kv_rep;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);       // token * (kv heads) + kv head
  if (row >= (long)a.total * hkv_r) return;
  const int tg = (int)(row / hkv_r);
  int sb = 0;
  {
    int hi = a.batch;
    while (hi - sb > 1) {
      const int mid = (sb + hi) >> 1;
      if (a.cu_seq[mid] <= tg) sb = mid; else hi = mid;
    }
  }
  const int Nc = a.cu_cmp[sb + 1] - a.cu_cmp[sb];
  int Ns = 0;
  if (Nc > 0 && Nc + 2 * a.pool_p >= a.pool_k) {
    Ns = (Nc + 2 * a.pool_p - a.pool_k + a.pool_s - 1) / a.pool_s + 1;
    if ((Ns - 1) * a.pool_s >= Nc + a.pool_p) --Ns;
  }
  Ns = min(Ns, a.max_ns);
  float* prow = a.pooled + row * a.kv_rep * a.pooled_stride;
  float v[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int b = lane + 64 * k;
    v[k] = b < Ns ? prow[b] : -1.f;
  }
  for (int r = 1; r < a.kv_rep; ++r) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int b = lane + 64 * k;
      if (b < Ns) v[k] += prow[(long)r * a.pooled_stride + b];
    }
  }
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int b = lane + 64 * k;
    if (b < Ns) {
      const int lo = b * a.pool_s - a.pool_p;
      const int div = min(lo + a.pool_k, Nc + a.pool_p) - lo;
      v[k] = v[k] / (float)div;
      if (a.keep_pooled) prow[b] = v[k];
    } else if (b < a.max_ns && a.keep_pooled) {
      prow[b] = 0.f;
    }
  }
  // lane r keeps the r-th pick; one coalesced store per row at the end (top_n <= 64)
  int picked = -1;
  auto emit = [&](int r, int val) { picked = lane == r ? val : picked; };
  auto flush = [&]() {
    if (lane < a.top_n) {
      const long pos = row * a.top_n + lane;
      if (a.idx64) reinterpret_cast<int64_t*>(a.indices)[pos] = picked;
      else reinterpret_cast<int32_t*>(a.indices)[pos] = picked;
    }
  };

  __shared__ float cand_v[4][128];
  __shared__ int cand_i[4][128];
  const int w = threadIdx.x >> 6;
  wave_topn_shortlist<PER>(v, a.top_n, lane, cand_v[w], cand_i[w], emit);
  flush();
}

int set_smem(const void* fn, size_t bytes);
int group_pow2(int G);

template <typename T, int DK, int NG>
static int launch_select_ng(const CmpArgs& a, hipStream_t st) {
  constexpr int CH = 32, NW = 4;
  const int Gp = group_pow2(a.hq / a.hkv);
  const int TQ = NW * NG * 16 / Gp;
  const size_t smem = 2 * (size_t)CH * (DK + kLdsRowPad<T>) * sizeof(T) + (size_t)TQ * a.max_ns * sizeof(float);
  if (smem > 160 * 1024) return -3;
  auto fn = importance_select_kernel<T, DK, NG, CH, NW>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  const int tiles = a.total / TQ + a.batch;
  hipLaunchKernelGGL(fn, dim3(tiles, a.hkv), dim3(NW * 64), smem, st, a);
  return 0;
}

#ifndef NSA_STREAM_NW
#define NSA_STREAM_NW 8
#endif
#ifndef NSA_STREAM_NG
#define NSA_STREAM_NG 2
#endif

// Two kernels: window sums into a.pooled, then averages + top-n per (token, head).
template <typename T, int DK, int TP>
static int launch_importance(const CmpArgs& a, hipStream_t st) {
  constexpr int NW = NSA_STREAM_NW, NG = sizeof(T) == 2 ? NSA_STREAM_NG : NSA_STREAM_NG / 2, TQ = NW * NG * TP;
  const size_t smem = 2 * (size_t)64 * (DK + kLdsRowPad<T>) * sizeof(T);
  auto fn = importance_stream_kernel<T, DK, NG, NW, TP>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  const int tiles = a.total / TQ + a.batch;
  hipLaunchKernelGGL(fn, dim3(tiles, a.hkv), dim3(NW * 64), smem, st, a);
  return 0;
}

template <typename T, int DK>
static int launch_select_stream(const CmpArgs& a, hipStream_t st) {
  const int G = a.hq / a.hkv;      // 16 rows of a score tile = 1, 2 or 4 tokens
  const int rc = G <= 4 ? launch_importance<T, DK, 4>(a, st)
                        : G <= 8 ? launch_importance<T, DK, 2>(a, st) : launch_importance<T, DK, 1>(a, st);
  if (rc) return rc;
  const int rows = (int)(((long)a.total * (a.hkv / a.kv_rep) + 3) / 4);
  if (a.max_ns <= 512) hipLaunchKernelGGL(topn_kernel<8>, dim3(rows), dim3(256), 0, st, a);
  else if (a.max_ns <= 1024) hipLaunchKernelGGL(topn_kernel<16>, dim3(rows), dim3(256), 0, st, a);
  else if (a.max_ns <= 2048) hipLaunchKernelGGL(topn_kernel<32>, dim3(rows), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(topn_kernel<64>, dim3(rows), dim3(256), 0, st, a);
  return 0;
}

template <typename T, int DK>
static int launch_select_t(const CmpArgs& a, hipStream_t st) {
  // (groups below 16 heads run with the missing heads as padded rows: their log-sum-exp is +inf, their weight 0)
  if (a.pooled != nullptr && a.max_ns <= 4096 && a.top_n <= 64 && a.hq / a.hkv <= 16 &&
      (a.pool_s == 1 || a.pool_s == 2 || a.pool_s == 4 || a.pool_s == 8) && a.pool_k == a.pool_s + 1 &&
      a.pool_p >= 0 && a.pool_p < 64)
    return launch_select_stream<T, DK>(a, st);
  if (a.kv_rep > 1) return -6;      // groups beyond 16 heads exist on the two-kernel schedule only
  CmpArgs b = a;
  if (!a.keep_pooled) b.pooled = nullptr;   // this kernel keeps its bins in LDS: nothing to hand over
  // four row groups per wavefront unless the per-token bins of such a tile outgrow the LDS
  constexpr int NGBIG = sizeof(T) == 2 ? 4 : 2;
  const int rc = launch_select_ng<T, DK, NGBIG>(b, st);
  if (rc != -3) return rc;
  return launch_select_ng<T, DK, 1>(b, st);
}

int launch_select(const CmpArgs& a, hipStream_t st) {
  if (a.dtype == 0) {
    switch (a.dk) {
      case 32: return launch_select_t<bf16_t, 32>(a, st);
      case 64: return launch_select_t<bf16_t, 64>(a, st);
      case 128: return launch_select_t<bf16_t, 128>(a, st);
      case 192: return launch_select_t<bf16_t, 192>(a, st);
      default: return -2;
    }
  }
  if (a.dtype == 2) {
    switch (a.dk) {
      case 32: return launch_select_t<f16_t, 32>(a, st);
      case 64: return launch_select_t<f16_t, 64>(a, st);
      case 128: return launch_select_t<f16_t, 128>(a, st);
      case 192: return launch_select_t<f16_t, 192>(a, st);
      default: return -2;
    }
  }
  switch (a.dk) {
    case 32: return launch_select_t<float, 32>(a, st);
    case 64: return launch_select_t<float, 64>(a, st);
    case 128: return launch_select_t<float, 128>(a, st);
    case 192: return launch_select_t<float, 192>(a, st);
    default: return -2;
  }
}

}  // namespace nsa
