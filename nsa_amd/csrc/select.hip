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

// FAST: GQA group of 16 (one token per row group) and the default pooling (5 columns every 4, no
// padding); everything else takes the generic path with LDS atomics.
template <typename T, int DK, int NG, int CH, int NW, bool FAST>
__global__ void __launch_bounds__(NW * 64)
importance_select_kernel(const CmpArgs a) {
  constexpr int KLD = DK + 8, ROWS = NW * NG * 16, NT = NW * 64;
  constexpr int KPIECES = CH * DK / 8;
  constexpr int KPT = (KPIECES + NT - 1) / NT;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* ldsK = reinterpret_cast<T*>(smem_raw);                       // [2][CH][KLD]
  float* bins = reinterpret_cast<float*>(ldsK + 2 * CH * KLD);    // [TQ][Ns]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv, Gp = FAST ? 16 : next_pow2(G), lgp = FAST ? 4 : ilog2(Gp);
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

  float pend[NG];   // FAST: the unfinished last bin of the previous tile (lane 12 of the g == 0 row)
#pragma unroll
  for (int j = 0; j < NG; ++j) pend[j] = 0.f;

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
      if (FAST) {
        // One token per row group, windows of 5 columns every 4: after the head sum every lane of
        // tile column n holds R[c].  Quad sums and the first column of the next quad come from DPP.
        // Bins 4t..4t+2 of tile t are complete at once; bin 4t+3 waits in a register of lane 12 for
        // the first column of the next tile.  Every bin is written exactly once by the g == 0 row.
#pragma unroll
        for (int j = 0; j < NG; ++j) {
          float e[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) e[i] = fast_exp2(fmaf(s[j][i], kLog2e, -lse_r[j][i]));
          float v = colgroup_sum((e[0] + e[1]) + (e[2] + e[3]));
          v = c < Nc ? v : 0.f;
          const float t2 = v + dpp_f32<0xB1>(v);            // quad_perm [1,0,3,2]
          const float quad = t2 + dpp_f32<0x4E>(t2);        // quad_perm [2,3,0,1]
          const float nextf = dpp_f32<0x104>(v);            // row_shl:4 -> R[c+4], 0 past the tile
          const float first = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
          if (g == 0 && (n & 3) == 0) {
            float* row = bins + (wave * NG + j) * Ns;
            const int b = (cb >> 2) + (n >> 2);
            if (n == 12) {
              if (cb > 0 && (cb >> 2) - 1 < Ns) row[(cb >> 2) - 1] = pend[j] + first;
              pend[j] = quad;
            } else if (b < Ns) {
              row[b] = quad + nextf;
            }
          }
        }
      } else {
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
    }
    if (has_next) lstore(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
  if (FAST && c_end > 0 && g == 0 && n == 12) {
    const int b = ((((c_end - 1) >> 4) << 4) >> 2) + 3;     // last bin of the last tile: no next column
#pragma unroll
    for (int j = 0; j < NG; ++j)
      if (b < Ns) bins[(wave * NG + j) * Ns + b] = pend[j];
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

int set_smem(const void* fn, size_t bytes);
int group_pow2(int G);

template <typename T, int DK, int NG>
static int launch_select_ng(const CmpArgs& a, hipStream_t st) {
  constexpr int CH = 32, NW = 4;
  const int Gp = group_pow2(a.hq / a.hkv);
  const int TQ = NW * NG * 16 / Gp;
  const size_t smem = 2 * (size_t)CH * (DK + 8) * sizeof(T) + (size_t)TQ * a.max_ns * sizeof(float);
  if (smem > 160 * 1024) return -3;
  const bool fast = Gp == 16 && a.pool_k == 5 && a.pool_s == 4 && a.pool_p == 0;
  auto fn = fast ? importance_select_kernel<T, DK, NG, CH, NW, true> : importance_select_kernel<T, DK, NG, CH, NW, false>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  const int tiles = a.total / TQ + a.batch;
  hipLaunchKernelGGL(fn, dim3(tiles, a.hkv), dim3(NW * 64), smem, st, a);
  return 0;
}

template <typename T, int DK>
static int launch_select_t(const CmpArgs& a, hipStream_t st) {
  // four row groups per wavefront unless the per-token bins of such a tile outgrow the LDS
  constexpr int NGBIG = sizeof(T) == 2 ? 4 : 2;
  const int rc = launch_select_ng<T, DK, NGBIG>(a, st);
  if (rc != -3) return rc;
  return launch_select_ng<T, DK, 1>(a, st);
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
  switch (a.dk) {
    case 32: return launch_select_t<float, 32>(a, st);
    case 64: return launch_select_t<float, 64>(a, st);
    case 128: return launch_select_t<float, 128>(a, st);
    case 192: return launch_select_t<float, 192>(a, st);
    default: return -2;
  }
}

}  // namespace nsa
