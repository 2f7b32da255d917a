// Compressed attention, block importance and top-n selection in ONE pass over the compressed keys.
//
// The reference multiplies q with the compressed keys once, keeps the scores in a [tokens][heads][rows] buffer and
// reads them back for the importance softmax, the pooling and the top-k (nsa/triton_attention.py:34,40,437,465-476).
// Here nothing is kept in memory: a wavefront owns ONE token (its up to 16 query heads are the 16 columns of a
// score tile) and, while the score tiles go by,
//   * runs the attention softmax of the visible rows (scaled scores, P V on the matrix unit), and
//   * exponentiates every raw score against the same reference, adds the pooling windows up PER HEAD and parks
//     each finished window sum in a register: 16 heads x 512 windows = 128 registers per lane, written once each.
// The importance softmax is normalised per head over ALL rows, so the window sums of different heads cannot be
// added before the pass is over; after it every head knows its normaliser, the lanes scale their 128 sums, a
// 4-level reduce-scatter over the 16 lanes of a lane row adds the heads and leaves 8 window sums per lane, and
// the wavefront picks the top_n windows.  Both softmaxes run against ONE FIXED reference per head (the largest raw
// score of the first 32 compressed rows): nothing is rescaled on the way.  A workgroup in which a sum left the safe
// range finds the exact maxima in a scores-only pass and repeats the pass with those as references.
//
// Pooling geometry: windows of 5 compressed rows every 4 (compression block of two strides, selection block of
// four), at most 2048 compressed rows per sequence (32768 tokens at stride 16), GQA groups of up to 16 heads,
// 16-bit inputs.  Everything else stays on the two-kernel schedule (attn.hip, select.hip).
//
// Where a window sum lives.  A 32-row step gives lane (n = head, g = lane row) the 8 rows 8g .. 8g+7: two window
// quads.  Window j = rows 4j .. 4j+4: its quad plus the first row of the next quad, which is the lane's own for the
// lower quad and sits one lane row further (or, for g = 3, in the next step) for the upper one.  Step i therefore
// writes slot 2i (window 8i + 2g) and slot 2i + 1 (window 8i + 2g + 1; in lane row 3 the window 8i - 1 of the step
// before, completed by this step's first row).  The last step's upper quad of lane row 3 has no next row and
// stays in `pend`, a 129th value per lane.
#include <type_traits>

#include "tiles.h"

namespace nsa {

typedef float f32x32_t __attribute__((ext_vector_type(32)));

int set_smem(const void* fn, size_t bytes);

constexpr int kFusedMaxRows = 2048;      // compressed rows per sequence the bins have room for

// Top-n over the PER candidates every lane holds (score v[k] >= 0 with window number ix[k]; -1 = no candidate),
// descending, ties to the lower window number; emit(r, window or -1).  The shortlist of tiles.h with explicit
// window numbers: the candidates of a lane need not be in any order.
template <int PER, typename Emit>
__device__ __forceinline__ void wave_topn_indexed(const float (&v)[PER], const int (&ix)[PER], int top_n, int lane,
                                                  float* cand_v, int* cand_i, Emit emit) {
  int total = 129;
  if (top_n <= 16) {
    float m = v[0];
#pragma unroll
    for (int k = 1; k < PER; ++k) m = fmaxf(m, v[k]);
    m = fmaxf(m, dpp_f32<0xB1>(m));
    m = fmaxf(m, dpp_f32<0x4E>(m));                       // quad maximum (-1 for a quad without candidates)
    const float L = wave_min_f32(m);                      // 16 quads: at least 16 candidates are >= L
    total = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const bool c = v[k] >= L && v[k] >= 0.f;
      const unsigned long long mask = __ballot(c);
      const int pos = total + (int)__builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32),
                                                             __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
      if (c && pos < 128) {
        cand_v[pos] = v[k];
        cand_i[pos] = ix[k];
      }
      total += __popcll(mask);
    }
  }
  if (total <= 128) {
    __builtin_amdgcn_wave_barrier();
    float c0 = lane < total ? cand_v[lane] : -1.f;
    float c1 = lane + 64 < total ? cand_v[lane + 64] : -1.f;
    const int i0 = lane < total ? cand_i[lane] : 0x7fffffff, i1 = lane + 64 < total ? cand_i[lane + 64] : 0x7fffffff;
    for (int r = 0; r < top_n; ++r) {
      const bool second = c1 > c0 || (c1 == c0 && i1 < i0);
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
        if (bi == win) {                                  // window numbers are unique: exactly one lane
          if (second) c1 = -1.f; else c0 = -1.f;
        }
      }
      emit(r, win);
    }
    return;
  }
  float w[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) w[k] = v[k];
  for (int r = 0; r < top_n; ++r) {
    float best = w[0];
    int bi = ix[0];
#pragma unroll
    for (int k = 1; k < PER; ++k)
      if (w[k] > best || (w[k] == best && ix[k] < bi)) { best = w[k]; bi = ix[k]; }
    long key = ((long)__float_as_int(best) << 32) | (unsigned int)(0x7fffffff - bi);
    key = wave_max_i64(key);
    const bool found = (int)(key >> 32) >= 0;
    const int win = 0x7fffffff - (int)(unsigned int)key;
    if (found) {
#pragma unroll
      for (int k = 0; k < PER; ++k)
        if (ix[k] == win && w[k] >= 0.f) w[k] = -1.f;
    }
    emit(r, found ? win : -1);
  }
}

// One level of the reduce-scatter over the 16 lanes of a lane row: of every pair (in[2j], in[2j + 1]) a lane keeps
// one (by `upper`), hands the other to its partner under the lane permutation CTRL (the partner keeps the other
// one) and adds what the partner hands over.  in: 2 * N values, out: N sums over twice as many lanes.
template <int CTRL, int N>
__device__ __forceinline__ void scatter_level(const float (&in)[2 * N], float (&out)[N], bool upper) {
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const float keep = upper ? in[2 * j + 1] : in[2 * j];
    const float give = upper ? in[2 * j] : in[2 * j + 1];
    out[j] = keep + dpp_f32<CTRL>(give);
  }
}

template <typename T, int DK, int DV>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
cmp_select_kernel(const CmpArgs a) {
  constexpr int NW = 8, CH = 64, NT = NW * 64, TQ = NW;
  constexpr int KLD = DK + kLdsRowPad<T>, VLD = CH + kLdsRowPad<T>;
  constexpr int KPIECES = CH * DK / 8, VPIECES = DV * CH / 8;
  constexpr int KPT = (KPIECES + NT - 1) / NT, VPT = (VPIECES + NT - 1) / NT;
  constexpr bool kNarrowP = std::is_same<T, f16_t>::value;      // packed probabilities narrower than the fp32 sums
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* ldsK = reinterpret_cast<T*>(smem_raw);          // [2][CH][KLD]
  T* ldsV = ldsK + 2 * CH * KLD;                     // [2][DV][VLD]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv;
  const SeqTile st = find_tile(a.cu_seq, a.batch, TQ, blockIdx.x);
  if (!st.valid) return;
  const int h = blockIdx.y;
  const int tok = st.t0 + wave;                      // this wavefront's token
  const bool tok_ok = tok < st.len;
  const int koff = a.cu_cmp[st.b];
  const int nkeys = min(a.cu_cmp[st.b + 1] - koff, kFusedMaxRows);
  const int vtoff = transposed_offset(koff, st.b);
  const T* kb = reinterpret_cast<const T*>(a.ck) + (long)koff * a.ck_row_stride + (long)h * a.ck_head_stride;
  const T* vtb = reinterpret_cast<const T*>(a.cvt) + (long)h * DV * a.cvt_cols + vtoff;

  auto last_visible = [&](int t) -> int {            // largest compressed row token t may attend
    if (!a.causal) return nkeys - 1;
    return t >= a.block ? min((t - a.block) / a.stride, nkeys - 1) : -1;
  };
  const int hi = tok_ok ? last_visible(tok) : -1;    // the same for all lanes: one token per wavefront
  const int attn_end = last_visible(min(st.t0 + TQ, st.len) - 1);
  const int c_end = nkeys;
  const int steps = (c_end + 31) >> 5;               // 32-row steps of the pass
  int Ns = 0;                                        // pooling windows of this sequence
  if (nkeys >= 5) {
    Ns = (nkeys - 2) / 4 + 1;
    if ((Ns - 1) * 4 >= nkeys) --Ns;
  }
  Ns = min(Ns, a.max_ns);

  RowGroup<T, DK, DV> grp[1];
  const RowMap rm = map_row(st.t0, wave, n, 4, G, st.len);
  load_q(grp[0], reinterpret_cast<const T*>(a.q), (long)st.start, rm, st.len, a.hq, h, G, g);
  group_reset(grp[0]);

  // The gating Linear on the query rows this wavefront holds: logits^T = W q^T as one more 16 x 16 tile (W's three
  // rows in rows 0..2 of the A operand), so lane row 0 ends with the three logits of column n.
  if (a.gate_w != nullptr) {
    const T* wp = reinterpret_cast<const T*>(a.gate_w) + (long)min(n, 2) * DK + 8 * g;
    const T* bp = reinterpret_cast<const T*>(a.gate_b);
    f32x4_t gt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < DK / 32; ++kk) gt = mma16(n < 3 ? load8(wp + 32 * kk) : zero8<T>(), grp[0].q[kk], gt);
    if (g == 0 && rm.valid) {
      T* gp = reinterpret_cast<T*>(a.gates) + (((long)st.start + rm.tok) * a.hq + h * G + rm.gidx) * 3;
#pragma unroll
      for (int i = 0; i < 3; ++i) gp[i] = (T)(gt[i] + (bp != nullptr ? (float)bp[i] : 0.f));
    }
  }
  const float c_attn = a.scale * kLog2e;

  // staging: every thread moves KPT + VPT 16-byte pieces of a 64-row chunk
  vec8_t<T> kr[KPT], vr[VPT];
  unsigned kpo[KPT], vpo[VPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    const int p = tid + i * NT;
    kpo[i] = (unsigned)((p / (DK / 8)) * (int)a.ck_row_stride + (p % (DK / 8)) * 8);
  }
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int p = tid + i * NT;
    vpo[i] = (unsigned)((p / (CH / 8)) * a.cvt_cols + (p % (CH / 8)) * 8);
  }
  auto gload = [&](int c0, bool with_v) {
    if (c0 + CH <= nkeys) {
      const unsigned base = (unsigned)c0 * (unsigned)a.ck_row_stride;
#pragma unroll
      for (int i = 0; i < KPT; ++i)
        if (KPIECES % NT == 0 || tid + i * NT < KPIECES) kr[i] = load8(kb + (base + kpo[i]));
    } else {                                         // last chunk of the sequence: clamp the row
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        const int p = tid + i * NT;
        if (KPIECES % NT == 0 || p < KPIECES) {
          const int sr = min(c0 + p / (DK / 8), nkeys - 1);
          kr[i] = load8(kb + (long)sr * a.ck_row_stride + (p % (DK / 8)) * 8);
        }
      }
    }
    if (with_v) {
#pragma unroll
      for (int i = 0; i < VPT; ++i)
        if (VPIECES % NT == 0 || tid + i * NT < VPIECES) vr[i] = load8(vtb + ((unsigned)c0 + vpo[i]));
    }
  };
  auto lstore = [&](int buf, bool with_v) {
    T* dk = ldsK + buf * CH * KLD;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int p = tid + i * NT;
      if (KPIECES % NT == 0 || p < KPIECES) store8(dk + (p / (DK / 8)) * KLD + (p % (DK / 8)) * 8, kr[i]);
    }
    if (with_v) {
      T* dv = ldsV + buf * DV * VLD;
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int p = tid + i * NT;
        if (VPIECES % NT == 0 || p < VPIECES) {
          // rows 16..31 of every 32-row step: the two 4-row halves trade places (see lds_key_of_row)
          const int pc = p % (CH / 8);
          vec8_t<T> x = vr[i];
          if (pc & 2) {
            vec8_t<T> y;
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = x[e ^ 4];
            x = y;
          }
          store8(dv + (p / (CH / 8)) * VLD + pc * 8, x);
        }
      }
    }
  };

  const bool swapped = (g >> 1) != 0;        // value i of this lane is row 8g + (i ^ 4) of the step instead of 8g + i
  const int swp = lds_key_swap(g);
  const bool last_row = g == 3;
  const int next_lane = ((lane + 16) & 63) << 2;

  f32x32_t bq0, bq1, bq2, bq3;               // the window sums of this lane's head: slot s = bq<s / 32>[s % 32]
#pragma unroll
  for (int i = 0; i < 32; ++i) { bq0[i] = 0.f; bq1[i] = 0.f; bq2[i] = 0.f; bq3[i] = 0.f; }
  float li = 0.f;                            // this lane's share of the importance denominator
  float pend = 0.f;                          // lane row 3: the upper quad of the step before
  float pmax = 0.f;                          // float16: the largest 8-row sum of packed probabilities
  float m_i = 0.f, m_a = 0.f;                // references of the two softmaxes (raw score units)
  float off_i = 0.f, off_a = 0.f;

  wait_all_loads();

  // One 32-row step.  derive: the first step sets the references.
  auto step32 = [&](f32x32_t& bins, int slot, int cb, const T* bk, const T* bv, bool derive) {
    f32x4_t s0[1], s1[1];
    const T* ks = bk + 8 * g;
    scores32<T, DK, DV, 1>(ks + lds_key_of_row(0, n) * KLD, ks + lds_key_of_row(1, n) * KLD, grp, s0, s1);
    float s[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) { s[i] = s0[0][i]; s[4 + i] = s1[0][i]; }
    const int key0 = cb + 8 * g;
    if (cb + 32 > nkeys) {                           // last step of the sequence only
      asm volatile("" ::: "memory");
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (key0 + (i ^ swp) >= nkeys) s[i] = kNegInf;
    }
    if (derive && cb == 0) {                         // the reference: largest score of the first 32 rows
      float mx = s[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) mx = fmaxf(mx, s[i]);
      m_i = m_a = colgroup_max(mx);                  // finite: row 0 exists
      off_i = -m_i * kLog2e;
      off_a = -m_a * c_attn;
    }
    float e[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) e[i] = fast_exp2(fmaf(s[i], kLog2e, off_i));
    const float qlo = (e[0] + e[1]) + (e[2] + e[3]), qhi = (e[4] + e[5]) + (e[6] + e[7]);
    li += qlo + qhi;
    const float first = swapped ? e[4] : e[0];       // row 8g: completes the upper window of the lane row before
    const float fifth = swapped ? e[0] : e[4];       // row 8g + 4: completes this lane's lower window
    const float qa = swapped ? qhi : qlo, qb = swapped ? qlo : qhi;
    const float nxt = __int_as_float(__builtin_amdgcn_ds_bpermute(next_lane, __float_as_int(first)));
    bins[slot] = qa + fifth;
    bins[slot + 1] = (last_row ? pend : qb) + nxt;
    pend = qb;
    if (cb <= hi) {                                  // the token attends rows of this step
      float p[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = fast_exp2(fmaf(s[i], c_attn, off_a));
      if (cb + 31 > hi) {                            // the step on the causal edge
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (key0 + (i ^ swp) > hi) p[i] = 0.f;
      }
      const float p8 = sum8(p);
      grp[0].l += p8;
      if constexpr (kNarrowP) pmax = fmaxf(pmax, p8);
      vec8_t<T> pb[1];
      pb[0] = pack8<T>(p);
      pv32_all<T, DK, DV, 1>(bv + n * VLD + 8 * g, 16 * VLD, grp, pb);
    }
  };

  auto run_pass = [&](bool derive) {
    if (c_end > 0) {
      gload(0, 0 <= attn_end);
      lstore(0, 0 <= attn_end);
    }
    __syncthreads();
    int buf = 0;
    // 512 rows = 16 steps = 32 slots per section: inside a section the slots of one register block are written
    // in place with a scalar index
    auto section = [&](f32x32_t& bins, int c_first) {
      const int c_stop = min(c_first + 512, c_end);
      for (int c0 = c_first; c0 < c_stop; c0 += CH) {
        const int cn = c0 + CH;
        const bool has_next = cn < c_end;
        const bool next_v = has_next && cn <= attn_end;
        if (has_next) gload(cn, next_v);
        const T* bk = ldsK + buf * CH * KLD;
        const T* bv = ldsV + buf * DV * VLD;
        const int slot = (c0 - c_first) >> 4;
        step32(bins, slot, c0, bk, bv, derive);
        if (c0 + 32 < c_end) step32(bins, slot + 2, c0 + 32, bk + 32 * KLD, bv + 32, derive);
        if (has_next) lstore(buf ^ 1, next_v);
        __syncthreads();
        buf ^= 1;
      }
    };
    section(bq0, 0);
    section(bq1, 512);
    section(bq2, 1024);
    section(bq3, 1536);
  };

  run_pass(true);
  float lt = colgroup_sum(grp[0].l), lit = colgroup_sum(li);
  {
    const bool sees = rm.valid && hi >= 0;
    int bad = !(lit < 1e30f) || !(lt < 1e30f) || (sees && !(lt > 1e-30f));
    if constexpr (kNarrowP) {
      // every packed probability is at most its 8-row sum: below 3e4 none overflowed float16, and a largest 8-row
      // sum of at least 2^-7 puts the row's largest probability at 2^-10 or more, a normal float16
      const float pm = colgroup_max(pmax);
      bad |= !(pm < 3e4f) || (sees && !(pm >= 0.0078125f));
    }
    if (__syncthreads_or(bad)) {
      // Rare: exact maxima first (scores only: the importance one over all rows, the attention one over the
      // visible rows), then the same pass with those as references -- no exponential exceeds 1.
      float mx_all = kNegInf, mx_vis = kNegInf;
      if (c_end > 0) {
        gload(0, false);
        lstore(0, false);
      }
      __syncthreads();
      int buf = 0;
      for (int c0 = 0; c0 < c_end; c0 += CH) {
        const bool has_next = c0 + CH < c_end;
        if (has_next) gload(c0 + CH, false);
        const T* bk = ldsK + buf * CH * KLD;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
          const int cb = c0 + 32 * sub;
          if (cb >= c_end) break;
          f32x4_t s0[1], s1[1];
          const T* ks = bk + 32 * sub * KLD + 8 * g;
          scores32<T, DK, DV, 1>(ks + lds_key_of_row(0, n) * KLD, ks + lds_key_of_row(1, n) * KLD, grp, s0, s1);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float sv = i < 4 ? s0[0][i] : s1[0][i - 4];
            const int key = cb + 8 * g + (i ^ swp);
            if (key < nkeys) mx_all = fmaxf(mx_all, sv);
            if (key <= hi) mx_vis = fmaxf(mx_vis, sv);
          }
        }
        if (has_next) lstore(buf ^ 1, false);
        __syncthreads();
        buf ^= 1;
      }
      m_i = colgroup_max(mx_all);
      m_a = colgroup_max(mx_vis);
      if (m_i == kNegInf) m_i = 0.f;
      if (m_a == kNegInf) m_a = 0.f;
      off_i = -m_i * kLog2e;
      off_a = -m_a * c_attn;
      group_reset(grp[0]);
      li = 0.f;
      pend = 0.f;
      run_pass(false);
      lt = colgroup_sum(grp[0].l);
      lit = colgroup_sum(li);
    }
  }

  // ---- attention output: rows leave through LDS (the K buffers are free after the pass's last barrier)
  constexpr int OLD = DV + 8, PIECES = DV / 8;
  static_assert(NW * 16 * OLD * sizeof(T) + NW * 1024 <= (2 * CH * KLD + 2 * DV * VLD) * sizeof(T),
                "output staging and the top-n shortlists must fit the K/V buffers");
  {
    T* stage = ldsK + wave * 16 * OLD;
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    store_rows<T, DV>(stage + n * OLD, grp[0].o, inv, g);
    T* ob = reinterpret_cast<T*>(a.o);
#pragma unroll
    for (int k = 0; k < (16 * PIECES + 63) / 64; ++k) {
      const int e = lane + 64 * k;
      const int r = e / PIECES, pc = e % PIECES;
      if ((16 * PIECES % 64 == 0 || r < 16) && tok_ok && r < G) {
        const long orow = ((long)st.start + tok) * a.hq + h * G + r;
        store8(ob + orow * DV + pc * 8, load8(stage + r * OLD + pc * 8));
      }
    }
    if (rm.valid && g == 0) {
      const long row = ((long)st.start + tok) * a.hq + h * G + n;
      if (a.lse_attn != nullptr)
        a.lse_attn[row] = lt > 0.f ? fmaf(m_a, a.scale, __logf(lt)) : __builtin_huge_valf();
      if (a.lse != nullptr) a.lse[row] = nkeys > 0 ? m_i + __logf(lit) : 0.f;
    }
  }
  if (a.indices == nullptr || !tok_ok) return;

  // ---- block importance: scale by the head's normaliser, add the heads, average, pick
  const long orow = ((long)st.start + tok) * a.hkv + h;
  float v[9];
  int ix[9];
  {
    const float w = (rm.valid && lit > 0.f) ? 1.0f / lit : 0.f;     // padded heads weigh nothing
    float x[128];
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      x[i] = bq0[i] * w; x[32 + i] = bq1[i] * w; x[64 + i] = bq2[i] * w; x[96 + i] = bq3[i] * w;
    }
    // Partners: lane ^ 15 (row_mirror), ^ 7 (row_half_mirror), ^ 2, ^ 1 (quad permutations); each level is keyed on
    // a lane bit that its own partner flips and the later partners keep.  Lane n ends with the slots 16 k + c(n),
    // c = bit3 + 2 bit2 + 4 bit1 + 8 bit0, summed over the 16 heads.
    float y[64], z[32], u[16], r8[8];
    scatter_level<0x140, 64>(x, y, (n & 8) != 0);
    scatter_level<0x141, 32>(y, z, (n & 4) != 0);
    scatter_level<0x4E, 16>(z, u, (n & 2) != 0);
    scatter_level<0xB1, 8>(u, r8, (n & 1) != 0);
    const int c = ((n >> 3) & 1) + 2 * ((n >> 2) & 1) + 4 * ((n >> 1) & 1) + 8 * (n & 1);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int slot = 16 * k + c, i = slot >> 1, ab = slot & 1;
      int bin = 8 * i + 2 * g + ab;
      bool ok = true;
      if (last_row && ab) {                     // lane row 3 keeps the upper window of the step BEFORE in slot 2i + 1
        bin = 8 * i - 1;
        ok = i >= 1 && i < steps;
      }
      ok = ok && bin < Ns;
      const int lo = 4 * bin;
      v[k] = ok ? r8[k] / (float)(min(lo + 5, nkeys) - lo) : -1.f;
      ix[k] = ok ? bin : 0x7fffffff;
    }
    // the 129th value: the last step's upper window of lane row 3 (no next row), owned by lane (n = 0, g = 3)
    float tail = last_row ? pend * w : 0.f;
    tail += dpp_f32<0xB1>(tail);
    tail += dpp_f32<0x4E>(tail);
    tail += dpp_f32<0x141>(tail);
    tail += dpp_f32<0x140>(tail);
    {
      const int bin = 8 * steps - 1, lo = 4 * bin;
      const bool ok = last_row && n == 0 && steps > 0 && bin < Ns;
      v[8] = ok ? tail / (float)(min(lo + 5, nkeys) - lo) : -1.f;
      ix[8] = ok ? bin : 0x7fffffff;
    }
  }
  if (a.pooled != nullptr && a.keep_pooled) {
    float* prow = a.pooled + orow * a.pooled_stride;
#pragma unroll
    for (int k = 0; k < 9; ++k)
      if (ix[k] != 0x7fffffff) prow[ix[k]] = v[k];
    for (int b = Ns + lane; b < a.max_ns; b += 64) prow[b] = 0.f;
  }
  int picked = -1;
  auto emit = [&](int r, int val) { picked = lane == r ? val : picked; };
  float* cand_v = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(ldsK) + NW * 16 * OLD * sizeof(T)) + wave * 256;
  int* cand_i = reinterpret_cast<int*>(cand_v + 128);
  wave_topn_indexed<9>(v, ix, a.top_n, lane, cand_v, cand_i, emit);
  if (lane < a.top_n) {
    const long pos = orow * a.top_n + lane;
    if (a.idx64) reinterpret_cast<int64_t*>(a.indices)[pos] = picked;
    else reinterpret_cast<int32_t*>(a.indices)[pos] = picked;
  }
}

// ------------------------------------------------------------------------------------------------

bool cmp_select_single_pass_ok(const CmpArgs& a, int max_nc) {
  const int G = a.hq / a.hkv;
  return a.kv_rep == 1 && G >= 9 && G <= 16 && (a.dtype == 0 || a.dtype == 2) && a.pool_k == 5 && a.pool_s == 4 &&
         a.pool_p == 0 && max_nc <= kFusedMaxRows && a.max_ns <= 512 && a.top_n <= 64 && a.indices != nullptr &&
         a.cvt != nullptr && a.o != nullptr &&
         ((a.dk == 64 && a.dv == 64) || (a.dk == 128 && a.dv == 128) || (a.dk == 192 && a.dv == 128));
}

template <typename T, int DK, int DV>
static int launch_cmp_select_t(const CmpArgs& a, hipStream_t st) {
  constexpr int CH = 64;
  const size_t smem = 2 * ((size_t)CH * (DK + kLdsRowPad<T>) + (size_t)DV * (CH + kLdsRowPad<T>)) * sizeof(T);
  auto fn = cmp_select_kernel<T, DK, DV>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  const int tiles = a.total / 8 + a.batch;
  hipLaunchKernelGGL(fn, dim3(tiles, a.hkv), dim3(512), smem, st, a);
  return 0;
}

int launch_cmp_select(const CmpArgs& a, hipStream_t st) {
  const int key = a.dk * 1000 + a.dv;
  if (a.dtype == 0) {
    switch (key) {
      case 64064: return launch_cmp_select_t<bf16_t, 64, 64>(a, st);
      case 128128: return launch_cmp_select_t<bf16_t, 128, 128>(a, st);
      case 192128: return launch_cmp_select_t<bf16_t, 192, 128>(a, st);
      default: return -2;
    }
  }
  if (a.dtype == 2) {
    switch (key) {
      case 64064: return launch_cmp_select_t<f16_t, 64, 64>(a, st);
      case 128128: return launch_cmp_select_t<f16_t, 128, 128>(a, st);
      case 192128: return launch_cmp_select_t<f16_t, 192, 128>(a, st);
      default: return -2;
    }
  }
  return -2;
}

}  // namespace nsa
