// Attention over a contiguous key stream shared by a whole token tile: the compressed branch
// (keys = compressed rows, plus the log-sum-exp of the raw scores that the block-importance kernel
// needs) and the sliding-window branch (keys = the union of the tile's windows).
//
// One workgroup of NW wavefronts owns NW*NG row groups (NW*NG*16 rows: 16 tokens for a GQA group
// of 16).  Keys stream through LDS in chunks of CH rows, K row-major and V key-contiguous, double
// buffered: the global loads of chunk i+1 are issued into registers before chunk i is computed and
// written to the other buffer afterwards, one barrier per chunk.  Every wavefront reads each K/V
// fragment from LDS once and feeds it to NG MFMAs (register blocking over row groups).
//
// Softmax bookkeeping of the compressed branch: two sums per row off one score tile,
//   li += exp(s - M)                         every row      -> lse = M + log(li)   (importance softmax, not causal)
//   l  += exp(scale*(s - M)), O += p V       visible rows   -> o = O / l
// In the common pass M is fixed after the first 32 rows (no maximum, no rescale, no branch per chunk); a row
// whose sums leave the safe range sends its workgroup through an exact second pass with a running maximum per
// softmax (the attention one over the visible rows only), so neither a large hidden score nor a late large
// score can cost a visible one its precision.
//
// The selected-block branch (one wavefront per row group, blocks read straight from global memory
// in fragment layout) and the gated combine of the three branches live here as well.
#include <type_traits>

#include "slc_merge.h"

namespace nsa {


struct StreamParams {
  const void* q; const void* k; const void* vt; void* o; float* lse;
  const int32_t* cu_seq; const int32_t* cu_key;
  int batch, hq, hkv;
  long k_row_stride, k_head_stride; int vt_cols;
  int block, stride, window, causal;
  float scale;
  MergeArgs mg;      // MERGE kernels only: the selected-attention partials and the other branches
  float* lse_attn;   // optional: log-sum-exp (natural log) of the scaled visible scores, for the backward
  int kv_rep;        // sub-groups of 16 query heads per kv head (1 unless the GQA group exceeds 16): hkv counts
                     // sub-groups, and sub-group h reads the keys / values of kv head h / kv_rep
  int split_hidden;  // compressed branch: stop at cmp_visible_end(): the rows beyond carry no attention, they only feed
                     // the importance log-sum-exp, which this caller did not ask for
  int tile_base = 0; // first token tile of this launch (workgroup x takes tile tile_base + x)
  const void* gate_w = nullptr; const void* gate_b = nullptr; void* gates = nullptr;   // as CmpArgs
};

// MERGE (sliding window only): 0 = write the branch output; otherwise the epilogue merges the
// block-major selected-attention partials of its rows, applies the gates, adds the compressed
// branch and writes the final output, so the window result never goes to memory (16 = top_n of exactly 16, all
// partial loads in flight; 2 = any top_n, the picks in rounds of 16; 1 = one partial at a time, kept for reference).
template <typename T, int DK, int DV, int NG, int CH, int NW, bool CMP, int MERGE = 0>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
stream_attn_kernel(const StreamParams a) {
  constexpr int KLD = DK + kLdsRowPad<T>, VLD = CH + kLdsRowPad<T>, ROWS = NW * NG * 16, NT = NW * 64;
  constexpr int KPIECES = CH * DK / 8, VPIECES = DV * CH / 8;
  constexpr int KPT = (KPIECES + NT - 1) / NT, VPT = (VPIECES + NT - 1) / NT;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* ldsK = reinterpret_cast<T*>(smem_raw);          // [2][CH][KLD]
  T* ldsV = ldsK + 2 * CH * KLD;                     // [2][DV][VLD]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: group bounds stay in SGPRs
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv, Gp = next_pow2(G), lgp = ilog2(Gp);
  const int TQ = ROWS >> lgp;
  const SeqTile st = find_tile(a.cu_seq, a.batch, TQ, a.tile_base + blockIdx.x);
  if (!st.valid) return;
  const int h = blockIdx.y;
  const int hk = h / a.kv_rep;                 // kv head whose keys / values this (sub-)group reads
  const int t_last = min(st.t0 + TQ, st.len) - 1;

  // key space of this sequence
  int nkeys, koff, vtoff;
  if (CMP) {
    koff = a.cu_key[st.b];
    nkeys = a.cu_key[st.b + 1] - koff;
    vtoff = transposed_offset(koff, st.b);
  } else {
    koff = st.start;
    nkeys = st.len;
    vtoff = transposed_offset(st.start, st.b);
  }
  const T* kb = reinterpret_cast<const T*>(a.k) + (long)koff * a.k_row_stride + (long)hk * a.k_head_stride;
  const T* vtb = reinterpret_cast<const T*>(a.vt) + (long)hk * DV * a.vt_cols + vtoff;
  const int W = a.window;

  auto last_visible = [&](int t) -> int {      // largest key index token t may attend
    if (!CMP) return t;
    if (!a.causal) return nkeys - 1;
    return t >= a.block ? min((t - a.block) / a.stride, nkeys - 1) : -1;
  };

  RowGroup<T, DK, DV> grp[NG];
  RowMap rm[NG];
  int hi[NG], lo[NG];            // per lane: visible keys are lo..hi
  int g_hi_max[NG], g_hi_min[NG], g_lo_min[NG], g_lo_max[NG];   // wave uniform bounds over the group
  float li[NG];                  // compressed branch: this lane's share of the importance denominator ...
  float mi[NG];                  // ... and its reference (the attention softmax keeps its own in grp[j].m)
  // float16 only: the largest 8-key sum of probabilities this lane has packed.  The sums are fp32, the packed
  // probabilities are not: a float16 probability overflows at 65504 and loses its mantissa below 6e-5, ranges that
  // the fp32 sums pass through unnoticed.
  constexpr bool kNarrowP = std::is_same<T, f16_t>::value;
  float pmax[NG];
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    const int gi = wave * NG + j;
    rm[j] = map_row(st.t0, gi, n, lgp, G, st.len);
    load_q(grp[j], reinterpret_cast<const T*>(a.q), (long)st.start, rm[j], st.len, a.hq, h, G, g);
    group_reset(grp[j]);
    li[j] = 0.f;
    mi[j] = kNegInf;
    pmax[j] = 0.f;
    hi[j] = last_visible(rm[j].tok);
    lo[j] = CMP ? 0 : rm[j].tok - W + 1;
    const int tf = st.t0 + ((gi * 16) >> lgp);
    const int tl = min(st.t0 + ((gi * 16 + 15) >> lgp), st.len - 1);
    g_hi_min[j] = last_visible(tf);
    g_hi_max[j] = last_visible(tl);          // below g_hi_min when the group lies past the sequence end
    g_lo_min[j] = CMP ? 0 : tf - W + 1;
    g_lo_max[j] = CMP ? 0 : tl - W + 1;
  }
  if constexpr (CMP) {
    // The gating Linear on the query rows this wavefront holds: logits^T = W q^T as one more 16 x 16 tile per row
    // group (W's three rows in rows 0..2 of the A operand), so lane group 0 ends with the three logits of column n.
    if (a.gate_w != nullptr) {
      const T* wp = reinterpret_cast<const T*>(a.gate_w) + (long)min(n, 2) * DK + 8 * g;
      const T* bp = reinterpret_cast<const T*>(a.gate_b);
      vec8_t<T> wf[DK / 32];
#pragma unroll
      for (int kk = 0; kk < DK / 32; ++kk) wf[kk] = n < 3 ? load8(wp + 32 * kk) : zero8<T>();
      float bias[3] = {0.f, 0.f, 0.f};
      if (bp != nullptr) { bias[0] = (float)bp[0]; bias[1] = (float)bp[1]; bias[2] = (float)bp[2]; }
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        f32x4_t gt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < DK / 32; ++kk) gt = mma16(wf[kk], grp[j].q[kk], gt);
        if (g == 0 && rm[j].valid) {
          T* gp = reinterpret_cast<T*>(a.gates) + (((long)st.start + rm[j].tok) * a.hq + h * G + rm[j].gidx) * 3;
#pragma unroll
          for (int i = 0; i < 3; ++i) gp[i] = (T)(gt[i] + bias[i]);
        }
      }
    }
  }
  const float c_attn = a.scale * kLog2e;
  const int attn_end = last_visible(t_last);                      // last key any row of the tile attends
  const int c_begin = CMP ? 0 : (max(st.t0 - W + 1, 0) / CH) * CH;
  const int c_end = CMP ? (a.split_hidden ? cmp_visible_end(st.t0, TQ, st.len, nkeys, a.block, a.stride, a.causal) : nkeys)
                        : t_last + 1;

  // Per-thread element offsets of its staging pieces for chunk 0; a chunk adds one scalar.  Only the
  // last chunk of a sequence needs the row clamp.
  vec8_t<T> kr[KPT], vr[VPT];
  unsigned kpo[KPT], vpo[VPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    const int p = tid + i * NT;
    kpo[i] = (unsigned)((p / (DK / 8)) * (int)a.k_row_stride + (p % (DK / 8)) * 8);
  }
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int p = tid + i * NT;
    vpo[i] = (unsigned)((p / (CH / 8)) * a.vt_cols + (p % (CH / 8)) * 8);
  }
  auto gload = [&](int c0, bool with_v) {
    if (c0 + CH <= nkeys) {
      const unsigned base = (unsigned)c0 * (unsigned)a.k_row_stride;
#pragma unroll
      for (int i = 0; i < KPT; ++i)
        if (KPIECES % NT == 0 || tid + i * NT < KPIECES) kr[i] = load8(kb + (base + kpo[i]));
    } else {
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        const int p = tid + i * NT;
        if (KPIECES % NT == 0 || p < KPIECES) {
          const int r = p / (DK / 8), pc = p % (DK / 8);
          const int sr = min(c0 + r, nkeys - 1);
          kr[i] = load8(kb + (long)sr * a.k_row_stride + pc * 8);
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
          // keys 16..31 of every 32-key sub-chunk: the two 4-key halves trade places (see lds_key_of_row)
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

  wait_all_loads();
  // One pass over the key chunks.  FAST (compressed branch only): both softmaxes of a row run against one
  // FIXED reference, the largest raw score of the first 32 compressed rows, so a chunk costs neither a
  // maximum nor a branch; scores above the reference simply give exponentials above 1 (fp32 sums and bf16
  // probabilities keep their relative precision at any magnitude).  What a fixed reference cannot rule out --
  // a sum that overflows, or visible scores so far below the reference that their sum underflows -- is
  // checked once per row after the pass, and a workgroup that finds such a row runs the pass again in the
  // exact form (FAST = false): a running maximum per softmax, the importance one over all rows, the
  // attention one over the visible rows only.
  auto run_chunks = [&](auto fast_tag) {
    constexpr bool FAST = decltype(fast_tag)::value;
    if (c_begin < c_end) {
      const bool v0 = c_begin <= attn_end;
      gload(c_begin, v0);
      lstore(0, v0);
    }
    __syncthreads();
    int buf = 0;
    for (int c0 = c_begin; c0 < c_end; c0 += CH) {
      const int cn = c0 + CH;
      const bool has_next = cn < c_end;
      const bool next_v = has_next && cn <= attn_end;
      if (has_next) gload(cn, next_v);

      const T* bk = ldsK + buf * CH * KLD;
      const T* bv = ldsV + buf * DV * VLD;
#pragma unroll
      for (int sub = 0; sub < CH / 32; ++sub) {
        const int cb = c0 + 32 * sub;
        if (cb >= c_end) break;
        bool act[NG];
        bool any_act = false;
#pragma unroll
        for (int j = 0; j < NG; ++j) {
          act[j] = cb <= g_hi_max[j] && (CMP || cb + 31 >= g_lo_min[j]);
          any_act |= act[j];
        }
        if (!CMP && !any_act) continue;
        f32x4_t s0[NG], s1[NG];
        const T* ks = bk + 32 * sub * KLD + 8 * g;
        scores32<T, DK, DV, NG>(ks + lds_key_of_row(0, n) * KLD, ks + lds_key_of_row(1, n) * KLD, grp, s0, s1);
        const int swp = lds_key_swap(g);       // value i of this lane belongs to key cb + 8g + (i ^ swp)
        vec8_t<T> pb[NG];
        if constexpr (CMP) {
          float s[NG][8];
#pragma unroll
          for (int j = 0; j < NG; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i) { s[j][i] = s0[j][i]; s[j][4 + i] = s1[j][i]; }
          }
          const int key0 = cb + 8 * g;
          if (cb + 32 > nkeys) {                         // last chunk of the sequence only
            asm volatile("" ::: "memory");
#pragma unroll
            for (int j = 0; j < NG; ++j)
#pragma unroll
              for (int i = 0; i < 8; ++i)
                if (key0 + (i ^ swp) >= nkeys) s[j][i] = kNegInf;
          }
          if constexpr (FAST) {
            if (cb == c_begin) {                         // the reference: largest score of the first 32 rows
#pragma unroll
              for (int j = 0; j < NG; ++j) {
                float mx = s[j][0];
#pragma unroll
                for (int i = 1; i < 8; ++i) mx = fmaxf(mx, s[j][i]);
                mi[j] = colgroup_max(mx);                // finite: key cb exists
                grp[j].m = mi[j];
              }
            }
#pragma unroll
            for (int j = 0; j < NG; ++j) {
              const float off_i = -mi[j] * kLog2e;
              float ei[8];
#pragma unroll
              for (int i = 0; i < 8; ++i) ei[i] = fast_exp2(fmaf(s[j][i], kLog2e, off_i));
              li[j] += sum8(ei);
              if (act[j]) {
                const float off_a = -mi[j] * c_attn;
                const bool full = cb + 31 <= g_hi_min[j];
                float p[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) p[i] = fast_exp2(fmaf(s[j][i], c_attn, off_a));
                if (!full) {                             // the one or two chunks on the causal edge
                  asm volatile("" ::: "memory");
#pragma unroll
                  for (int i = 0; i < 8; ++i)
                    if (key0 + (i ^ swp) > hi[j]) p[i] = 0.f;
                }
                const float p8 = sum8(p);
                grp[j].l += p8;
                if constexpr (kNarrowP) pmax[j] = fmaxf(pmax[j], p8);
                pb[j] = pack8<T>(p);
              } else {
                pb[j] = zero8<T>();
              }
            }
          } else {
#pragma unroll
            for (int j = 0; j < NG; ++j) {
              float mx = s[j][0];
#pragma unroll
              for (int i = 1; i < 8; ++i) mx = fmaxf(mx, s[j][i]);
              mx = colgroup_max(mx);                     // finite: key cb exists
              const float m_new = fmaxf(mi[j], mx);
              const float off_i = -m_new * kLog2e;
              float ei[8];
#pragma unroll
              for (int i = 0; i < 8; ++i) ei[i] = fast_exp2(fmaf(s[j][i], kLog2e, off_i));
              li[j] = li[j] * fast_exp2((mi[j] - m_new) * kLog2e) + sum8(ei);     // exp2(-inf) = 0 on the first chunk
              mi[j] = m_new;
              if (act[j]) {
                float sv[8], p[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) sv[i] = key0 + (i ^ swp) > hi[j] ? kNegInf : s[j][i];
                softmax_update(grp[j], sv, c_attn, p);   // running maximum of the visible scores only
                pb[j] = pack8<T>(p);
              } else {
                pb[j] = zero8<T>();
              }
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < NG; ++j) {
            float s[8], p[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) { s[i] = s0[j][i]; s[4 + i] = s1[j][i]; }
            const int key0 = cb + 8 * g;
            const bool full = cb + 31 <= g_hi_min[j] && cb >= g_lo_max[j];
            if (act[j]) {
              if (!full) {                               // window edges
                asm volatile("" ::: "memory");
#pragma unroll
                for (int i = 0; i < 8; ++i)
                  if (!(key0 + (i ^ swp) <= hi[j] && key0 + (i ^ swp) >= lo[j])) s[i] = kNegInf;
              }
              softmax_update(grp[j], s, c_attn, p);
              pb[j] = pack8<T>(p);
            } else {
              pb[j] = zero8<T>();
            }
          }
        }
        // a group without visible keys in this chunk carries all-zero probabilities: one MFMA chain
        // for all groups keeps the accumulators in place (no per-group control flow around them)
        if (any_act) pv32_all<T, DK, DV, NG>(bv + n * VLD + 32 * sub + 8 * g, 16 * VLD, grp, pb);
      }

      if (has_next) lstore(buf ^ 1, next_v);
      __syncthreads();
      buf ^= 1;
    }
  };

  float lt[NG], lit[NG];                       // denominators summed over the four lanes of a column
  auto row_sums = [&]() {
#pragma unroll
    for (int j = 0; j < NG; ++j) {
      lt[j] = colgroup_sum(grp[j].l);
      lit[j] = CMP ? colgroup_sum(li[j]) : 0.f;
    }
  };
  if constexpr (CMP) {
    run_chunks(std::true_type{});
    row_sums();
    int bad = 0;
#pragma unroll
    for (int j = 0; j < NG; ++j) {
      const bool sees = rm[j].valid && hi[j] >= 0 && c_begin < c_end;
      bad |= !(lit[j] < 1e30f) || !(lt[j] < 1e30f) || (sees && !(lt[j] > 1e-30f));
      if constexpr (kNarrowP) {
        // every packed probability is at most its 8-key sum: below 3e4 none overflowed.  The largest 8-key sum of
        // the row at or above 2^-7 puts the row's largest probability at or above 2^-10, a normal float16 with its
        // whole mantissa; what lies 2^-14 and more below it is subnormal, as under a running maximum.
        const float pm = colgroup_max(pmax[j]);
        bad |= !(pm < 3e4f) || (sees && !(pm >= 0.0078125f));
      }
    }
    if (__syncthreads_or(bad)) {               // rare: the whole workgroup repeats the pass in the exact form
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        group_reset(grp[j]);
        li[j] = 0.f;
        mi[j] = kNegInf;
      }
      run_chunks(std::false_type{});
      row_sums();
    }
  } else {
    run_chunks(std::false_type{});
    row_sums();
  }

  // Output rows leave through LDS (the K buffers are free after the loop's last barrier): the
  // accumulators hold 4 channels of 16 different rows per lane, whole 16-byte pieces of one row
  // per lane make full cache lines.
  T* ob = reinterpret_cast<T*>(a.o);
  constexpr int OLD = DV + 8;
  static_assert(NW * 16 * OLD <= 2 * CH * KLD + 2 * DV * VLD, "output staging must fit the K/V buffers");
  T* stage = ldsK + wave * 16 * OLD;
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    const float inv = lt[j] > 0.f ? 1.0f / lt[j] : 0.f;
    const long row = ((long)st.start + rm[j].tok) * a.hq + h * G + rm[j].gidx;
    store_rows<T, DV>(stage + n * OLD, grp[j].o, inv, g);
    constexpr int PIECES = DV / 8;
    const int gi = wave * NG + j;
    if constexpr (MERGE == 16 || MERGE == 2) {
      // a lane takes two pieces (pc, pc + PIECES / 2) of one row, so that 32 partial loads are in flight per lane
      constexpr int HALF = PIECES / 2;
#pragma unroll
      for (int k = 0; k < (16 * HALF + 63) / 64; ++k) {
        const int e = lane + 64 * k;
        const int r = e / HALF, pc = e % HALF;
        if (16 * HALF % 64 == 0 || r < 16) {
          const RowMap rr = map_row(st.t0, gi, r, lgp, G, st.len);
          if (rr.valid) {
            const long tg = (long)st.start + rr.tok;
            const long orow = tg * a.hq + h * G + rr.gidx;
            const vec8_t<T> pa = load8(stage + r * OLD + pc * 8), pb = load8(stage + r * OLD + (pc + HALF) * 8);
            vec8_t<T> ra, rb;
            merge_two<T, DV, 16, MERGE == 16>(a.mg, tg, h, rr.gidx, orow, pc, pc + HALF, pa, pb, ra, rb);
            store8(reinterpret_cast<T*>(a.mg.out) + orow * DV + pc * 8, ra);
            store8(reinterpret_cast<T*>(a.mg.out) + orow * DV + (pc + HALF) * 8, rb);
          }
        }
      }
    } else {
#pragma unroll
      for (int k = 0; k < (16 * PIECES + 63) / 64; ++k) {
        const int e = lane + 64 * k;
        const int r = e / PIECES, pc = e % PIECES;
        if (16 * PIECES % 64 == 0 || r < 16) {
          const RowMap rr = map_row(st.t0, gi, r, lgp, G, st.len);
          if (rr.valid) {
            const long tg = (long)st.start + rr.tok;
            const long orow = tg * a.hq + h * G + rr.gidx;
            const vec8_t<T> piece = load8(stage + r * OLD + pc * 8);
            if constexpr (MERGE == 0) {
              store8(ob + orow * DV + pc * 8, piece);
            } else {
              const vec8_t<T> res = merge_piece<T, DV, 0>(a.mg, tg, h, rr.gidx, orow, pc, true, piece);
              store8(reinterpret_cast<T*>(a.mg.out) + orow * DV + pc * 8, res);
            }
          }
        }
      }
    }
    if (a.lse_attn != nullptr && rm[j].valid && g == 0)
      a.lse_attn[row] = lt[j] > 0.f ? fmaf(grp[j].m, a.scale, __logf(lt[j])) : __builtin_huge_valf();
    if (CMP && a.lse != nullptr) {
      if (rm[j].valid && g == 0) a.lse[row] = nkeys > 0 ? mi[j] + __logf(lit[j]) : 0.f;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// selected blocks + gated combine

__device__ __forceinline__ float gate_value(float x, int act) {
  return act == 1 ? 1.0f / (1.0f + __expf(-x)) : x;
}

// One wavefront per row group.  The usable blocks of a token are walked as a flat sequence of
// 32-key chunks; the K fragments (two tiles) and V^T fragments of chunk i+1 are requested from
// global memory before chunk i is multiplied, so a wavefront keeps one full chunk (K and V) in
// flight while it computes.  Workgroups are dealt to kv heads so that, with the hardware's
// round-robin placement of workgroups on the 8 XCDs, an XCD's L2 only ever holds one head's K/V.
template <typename T, int DK, int DV>
__global__ void __launch_bounds__(256)
slc_combine_kernel(const SlcArgs a) {
  constexpr int NK = DK / 32, NV = DV / 16;
  constexpr bool PIPE = sizeof(T) == 2;       // fp32 fragments are twice as wide: no second buffer
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv, Gp = next_pow2(G), lgp = ilog2(Gp);
  const int TQ = 64 >> lgp;
  int h, tile;
  {
    const int id = blockIdx.x, hkv = a.hkv;
    if (8 % hkv == 0) {
      const int per = 8 / hkv, x = id & 7;
      h = x % hkv;
      tile = (id >> 3) * per + x / hkv;
    } else {
      h = id % hkv;
      tile = id / hkv;
    }
  }
  const SeqTile st = find_tile(a.cu_seq, a.batch, TQ, tile);
  if (!st.valid) return;
  const int S = a.top_n, BS = a.block_size;
  const int hk = h / a.kv_rep, hkv_r = a.hkv / a.kv_rep;     // kv head of this (sub-)group, number of kv heads
  const T* qb = reinterpret_cast<const T*>(a.q);
  const T* kb = reinterpret_cast<const T*>(a.k) + ((long)st.start * hkv_r + hk) * DK + 8 * g;
  const T* vtb = reinterpret_cast<const T*>(a.vt) + (long)hk * DV * a.vt_cols + transposed_offset(st.start, st.b)
                 + (long)n * a.vt_cols + 8 * g;
  const long krow = (long)hkv_r * DK;
  const long vstep = 16L * a.vt_cols;

  RowGroup<T, DK, DV> grp[1];
  const RowMap rm = map_row(st.t0, wave, n, lgp, G, st.len);
  load_q(grp[0], qb, (long)st.start, rm, st.len, a.hq, h, G, g);
  group_reset(grp[0]);
  const float c_attn = a.scale * kLog2e;
  const int tpg = lgp >= 4 ? 1 : (16 >> lgp);          // tokens per row group
  const int tfirst = st.t0 + ((wave * 16) >> lgp);
  const int key_r0 = chunk_key_of_row(0, n), key_r1 = chunk_key_of_row(1, n);

  struct Frags { vec8_t<T> k0[NK], k1[NK], v[NV]; };
  wait_all_loads();

  for (int tk = 0; tk < tpg; ++tk) {
    const int tt = tfirst + tk;
    if (tt >= st.len) break;
    const long irow = ((long)st.start + tt) * hkv_r + hk;
    int cnt = S;
    if (a.counts != nullptr) cnt = min(max(a.counts[irow], 0), S);
    long myidx = -1;
    if (lane < cnt) {
      myidx = a.idx64 ? reinterpret_cast<const int64_t*>(a.indices)[irow * S + lane]
                      : (long)reinterpret_cast<const int32_t*>(a.indices)[irow * S + lane];
    }
    const bool usable = myidx >= 0 && myidx <= tt && myidx * BS <= tt;   // bi <= tt keeps bi*BS in range
    unsigned long long todo = __ballot(usable);
    int cur = 0, cur_last = -1;                          // next chunk start / last visible key of the block
    auto next_chunk = [&](int& cb, int& last) -> bool {
      if (cur > cur_last) {
        if (todo == 0) return false;
        const int i = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const int k0 = (int)__shfl(myidx, i) * BS;
        cur = k0;
        cur_last = min(k0 + BS - 1, tt);
      }
      cb = cur;
      last = cur_last;
      cur += 32;
      return true;
    };
    auto issue = [&](Frags& f, int cb) {
      const T* p0 = kb + (long)min(cb + key_r0, st.len - 1) * krow;
      const T* p1 = kb + (long)min(cb + key_r1, st.len - 1) * krow;
#pragma unroll
      for (int kk = 0; kk < NK; ++kk) { f.k0[kk] = load8(p0 + 32 * kk); f.k1[kk] = load8(p1 + 32 * kk); }
#pragma unroll
      for (int t = 0; t < NV; ++t) f.v[t] = load8(vtb + t * vstep + cb);
    };
    auto compute = [&](const Frags& f, int cb, int last) {
      f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NK; ++kk) {
        s0 = mma16(f.k0[kk], grp[0].q[kk], s0);
        s1 = mma16(f.k1[kk], grp[0].q[kk], s1);
      }
      float s[8], p[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) { s[e] = s0[e]; s[4 + e] = s1[e]; }
      if (cb + 31 > last || tpg > 1) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (!(cb + 8 * g + e <= last && rm.tok == tt)) s[e] = kNegInf;
      }
      softmax_update(grp[0], s, c_attn, p);
      const vec8_t<T> pb = pack8<T>(p);
#pragma unroll
      for (int t = 0; t < NV; ++t) grp[0].o[t] = mma16(f.v[t], pb, grp[0].o[t]);
    };

    Frags fa;
    int cba, lasta;
    bool ha = next_chunk(cba, lasta);
    if (ha) issue(fa, cba);
    if (PIPE) {
      Frags fb;
      int cbb, lastb;
      while (ha) {
        const bool hb = next_chunk(cbb, lastb);
        if (hb) issue(fb, cbb);
        compute(fa, cba, lasta);
        if (!hb) break;
        ha = next_chunk(cba, lasta);
        if (ha) issue(fa, cba);
        compute(fb, cbb, lastb);
      }
    } else {
      while (ha) {
        compute(fa, cba, lasta);
        ha = next_chunk(cba, lasta);
        if (ha) issue(fa, cba);
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

template <typename T, bool CMP> struct StreamTile {
  // row groups per wavefront, keys per LDS chunk, wavefronts per workgroup.  The compressed branch
  // walks ~2000 keys per tile and gains from half as many barriers (64-key chunks, 16 tokens per
  // workgroup); the window branch walks ~550 and is better off with small workgroups.
  static constexpr int NG = sizeof(T) == 2 ? 2 : 1;
  static constexpr int CH = (CMP && sizeof(T) == 2) ? 64 : 32;
  static constexpr int NW = (CMP && sizeof(T) == 2) ? 8 : 4;
};

int set_smem(const void* fn, size_t bytes) {
  if (bytes > 160 * 1024) return -3;
  if (bytes > 48 * 1024) {
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return -4;
  }
  return 0;
}

int group_pow2(int G) {
  int p = 1;
  while (p < G) p <<= 1;
  return p;
}

template <typename T, int DK, int DV, bool CMP, int MERGE = 0>
static int launch_stream_t(const StreamParams& a, int total, hipStream_t st, int tile_count = 0) {
  constexpr int NG = StreamTile<T, CMP>::NG, CH = StreamTile<T, CMP>::CH, NW = StreamTile<T, CMP>::NW;
  const int Gp = group_pow2(a.hq / a.hkv);
  const int TQ = NW * NG * 16 / Gp;
  const size_t smem = 2 * ((size_t)CH * (DK + kLdsRowPad<T>) + (size_t)DV * (CH + kLdsRowPad<T>)) * sizeof(T);
  auto fn = stream_attn_kernel<T, DK, DV, NG, CH, NW, CMP, MERGE>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  const int tiles = tile_count > 0 ? tile_count : total / TQ + a.batch;
  hipLaunchKernelGGL(fn, dim3(tiles, a.hkv), dim3(NW * 64), smem, st, a);
  return 0;
}

// tokens per tile of the window kernel (what SlcArgs::tile_tokens / SwaArgs::tile_begin count in)
int swa_tile_tokens(int hq, int hkv, int dtype) {
  const int rows = dtype == 1 ? StreamTile<float, false>::NW * StreamTile<float, false>::NG * 16
                              : StreamTile<bf16_t, false>::NW * StreamTile<bf16_t, false>::NG * 16;
  return rows / group_pow2(hq / hkv);
}

template <typename T, int DK, int DV>
static int launch_cmp_t(const CmpArgs& a, hipStream_t st) {
  StreamParams p{a.q, a.ck, a.cvt, a.o, a.lse, a.cu_seq, a.cu_cmp, a.batch, a.hq, a.hkv, a.ck_row_stride,
                 a.ck_head_stride, a.cvt_cols, a.block, a.stride, 0, a.causal, a.scale, MergeArgs{}, a.lse_attn, a.kv_rep, 0};
  p.gate_w = a.gate_w; p.gate_b = a.gate_b; p.gates = a.gates;
  // rows beyond the last one a tile's tokens may attend only feed the importance log-sum-exp: skipped when that
  // is not asked for
  if (a.causal && a.lse == nullptr) p.split_hidden = 1;
  return launch_stream_t<T, DK, DV, true>(p, a.total, st);
}

template <typename T, int DK, int DV>
static int launch_swa_t(const SwaArgs& a, hipStream_t st) {
  StreamParams p{a.q, a.k, a.vt, a.o, nullptr, a.cu_seq, a.cu_seq, a.batch, a.hq, a.hkv, (long)(a.hkv / a.kv_rep) * DK,
                 (long)DK, a.vt_cols, 0, 0, a.window, 1, a.scale, MergeArgs{}, a.lse, a.kv_rep, 0};
  return launch_stream_t<T, DK, DV, false>(p, a.total, st);
}

template <typename T, int DK, int DV>
static int launch_swa_merge_t(const SwaArgs& a, const MergeArgs& m, hipStream_t st) {
  StreamParams p{a.q, a.k, a.vt, nullptr, nullptr, a.cu_seq, a.cu_seq, a.batch, a.hq, a.hkv, (long)(a.hkv / a.kv_rep) * DK,
                 (long)DK, a.vt_cols, 0, 0, a.window, 1, a.scale, m, a.lse, a.kv_rep, 0, a.tile_begin};
  if (m.top_n == 16) return launch_stream_t<T, DK, DV, false, 16>(p, a.total, st, a.tile_count);
  return launch_stream_t<T, DK, DV, false, 2>(p, a.total, st, a.tile_count);    // picks merged in rounds of 16
}

template <typename T, int DK, int DV>
static int launch_slc_t(const SlcArgs& a, hipStream_t st) {
  const int Gp = group_pow2(a.hq / a.hkv);
  const int TQ = 64 / Gp;
  int tiles = a.total / TQ + a.batch;
  if (8 % a.hkv == 0) tiles = (tiles + 8 / a.hkv - 1) / (8 / a.hkv) * (8 / a.hkv);   // whole rounds of 8 workgroups
  hipLaunchKernelGGL((slc_combine_kernel<T, DK, DV>), dim3(tiles * a.hkv), dim3(256), 0, st, a);
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
    } else if ((ARGS).dtype == 2) {                                                   \
      switch (key) {                                                                  \
        case 32032: return FN<f16_t, 32, 32>(ARGS, ST);                               \
        case 64064: return FN<f16_t, 64, 64>(ARGS, ST);                               \
        case 128128: return FN<f16_t, 128, 128>(ARGS, ST);                            \
        case 192128: return FN<f16_t, 192, 128>(ARGS, ST);                            \
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

int launch_cmp_attn(const CmpArgs& a, hipStream_t st) { NSA_DISPATCH(launch_cmp_t, a, st); }
int launch_swa(const SwaArgs& a, hipStream_t st) { NSA_DISPATCH(launch_swa_t, a, st); }
int launch_swa_merge(const SwaArgs& a, const MergeArgs& m, hipStream_t st) {
  if (a.dtype == 1) return -2;             // the partials are 16-bit
  switch (a.dk * 1000 + a.dv + (a.dtype == 2 ? 1000000 : 0)) {
    case 32032: return launch_swa_merge_t<bf16_t, 32, 32>(a, m, st);
    case 64064: return launch_swa_merge_t<bf16_t, 64, 64>(a, m, st);
    case 128128: return launch_swa_merge_t<bf16_t, 128, 128>(a, m, st);
    case 192128: return launch_swa_merge_t<bf16_t, 192, 128>(a, m, st);
    case 1032032: return launch_swa_merge_t<f16_t, 32, 32>(a, m, st);
    case 1064064: return launch_swa_merge_t<f16_t, 64, 64>(a, m, st);
    case 1128128: return launch_swa_merge_t<f16_t, 128, 128>(a, m, st);
    case 1192128: return launch_swa_merge_t<f16_t, 192, 128>(a, m, st);
    default: return -2;
  }
}
int launch_slc_combine(const SlcArgs& a, hipStream_t st) {
  // block-major path when the caller lent a large enough workspace and the shape qualifies
  if (a.workspace != nullptr && slc_block_major_ok(a) && a.workspace_bytes >= slc_workspace_bytes(a))
    return launch_slc_block_major(a, a.workspace, st);
  if (a.lse != nullptr) return -5;              // only the block-major schedule produces the log-sum-exp
  NSA_DISPATCH(launch_slc_t, a, st);
}

}  // namespace nsa
