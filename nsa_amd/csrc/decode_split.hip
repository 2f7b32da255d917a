// Decode step for small batches: the work of one (sequence, kv head) spread over many workgroups.
//
// The one-workgroup kernel streams 1.8 MB through a single CU, which takes ~60 us however few sequences
// there are; with fewer than 128 (sequence, kv head) pairs most of the chip idles.  Here the step runs as
// three launches on the same stream, each over (pair, split) workgroups of 4 wavefronts:
//   A  compressed rows cut into SA slices: raw scores, per-slice max / sum per head, per-head pooled
//      window sums relative to the slice maximum (the head sum needs every head's global normaliser, which
//      only B knows), partial compressed attention of the visible rows
//   B  every workgroup rebuilds the global statistics from the SA slices (a few KB), normalises and adds the
//      window sums, takes the top-n blocks (all SB workgroups get the same answer), then attends its share
//      of the 32-key chunks of the window and of the selected blocks; partial states per branch
//   C  merges the partial states of the three branches, gates, stores
// Same arithmetic as the one-workgroup kernel up to the order of fp32 sums.  Any pooling geometry; windows of 5
// compressed rows every 4 (the default) add their rows to the bins three sums at a time, others row by row.
#include <mutex>

#include "decode_common.h"

namespace nsa {

constexpr int kSplitWaves = 4;
constexpr int kSplitMaxChunks = 3;                                   // compressed 32-row chunks per wavefront of a slice
constexpr int kSplitMaxSlice = 32 * kSplitWaves * kSplitMaxChunks;   // 384 rows

// floats per (sequence, kv head) in the workspace
struct SplitLayout {
  int sa, sb, slice, nb, dv;
  int ns_cap;                          // bound of the pooled bins of a sequence
  int pool_k, pool_s, pool_p;
  // bin of a sequence that local bin 0 of the slice starting at row c_lo stands for: the first one a row of the
  // slice can belong to (bin j pools rows j * s - p .. j * s - p + k - 1); may be -1 for the first slice
  __host__ __device__ int first_bin(int c_lo) const {
    const int x = c_lo + pool_p - pool_k + pool_s;
    return x >= 0 ? x / pool_s : -((-x + pool_s - 1) / pool_s);
  }
  __host__ __device__ long stat() const { return 0; }                                   // [sa][2][16]
  __host__ __device__ long bins() const { return (long)sa * 32; }                       // [sa][nb][16]
  __host__ __device__ long cmp() const { return bins() + (long)sa * nb * 16; }          // [sa][1 + dv][16]
  __host__ __device__ long att() const { return cmp() + (long)sa * (1 + dv) * 16; }     // [2][sb][2 + dv][16]
  __host__ __device__ long total() const { return att() + 2L * sb * (2 + dv) * 16; }
};

static SplitLayout split_layout(const DecodeArgs& a, int splits) {
  SplitLayout l;
  l.sa = max(splits, (a.nc_cap + kSplitMaxSlice - 1) / kSplitMaxSlice);
  l.slice = ((a.nc_cap + l.sa - 1) / l.sa + 31) / 32 * 32;
  l.sb = splits;
  l.pool_k = max(a.pool_k, 1); l.pool_s = max(a.pool_s, 1); l.pool_p = max(a.pool_p, 0);
  l.nb = (l.slice + l.pool_k - 2) / l.pool_s + 2;            // bins that the rows of one slice can belong to
  const int span = a.nc_cap + 2 * l.pool_p - l.pool_k;
  l.ns_cap = span < 0 ? 0 : (span + l.pool_s - 1) / l.pool_s + 1;
  l.dv = a.dv;
  return l;
}

long decode_split_workspace_bytes(const DecodeArgs& a, int splits) {
  return split_layout(a, splits).total() * (long)a.batch * a.hkv * max(a.kv_rep, 1) * (long)sizeof(float);
}

// ---- A: compressed rows of one slice ---------------------------------------------------------------
template <typename T, int DK, int DV>
__global__ void __launch_bounds__(kSplitWaves * 64)
decode_split_cmp_kernel(const DecodeArgs a, const SplitLayout L, float* __restrict__ ws) {
  constexpr int NW = kSplitWaves, MAXC = kSplitMaxChunks, PLD = 17;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  float* part = reinterpret_cast<float*>(smem_raw);            // [NW][DV][PLD]
  float* pstat = part + NW * DV * PLD;                         // [NW][2][16]
  float* pl = pstat + NW * 2 * 16;                             // [NW][16]
  float* binsL = pl + NW * 16;                                 // [nb][16]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int bh = blockIdx.x, s = blockIdx.y;
  const int hs = a.hkv * a.kv_rep;                         // sub-groups of at most 16 query heads per sequence
  const int b = bh / hs, h = bh % hs, hc = h / a.kv_rep;   // h: sub-group (query heads h * G ..), hc: its kv head
  const int G = a.hq / hs;
  float* wsp = ws + (long)bh * L.total();
  float* w_stat = wsp + L.stat() + (long)s * 32;
  float* w_bins = wsp + L.bins() + (long)s * L.nb * 16;
  float* w_cmp = wsp + L.cmp() + (long)s * (1 + DV) * 16;

  const int cap = a.block_table != nullptr ? a.max_pages * 64 : a.ctx_cap;
  const int ctx = min(a.ctx_lens[b], cap);
  const int t = ctx - 1;
  const int Nc = ctx >= a.block ? min((ctx - a.block) / a.stride + 1, a.nc_cap) : 0;
  const int c_lo = s * L.slice, c_hi = min(c_lo + L.slice, Nc);
  if (c_lo >= c_hi) {                        // nothing in this slice: neutral statistics, no partial
    if (tid < 16) { w_stat[tid] = kNegInf; w_stat[16 + tid] = 0.f; w_cmp[tid] = 0.f; }
    return;
  }
  const int cmaxv = t >= a.block ? min((t - a.block) / a.stride, Nc - 1) : -1;   // last visible compressed row
  const float c_attn = a.scale * kLog2e;
  const long krow = (long)a.hkv * DK;
  const T* ckseq = reinterpret_cast<const T*>(a.ck_cache) + ((long)b * a.nc_cap * a.hkv + hc) * DK;
  const T* cvt = reinterpret_cast<const T*>(a.cv_cache_t) + (((long)b * a.hkv + hc) * DV + n) * a.nc_cap + 8 * g;
  const long cvstep = 16L * a.nc_cap;

  vec8_t<T> qf[DK / 32];
  {
    const int gc = n < G ? n : G - 1;
    const T* qp = reinterpret_cast<const T*>(a.q) + ((long)b * a.hq + h * G + gc) * DK + 8 * g;
#pragma unroll
    for (int kk = 0; kk < DK / 32; ++kk) qf[kk] = load8(qp + 32 * kk);
  }
  for (int i = tid; i < L.nb * 16; i += NW * 64) binsL[i] = 0.f;

  // raw scores of this wavefront's chunks, all K fragments requested before the first product
  vec8_t<T> kf[MAXC][2][DK / 32];
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int cb = c_lo + 32 * (wave + NW * i);
    if (cb < c_hi) {
      const T* k0p = ckseq + (long)min(cb + chunk_key_of_row(0, n), Nc - 1) * krow + 8 * g;
      const T* k1p = ckseq + (long)min(cb + chunk_key_of_row(1, n), Nc - 1) * krow + 8 * g;
#pragma unroll
      for (int kk = 0; kk < DK / 32; ++kk) { kf[i][0][kk] = load8(k0p + 32 * kk); kf[i][1][kk] = load8(k1p + 32 * kk); }
    }
  }
  float sc[MAXC][8];
  float mi = kNegInf, li = 0.f;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int cb = c_lo + 32 * (wave + NW * i);
    if (cb < c_hi) {
      f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < DK / 32; ++kk) {
        s0 = mma16(kf[i][0][kk], qf[kk], s0);
        s1 = mma16(kf[i][1][kk], qf[kk], s1);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) { sc[i][e] = s0[e]; sc[i][4 + e] = s1[e]; }
      float mx = kNegInf;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (cb + 8 * g + e >= c_hi) sc[i][e] = kNegInf;
        mx = fmaxf(mx, sc[i][e]);
      }
      mx = colgroup_max(mx);                            // finite: row cb exists
      const float m_new = fmaxf(mi, mx);
      float sum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) sum += fast_exp2((sc[i][e] - m_new) * kLog2e);
      li = li * fast_exp2((mi - m_new) * kLog2e) + sum;
      mi = m_new;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) sc[i][e] = kNegInf;
    }
  }
  // the visible chunks' value fragments: requested now, used after the statistics are combined
  vec8_t<T> vf[MAXC][DV / 16];
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int cb = c_lo + 32 * (wave + NW * i);
    if (cb < c_hi && cb <= cmaxv) {
#pragma unroll
      for (int tt = 0; tt < DV / 16; ++tt) vf[i][tt] = load8(cvt + tt * cvstep + cb);
    }
  }
  li = colgroup_sum(li);
  if (g == 0) { pstat[(wave * 2 + 0) * 16 + n] = mi; pstat[(wave * 2 + 1) * 16 + n] = li; }
  __syncthreads();                                      // also: binsL is zero
  float M = kNegInf;
#pragma unroll
  for (int w = 0; w < NW; ++w) M = fmaxf(M, pstat[(w * 2) * 16 + n]);
  float Z = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    const float mw = pstat[(w * 2) * 16 + n];
    if (mw != kNegInf) Z += pstat[(w * 2 + 1) * 16 + n] * fast_exp2((mw - M) * kLog2e);
  }
  if (tid < 16) { w_stat[tid] = M; w_stat[16 + tid] = Z; }          // head n = tid (wavefront 0, g = 0)

  // pooled window sums per head, relative to the slice maximum; local bin index = j - L.first_bin(c_lo).
  // Windows of 5 every 4: rows 4j .. 4j+4 make bin j, first_bin = c_lo / 4 - 1 (the bin that the slice's first
  // row completes).
  const float Ml2 = M * kLog2e;
  const bool fast_pool = L.pool_k == 5 && L.pool_s == 4 && L.pool_p == 0;
  // windows of s + 1 rows every s, s = 1, 2, 4 or 8, any padding: a lane's 8 rows are runs of equal bin
  const bool run_pool = L.pool_k == L.pool_s + 1 && (L.pool_s == 1 || L.pool_s == 2 || L.pool_s == 4 || L.pool_s == 8);
  const int ls = L.pool_s == 1 ? 0 : L.pool_s == 2 ? 1 : L.pool_s == 4 ? 2 : 3;
  const int jf = L.first_bin(c_lo);
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int cb = c_lo + 32 * (wave + NW * i);
    if (cb < c_hi) {
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = fast_exp2(fmaf(sc[i][e], kLog2e, -Ml2));     // 0 past c_hi
      const int c0 = cb + 8 * g;
      if (fast_pool) {
        if (c0 < c_hi) {
          const int b0 = (c0 - c_lo) / 4 + 1;
          atomicAdd(&binsL[(b0 - 1) * 16 + n], v[0]);
          atomicAdd(&binsL[b0 * 16 + n], (v[0] + v[1]) + (v[2] + v[3]) + v[4]);
          atomicAdd(&binsL[(b0 + 1) * 16 + n], (v[4] + v[5]) + (v[6] + v[7]));
        }
      } else if (run_pool) {
        // bin j pools positions j * s .. j * s + s of the padded row (position = row + padding): one atomic per run
        // of rows of equal bin; a position that is a multiple of s is the first of its bin and the last of the bin
        // before.  Rows past c_hi carry 0; local bins stay within [0, L.nb).
        if (c0 < c_hi) {
          const int x0 = c0 + L.pool_p;
          int cur = x0 >> ls;
          float run = 0.f;
          auto add = [&](int j, float val) {
            const int lb = j - jf;
            if (lb >= 0 && lb < L.nb) atomicAdd(&binsL[lb * 16 + n], val);
          };
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int x = x0 + e;
            if ((x & (L.pool_s - 1)) == 0) {
              if (e == 0) add(cur - 1, v[0]);
              else { add(cur, run + v[e]); cur = x >> ls; }
              run = v[e];
            } else {
              run += v[e];
            }
          }
          add(cur, run);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int c = c0 + e;
          if (c < c_hi) {
            const int num = c + L.pool_p - L.pool_k + 1;
            const int b_lo = num <= 0 ? 0 : (num + L.pool_s - 1) / L.pool_s;
            const int b_hi = min((c + L.pool_p) / L.pool_s, jf + L.nb - 1);
            for (int bb = b_lo; bb <= b_hi; ++bb) atomicAdd(&binsL[(bb - jf) * 16 + n], v[e]);
          }
        }
      }
    }
  }

  // partial compressed attention of the visible rows, reference = the slice maximum
  DecState<T, DK, DV> cmp;
  dec_reset(cmp);
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int cb = c_lo + 32 * (wave + NW * i);
    if (cb < c_hi && cb <= cmaxv) {
      float p[8], psum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int c = cb + 8 * g + e;
        p[e] = (c <= cmaxv && c < c_hi) ? fast_exp2((sc[i][e] - M) * c_attn) : 0.f;
        psum += p[e];
      }
      cmp.l += psum;
      const vec8_t<T> pb = pack8<T>(p);
#pragma unroll
      for (int tt = 0; tt < DV / 16; ++tt) cmp.o[tt] = mma16(vf[i][tt], pb, cmp.o[tt]);
    }
  }
#pragma unroll
  for (int tt = 0; tt < DV / 16; ++tt)
#pragma unroll
    for (int i = 0; i < 4; ++i) part[(wave * DV + tt * 16 + 4 * g + i) * PLD + n] = cmp.o[tt][i];
  const float lt = colgroup_sum(cmp.l);
  if (g == 0) pl[wave * 16 + n] = lt;
  __syncthreads();
  for (int i = tid; i < L.nb * 16; i += NW * 64) w_bins[i] = binsL[i];
  // every wavefront used the same reference: the partial states just add up
  const int r = tid & 15;
  if (tid < 16) {
    float l = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) l += pl[w * 16 + tid];
    w_cmp[tid] = l;
  }
  for (int d = tid >> 4; d < DV; d += NW * 4) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) o += part[(w * DV + d) * PLD + r];
    w_cmp[(1 + d) * 16 + r] = o;
  }
}

// ---- B: selection, then window and selected chunks ---------------------------------------------------
template <typename T, int DK, int DV, bool PAGED, int PER>
__global__ void __launch_bounds__(kSplitWaves * 64)
decode_split_attend_kernel(const DecodeArgs a, const SplitLayout L, float* __restrict__ ws) {
  constexpr int NW = kSplitWaves, PLD = 17;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  float* part = reinterpret_cast<float*>(smem_raw);            // [NW][DV][PLD]
  float* pstat = part + NW * DV * PLD;                         // [NW][2][16]
  float* fac = pstat + NW * 2 * 16;                            // [kv_rep][sa][16]
  float* pooled = fac + a.kv_rep * L.sa * 16;                  // [Ns]
  int* sel = reinterpret_cast<int*>(pooled + L.ns_cap + 4);    // [top_n]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int bh = blockIdx.x, sb = blockIdx.y;
  const int hs = a.hkv * a.kv_rep;
  const int b = bh / hs, h = bh % hs, hc = h / a.kv_rep;     // as in kernel A
  const int G = a.hq / hs;
  float* wsp = ws + (long)bh * L.total();
  // the selection sums the importance over every query head of the kv head: the statistics and window sums of
  // all its sub-groups (consecutive pairs of the workspace) are read, so each of them takes the same blocks
  const float* wsib = ws + (long)(bh - h % a.kv_rep) * L.total();

  const int cap = PAGED ? a.max_pages * 64 : a.ctx_cap;
  const int ctx = min(a.ctx_lens[b], cap);
  if (ctx <= 0) return;
  const int t = ctx - 1;
  const int Nc = ctx >= a.block ? min((ctx - a.block) / a.stride + 1, a.nc_cap) : 0;
  int Ns = 0;
  if (Nc > 0 && Nc + 2 * L.pool_p >= L.pool_k) {
    Ns = (Nc + 2 * L.pool_p - L.pool_k + L.pool_s - 1) / L.pool_s + 1;
    if ((Ns - 1) * L.pool_s >= Nc + L.pool_p) --Ns;
  }
  const float c_attn = a.scale * kLog2e;

  // ---- this workgroup's share of the 32-key chunks: item k goes to workgroup k % sb, wavefront (k / sb) % NW
  const T* kseq = reinterpret_cast<const T*>(a.k_cache) + (PAGED ? (long)hc * DK : ((long)b * a.ctx_cap * a.hkv + hc) * DK);
  const long krow = (long)a.hkv * DK;
  const T* vt = reinterpret_cast<const T*>(a.v_cache_t) +
                (PAGED ? ((long)hc * DV + n) * 64 + 8 * g : (((long)b * a.hkv + hc) * DV + n) * a.ctx_cap + 8 * g);
  const long vstep = PAGED ? 16L * 64 : 16L * a.ctx_cap;
  auto issue_kv = [&](ChunkFrags<T, DK, DV>& f, int cb) {
    if constexpr (PAGED) {
      const long pg = a.block_table[(long)b * a.max_pages + (cb >> 6)];
      chunk_issue<T, DK, DV>(f, kseq + pg * 64 * krow, krow, vt + pg * a.hkv * DV * 64, vstep, cb & 63,
                             min(t - (cb & ~63), 63), n, g);
    } else {
      chunk_issue<T, DK, DV>(f, kseq, krow, vt, vstep, cb, t, n, g);
    }
  };
  vec8_t<T> qf[DK / 32];
  {
    const int gc = n < G ? n : G - 1;
    const T* qp = reinterpret_cast<const T*>(a.q) + ((long)b * a.hq + h * G + gc) * DK + 8 * g;
#pragma unroll
    for (int kk = 0; kk < DK / 32; ++kk) qf[kk] = load8(qp + 32 * kk);
  }
  const int r = tid & 15;
  // partial state of a branch: wavefronts merged through LDS, left un-normalised for kernel C
  auto put = [&](const DecState<T, DK, DV>& st, int branch) {
    float* dst = wsp + L.att() + ((long)branch * L.sb + sb) * (2 + DV) * 16;
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < DV / 16; ++tt)
#pragma unroll
      for (int i = 0; i < 4; ++i) part[(wave * DV + tt * 16 + 4 * g + i) * PLD + n] = st.o[tt][i];
    const float lt = colgroup_sum(st.l);
    if (g == 0) { pstat[(wave * 2 + 0) * 16 + n] = st.m; pstat[(wave * 2 + 1) * 16 + n] = lt; }
    __syncthreads();
    float mm = kNegInf;
#pragma unroll
    for (int w = 0; w < NW; ++w) mm = fmaxf(mm, pstat[(w * 2) * 16 + r]);
    float wgt[NW], den = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = pstat[(w * 2) * 16 + r];
      wgt[w] = mw == kNegInf ? 0.f : fast_exp2((mw - mm) * c_attn);
      den += wgt[w] * pstat[(w * 2 + 1) * 16 + r];
    }
    if (tid < 16) { dst[tid] = mm; dst[16 + tid] = den; }
    for (int d = tid >> 4; d < DV; d += NW * 4) {
      float o = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) o += wgt[w] * part[(w * DV + d) * PLD + r];
      dst[(2 + d) * 16 + r] = o;
    }
  };

  // chunk items are numbered window first, then the selected blocks in pick order; this wavefront takes the
  // items sb + L.sb * (wave + NW * i), i = 0, 1, ...
  const int item_step = L.sb * NW;
  int next = sb + L.sb * wave;
  // The window does not depend on the selection: this wavefront's first window chunk is requested before the
  // statistics and the top-n (which only wavefront 0 computes) and attended while they are under way.
  ChunkFrags<T, DK, DV> f;
  const int w_lo = max(t - a.window + 1, 0);
  const int w_first = (w_lo / 32) * 32;
  const int nwin = a.window > 0 ? (t - w_first) / 32 + 1 : 0;
  const int my_win = next < nwin ? next : -1;                // first window item of this wavefront
  if (my_win >= 0) issue_kv(f, w_first + 32 * my_win);

  // global log-sum-exp of the raw scores per head, and each slice's factor exp(M_s - lse).  One thread per
  // (slice, statistic, head) fetches its value (sa <= 32: at most 1024 of them) so that the 16 threads that
  // combine them read LDS, not a chain of dependent global loads.
  float* st_l = part;                                          // [kv_rep][sa][32], free until the first put()
  for (int i = tid; i < a.kv_rep * L.sa * 32; i += NW * 64)
    st_l[i] = wsib[(long)(i / (L.sa * 32)) * L.total() + L.stat() + i % (L.sa * 32)];
  __syncthreads();
  if (tid < 16 * a.kv_rep) {                                   // (sub-group, head)
    const int hd = tid & 15;
    const float* sj = st_l + (tid >> 4) * L.sa * 32;
    float* fj = fac + (tid >> 4) * L.sa * 16;
    float M = kNegInf;
    for (int s = 0; s < L.sa; ++s) M = fmaxf(M, sj[s * 32 + hd]);
    float Z = 0.f;
    for (int s = 0; s < L.sa; ++s) {
      const float ms = sj[s * 32 + hd];
      if (ms != kNegInf) Z += sj[s * 32 + 16 + hd] * fast_exp2((ms - M) * kLog2e);
    }
    const float lse2 = (Nc > 0 && hd < G) ? (M + __logf(Z)) * kLog2e : __builtin_huge_valf();   // padding heads drop out
    for (int s = 0; s < L.sa; ++s) {
      const float ms = sj[s * 32 + hd];
      fj[s * 16 + hd] = ms == kNegInf ? 0.f : fast_exp2(fmaf(ms, kLog2e, -lse2));
    }
  }
  for (int i = tid; i < Ns; i += NW * 64) pooled[i] = 0.f;
  __syncthreads();
  const int per_sub = L.sa * L.nb;
  for (int base = 0; base < a.kv_rep * per_sub; base += 4 * NW * 64) {
    f32x4_t x[4][4];
    int js[4], ss[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {                     // all loads of this pass first
      const int idx = base + u * NW * 64 + tid;
      const int sub = idx / per_sub, rem = idx % per_sub;
      const int s = rem / L.nb, lb = rem % L.nb;
      const int j = L.first_bin(s * L.slice) + lb;
      const bool ok = idx < a.kv_rep * per_sub && j >= 0 && j < Ns && s * L.slice < Nc;
      js[u] = ok ? j : -1;
      ss[u] = sub * L.sa + s;
      if (ok) {
        const float* src = wsib + (long)sub * L.total() + L.bins() + ((long)s * L.nb + lb) * 16;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) x[u][q4] = *reinterpret_cast<const f32x4_t*>(src + 4 * q4);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (js[u] >= 0) {
        float v = 0.f;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const f32x4_t fc = *reinterpret_cast<const f32x4_t*>(fac + ss[u] * 16 + 4 * q4);
          v += x[u][q4][0] * fc[0] + x[u][q4][1] * fc[1] + x[u][q4][2] * fc[2] + x[u][q4][3] * fc[3];
        }
        atomicAdd(&pooled[js[u]], v);
      }
    }
  }
  __syncthreads();
  if (wave == 0) {
    __shared__ float cand_v[128];
    __shared__ int cand_i[128];
    float v[PER];                                              // the launcher picks PER with 64 * PER >= Ns
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int bb = lane + 64 * k;
      v[k] = -1.f;
      if (bb < Ns) {
        const int lo = bb * L.pool_s - L.pool_p;
        v[k] = pooled[bb] / (float)(min(lo + L.pool_k, Nc + L.pool_p) - lo);
      }
    }
    wave_topn_shortlist<PER>(v, a.top_n, lane, cand_v, cand_i, [&](int rr, int val) {
      if (lane == 0) {
        sel[rr] = val;
        if (a.indices != nullptr && sb == 0 && h % a.kv_rep == 0) a.indices[((long)b * a.hkv + hc) * a.top_n + rr] = val;
      }
    });
  }
  {
    DecState<T, DK, DV> swa;
    dec_reset(swa);
    for (; next < nwin; next += item_step) {
      const int cb = w_first + 32 * next;
      if (next != my_win) issue_kv(f, cb);
      chunk_attend<T, DK, DV>(swa, f, qf, cb, w_lo, t, c_attn, g);
    }
    put(swa, 1);                                             // its barriers also publish the selected blocks
  }

  // selected blocks: their chunks continue the item count of the window
  {
    DecState<T, DK, DV> slc;
    dec_reset(slc);
    int item = nwin;
    for (int rr = 0; rr < a.top_n; ++rr) {
      const int bi = sel[rr];
      if (bi < 0 || (long)bi * a.sel_block > t) continue;
      const int k0 = bi * a.sel_block, k1 = min(k0 + a.sel_block - 1, t);
      for (int cb = k0; cb <= k1; cb += 32, ++item) {
        if (item != next) continue;
        next += item_step;
        issue_kv(f, cb);
        chunk_attend<T, DK, DV>(slc, f, qf, cb, k0, k1, c_attn, g);
      }
    }
    put(slc, 0);
  }
}

// ---- C: merge of the partial states, gates, output ---------------------------------------------------
// grid (pair, DV / 16): thread = (head r, channel d).  The weights of all partial states go through LDS first
// (one thread per state and head), and the weighted sums are unrolled over the most states there can be, so
// that every load of a thread is in flight at once: the launch is pure latency otherwise.
constexpr int kSplitMaxSplits = 16;      // workgroups per pair in kernel B (and the least number of slices in A)
constexpr int kSplitMaxSlices = 32;      // slices of kernel A: up to 32 * 384 = 12288 compressed rows

template <typename T, int DV, int MAXS>
__global__ void __launch_bounds__(256)
decode_split_merge_kernel(const DecodeArgs a, const SplitLayout L, const float* __restrict__ ws) {
  __shared__ float sm[3][MAXS][16], sl[3][MAXS][16];           // branch 0 selected, 1 window, 2 compressed
  const int tid = threadIdx.x, r = tid & 15, dg = tid >> 4;
  const int bh = blockIdx.x, d = blockIdx.y * 16 + dg;
  const int hs = a.hkv * a.kv_rep;
  const int b = bh / hs, h = bh % hs;                       // h: sub-group, as in kernel A
  const int G = a.hq / hs;
  const float* wsp = ws + (long)bh * L.total();
  const int cap = a.block_table != nullptr ? a.max_pages * 64 : a.ctx_cap;
  if (min(a.ctx_lens[b], cap) <= 0) return;
  const float c_attn = a.scale * kLog2e;
  for (int i = tid; i < 3 * MAXS * 16; i += 256) {
    const int br = i / (MAXS * 16), s = (i / 16) % MAXS, hh = i % 16;
    float m = kNegInf, l = 0.f;
    if (br < 2) {
      if (s < L.sb) {
        const float* p = wsp + L.att() + ((long)br * L.sb + s) * (2 + DV) * 16;
        m = p[hh]; l = p[16 + hh];
      }
    } else if (s < L.sa) {
      m = wsp[L.stat() + s * 32 + hh];
      l = wsp[L.cmp() + (long)s * (1 + DV) * 16 + hh];
    }
    sm[br][s][hh] = m; sl[br][s][hh] = l;
  }
  __syncthreads();
  if (r >= G) return;
  const T* gp = reinterpret_cast<const T*>(a.gates);
  float acc = 0.f;
#pragma unroll
  for (int br = 0; br < 3; ++br) {
    float mm = kNegInf;
#pragma unroll
    for (int s = 0; s < MAXS; ++s) mm = fmaxf(mm, sm[br][s][r]);
    float w[MAXS], den = 0.f;
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
      const float ms = sm[br][s][r];
      w[s] = ms == kNegInf ? 0.f : fast_exp2((ms - mm) * c_attn);
      den += w[s] * sl[br][s][r];
    }
    const float* p = br < 2 ? wsp + L.att() + (long)br * L.sb * (2 + DV) * 16 + (2 + d) * 16 + r
                            : wsp + L.cmp() + (1 + d) * 16 + r;
    const long step = br < 2 ? (2 + DV) * 16 : (1 + DV) * 16;
    float x[MAXS];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) x[s] = w[s] != 0.f ? p[s * step] : 0.f;    // zero weight: unwritten or empty state
    float num = 0.f;
#pragma unroll
    for (int s = 0; s < MAXS; ++s) num += w[s] * x[s];
    float gate = 1.f;
    if (gp != nullptr) {
      const float gx = (float)gp[((long)b * a.hq + h * G + r) * 3 + br];
      gate = a.gate_act == 1 ? 1.0f / (1.0f + __expf(-gx)) : gx;
    }
    if (den > 0.f) acc += num * gate / den;
  }
  reinterpret_cast<T*>(a.out)[((long)b * a.hq + h * G + r) * DV + d] = (T)acc;
}

int set_smem(const void* fn, size_t bytes);

template <typename T, int DK, int DV>
static int launch_decode_split_t(const DecodeArgs& a, int splits, float* ws, hipStream_t st) {
  const SplitLayout L = split_layout(a, splits);
  if (L.sa > kSplitMaxSlices || L.sb > kSplitMaxSplits) return -2;
  if (a.kv_rep < 1 || (long)a.kv_rep * L.sa * 32 > (long)kSplitWaves * DV * 17 || 16 * a.kv_rep > kSplitWaves * 64) return -2;
  const bool big = L.ns_cap > 64 * 10;                        // more bins than ten per lane: the wide top-n
  const int pairs = a.batch * a.hkv * a.kv_rep;
  const size_t base = ((size_t)kSplitWaves * DV * 17 + kSplitWaves * 32) * sizeof(float);
  const size_t smem_a = base + ((size_t)kSplitWaves * 16 + (size_t)L.nb * 16) * sizeof(float);
  const size_t smem_b = base + ((size_t)a.kv_rep * L.sa * 16 + L.ns_cap + 4) * sizeof(float) + (size_t)a.top_n * sizeof(int) + 64;
  {
    auto fn = decode_split_cmp_kernel<T, DK, DV>;
    if (int rc = set_smem(reinterpret_cast<const void*>(fn), smem_a)) return rc;
    hipLaunchKernelGGL(fn, dim3(pairs, L.sa), dim3(kSplitWaves * 64), smem_a, st, a, L, ws);
  }
  auto launch_b = [&](auto fn) -> int {
    if (int rc = set_smem(reinterpret_cast<const void*>(fn), smem_b)) return rc;
    hipLaunchKernelGGL(fn, dim3(pairs, L.sb), dim3(kSplitWaves * 64), smem_b, st, a, L, ws);
    return 0;
  };
  constexpr int PER_BIG = (kSplitMaxSlices * kSplitMaxSlice / 4 + 1 + 63) / 64;   // 3073 bins (the longest cache, windows every 4)
  if (L.ns_cap > 64 * PER_BIG) return -3;
  static_assert(64 * 10 >= 32 * kDecWaves * kDecMaxChunks / 4 + 1, "ten bins per lane cover the short caches");
  int rc;
  if (a.block_table != nullptr)
    rc = big ? launch_b(decode_split_attend_kernel<T, DK, DV, true, PER_BIG>)
             : launch_b(decode_split_attend_kernel<T, DK, DV, true, 10>);
  else
    rc = big ? launch_b(decode_split_attend_kernel<T, DK, DV, false, PER_BIG>)
             : launch_b(decode_split_attend_kernel<T, DK, DV, false, 10>);
  if (rc) return rc;
  if (L.sa > 16)
    hipLaunchKernelGGL((decode_split_merge_kernel<T, DV, kSplitMaxSlices>), dim3(pairs, DV / 16), dim3(256), 0, st, a, L, ws);
  else
    hipLaunchKernelGGL((decode_split_merge_kernel<T, DV, 16>), dim3(pairs, DV / 16), dim3(256), 0, st, a, L, ws);
  return 0;
}

int decode_split_max_nc() { return kSplitMaxSlices * kSplitMaxSlice; }

// ---- the same step for callers that cannot allocate --------------------------------------------------
// The partial results live in a fixed array of the library instead of a caller workspace.  Every GPU the
// library runs on holds its own copy of the array at its own address; `scratch` itself is only the host-side
// name of the symbol, so the device address is looked up once per device and that pointer is what the kernels
// get.  All calls on one GPU share the array: calls that overlap in time race.
constexpr long kStaticScratchBytes = 16L << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];           // device address of `scratch` on each GPU, null = not looked up yet
static std::mutex g_scratch_mutex;

long decode_split_static_bytes() { return kStaticScratchBytes; }

// -1: the workspace of this call does not fit the array; -4: the symbol lookup failed
int launch_decode_split_static(const DecodeArgs& a, int splits, hipStream_t st) {
  if (decode_split_workspace_bytes(a, splits) > kStaticScratchBytes) return -1;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -4;
  void* ptr;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
      void* p = nullptr;
      if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return -4;
      g_scratch_ptr[dev] = p;
    }
    ptr = g_scratch_ptr[dev];
  }
  return launch_decode_split(a, splits, ptr, st);
}

int launch_decode_split(const DecodeArgs& a, int splits, void* workspace, hipStream_t st) {
  float* ws = reinterpret_cast<float*>(workspace);
  const int key = a.dk * 1000 + a.dv;
  if (a.dtype == 0) {
    switch (key) {
      case 64064: return launch_decode_split_t<bf16_t, 64, 64>(a, splits, ws, st);
      case 128128: return launch_decode_split_t<bf16_t, 128, 128>(a, splits, ws, st);
      case 192128: return launch_decode_split_t<bf16_t, 192, 128>(a, splits, ws, st);
      default: return -2;
    }
  }
  if (a.dtype == 2) {
    switch (key) {
      case 64064: return launch_decode_split_t<f16_t, 64, 64>(a, splits, ws, st);
      case 128128: return launch_decode_split_t<f16_t, 128, 128>(a, splits, ws, st);
      case 192128: return launch_decode_split_t<f16_t, 192, 128>(a, splits, ws, st);
      default: return -2;
    }
  }
  switch (key) {
    case 64064: return launch_decode_split_t<float, 64, 64>(a, splits, ws, st);
    case 128128: return launch_decode_split_t<float, 128, 128>(a, splits, ws, st);
    default: return -2;
  }
}

}  // namespace nsa
