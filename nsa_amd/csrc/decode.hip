// One-token NSA decode step: for every sequence the query at position ctx-1 against its caches.
//
// Cache layout (owned by this library; the reference has no decode path):
//   k_cache    [B][ctx_cap][Hkv][Dk]   row-major keys, the current token already appended
//   v_cache_t  [B][Hkv][Dv][ctx_cap]   key-contiguous values (ctx_cap a multiple of 64, zero-filled)
//   ck_cache   [B][nc_cap][Hkv][Dk]    compressed keys,  row n = mean of tokens [n*stride, n*stride+block)
//   cv_cache_t [B][Hkv][Dv][nc_cap]    compressed values, key-contiguous (nc_cap a multiple of 64)
// so every MFMA operand of the step is a plain 16-byte global load: K fragments are rows, V^T
// fragments are 8 contiguous keys of one channel.
// Paged variant: k / v live in a pool of 64-token pages (one selection block = one page),
//   k_pool [page][64][Hkv][Dk],  v_pool_t [page][Hkv][Dv][64],  block_table [B][max_pages]
// and a 32-key chunk looks its page up (a wavefront-uniform scalar load) before requesting its
// fragments; the compressed caches stay contiguous.  The step is bound by HBM: per sequence and kv
// head it reads all compressed keys once (block importance is scored over every compressed row),
// the visible compressed values, the selected blocks and the window.
//
// One workgroup of 8 wavefronts per (sequence, kv head); the G <= 16 query heads are the 16
// columns of the MFMA tiles.  Phases (barriers between them):
//   1  compressed scores: 32-row chunks dealt round-robin to the wavefronts, raw scores kept in
//      registers; per-wavefront running max / sum of the raw scores.  Sliding window chunks are
//      dealt the same way (online softmax state per wavefront).
//   2  combine the score statistics -> lse per head.  From the registers: exp(s - lse) summed over
//      heads and added to the pooled bins in LDS; exp(scale*(s - M)) times cv^T for the visible rows.
//   3  wavefront 0 normalises the bins and takes the top-n blocks.
//   4  selected blocks: 32-key chunks of the usable blocks dealt round-robin.
//   5  partial states of the three branches are merged through LDS, gated and stored.
#include "decode_common.h"

namespace nsa {

// WIDE: room for twice the pooled bins (pooling stride 2: selection blocks of two compression strides)
template <typename T, int DK, int DV, bool PAGED, bool WIDE>
__global__ void __launch_bounds__(kDecWaves * 64)
decode_step_kernel(const DecodeArgs a) {
  constexpr int NW = kDecWaves, MAXC = kDecMaxChunks, PLD = 17;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  float* part = reinterpret_cast<float*>(smem_raw);            // [NW][DV][PLD] partial O^T of one branch
  float* pstat = part + NW * DV * PLD;                         // [NW][2][16]   (m, l) per wavefront
  float* pstat1 = pstat + NW * 2 * 16;                         // [NW][2][16]   score statistics of phase 1
  float* bins = pstat1 + NW * 2 * 16;                          // [Ns]
  int* sel = reinterpret_cast<int*>(bins + decode_bins_cap(a.nc_cap, WIDE));   // [top_n]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int b = blockIdx.x / a.hkv, h = blockIdx.x % a.hkv;
  const int G = a.hq / a.hkv;
  // a length beyond the cache would index past the K/V rows (or the page table): clamp it
  const int ctx = min(a.ctx_lens[b], PAGED ? a.max_pages * 64 : a.ctx_cap);
  if (ctx <= 0) return;
  const int t = ctx - 1;
  const int Nc = ctx >= a.block ? min((ctx - a.block) / a.stride + 1, a.nc_cap) : 0;
  int Ns = 0;
  if (Nc > 0 && Nc + 2 * a.pool_p >= a.pool_k) {
    Ns = (Nc + 2 * a.pool_p - a.pool_k + a.pool_s - 1) / a.pool_s + 1;
    if ((Ns - 1) * a.pool_s >= Nc + a.pool_p) --Ns;
  }
  const int cmaxv = t >= a.block ? min((t - a.block) / a.stride, Nc - 1) : -1;   // last visible compressed row
  const float c_attn = a.scale * kLog2e;

  const T* kseq = reinterpret_cast<const T*>(a.k_cache) + (PAGED ? (long)h * DK : ((long)b * a.ctx_cap * a.hkv + h) * DK);
  const long krow = (long)a.hkv * DK;
  const T* vt = reinterpret_cast<const T*>(a.v_cache_t) +
                (PAGED ? ((long)h * DV + n) * 64 + 8 * g : (((long)b * a.hkv + h) * DV + n) * a.ctx_cap + 8 * g);
  const long vstep = PAGED ? 16L * 64 : 16L * a.ctx_cap;
  // fragments of keys [cb, cb+32) of this sequence (rows past the newest token t are clamped to it)
  auto issue_kv = [&](ChunkFrags<T, DK, DV>& f, int cb) {
    if constexpr (PAGED) {
      const long pg = a.block_table[(long)b * a.max_pages + (cb >> 6)];
      chunk_issue<T, DK, DV>(f, kseq + pg * 64 * krow, krow, vt + pg * a.hkv * DV * 64, vstep, cb & 63,
                             min(t - (cb & ~63), 63), n, g);
    } else {
      chunk_issue<T, DK, DV>(f, kseq, krow, vt, vstep, cb, t, n, g);
    }
  };
  const T* ckseq = reinterpret_cast<const T*>(a.ck_cache) + ((long)b * a.nc_cap * a.hkv + h) * DK;
  const T* cvt = reinterpret_cast<const T*>(a.cv_cache_t) + (((long)b * a.hkv + h) * DV + n) * a.nc_cap + 8 * g;
  const long cvstep = 16L * a.nc_cap;

  // query fragments: column n = head n of this kv head's group (columns >= G are padding)
  vec8_t<T> qf[DK / 32];
  {
    const int gc = n < G ? n : G - 1;
    const T* qp = reinterpret_cast<const T*>(a.q) + ((long)b * a.hq + h * G + gc) * DK + 8 * g;
#pragma unroll
    for (int kk = 0; kk < DK / 32; ++kk) qf[kk] = load8(qp + 32 * kk);
  }
  for (int i = tid; i < Ns; i += NW * 64) bins[i] = 0.f;

  // merging of per-wavefront partial states (used as soon as a branch is complete), gate, accumulate
  // thread -> head r = tid % 16, channels 4*(tid/16) .. +3
  const int r = tid & 15, d0 = (tid >> 4) * 4;
  // The output is (compressed + window) + selected whatever the order the phases ran in, so that an output row does
  // not depend on the batch slot of its sequence: the first two share an accumulator (their sum does not depend on
  // which came first), the selected branch keeps its own until the end.
  float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  const T* gp = reinterpret_cast<const T*>(a.gates);
  auto gate = [&](int which) -> float {
    if (gp == nullptr || r >= G) return 1.f;
    const float x = (float)gp[((long)b * a.hq + h * G + r) * 3 + which];
    return a.gate_act == 1 ? 1.0f / (1.0f + __expf(-x)) : x;
  };
  auto merge = [&](const DecState<T, DK, DV>& st, float gate_w, float (&dst)[4]) {
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
    float den = 0.f, num[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = pstat[(w * 2) * 16 + r];
      if (mw == kNegInf) continue;
      const float wgt = fast_exp2((mw - mm) * c_attn);
      den += wgt * pstat[(w * 2 + 1) * 16 + r];
#pragma unroll
      for (int i = 0; i < 4; ++i) num[i] += wgt * part[(w * DV + ((d0 + i) & (DV - 1))) * PLD + r];
    }
    const float inv = den > 0.f ? gate_w / den : 0.f;
    if (d0 < DV) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float pr = num[i] * inv;
        asm volatile("" : "+v"(pr));       // keeps the product out of a fused multiply-add: only a + b == b + a
        dst[i] += pr;
      }
    }
  };

  // ---- phase 0: sliding window, chunks dealt round-robin, next chunk in flight while one is multiplied
  auto window_phase = [&]() {
    DecState<T, DK, DV> swa;
    dec_reset(swa);
    const int w_lo = max(t - a.window + 1, 0);
    ChunkFrags<T, DK, DV> fa, fb;
    int cb = (w_lo / 32) * 32 + 32 * wave;
    if (cb <= t) issue_kv(fa, cb);
    while (cb <= t) {
      const int cb2 = cb + 32 * NW;
      if (cb2 <= t) issue_kv(fb, cb2);
      chunk_attend<T, DK, DV>(swa, fa, qf, cb, w_lo, t, c_attn, g);
      if (cb2 > t) break;
      const int cb3 = cb2 + 32 * NW;
      if (cb3 <= t) issue_kv(fa, cb3);
      chunk_attend<T, DK, DV>(swa, fb, qf, cb2, w_lo, t, c_attn, g);
      cb = cb3;
    }
    merge(swa, gate(1), acc[1]);
  };
  // Where the window phase runs: 0 first, 1 between the compressed and the selected phase, 2 last.  The phases of
  // a step ramp up and drain one after the other, and with one workgroup per CU all CUs would do so at the same
  // moments; three orders spread the ramps of one third of the chip over the streaming of the rest (95.7 -> 91.4 us
  // at batch 64 x 32768 tokens; two orders 93.3 us).  The branch results are kept apart and summed in one order.
  const int window_pos = (int)(blockIdx.x % 3);
  if (a.window > 0 && window_pos == 0) window_phase();

  // ---- phase 1: compressed scores (kept in registers), next chunk's K fragments in flight
  float sc[MAXC][8];
  float mi = kNegInf, li = 0.f;
  {
    vec8_t<T> ka[2][DK / 32], kb2[2][DK / 32];
    auto issue = [&](vec8_t<T> (&f)[2][DK / 32], int cb) {
      const T* k0p = ckseq + (long)min(cb + chunk_key_of_row(0, n), Nc - 1) * krow + 8 * g;
      const T* k1p = ckseq + (long)min(cb + chunk_key_of_row(1, n), Nc - 1) * krow + 8 * g;
#pragma unroll
      for (int kk = 0; kk < DK / 32; ++kk) { f[0][kk] = load8(k0p + 32 * kk); f[1][kk] = load8(k1p + 32 * kk); }
    };
    if (32 * wave < Nc) issue(ka, 32 * wave);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int cb = 32 * (wave + NW * i);
      vec8_t<T> (&cur)[2][DK / 32] = (i & 1) ? kb2 : ka;
      vec8_t<T> (&nxt)[2][DK / 32] = (i & 1) ? ka : kb2;
      if (i + 1 < MAXC && cb + 32 * NW < Nc) issue(nxt, cb + 32 * NW);
      if (cb < Nc) {
        f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < DK / 32; ++kk) {
          s0 = mma16(cur[0][kk], qf[kk], s0);
          s1 = mma16(cur[1][kk], qf[kk], s1);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) { sc[i][e] = s0[e]; sc[i][4 + e] = s1[e]; }
        float mx = kNegInf;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if (cb + 8 * g + e >= Nc) sc[i][e] = kNegInf;
          mx = fmaxf(mx, sc[i][e]);
        }
        mx = colgroup_max(mx);
        const float m_new = fmaxf(mi, mx);              // finite: row cb exists
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
  }
  li = colgroup_sum(li);
  if (g == 0) { pstat1[(wave * 2 + 0) * 16 + n] = mi; pstat1[(wave * 2 + 1) * 16 + n] = li; }
  __syncthreads();

  // ---- phase 2: lse per head, importance bins, compressed attention
  float M = kNegInf;
#pragma unroll
  for (int w = 0; w < NW; ++w) M = fmaxf(M, pstat1[(w * 2) * 16 + n]);
  float Z = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    const float mw = pstat1[(w * 2) * 16 + n];
    if (mw != kNegInf) Z += pstat1[(w * 2 + 1) * 16 + n] * fast_exp2((mw - M) * kLog2e);
  }
  const float lse2 = (Nc > 0 && n < G) ? (M + __logf(Z)) * kLog2e : __builtin_huge_valf();  // padding heads drop out
  // ---- phase 2a: importance bins from the registers (no memory traffic).  The head sum is a DPP
  // all-reduce over the 16 lanes of a row; lane n == 0 of every row then owns 8 consecutive columns.
  const bool fast_pool = a.pool_k == 5 && a.pool_s == 4 && a.pool_p == 0;
  // windows of s + 1 columns every s, s = 1, 2, 4 or 8, any padding: see the runs below
  const bool run_pool = a.pool_k == a.pool_s + 1 && (a.pool_s == 1 || a.pool_s == 2 || a.pool_s == 4 || a.pool_s == 8);
  const int ls = a.pool_s == 1 ? 0 : a.pool_s == 2 ? 1 : a.pool_s == 4 ? 2 : 3;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int cb = 32 * (wave + NW * i);
    if (cb < Nc && Ns > 0) {
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float x = fast_exp2(fmaf(sc[i][e], kLog2e, -lse2));
        x += dpp_f32<0xB1>(x);          // quad_perm [1,0,3,2]
        x += dpp_f32<0x4E>(x);          // quad_perm [2,3,0,1]
        x += dpp_f32<0x141>(x);         // row_half_mirror
        x += dpp_f32<0x140>(x);         // row_mirror
        v[e] = x;
      }
      const int c0 = cb + 8 * g;
      if (n == 0 && c0 < Nc) {
        if (fast_pool) {
          // windows of 5 columns every 4: columns c0..c0+7 touch bins c0/4-1 (first column only),
          // c0/4 and c0/4+1; columns past Nc carry 0
          const int b0 = c0 >> 2;
          if (b0 >= 1 && b0 - 1 < Ns) atomicAdd(&bins[b0 - 1], v[0]);
          if (b0 < Ns) atomicAdd(&bins[b0], (v[0] + v[1]) + (v[2] + v[3]) + v[4]);
          if (b0 + 1 < Ns) atomicAdd(&bins[b0 + 1], (v[4] + v[5]) + (v[6] + v[7]));
        } else if (run_pool) {
          // bin j pools positions j * s .. j * s + s of the padded row (position = column + padding): the lane's 8
          // consecutive columns are runs of equal bin, one atomic per run; a position that is a multiple of s is the
          // first of its bin and also the last of the bin before
          const int x0 = c0 + a.pool_p;
          int cur = x0 >> ls;
          float run = 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int x = x0 + e;
            if ((x & (a.pool_s - 1)) == 0) {
              if (e == 0) {
                if (cur >= 1 && cur - 1 < Ns) atomicAdd(&bins[cur - 1], v[0]);
              } else {
                if (cur < Ns) atomicAdd(&bins[cur], run + v[e]);
                cur = x >> ls;
              }
              run = v[e];
            } else {
              run += v[e];
            }
          }
          if (cur < Ns) atomicAdd(&bins[cur], run);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int c = c0 + e;
            if (c >= Nc) break;
            const int num = c + a.pool_p - a.pool_k + 1;
            const int b_lo = num <= 0 ? 0 : (num + a.pool_s - 1) / a.pool_s;
            const int b_hi = min((c + a.pool_p) / a.pool_s, Ns - 1);
            for (int bb = b_lo; bb <= b_hi; ++bb) atomicAdd(&bins[bb], v[e]);
          }
        }
      }
    }
  }
  __syncthreads();

  // ---- phase 3 (wavefront 0 only): top-n blocks; each lane owns the bins b == lane (mod 64)
  if (wave == 0) {
    constexpr int PER = (32 * kDecWaves * kDecMaxChunks / (WIDE ? 2 : 4) + 63) / 64 + 1;
    static_assert(64 * PER >= kDecBinsMax<WIDE>, "every bin needs a lane slot");
    __shared__ float cand_v[128];
    __shared__ int cand_i[128];
    float v[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int bb = lane + 64 * k;
      v[k] = -1.f;
      if (bb < Ns) {
        const int lo = bb * a.pool_s - a.pool_p;
        const int div = min(lo + a.pool_k, Nc + a.pool_p) - lo;
        v[k] = bins[bb] / (float)div;
      }
    }
    wave_topn_shortlist<PER>(v, a.top_n, lane, cand_v, cand_i, [&](int rr, int val) {
      if (lane == 0) {
        sel[rr] = val;
        if (a.indices != nullptr) a.indices[((long)b * a.hkv + h) * a.top_n + rr] = val;
      }
    });
  }

  // ---- phase 2b: compressed attention from the registers, cv^T fragments one chunk ahead
  DecState<T, DK, DV> cmp;
  dec_reset(cmp);
  {
    vec8_t<T> va[DV / 16], vb2[DV / 16];
    auto issue = [&](vec8_t<T> (&f)[DV / 16], int cb) {
#pragma unroll
      for (int tt = 0; tt < DV / 16; ++tt) f[tt] = load8(cvt + tt * cvstep + cb);
    };
    if (32 * wave <= cmaxv) issue(va, 32 * wave);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int cb = 32 * (wave + NW * i);
      vec8_t<T> (&cur)[DV / 16] = (i & 1) ? vb2 : va;
      vec8_t<T> (&nxt)[DV / 16] = (i & 1) ? va : vb2;
      if (i + 1 < MAXC && cb + 32 * NW <= cmaxv) issue(nxt, cb + 32 * NW);
      if (cb <= cmaxv) {
        float p[8], psum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int c = cb + 8 * g + e;
          p[e] = c <= cmaxv ? fast_exp2((sc[i][e] - M) * c_attn) : 0.f;   // reference M >= every visible score
          psum += p[e];
        }
        cmp.l += psum;
        const vec8_t<T> pb = pack8<T>(p);
#pragma unroll
        for (int tt = 0; tt < DV / 16; ++tt) cmp.o[tt] = mma16(cur[tt], pb, cmp.o[tt]);
      }
    }
  }
  cmp.m = cmaxv >= 0 ? M : kNegInf;   // every wavefront used the common reference M
  merge(cmp, gate(2), acc[1]);               // its barriers also publish the selected blocks
  if (a.window > 0 && window_pos == 1) window_phase();

  // ---- phase 4: selected blocks, 32-key chunks dealt round-robin, next chunk in flight
  DecState<T, DK, DV> slc;
  dec_reset(slc);
  {
    int rr = 0, item = 0, cur = 0, cur_last = -1, cur_k0 = 0;
    // next 32-key chunk of this wavefront: (cb, k0, k1) of its block; false when the picks are exhausted
    auto next_chunk = [&](int& cb, int& k0, int& k1) -> bool {
      while (true) {
        if (cur > cur_last) {
          if (rr >= a.top_n) return false;
          const int bi = sel[rr++];
          if (bi < 0 || (long)bi * a.sel_block > t) continue;
          cur_k0 = bi * a.sel_block;
          cur = cur_k0;
          cur_last = min(cur_k0 + a.sel_block - 1, t);
        }
        const bool mine = (item & (NW - 1)) == wave;
        cb = cur; k0 = cur_k0; k1 = cur_last;
        cur += 32;
        ++item;
        if (mine) return true;
      }
    };
    ChunkFrags<T, DK, DV> fa, fb;
    int cba, k0a, k1a, cbb, k0b, k1b;
    bool ha = next_chunk(cba, k0a, k1a);
    if (ha) issue_kv(fa, cba);
    while (ha) {
      const bool hb = next_chunk(cbb, k0b, k1b);
      if (hb) issue_kv(fb, cbb);
      chunk_attend<T, DK, DV>(slc, fa, qf, cba, k0a, k1a, c_attn, g);
      if (!hb) break;
      ha = next_chunk(cba, k0a, k1a);
      if (ha) issue_kv(fa, cba);
      chunk_attend<T, DK, DV>(slc, fb, qf, cbb, k0b, k1b, c_attn, g);
    }
  }
  merge(slc, gate(0), acc[0]);
  if (a.window > 0 && window_pos == 2) window_phase();
  if (r < G && d0 < DV) {
    T* op = reinterpret_cast<T*>(a.out) + ((long)b * a.hq + h * G + r) * DV + d0;
#pragma unroll
    for (int i = 0; i < 4; ++i) op[i] = (T)(acc[1][i] + acc[0][i]);
  }
}

// Appends one token per sequence to the caches: k row, v column, and - when the token completes a
// compression block - the new compressed row (mean of the last `block` tokens).
template <typename T>
__global__ void __launch_bounds__(256)
decode_append_kernel(const T* __restrict__ k_new, const T* __restrict__ v_new, T* __restrict__ k_cache,
                     T* __restrict__ v_cache_t, T* __restrict__ ck_cache, T* __restrict__ cv_cache_t,
                     const int32_t* __restrict__ pos, int hkv, int dk, int dv, int ctx_cap, int nc_cap,
                     int block, int stride) {
  const int b = blockIdx.x;
  const int p = pos[b];
  if (p < 0 || p >= ctx_cap) return;
  T* krow = k_cache + ((long)b * ctx_cap + p) * hkv * dk;
  for (int i = threadIdx.x; i < hkv * dk; i += 256) krow[i] = k_new[(long)b * hkv * dk + i];
  for (int i = threadIdx.x; i < hkv * dv; i += 256)
    v_cache_t[((long)b * hkv * dv + i) * ctx_cap + p] = v_new[(long)b * hkv * dv + i];
  const int ctx = p + 1;
  if (ctx < block || (ctx - block) % stride != 0) return;
  const int nrow = (ctx - block) / stride;
  if (nrow >= nc_cap) return;
  __syncthreads();   // the row and column written above are part of the window below
  const float inv = 1.0f / (float)block;
  for (int i = threadIdx.x; i < hkv * dk; i += 256) {
    float s = 0.f;
    for (int j = 0; j < block; ++j) s += (float)k_cache[((long)b * ctx_cap + (ctx - block + j)) * hkv * dk + i];
    ck_cache[((long)b * nc_cap + nrow) * hkv * dk + i] = (T)(s * inv);
  }
  for (int i = threadIdx.x; i < hkv * dv; i += 256) {
    const T* col = v_cache_t + ((long)b * hkv * dv + i) * ctx_cap + (ctx - block);
    float s = 0.f;
    for (int j = 0; j < block; ++j) s += (float)col[j];
    cv_cache_t[((long)b * hkv * dv + i) * nc_cap + nrow] = (T)(s * inv);
  }
}

// The same for the paged pool: the token goes to slot pos % 64 of page block_table[b][pos / 64]; a
// compression window may straddle two pages.
template <typename T>
__global__ void __launch_bounds__(256)
decode_append_paged_kernel(const T* __restrict__ k_new, const T* __restrict__ v_new, T* __restrict__ k_pool,
                           T* __restrict__ v_pool_t, const int32_t* __restrict__ block_table, int max_pages,
                           T* __restrict__ ck_cache, T* __restrict__ cv_cache_t, const int32_t* __restrict__ pos,
                           int hkv, int dk, int dv, int nc_cap, int block, int stride) {
  const int b = blockIdx.x;
  const int p = pos[b];
  if (p < 0 || p >= max_pages * 64) return;
  const int32_t* table = block_table + (long)b * max_pages;
  const long pg = table[p >> 6];
  T* krow = k_pool + (pg * 64 + (p & 63)) * hkv * dk;
  for (int i = threadIdx.x; i < hkv * dk; i += 256) krow[i] = k_new[(long)b * hkv * dk + i];
  for (int i = threadIdx.x; i < hkv * dv; i += 256)
    v_pool_t[(pg * hkv * dv + i) * 64 + (p & 63)] = v_new[(long)b * hkv * dv + i];
  const int ctx = p + 1;
  if (ctx < block || (ctx - block) % stride != 0) return;
  const int nrow = (ctx - block) / stride;
  if (nrow >= nc_cap) return;
  __syncthreads();   // the row and column written above are part of the window below
  const float inv = 1.0f / (float)block;
  for (int i = threadIdx.x; i < hkv * dk; i += 256) {
    float s = 0.f;
    for (int j = 0; j < block; ++j) {
      const int tk = ctx - block + j;
      s += (float)k_pool[((long)table[tk >> 6] * 64 + (tk & 63)) * hkv * dk + i];
    }
    ck_cache[((long)b * nc_cap + nrow) * hkv * dk + i] = (T)(s * inv);
  }
  for (int i = threadIdx.x; i < hkv * dv; i += 256) {
    float s = 0.f;
    for (int j = 0; j < block; ++j) {
      const int tk = ctx - block + j;
      s += (float)v_pool_t[((long)table[tk >> 6] * hkv * dv + i) * 64 + (tk & 63)];
    }
    cv_cache_t[((long)b * hkv * dv + i) * nc_cap + nrow] = (T)(s * inv);
  }
}

int set_smem(const void* fn, size_t bytes);

template <typename T, int DK, int DV, bool PAGED, bool WIDE>
static int launch_decode_v(const DecodeArgs& a, hipStream_t st) {
  const size_t smem = ((size_t)kDecWaves * DV * 17 + kDecWaves * 64 + decode_bins_cap(a.nc_cap, WIDE)) * sizeof(float) +
                      (size_t)a.top_n * sizeof(int) + 64;
  auto fn = decode_step_kernel<T, DK, DV, PAGED, WIDE>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  hipLaunchKernelGGL(fn, dim3(a.batch * a.hkv), dim3(kDecWaves * 64), smem, st, a);
  return 0;
}

template <typename T, int DK, int DV>
static int launch_decode_t(const DecodeArgs& a, hipStream_t st) {
  const int bins = decode_pooled_bins(a.nc_cap, a.pool_k, a.pool_s, a.pool_p);
  if (bins > decode_bins_room(a.nc_cap, true)) return -3;
  const bool wide = bins > decode_bins_room(a.nc_cap, false);
  if (a.block_table != nullptr)
    return wide ? launch_decode_v<T, DK, DV, true, true>(a, st) : launch_decode_v<T, DK, DV, true, false>(a, st);
  return wide ? launch_decode_v<T, DK, DV, false, true>(a, st) : launch_decode_v<T, DK, DV, false, false>(a, st);
}

int decode_max_bins(int nc_cap) { return decode_bins_room(nc_cap, true); }

int launch_decode(const DecodeArgs& a, hipStream_t st) {
  const int key = a.dk * 1000 + a.dv;
  if (a.dtype == 0) {
    switch (key) {
      case 64064: return launch_decode_t<bf16_t, 64, 64>(a, st);
      case 128128: return launch_decode_t<bf16_t, 128, 128>(a, st);
      case 192128: return launch_decode_t<bf16_t, 192, 128>(a, st);
      default: return -2;
    }
  }
  if (a.dtype == 2) {
    switch (key) {
      case 64064: return launch_decode_t<f16_t, 64, 64>(a, st);
      case 128128: return launch_decode_t<f16_t, 128, 128>(a, st);
      case 192128: return launch_decode_t<f16_t, 192, 128>(a, st);
      default: return -2;
    }
  }
  switch (key) {
    case 64064: return launch_decode_t<float, 64, 64>(a, st);
    case 128128: return launch_decode_t<float, 128, 128>(a, st);
    default: return -2;
  }
}

int launch_decode_append(const void* k_new, const void* v_new, void* k_cache, void* v_cache_t, void* ck_cache,
                         void* cv_cache_t, const int32_t* pos, int batch, int hkv, int dk, int dv, int ctx_cap,
                         int nc_cap, int block, int stride, int dtype, hipStream_t st) {
  if (dtype == 0)
    hipLaunchKernelGGL(decode_append_kernel<bf16_t>, dim3(batch), dim3(256), 0, st, (const bf16_t*)k_new,
                       (const bf16_t*)v_new, (bf16_t*)k_cache, (bf16_t*)v_cache_t, (bf16_t*)ck_cache,
                       (bf16_t*)cv_cache_t, pos, hkv, dk, dv, ctx_cap, nc_cap, block, stride);
  else if (dtype == 2)
    hipLaunchKernelGGL(decode_append_kernel<f16_t>, dim3(batch), dim3(256), 0, st, (const f16_t*)k_new,
                       (const f16_t*)v_new, (f16_t*)k_cache, (f16_t*)v_cache_t, (f16_t*)ck_cache,
                       (f16_t*)cv_cache_t, pos, hkv, dk, dv, ctx_cap, nc_cap, block, stride);
  else
    hipLaunchKernelGGL(decode_append_kernel<float>, dim3(batch), dim3(256), 0, st, (const float*)k_new,
                       (const float*)v_new, (float*)k_cache, (float*)v_cache_t, (float*)ck_cache,
                       (float*)cv_cache_t, pos, hkv, dk, dv, ctx_cap, nc_cap, block, stride);
  return 0;
}

int launch_decode_append_paged(const void* k_new, const void* v_new, void* k_pool, void* v_pool_t,
                               const int32_t* block_table, int max_pages, void* ck_cache, void* cv_cache_t,
                               const int32_t* pos, int batch, int hkv, int dk, int dv, int nc_cap, int block,
                               int stride, int dtype, hipStream_t st) {
  if (dtype == 0)
    hipLaunchKernelGGL(decode_append_paged_kernel<bf16_t>, dim3(batch), dim3(256), 0, st, (const bf16_t*)k_new,
                       (const bf16_t*)v_new, (bf16_t*)k_pool, (bf16_t*)v_pool_t, block_table, max_pages,
                       (bf16_t*)ck_cache, (bf16_t*)cv_cache_t, pos, hkv, dk, dv, nc_cap, block, stride);
  else if (dtype == 2)
    hipLaunchKernelGGL(decode_append_paged_kernel<f16_t>, dim3(batch), dim3(256), 0, st, (const f16_t*)k_new,
                       (const f16_t*)v_new, (f16_t*)k_pool, (f16_t*)v_pool_t, block_table, max_pages,
                       (f16_t*)ck_cache, (f16_t*)cv_cache_t, pos, hkv, dk, dv, nc_cap, block, stride);
  else
    hipLaunchKernelGGL(decode_append_paged_kernel<float>, dim3(batch), dim3(256), 0, st, (const float*)k_new,
                       (const float*)v_new, (float*)k_pool, (float*)v_pool_t, block_table, max_pages,
                       (float*)ck_cache, (float*)cv_cache_t, pos, hkv, dk, dv, nc_cap, block, stride);
  return 0;
}

int decode_max_nc() { return 32 * kDecWaves * kDecMaxChunks; }

}  // namespace nsa
