// One-token NSA decode step: for every sequence the query at position ctx-1 against its caches.
//
// Cache layout (owned by this library; the reference has no decode path):
//   k_cache    [B][ctx_cap][Hkv][Dk]   row-major keys, the current token already appended
//   v_cache_t  [B][Hkv][Dv][ctx_cap]   key-contiguous values (ctx_cap a multiple of 64, zero-filled)
//   ck_cache   [B][nc_cap][Hkv][Dk]    compressed keys,  row n = mean of tokens [n*stride, n*stride+block)
//   cv_cache_t [B][Hkv][Dv][nc_cap]    compressed values, key-contiguous (nc_cap a multiple of 64)
// so every MFMA operand of the step is a plain 16-byte global load: K fragments are rows, V^T
// fragments are 8 contiguous keys of one channel.  The step is bound by HBM: per sequence and kv
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
#include "tiles.h"

namespace nsa {

constexpr int kDecWaves = 8;
constexpr int kDecMaxChunks = 9;   // compressed 32-row chunks per wavefront kept in registers

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

// one chunk of ordinary attention (window / selected block): keys [cb, cb+32) of the sequence,
// visible keys are lo..hi
template <typename T, int DK, int DV>
__device__ __forceinline__ void dec_attend(DecState<T, DK, DV>& st, const vec8_t<T> (&q)[DK / 32],
                                           const T* __restrict__ kseq, long krow, const T* __restrict__ vt,
                                           long vstep, int cb, int lo, int hi, int last_row, float c_attn,
                                           int n, int g) {
  float s[8], p[8];
  const T* k0p = kseq + (long)min(cb + chunk_key_of_row(0, n), last_row) * krow + 8 * g;
  const T* k1p = kseq + (long)min(cb + chunk_key_of_row(1, n), last_row) * krow + 8 * g;
  dec_scores<T, DK>(k0p, k1p, q, s);
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
    st.o[t] = mma16(load8(vt + t * vstep + cb), pb, st.o[t]);
  }
}

template <typename T, int DK, int DV>
__global__ void __launch_bounds__(kDecWaves * 64)
decode_step_kernel(const DecodeArgs a) {
  constexpr int NW = kDecWaves, MAXC = kDecMaxChunks, PLD = 17;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  float* part = reinterpret_cast<float*>(smem_raw);            // [NW][DV][PLD] partial O^T of one branch
  float* pstat = part + NW * DV * PLD;                         // [NW][2][16]   (m, l) per wavefront
  float* bins = pstat + NW * 2 * 16;                           // [Ns]
  int* sel = reinterpret_cast<int*>(bins + ((a.nc_cap + 3) / 4 + 4));   // [top_n]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int b = blockIdx.x / a.hkv, h = blockIdx.x % a.hkv;
  const int G = a.hq / a.hkv;
  const int ctx = a.ctx_lens[b];
  if (ctx <= 0) return;
  const int t = ctx - 1;
  const int Nc = ctx >= a.block ? (ctx - a.block) / a.stride + 1 : 0;
  int Ns = 0;
  if (Nc > 0 && Nc + 2 * a.pool_p >= a.pool_k) {
    Ns = (Nc + 2 * a.pool_p - a.pool_k + a.pool_s - 1) / a.pool_s + 1;
    if ((Ns - 1) * a.pool_s >= Nc + a.pool_p) --Ns;
  }
  const int cmaxv = t >= a.block ? min((t - a.block) / a.stride, Nc - 1) : -1;   // last visible compressed row
  const float c_attn = a.scale * kLog2e;

  const T* kseq = reinterpret_cast<const T*>(a.k_cache) + ((long)b * a.ctx_cap * a.hkv + h) * DK;
  const long krow = (long)a.hkv * DK;
  const T* vt = reinterpret_cast<const T*>(a.v_cache_t) + (((long)b * a.hkv + h) * DV + n) * a.ctx_cap + 8 * g;
  const long vstep = 16L * a.ctx_cap;
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
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const T* gp = reinterpret_cast<const T*>(a.gates);
  auto gate = [&](int which) -> float {
    if (gp == nullptr || r >= G) return 1.f;
    const float x = (float)gp[((long)b * a.hq + h * G + r) * 3 + which];
    return a.gate_act == 1 ? 1.0f / (1.0f + __expf(-x)) : x;
  };
  auto merge = [&](const DecState<T, DK, DV>& st, float gate_w) {
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
      for (int i = 0; i < 4; ++i) acc[i] += num[i] * inv;
    }
  };

  // ---- phase 1: compressed scores (registers) + sliding window
  float sc[MAXC][8];
  float mi = kNegInf, li = 0.f;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int cb = 32 * (wave + NW * i);
    if (cb < Nc) {
      const T* k0p = ckseq + (long)min(cb + chunk_key_of_row(0, n), Nc - 1) * krow + 8 * g;
      const T* k1p = ckseq + (long)min(cb + chunk_key_of_row(1, n), Nc - 1) * krow + 8 * g;
      dec_scores<T, DK>(k0p, k1p, qf, sc[i]);
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
  DecState<T, DK, DV> swa;
  dec_reset(swa);
  if (a.window > 0) {
    const int w_lo = max(t - a.window + 1, 0);
    for (int cb = (w_lo / 32) * 32 + 32 * wave; cb <= t; cb += 32 * NW)
      dec_attend<T, DK, DV>(swa, qf, kseq, krow, vt, vstep, cb, w_lo, t, t, c_attn, n, g);
  }
  li = colgroup_sum(li);
  if (g == 0) { pstat[(wave * 2 + 0) * 16 + n] = mi; pstat[(wave * 2 + 1) * 16 + n] = li; }
  __syncthreads();

  // ---- phase 2: lse per head, importance bins, compressed attention
  float M = kNegInf;
#pragma unroll
  for (int w = 0; w < NW; ++w) M = fmaxf(M, pstat[(w * 2) * 16 + n]);
  float Z = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    const float mw = pstat[(w * 2) * 16 + n];
    if (mw != kNegInf) Z += pstat[(w * 2 + 1) * 16 + n] * fast_exp2((mw - M) * kLog2e);
  }
  const float lse2 = (Nc > 0 && n < G) ? (M + __logf(Z)) * kLog2e : __builtin_huge_valf();  // padding heads drop out
  if (a.window > 0) merge(swa, gate(1));
  DecState<T, DK, DV> cmp;
  dec_reset(cmp);
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int cb = 32 * (wave + NW * i);
    if (cb < Nc) {
      float p[8];
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int c = cb + 8 * g + e;
        // importance: sum over the 16 lanes (heads) of this lane row
        float v = fast_exp2(fmaf(sc[i][e], kLog2e, -lse2));
        v += __shfl_xor(v, 1); v += __shfl_xor(v, 2); v += __shfl_xor(v, 4); v += __shfl_xor(v, 8);
        if (n == 0 && c < Nc && Ns > 0) {
          const int num = c + a.pool_p - a.pool_k + 1;
          const int b_lo = num <= 0 ? 0 : (num + a.pool_s - 1) / a.pool_s;
          const int b_hi = min((c + a.pool_p) / a.pool_s, Ns - 1);
          for (int bb = b_lo; bb <= b_hi; ++bb) atomicAdd(&bins[bb], v);
        }
        // attention over the visible rows, reference M (>= every visible score)
        p[e] = c <= cmaxv ? fast_exp2((sc[i][e] - M) * c_attn) : 0.f;
        psum += p[e];
      }
      if (cb <= cmaxv) {
        cmp.l += psum;
        const vec8_t<T> pb = pack8<T>(p);
#pragma unroll
        for (int tt = 0; tt < DV / 16; ++tt) cmp.o[tt] = mma16(load8(cvt + tt * cvstep + cb), pb, cmp.o[tt]);
      }
    }
  }
  cmp.m = cmaxv >= 0 ? M : kNegInf;   // every wavefront used the common reference M
  merge(cmp, gate(2));               // its barriers also complete the bins
  __syncthreads();

  // ---- phase 3: top-n blocks (wavefront 0); each lane owns the bins b == lane (mod 64)
  if (wave == 0) {
    volatile float* vb = bins;
    for (int bb = lane; bb < Ns; bb += 64) {
      const int lo = bb * a.pool_s - a.pool_p;
      const int div = min(lo + a.pool_k, Nc + a.pool_p) - lo;
      vb[bb] = vb[bb] / (float)div;
    }
    for (int r = 0; r < a.top_n; ++r) {
      float best = -1.f;
      int bi = 0x7fffffff;
      for (int bb = lane; bb < Ns; bb += 64) {
        const float v = vb[bb];
        if (v > best) { best = v; bi = bb; }
      }
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const float ov = __shfl_xor(best, off);
        const int oi = __shfl_xor(bi, off);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
      }
      const bool found = best >= 0.f;
      if (found && (bi & 63) == lane) vb[bi] = -1.f;
      if (lane == 0) {
        sel[r] = found ? bi : -1;
        if (a.indices != nullptr) a.indices[((long)b * a.hkv + h) * a.top_n + r] = found ? bi : -1;
      }
    }
  }
  __syncthreads();

  // ---- phase 4: selected blocks, 32-key chunks dealt round-robin
  DecState<T, DK, DV> slc;
  dec_reset(slc);
  {
    int item = 0;
    for (int r = 0; r < a.top_n; ++r) {
      const int bi = sel[r];
      if (bi < 0 || (long)bi * a.sel_block > t) continue;
      const int k0 = bi * a.sel_block;
      const int k1 = min(k0 + a.sel_block - 1, t);
      for (int cb = k0; cb <= k1; cb += 32, ++item)
        if ((item & (NW - 1)) == wave)
          dec_attend<T, DK, DV>(slc, qf, kseq, krow, vt, vstep, cb, k0, k1, t, c_attn, n, g);
    }
  }

  merge(slc, gate(0));
  if (r < G && d0 < DV) {
    T* op = reinterpret_cast<T*>(a.out) + ((long)b * a.hq + h * G + r) * DV + d0;
#pragma unroll
    for (int i = 0; i < 4; ++i) op[i] = (T)acc[i];
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

int set_smem(const void* fn, size_t bytes);

template <typename T, int DK, int DV>
static int launch_decode_t(const DecodeArgs& a, hipStream_t st) {
  const size_t smem = ((size_t)kDecWaves * DV * 17 + kDecWaves * 32 + (a.nc_cap + 3) / 4 + 4) * sizeof(float) +
                      (size_t)a.top_n * sizeof(int) + 64;
  auto fn = decode_step_kernel<T, DK, DV>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  hipLaunchKernelGGL(fn, dim3(a.batch * a.hkv), dim3(kDecWaves * 64), smem, st, a);
  return 0;
}

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
  else
    hipLaunchKernelGGL(decode_append_kernel<float>, dim3(batch), dim3(256), 0, st, (const float*)k_new,
                       (const float*)v_new, (float*)k_cache, (float*)v_cache_t, (float*)ck_cache,
                       (float*)cv_cache_t, pos, hkv, dk, dv, ctx_cap, nc_cap, block, stride);
  return 0;
}

int decode_max_nc() { return 32 * kDecWaves * kDecMaxChunks; }

}  // namespace nsa
