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
// stays in `pend`, a 129th value per lane.  Slots 0 .. 95 (rows 0 .. 1535) are registers; the slots of the last 512
// rows go to a lane-private column of LDS (8 KB per wavefront): 128 more registers would not leave room for the
// query fragments and the output accumulators of a 192-wide head at two wavefronts per SIMD.
#include <type_traits>
#include <utility>

#include "tiles.h"

namespace nsa {

typedef float f32x32_t __attribute__((ext_vector_type(32)));

int set_smem(const void* fn, size_t bytes);

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}
// keeps a value (and the instruction that made it) at this point of the program
__device__ __forceinline__ void pin(float& x) { asm volatile("" : "+v"(x)); }

// ------------------------------------------------------------------------------------------------
// Fragment-major copy of the compressed keys and values.
//
// The pass streams every 64-row chunk of a sequence's compressed K and V through LDS once per token tile.  With the
// chunk stored in memory exactly as the matrix instructions consume it -- one 1 KB block per operand fragment, lane
// l's 16 bytes at byte 16 l -- the global -> LDS copy is a straight run of bytes (done by the load unit itself,
// global_load_lds, no staging registers and no LDS store instructions) and every fragment read is 64 consecutive
// 16-byte pieces: no padding, no bank conflicts, whatever the row -> lane map.
//   chunk = [ K part: step s (32 rows) | tile t (0/1) | depth block kk | lane | 8 elements ]
//           [ V part: step s           | channel tile tv (16 channels)  | lane | 8 elements ]
//   K fragment (s, t, kk), lane (m, g):  K[32 s + chunk_key_of_row(t, m)][32 kk + 8 g .. + 7]
//   V fragment (s, tv),    lane (m, g):  V[32 s + 8 g .. + 7][16 tv + m]   (8 rows of one channel)
// Chunk c of sequence b of kv head h sits at chunk slot cu_cmp[b] / 64 + b + c of that head (slots of different
// sequences never overlap; at most total_rows / 64 + batch + 1 slots).  Rows past the sequence's last one are zero.
// 16 bytes per lane from global memory straight into LDS: lane i's piece lands at lds + 16 i bytes (lds is the same
// for the whole wavefront).  Counts as a vector-memory load of the wavefront until the data is in LDS.
// Written as assembly on purpose: the compiler books the built-in form as an access that may touch both memories,
// and from then on answers every wait for an LDS read with "wait for all of them" -- which undoes a ring of
// fragment reads in flight.  The callers wait for these loads themselves (s_waitcnt vmcnt(0) before the barrier
// that publishes the chunk).  m0 is not named as clobbered: the compiler reserves it and sets it anew before every
// use of its own (register indexing), never across a statement.
__device__ __forceinline__ unsigned lds_address(const void* p) {
  return (unsigned)(uintptr_t)((__attribute__((address_space(3))) const char*)p);
}
template <typename T>
__device__ __forceinline__ void global_to_lds16(const T* src, T* lds) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :: "v"(src), "s"(lds_address(lds)) : "memory");
}

__host__ __device__ __forceinline__ int frag_chunk_slot(int cu_b, int b) { return (cu_b >> 6) + b; }

template <typename T, int DK, int DV>
__global__ void __launch_bounds__(256)
frag_pack_kernel(const T* __restrict__ ck, const T* __restrict__ cv, T* __restrict__ frag, const int32_t* cu_cmp,
                 int batch, long ck_row_stride, long ck_head_stride, long cv_row_stride, long cv_head_stride,
                 int frag_chunks) {
  constexpr int KLD = DK + 8, VLD = DV + 2, NKK = DK / 32, NV = DV / 16, CHUNK = 64 * (DK + DV);
  __shared__ __attribute__((aligned(16))) T sk[64 * KLD];
  __shared__ T sv[64 * VLD];
  const SeqTile st = find_tile(cu_cmp, batch, 64, blockIdx.x);
  if (!st.valid) return;
  const int h = blockIdx.y, tid = threadIdx.x;
  const T* kb = ck + (long)(st.start + st.t0) * ck_row_stride + (long)h * ck_head_stride;
  const T* vb = cv + (long)(st.start + st.t0) * cv_row_stride + (long)h * cv_head_stride;
  const int rows = min(64, st.len - st.t0);
  for (int p = tid; p < 64 * (DK / 8); p += 256) {
    const int r = p / (DK / 8), pc = p % (DK / 8);
    store8(sk + r * KLD + pc * 8, r < rows ? load8(kb + (long)r * ck_row_stride + pc * 8) : zero8<T>());
  }
  for (int p = tid; p < 64 * (DV / 8); p += 256) {
    const int r = p / (DV / 8), pc = p % (DV / 8);
    const vec8_t<T> x = r < rows ? load8(vb + (long)r * cv_row_stride + pc * 8) : zero8<T>();
#pragma unroll
    for (int e = 0; e < 8; ++e) sv[r * VLD + pc * 8 + e] = x[e];
  }
  __syncthreads();
  T* out = frag + ((long)h * frag_chunks + frag_chunk_slot(st.start, st.b) + (st.t0 >> 6)) * CHUNK;
  for (int p = tid; p < 64 * (DK / 8); p += 256) {
    const int l = p & 63, f = p >> 6;                 // fragment f = (s * 2 + t) * NKK + kk
    const int kk = f % NKK, t = (f / NKK) & 1, sstep = f / (2 * NKK);
    const int m = l & 15, g = l >> 4;
    store8(out + p * 8, load8(sk + (32 * sstep + chunk_key_of_row(t, m)) * KLD + 32 * kk + 8 * g));
  }
  for (int p = tid; p < 64 * (DV / 8); p += 256) {
    const int l = p & 63, f = p >> 6;                 // fragment f = s * NV + tv
    const int tv = f % NV, sstep = f / NV;
    const int m = l & 15, g = l >> 4;
    vec8_t<T> x;
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = sv[(32 * sstep + 8 * g + e) * VLD + 16 * tv + m];
    store8(out + 64 * DK + p * 8, x);
  }
}

#ifndef NSA_FUSED_GS
#define NSA_FUSED_GS 2
#endif
constexpr int kFusedMaxRows = 2048;      // compressed rows per sequence the window sums have room for

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
  constexpr int NW = 8, TQ = NW, NKK = DK / 32, NV = DV / 16;
  constexpr int KPART = 64 * DK, CHUNK = 64 * (DK + DV);          // elements of a chunk's K part / of a chunk
  constexpr int NKB = KPART / 512, NVB = 64 * DV / 512;           // 1 KB blocks of the two parts
  constexpr bool kNarrowP = std::is_same<T, f16_t>::value;      // packed probabilities narrower than the fp32 sums
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* ldsC = reinterpret_cast<T*>(smem_raw);                        // [2][CHUNK]: chunks in fragment order
  float* ldsB = reinterpret_cast<float*>(ldsC + 2 * CHUNK);        // [NW][32 slots][64 lanes]

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
  const T* fragb = reinterpret_cast<const T*>(a.frag) + ((long)h * a.frag_chunks + frag_chunk_slot(koff, st.b)) * CHUNK;

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
    for (int kk = 0; kk < NKK; ++kk) gt = mma16(n < 3 ? load8(wp + 32 * kk) : zero8<T>(), grp[0].q[kk], gt);
    if (g == 0 && rm.valid) {
      T* gp = reinterpret_cast<T*>(a.gates) + (((long)st.start + rm.tok) * a.hq + h * G + rm.gidx) * 3;
#pragma unroll
      for (int i = 0; i < 3; ++i) gp[i] = (T)(gt[i] + (bp != nullptr ? (float)bp[i] : 0.f));
    }
  }
  const float c_attn = a.scale * kLog2e;

  // staging: the load unit copies the chunk, 1 KB per wavefront instruction; wavefront w takes blocks w, w + 8, ..
  auto stage_chunk = [&](int c0, int buf, bool with_v) __attribute__((always_inline)) {
    const T* src = fragb + (long)(c0 >> 6) * CHUNK + lane * 8;
    T* dst = ldsC + buf * CHUNK;
#pragma unroll
    for (int i = 0; i < (NKB + NW - 1) / NW; ++i)
      if (NKB % NW == 0 || wave + i * NW < NKB) global_to_lds16(src + (wave + i * NW) * 512, dst + (wave + i * NW) * 512);
    if (with_v) {
#pragma unroll
      for (int i = 0; i < (NVB + NW - 1) / NW; ++i)
        if (NVB % NW == 0 || wave + i * NW < NVB)
          global_to_lds16(src + KPART + (wave + i * NW) * 512, dst + KPART + (wave + i * NW) * 512);
    }
  };
  auto staged = [&]() {                       // this wavefront's blocks have landed; then everybody's
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };

  const bool last_row = g == 3;
  const int next_lane = ((lane + 16) & 63) << 2;

  f32x32_t bq0, bq1, bq2;                    // the window sums of this lane's head: slot s < 96 = bq<s / 32>[s % 32]
#pragma unroll
  for (int i = 0; i < 32; ++i) { bq0[i] = 0.f; bq1[i] = 0.f; bq2[i] = 0.f; }
  float* binl = ldsB + (wave * 32) * 64 + lane;      // slot 96 + j = binl[64 j]
#pragma unroll
  for (int i = 0; i < 32; ++i) binl[64 * i] = 0.f;
  float li = 0.f;                            // this lane's share of the importance denominator
  float pend = 0.f;                          // lane row 3: the upper quad of the step before
  float pmax = 0.f;                          // float16: the largest 8-row sum of packed probabilities
  float m_i = 0.f, m_a = 0.f;                // references of the two softmaxes (raw score units)
  float off_i = 0.f, off_a = 0.f;

  wait_all_loads();

  // raw scores of one 32-row step: value i of lane (n, g) = row 8g + i of the step, head n
  auto scores = [&](const T* kf, float (&s)[8]) __attribute__((always_inline)) {
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      s0 = mma16(load8(kf + kk * 512), grp[0].q[kk], s0);
      s1 = mma16(load8(kf + (NKK + kk) * 512), grp[0].q[kk], s1);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) { s[i] = s0[i]; s[4 + i] = s1[i]; }
  };

  // ---- a chunk = two steps a, b; the common chunks are software-pipelined by hand
  // A wavefront that runs "scores, softmax, P V" one after the other leaves the matrix unit idle during its vector
  // work, and its SIMD partner, released by the same barrier, is in the same phase.  A chunk whose two steps are
  // both fully visible (or both hidden) therefore runs as one fixed schedule of matrix instructions with the
  // vector work of OTHER steps dealt out between them:
  //   visible:  QK(a) | B(prev b)    QK(b) | A(a)    PV(a) | A(b)    PV(b) | B(a)
  //   hidden:   QK(a) | B(prev b)    QK(b) | B(a)
  // A(x) = attention probabilities of step x (8 exponentials, their sum, the packed operand of PV(x)), B(x) = the
  // importance side (8 exponentials, the step's two window sums).  B of a chunk's second step is carried into the
  // next chunk.  Fragments come from LDS through a ring of 4 register sets, requested in pairs two matrix instructions ahead.
  // The visible schedule takes any chunk: the first one (its step a sets the references), the one on the causal edge
  // and a tail chunk switch its masks on.  Either schedule ends with the same four values -- the window sums of the
  // carried step and of step a -- and the register block of the section is written at ONE place behind the two
  // bodies: two bodies that each wrote it would meet in a merge that costs a copy of the 32-register block.
  constexpr int NQ = 2 * NKK;                      // matrix instructions of one step's scores
  constexpr int kOpsA = 25, kOpsB = 25;            // vector operations of A(x) / B(x)
  float cs[8];                                     // carried: scores of the previous chunk's second step ...
  int cslot = -1;                                  // ... and its slot (-1: nothing carried)
  bool creal = false;                              // ... and whether that step has rows at all
  float bt[4], bnxt;                               // B's temporaries
  float e_[8];
  // real = false: a stand-in for a carried step that does not exist (scores -inf: every exponential 0); its zeros go
  // to slots that the chunk's own first step overwrites right after, and it must leave `pend` alone
  auto opB = [&](auto I, const float (&s)[8], float& w0, float& w1, bool real) __attribute__((always_inline)) {   // kOpsB operations
    constexpr int i = decltype(I)::value;
    // the multiply-adds first, the exponentials after them: neighbours in the instruction stream are independent
    if constexpr (i < 8) { e_[i] = fmaf(s[i], kLog2e, off_i); pin(e_[i]); }
    else if constexpr (i < 16) { e_[i - 8] = fast_exp2(e_[i - 8]); pin(e_[i - 8]); }
    else if constexpr (i == 16) { bnxt = __int_as_float(__builtin_amdgcn_ds_bpermute(next_lane, __float_as_int(e_[0]))); }
    else if constexpr (i < 21) { bt[i - 17] = e_[2 * (i - 17)] + e_[2 * (i - 17) + 1]; pin(bt[i - 17]); }
    else if constexpr (i == 21) { bt[0] += bt[1]; pin(bt[0]); }                       // lower quad
    else if constexpr (i == 22) { bt[2] += bt[3]; pin(bt[2]); }                       // upper quad
    else if constexpr (i == 23) { li += bt[0] + bt[2]; pin(li); }
    else {
      // e_[0] (row 8g) completes the upper window of the lane row before, e_[4] this lane's lower window
      w0 = bt[0] + e_[4];
      w1 = (last_row ? pend : bt[2]) + bnxt;
      pend = real ? bt[2] : pend;
    }
  };
  auto stepB = [&](const float (&s)[8], float& w0, float& w1, bool real) __attribute__((always_inline)) {
    static_for<kOpsB>([&](auto O) { opB(O, s, w0, w1, real); });
  };
  float pt[4], p_[8];
  // cb: first row of the step; edge: some of its rows are past the last one the token attends (their probability is 0)
  auto opA = [&](auto I, const float (&s)[8], vec8_t<T>& pb, int cb, bool edge) __attribute__((always_inline)) {   // kOpsA operations
    constexpr int i = decltype(I)::value;
    if constexpr (i < 8) { p_[i] = fmaf(s[i], c_attn, off_a); pin(p_[i]); }
    else if constexpr (i < 16) { p_[i - 8] = fast_exp2(p_[i - 8]); pin(p_[i - 8]); }
    else if constexpr (i == 16) {
      if (edge) {
#pragma unroll
        for (int k = 0; k < 8; ++k)
          if (cb + 8 * g + k > hi) p_[k] = 0.f;
      }
    }
    else if constexpr (i < 21) { pt[i - 17] = p_[2 * (i - 17)] + p_[2 * (i - 17) + 1]; pin(pt[i - 17]); }
    else if constexpr (i == 21) { pt[0] += pt[1]; pin(pt[0]); }
    else if constexpr (i == 22) { pt[2] += pt[3]; pin(pt[2]); }
    else if constexpr (i == 23) {
      const float p8 = pt[0] + pt[2];
      grp[0].l += p8;
      if constexpr (kNarrowP) pmax = fmaxf(pmax, p8);
    } else { pb = pack8<T>(p_); }
  };
  // element offset of the fragment that matrix instruction J of a chunk reads (from this lane's piece of the chunk)
  auto frag_off = [](int J) constexpr -> int {
    if (J < 2 * NQ) { const int st = J / NQ, j = J % NQ; return (st * NQ + (j & 1) * NKK + (j >> 1)) * 512; }
    return KPART + (J - 2 * NQ) * 512;             // PV(a): channel tiles 0 .. NV-1, PV(b): NV .. 2 NV-1
  };
  // VIS = true: the token attends rows of the chunk (any chunk may take this body: rows past the sequence end or past
  // the token's last visible row are masked where the flags say so); false: a whole chunk the token does not attend.
  // Out: the window sums of the carried step (wc) and of step a (wa); the scores of step b replace the carried ones.
  auto chunk_piped = [&](auto vis_tag, const T* cf, int c0, bool carried, bool derive, float (&wc)[2], float (&wa)[2]) __attribute__((always_inline)) {
    constexpr bool VIS = decltype(vis_tag)::value;
    constexpr int NM = VIS ? 2 * NQ + 2 * NV : 2 * NQ, GS = NSA_FUSED_GS;
    const bool tail_a = VIS && c0 + 32 > nkeys, tail_b = VIS && c0 + 64 > nkeys;      // rows past the sequence end
    const bool edge_a = c0 + 31 > hi, edge_b = c0 + 63 > hi;                          // rows past the causal limit
    vec8_t<T> ring[2 * GS];
    f32x4_t a0 = {0.f, 0.f, 0.f, 0.f}, a1 = a0, b0 = a0, b1 = a0;
    float sa[8], sb[8];
    vec8_t<T> pa, pbb;
    // fragments are requested GS at a time, GS matrix instructions ahead: one wait per group
    static_for<GS>([&](auto J) { ring[J] = load8(cf + frag_off(J)); });
    static_for<NM>([&](auto Jc) {
      constexpr int J = decltype(Jc)::value;
      if constexpr (J % GS == 0) {
        static_for<GS>([&](auto Kc) {
          constexpr int F = J + GS + decltype(Kc)::value;
          if constexpr (F < NM) ring[F % (2 * GS)] = load8(cf + frag_off(F));
        });
      }
      // the matrix instruction
      if constexpr (J < NQ) {
        if constexpr ((J & 1) == 0) a0 = mma16(ring[J % (2 * GS)], grp[0].q[J >> 1], a0);
        else a1 = mma16(ring[J % (2 * GS)], grp[0].q[J >> 1], a1);
      } else if constexpr (J < 2 * NQ) {
        if constexpr ((J & 1) == 0) b0 = mma16(ring[J % (2 * GS)], grp[0].q[(J - NQ) >> 1], b0);
        else b1 = mma16(ring[J % (2 * GS)], grp[0].q[(J - NQ) >> 1], b1);
      } else if constexpr (J < 2 * NQ + NV) {
        grp[0].o[J - 2 * NQ] = mma16(ring[J % (2 * GS)], pa, grp[0].o[J - 2 * NQ]);
      } else {
        grp[0].o[J - 2 * NQ - NV] = mma16(ring[J % (2 * GS)], pbb, grp[0].o[J - 2 * NQ - NV]);
      }
      // the scores of a step leave the accumulators right after its last matrix instruction
      if constexpr (J == NQ - 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { sa[i] = a0[i]; sa[4 + i] = a1[i]; }
        if constexpr (VIS) {
          if (tail_a) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
              if (c0 + 8 * g + i >= nkeys) sa[i] = kNegInf;
          }
          if (derive && c0 == 0) {                   // the reference: largest score of the first 32 rows
            float mx = sa[0];
#pragma unroll
            for (int i = 1; i < 8; ++i) mx = fmaxf(mx, sa[i]);
            m_i = m_a = colgroup_max(mx);            // finite: row 0 exists
            off_i = -m_i * kLog2e;
            off_a = -m_a * c_attn;
          }
        }
      }
      if constexpr (J == 2 * NQ - 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { sb[i] = b0[i]; sb[4 + i] = b1[i]; }
        if constexpr (VIS) {
          if (tail_b) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
              if (c0 + 32 + 8 * g + i >= nkeys) sb[i] = kNegInf;
          }
        }
      }
      // this slot's share of the vector work
      if constexpr (J < NQ) {                                    // B(carried step)
        static_for<kOpsB>([&](auto O) {
          constexpr int o = decltype(O)::value;
          if constexpr (o >= J * kOpsB / NQ && o < (J + 1) * kOpsB / NQ) opB(O, cs, wc[0], wc[1], carried);
        });
      } else if constexpr (J < 2 * NQ) {                         // A(a) resp. B(a)
        constexpr int K = J - NQ;
        if constexpr (VIS) static_for<kOpsA>([&](auto O) {
          constexpr int o = decltype(O)::value;
          if constexpr (o >= K * kOpsA / NQ && o < (K + 1) * kOpsA / NQ) opA(O, sa, pa, c0, edge_a);
        });
        else static_for<kOpsB>([&](auto O) {
          constexpr int o = decltype(O)::value;
          if constexpr (o >= K * kOpsB / NQ && o < (K + 1) * kOpsB / NQ) opB(O, sa, wa[0], wa[1], true);
        });
      } else if constexpr (J < 2 * NQ + NV) {                    // A(b)
        constexpr int K = J - 2 * NQ;
        static_for<kOpsA>([&](auto O) {
          constexpr int o = decltype(O)::value;
          if constexpr (o >= K * kOpsA / NV && o < (K + 1) * kOpsA / NV) opA(O, sb, pbb, c0 + 32, edge_b);
        });
      } else {                                                   // B(a)
        constexpr int K = J - 2 * NQ - NV;
        static_for<kOpsB>([&](auto O) {
          constexpr int o = decltype(O)::value;
          if constexpr (o >= K * kOpsB / NV && o < (K + 1) * kOpsB / NV) opB(O, sa, wa[0], wa[1], true);
        });
      }
      if constexpr (J % GS == GS - 1) __builtin_amdgcn_sched_barrier(0);
    });
#pragma unroll
    for (int i = 0; i < 8; ++i) cs[i] = sb[i];
  };

  auto run_pass = [&](bool derive) __attribute__((always_inline)) {
    if (c_end > 0) stage_chunk(0, 0, true);        // the first chunk always runs the visible schedule
    staged();
    int buf = 0;
    cslot = -1;
    // 512 rows = 16 steps = 32 slots per section: inside a section the slots of one register block are written
    // in place with a scalar index
    auto section = [&](auto put, int c_first) __attribute__((always_inline)) {
      const int c_stop = min(c_first + 512, c_end);
      for (int c0 = c_first; c0 < c_stop; c0 += 64) {
        const int cn = c0 + 64;
        // values only where a wavefront runs the visible schedule: chunks some token attends, and a tail chunk
        if (cn < c_end) stage_chunk(cn, buf ^ 1, cn <= attn_end || cn + 64 > nkeys);
        const T* kf = ldsC + buf * CHUNK + lane * 8;
        const int slot = (c0 - c_first) >> 4;
        // nothing carried (first chunk of a section, or after a chunk of one step): a stand-in that writes zeros
        // to this chunk's first two slots, which the chunk's step a overwrites below
        const int slot_c = cslot >= 0 ? cslot : slot;
        const bool carried = cslot >= 0 && creal;
        if (cslot < 0) {
#pragma unroll
          for (int i = 0; i < 8; ++i) cs[i] = kNegInf;
        }
        float wc[2], wa[2];
        if (c0 > hi && c0 > 0 && cn <= nkeys) chunk_piped(std::false_type{}, kf, c0, carried, derive, wc, wa);
        else chunk_piped(std::true_type{}, kf, c0, carried, derive, wc, wa);
        // step b is carried; in a chunk of one step it is rows past the end (scores -inf, sums 0) and only its
        // zeros are written -- `pend` must keep the last real step's quad
        cslot = slot + 2;
        creal = c0 + 32 < c_end;
        put(slot_c, wc[0], wc[1]);
        put(slot, wa[0], wa[1]);
        staged();
        buf ^= 1;
      }
      // The step carried out of the section's last chunk belongs to this section's slots.  Nothing carried (the
      // sequence ends before this section): zeros into slot 0 of a section that no window uses.
      const bool carried = cslot >= 0 && creal;
      const int slot_c = cslot >= 0 ? cslot : 0;
      if (cslot < 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) cs[i] = kNegInf;
      }
      float wc[2];
      stepB(cs, wc[0], wc[1], carried);
      put(slot_c, wc[0], wc[1]);
      cslot = -1;
    };
    section([&](int s, float x0, float x1) { bq0[s] = x0; bq0[s + 1] = x1; }, 0);
    section([&](int s, float x0, float x1) { bq1[s] = x0; bq1[s + 1] = x1; }, 512);
    section([&](int s, float x0, float x1) { bq2[s] = x0; bq2[s + 1] = x1; }, 1024);
    section([&](int s, float x0, float x1) { binl[64 * s] = x0; binl[64 * s + 64] = x1; }, 1536);
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
      if (c_end > 0) stage_chunk(0, 0, false);
      staged();
      int buf = 0;
      for (int c0 = 0; c0 < c_end; c0 += 64) {
        if (c0 + 64 < c_end) stage_chunk(c0 + 64, buf ^ 1, false);
        const T* kf = ldsC + buf * CHUNK + lane * 8;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
          const int cb = c0 + 32 * sub;
          if (cb >= c_end) break;
          float s[8];
          scores(kf + sub * 2 * NKK * 512, s);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int key = cb + 8 * g + i;
            if (key < nkeys) mx_all = fmaxf(mx_all, s[i]);
            if (key <= hi) mx_vis = fmaxf(mx_vis, s[i]);
          }
        }
        staged();
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

  // ---- attention output: rows leave through LDS (the chunk buffers are free after the pass's last barrier)
  constexpr int OLD = DV + 8, PIECES = DV / 8;
  static_assert(NW * 16 * OLD * sizeof(T) + NW * 1024 <= 2 * CHUNK * sizeof(T),
                "output staging and the top-n shortlists must fit the chunk buffers");
  {
    T* stage = ldsC + wave * 16 * OLD;
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
  // 1 / rows of window `bin`: 5, fewer for the windows that reach past the sequence's last row
  auto window_rcp = [&](int bin) -> float {
    const int len = min(4 * bin + 5, nkeys) - 4 * bin;
    return len >= 5 ? 0.2f : len == 4 ? 0.25f : len == 3 ? (1.0f / 3.0f) : len == 2 ? 0.5f : 1.0f;
  };
  float v[9];
  int ix[9];
  {
    const float w = (rm.valid && lit > 0.f) ? 1.0f / lit : 0.f;     // padded heads weigh nothing
    float x[128];
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      x[i] = bq0[i] * w; x[32 + i] = bq1[i] * w; x[64 + i] = bq2[i] * w; x[96 + i] = binl[64 * i] * w;
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
      v[k] = ok ? r8[k] * window_rcp(bin) : -1.f;
      ix[k] = ok ? bin : 0x7fffffff;
    }
    // the 129th value: the last step's upper window of lane row 3 (no next row), owned by lane (n = 0, g = 3)
    float tail = last_row ? pend * w : 0.f;
    tail += dpp_f32<0xB1>(tail);
    tail += dpp_f32<0x4E>(tail);
    tail += dpp_f32<0x141>(tail);
    tail += dpp_f32<0x140>(tail);
    {
      const int bin = 8 * steps - 1;
      const bool ok = last_row && n == 0 && steps > 0 && bin < Ns;
      v[8] = ok ? tail * window_rcp(bin) : -1.f;
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
  float* cand_v = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(ldsC) + NW * 16 * OLD * sizeof(T)) + wave * 256;
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
         a.frag != nullptr && a.o != nullptr &&
         ((a.dk == 64 && a.dv == 64) || (a.dk == 128 && a.dv == 128) || (a.dk == 192 && a.dv == 128));
}

// chunk slots per kv head of the fragment-major copy for `total_rows` compressed rows in `batch` sequences
int cmp_frag_chunks(int total_rows, int batch) { return total_rows / 64 + batch + 1; }

template <typename T, int DK, int DV>
static int launch_cmp_select_t(const CmpArgs& a, hipStream_t st) {
  const size_t smem = 2 * (size_t)64 * (DK + DV) * sizeof(T) + 8 * 32 * 64 * sizeof(float);
  auto fn = cmp_select_kernel<T, DK, DV>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  const int tiles = a.total / 8 + a.batch;
  hipLaunchKernelGGL(fn, dim3(tiles, a.hkv), dim3(512), smem, st, a);
  return 0;
}

template <typename T, int DK, int DV>
static int launch_frag_pack_t(const CmpArgs& a, long cv_row_stride, long cv_head_stride, int rows_bound, hipStream_t st) {
  const int tiles = rows_bound / 64 + a.batch;
  hipLaunchKernelGGL((frag_pack_kernel<T, DK, DV>), dim3(tiles, a.hkv), dim3(256), 0, st,
                     reinterpret_cast<const T*>(a.ck), reinterpret_cast<const T*>(a.cvt),
                     reinterpret_cast<T*>(const_cast<void*>(a.frag)), a.cu_cmp, a.batch, a.ck_row_stride,
                     a.ck_head_stride, cv_row_stride, cv_head_stride, a.frag_chunks);
  return 0;
}

#define NSA_FUSED_DISPATCH(FN, ...)                                                   \
  do {                                                                                \
    const int key = a.dk * 1000 + a.dv;                                               \
    if (a.dtype == 0) {                                                               \
      switch (key) {                                                                  \
        case 64064: return FN<bf16_t, 64, 64>(__VA_ARGS__);                           \
        case 128128: return FN<bf16_t, 128, 128>(__VA_ARGS__);                        \
        case 192128: return FN<bf16_t, 192, 128>(__VA_ARGS__);                        \
        default: return -2;                                                           \
      }                                                                               \
    }                                                                                 \
    if (a.dtype == 2) {                                                               \
      switch (key) {                                                                  \
        case 64064: return FN<f16_t, 64, 64>(__VA_ARGS__);                            \
        case 128128: return FN<f16_t, 128, 128>(__VA_ARGS__);                         \
        case 192128: return FN<f16_t, 192, 128>(__VA_ARGS__);                         \
        default: return -2;                                                           \
      }                                                                               \
    }                                                                                 \
    return -2;                                                                        \
  } while (0)

int launch_cmp_select(const CmpArgs& a, hipStream_t st) { NSA_FUSED_DISPATCH(launch_cmp_select_t, a, st); }

// a.ck / a.cvt: the row-major compressed keys / VALUES (cv, not its transpose: rows at cv_row_stride, heads at
// cv_head_stride), a.frag: the destination, a.frag_chunks: its chunk slots per head
int launch_frag_pack(const CmpArgs& a, long cv_row_stride, long cv_head_stride, int rows_bound, hipStream_t st) {
  NSA_FUSED_DISPATCH(launch_frag_pack_t, a, cv_row_stride, cv_head_stride, rows_bound, st);
}

}  // namespace nsa
