// Backward of the three attention branches (reference: nsa/triton_attention.py:184-416,478-546 for
// the compressed branch, nsa/selection_attn.py:151-398,520-676 for the selected and sliding
// branches).  Given dO, the forward's O and log-sum-exp per row:
//   delta = rowsum(dO * O),  P = exp(scale*S - lse),  dP = dO V^T,  dS = P * (dP - delta)
//   dV = P^T dO,  dK = scale * dS^T Q,  dQ = scale * dS K
//
// Two kernel shapes, both built on 16x16x32 MFMA tiles and the fragment convention of tiles.h:
//
//  * key-stationary (dK, dV): a wavefront keeps 16 keys as B operands (K rows for S = Q K^T, V rows
//    for dP = dO V^T) and its dK^T / dV^T accumulators in registers; query rows stream through LDS in
//    chunks of 32 rows (2 tokens x 16 heads of the GQA group), Q and dO row-major.  The score tile
//    comes out with lane = key, registers = rows, which after the 8-row permutation of tiles.h is
//    directly the B operand of dV^T = dO^T P and dK^T = Q^T dS.  Their A operands (Q^T, dO^T: rows =
//    channels, depth = query rows) are read from the same row-major LDS tiles with the transposing
//    LDS load of gfx950 (ds_read_b64_tr_b16), so no transposed copy of Q or dO exists anywhere.
//    The three branches differ only in which tokens stream past a key tile: the tokens of a window
//    (sliding), all later tokens in segments (compressed), the tokens that picked the block
//    (selected, from the bucketed pair list of the block-major forward).  dK / dV go to fp32 buffers:
//    plain stores in the window mode (one work item per key tile), atomics in the other two.
//    The selected branch also produces dQ here: dS goes through LDS to become a B operand with
//    lane = query row, and dQ^T = K^T dS^T is written as one partial per (token, pick) pair, summed
//    per token by slc_dq_merge_kernel.
//
//  * query-stationary (dQ of the compressed and sliding branches): a wavefront keeps one token's 16
//    heads (Q and dO rows as B operands, dQ^T accumulators); keys stream through LDS in chunks of 32
//    (K and V row-major; K^T for dQ^T = K^T dS^T again through the transposing load).
#include "slc_ws.h"
#include "tiles.h"

namespace nsa {

int set_smem(const void* fn, size_t bytes);

constexpr int kBwdCmp = 0, kBwdSwa = 1, kBwdSlc = 2;
// Launch shapes, chosen by measurement on T = 32768, Hq64/Hkv4, Dk192/Dv128:
constexpr int kCmpSplit = 512;       // tokens of one compressed-branch work item (1024: 8.6 ms, 256: 5.4 ms; with conflict-free
                                     // LDS the whole backward call: 128: 9.48, 256: 7.89, 320: 7.87, 384: 7.71, 448: 7.68, 512: 7.75;
                                     // with the XCD-aware order 256: 7.25, 384: 7.2-7.4, 512: 7.07, 768: 7.74, 1024: 7.40)
constexpr int kXcds = 8;             // accelerator dies; workgroup w of a launch runs on die w % 8
constexpr int kKvWaves = 4;          // key-stationary: wavefronts (x16 keys) per workgroup, two workgroups per CU
constexpr int kQWaves = 12;          // query-stationary: tokens per workgroup = wavefronts, kQWaves / 4 per SIMD (8: 3.7 ms;
                                     // 16: 3.3 ms at 128 registers with the staged chunk spilled; 12: 170 registers, nothing
                                     // spilled, compressed / sliding calls 0.7 % / 3 % faster than 16)
constexpr int kSegGroup = 4;         // selected branch: consecutive 64-pair segments of a block per workgroup

struct BwdArgs {
  const void* q; const void* d_o; const float* lse; const float* delta;    // rows: [total][hq][.]
  const float* rowscale;          // optional [total][hq]: the branch's gate g; folded into the row statistics
                                  // (lse - ln|g| scales P and dS, sign(g) flips delta and the dO rows)
  const void* k; const void* v;                                          // keys: [key rows][hkv][.]
  const int32_t* cu_seq; const int32_t* cu_key;
  int batch, total, hq, hkv;
  int block, stride, causal, window;
  float scale;
  void* dq;                       // query-stationary: [total][hq][dk]
  float* dk_acc; float* dv_acc;   // key-stationary: fp32 [key rows][hkv][.]
  SlcWs ws;                       // selected branch: bucketed pairs; ws.po = dq partials [pair][16][dk]
  int slc_width;                  // selected branch: keys of a 64-key block one pair attends (the selection block
                                  // size when that is below 64, where ws.sub holds the pair's first key)
  int tiles, items;               // key-stationary launch: key tiles, token items (compressed branch)
};

// Two LDS layouts of a 32-row chunk.  X32: rows padded by 32 bytes, row ownership of lane_row32; no bank
// conflicts on either kind of read.  Otherwise: rows padded by 8 elements, lane group g owns rows 8g .. 8g+7
// (two-way conflicts on most reads).  The selected-block mode keeps the second one: it is bound by its global
// traffic, and with the first layout it measured 5 % slower although its LDS time halved.
template <typename T, bool X32> constexpr int kLdsPad = X32 ? 32 / (int)sizeof(T) : 8;
template <bool X32> __device__ __forceinline__ int chunk_row(int g, int j) { return X32 ? lane_row32(g, j) : 8 * g + j; }
template <bool X32, typename T> __device__ __forceinline__ vec8_t<T> chunk_tr(const T* tile, int ld, int lane) {
  if constexpr (X32) return load8_tr32(tile, ld, lane);
  else return load8_tr(tile, ld, lane);
}

// Two 16-row tiles of X[32 rows][D] (LDS) times the stationary fragments f[D/32]; lane group g receives the
// rows lane_row32(g, 0..7).
template <typename T, int D, bool X32>
__device__ __forceinline__ void tile_pair(const T* __restrict__ x, int ld, int n, int g, const vec8_t<T> (&f)[D / 32],
                                          float (&out)[8]) {
  f32x4_t t0 = {0.f, 0.f, 0.f, 0.f}, t1 = {0.f, 0.f, 0.f, 0.f};
  const T* r0 = x + (X32 ? tile_row32(0, n) : chunk_key_of_row(0, n)) * ld + 8 * g;
  const T* r1 = r0 + (X32 ? 8 : 4) * ld;
#pragma unroll
  for (int kk = 0; kk < D / 32; ++kk) {
    t0 = mma16(load8(r0 + 32 * kk), f[kk], t0);
    t1 = mma16(load8(r1 + 32 * kk), f[kk], t1);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) { out[i] = t0[i]; out[4 + i] = t1[i]; }
}

__device__ __forceinline__ void store4(bf16_t* p, const f32x4_t& v, float s) {
  typedef __bf16 bf16x4v __attribute__((ext_vector_type(4)));
  bf16x4v r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = (bf16_t)(v[i] * s);
  *reinterpret_cast<bf16x4v*>(p) = r;
}
__device__ __forceinline__ void store4(f16_t* p, const f32x4_t& v, float s) {
  typedef _Float16 f16x4v __attribute__((ext_vector_type(4)));
  f16x4v r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = (f16_t)(v[i] * s);
  *reinterpret_cast<f16x4v*>(p) = r;
}
__device__ __forceinline__ void store4(float* p, const f32x4_t& v, float s) {
  f32x4_t r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = v[i] * s;
  *reinterpret_cast<f32x4_t*>(p) = r;
}

// ---- key-stationary: dK, dV (and the dQ partials of the selected branch) ---------------------------

// Two wavefronts per SIMD: left alone the compiler takes 264 registers (one wavefront per SIMD); a budget of
// 168 (three) spills the accumulators and more than doubles the run time.
// TP: tokens (selected mode: pairs of the block's list) per 16 rows of a chunk for GQA groups of at most 16 / TP
// heads; row r of a chunk is head r % GP of the chunk's token or pair r / GP (GP = 16 / TP, TPC = 2 * TP per chunk).
template <typename T, int DK, int DV, int MODE, int NW, int TP = 1>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
bwd_kv_kernel(const BwdArgs a) {
  constexpr bool X32 = MODE != kBwdSlc;
  constexpr int GP = 16 / TP, TPC = 2 * TP;
  constexpr int QLD = DK + kLdsPad<T, X32>, OLD = DV + kLdsPad<T, X32>, NT = NW * 64, SLD = kBlk + 8;
  constexpr int QP = 32 * DK / 8, OP = 32 * DV / 8;                 // 16-byte pieces of one chunk
  constexpr int QPT = (QP + NT - 1) / NT, OPT = (OP + NT - 1) / NT;
  constexpr int STAGE = 32 * QLD + 32 * OLD;
  static_assert(MODE != kBwdSlc || NW * 16 == kBlk, "the selected branch keeps one 64-key block per workgroup");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* lds = reinterpret_cast<T*>(smem_raw);                          // [2][Q 32 x QLD | dO 32 x OLD]
  float* stat = reinterpret_cast<float*>(lds + 2 * STAGE);          // [2][lse2 32 | delta 32]
  T* kblk = reinterpret_cast<T*>(stat + 128);                       // selected branch: K block [64][QLD]
  T* dsl = kblk + kBlk * QLD;                                       //                  dS [32][SLD]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv;

  // ---- work item
  int h, seq_start, key0, nkeys, key_base;
  int t_begin = 0, t_end = 0, first = 0, count = 0, nchunks, rot = 0;
  if (MODE == kBwdSlc) {
    const int item = blockIdx.x;
    if (item >= *a.ws.n_items) return;
    const int key = a.ws.items[2 * item], seg = a.ws.items[2 * item + 1];
    if (seg % kSegGroup != 0) return;         // the workgroup of segment 4i also takes 4i+1 .. 4i+3
    h = key / a.ws.nb;
    const SeqTile st = find_tile(a.cu_seq, a.batch, kBlk, key % a.ws.nb);
    if (!st.valid) return;
    seq_start = st.start; key0 = st.t0; nkeys = st.len; key_base = st.start;
    first = a.ws.offsets[key] + seg * kSeg;
    count = min(a.ws.counts[key] - seg * kSeg, kSegGroup * kSeg);
    nchunks = (count + TPC - 1) / TPC;
  } else if (MODE == kBwdSwa) {
    // Workgroup w runs on XCD w % 8 (each XCD has its own L2).  Neighbouring key tiles stream almost the same
    // tokens (a 64-key tile and its 512-token window), so every XCD takes a contiguous run of key tiles: the
    // q / dO rows its resident workgroups stream are then fetched into that L2 once, not once per key tile.
    const int per_xcd = (a.tiles + kXcds - 1) / kXcds;
    const int xcd = blockIdx.x % kXcds, s = blockIdx.x / kXcds;
    h = s / per_xcd;
    const int tile = xcd * per_xcd + s % per_xcd;
    if (tile >= a.tiles) return;
    const SeqTile st = find_tile(a.cu_seq, a.batch, NW * 16, tile);
    if (!st.valid) return;
    seq_start = st.start; key0 = st.t0; nkeys = st.len; key_base = st.start;
    t_begin = key0;
    t_end = min(key0 + NW * 16 + a.window - 1, st.len);
    nchunks = (t_end - t_begin + TPC - 1) / TPC;
    // The key tiles resident on an XCD are 64 tokens apart, so in plain order tile i would stream a token 32
    // chunks after tile i + 1 did, long after it left the L2.  A full window spans `period` chunks and so holds
    // every chunk number modulo `period` once: each tile starts at its multiple of `period` and wraps around,
    // which makes the workgroups that run side by side stream the same tokens at the same time.
    const int period = (NW * 16 + a.window + TPC - 1) / TPC;
    rot = (period - (t_begin / TPC) % period) % period;
    if (rot >= nchunks) rot = 0;
  } else {
    // The same idea for the compressed branch: all key tiles of one token item stream the same q / dO rows,
    // so inside an XCD the key tile runs fastest and the token items are dealt to the XCDs round-robin.
    const int xcd = blockIdx.x % kXcds, s = blockIdx.x / kXcds;
    const int kt = s % a.tiles;
    const int per_xcd = (a.items + kXcds - 1) / kXcds;
    const int ti_local = (s / a.tiles) % per_xcd;
    h = s / (a.tiles * per_xcd);
    const int ti = ti_local * kXcds + xcd;
    if (ti >= a.items) return;
    const SeqTile st = find_tile(a.cu_key, a.batch, NW * 16, kt);
    if (!st.valid) return;
    key0 = st.t0; nkeys = st.len; key_base = st.start;
    seq_start = a.cu_seq[st.b];
    const int seq_len = a.cu_seq[st.b + 1] - seq_start;
    const int t_first = a.causal ? key0 * a.stride + a.block : 0;
    t_begin = max(ti * kCmpSplit, t_first) & ~(TPC - 1);
    t_end = min((ti + 1) * kCmpSplit, seq_len);
    if (t_begin >= t_end) return;
    nchunks = (t_end - t_begin + TPC - 1) / TPC;
  }
  if (nchunks <= 0) return;

  const T* qb = reinterpret_cast<const T*>(a.q);
  const T* dob = reinterpret_cast<const T*>(a.d_o);

  // Tokens of chunk c, as positions inside the sequence.  Window and compressed modes: `pos`, the chunk's first
  // token.  Selected branch: the chunk holds TPC pairs of the list, pair u in rows u * GP .. (its GQA group), and
  // lane l carries the word of pair l % TPC: 64 x the position of its token (the last pair's again past the end
  // of the list) + the first key it sees inside the block (selection blocks below 64 keys: a pair sees keys
  // [sub, sub + slc_width) of the block).  pair_word hands a lane the word of any pair of the chunk.
  const bool parts = MODE == kBwdSlc && a.slc_width < kBlk;
  auto chunk_first = [&](int c) -> int {
    if (MODE == kBwdSwa) { c += rot; if (c >= nchunks) c -= nchunks; }
    return t_begin + TPC * c;
  };

  // ---- stationary fragments: 16 keys of this wavefront
  const int keypos = key0 + 16 * wave + n;
  const bool keyvalid = keypos < nkeys;
  vec8_t<T> kf[DK / 32], vf[DV / 32];
  {
    const long krow = (long)(key_base + min(keypos, nkeys - 1)) * a.hkv + h;
    const T* kp = reinterpret_cast<const T*>(a.k) + krow * DK + 8 * g;
    const T* vp = reinterpret_cast<const T*>(a.v) + krow * DV + 8 * g;
#pragma unroll
    for (int kk = 0; kk < DK / 32; ++kk) kf[kk] = load8(kp + 32 * kk);
#pragma unroll
    for (int kk = 0; kk < DV / 32; ++kk) vf[kk] = load8(vp + 32 * kk);
  }
  if (MODE == kBwdSlc) {                      // the whole block row-major, for dQ^T = K^T dS^T
    for (int p = tid; p < kBlk * DK / 8; p += NT) {
      const int r = p / (DK / 8), pc = p % (DK / 8);
      const long krow = (long)(key_base + min(key0 + r, nkeys - 1)) * a.hkv + h;
      store8(kblk + r * QLD + pc * 8, load8(reinterpret_cast<const T*>(a.k) + krow * DK + pc * 8));
    }
  }
  f32x4_t dk_acc[DK / 16], dv_acc[DV / 16];
#pragma unroll
  for (int t = 0; t < DK / 16; ++t) dk_acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < DV / 16; ++t) dv_acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // ---- staging of one chunk: global -> registers -> LDS
  vec8_t<T> qr[QPT], orr[OPT];
  float ors[OPT], sr = 0.f, srs = 1.f;       // the gates of the staged rows (1 without a.rowscale)
#pragma unroll
  for (int i = 0; i < OPT; ++i) ors[i] = 1.f;
  // token (position in the sequence, clamped to the last one of the work item) and head of row r of a chunk
  auto pair_word = [&](int words, int u) -> int { return __builtin_amdgcn_ds_bpermute(u << 2, words); };
  auto row_tok = [&](int r, int pos, int words) -> int {
    if (MODE == kBwdSlc) return pair_word(words, r / GP) >> 6;
    return min(pos + r / GP, t_end - 1);
  };
  auto row_head = [&](int r) -> int { return min(r % GP, G - 1); };
  auto gload = [&](int pos, int words) {
#pragma unroll
    for (int i = 0; i < QPT; ++i) {
      const int p = tid + i * NT;
      if (QP % NT == 0 || p < QP) {
        const int r = p / (DK / 8), pc = p % (DK / 8);
        const long tg = seq_start + row_tok(r, pos, words);
        qr[i] = load8(qb + (tg * a.hq + h * G + row_head(r)) * DK + pc * 8);
      }
    }
#pragma unroll
    for (int i = 0; i < OPT; ++i) {
      const int p = tid + i * NT;
      if (OP % NT == 0 || p < OP) {
        const int r = p / (DV / 8), pc = p % (DV / 8);
        const long tg = seq_start + row_tok(r, pos, words);
        const long row = tg * a.hq + h * G + row_head(r);
        orr[i] = load8(dob + row * DV + pc * 8);
        if (a.rowscale != nullptr) ors[i] = a.rowscale[row];       // used in lstore: nothing here waits for a load
      }
    }
    if (tid < 64) {
      const int r = tid & 31;
      const long tg = seq_start + row_tok(r, pos, words);
      const long row = tg * a.hq + h * G + row_head(r);
      sr = tid < 32 ? a.lse[row] : a.delta[row];
      if (a.rowscale != nullptr) srs = a.rowscale[row];
    }
  };
  auto lstore = [&](int buf) {
    T* qs = lds + buf * STAGE;
    T* os = qs + 32 * QLD;
#pragma unroll
    for (int i = 0; i < QPT; ++i) {
      const int p = tid + i * NT;
      if (QP % NT == 0 || p < QP) store8(qs + (p / (DK / 8)) * QLD + (p % (DK / 8)) * 8, qr[i]);
    }
#pragma unroll
    for (int i = 0; i < OPT; ++i) {
      const int p = tid + i * NT;
      if (OP % NT == 0 || p < OP)
        store8(os + (p / (DV / 8)) * OLD + (p % (DV / 8)) * 8, ors[i] < 0.f ? -orr[i] : orr[i]);
    }
    // fold the gate g of a row: lse - ln|g| scales P and dS, sign(g) flips delta and (above) the dO row
    if (tid < 32) stat[buf * 64 + tid] = sr * kLog2e - __log2f(fabsf(srs));
    else if (tid < 64) stat[buf * 64 + tid] = srs < 0.f ? -sr : sr;
  };

  const float c_attn = a.scale * kLog2e;
  // Token positions are carried in registers: pos / words = chunk c, nxt / nwords = chunk c + 1.
  int pos = 0, nxt = 0, words = 0, nwords = 0;
  // selected mode: lane l reads the pair-list entry of the chunk's pair l % TPC (the last entry of the list for
  // pairs past its end) a chunk before its word is formed from it: the load is waited for where its value is
  // first used, not where it is issued.
  unsigned aftv = 0, afts = 0;
  auto list_entry = [&](int c) { return a.ws.list[first + min(TPC * c + (lane & (TPC - 1)), count - 1)]; };
  auto sub_entry = [&](int c) { return (unsigned)a.ws.sub[first + min(TPC * c + (lane & (TPC - 1)), count - 1)]; };
  auto word_of = [&](unsigned v, unsigned sb) -> int { return (int)(((v >> 6) - (unsigned)seq_start) << 6 | sb); };
  if (MODE == kBwdSlc) {
    words = word_of(list_entry(0), parts ? sub_entry(0) : 0u);
    if (nchunks > 1) nwords = word_of(list_entry(1), parts ? sub_entry(1) : 0u);
    if (nchunks > 2) {
      aftv = list_entry(2);
      if (parts) afts = sub_entry(2);
    }
  } else {
    pos = chunk_first(0);
    if (nchunks > 1) nxt = chunk_first(1);
  }
  gload(pos, words);
  lstore(0);
  __syncthreads();
  int buf = 0;
  for (int c = 0; c < nchunks; ++c) {
    // The last iteration stages its own chunk once more instead of branching around the loads and the LDS
    // stores: with both unconditional the compiler knows that nothing is in flight at the top of the loop and
    // puts no wait there (one that would also cover the dQ partial stores just issued).
    const bool has_next = c + 1 < nchunks;
    gload(has_next ? nxt : pos, has_next ? nwords : words);

    const T* qs = lds + buf * STAGE;
    const T* os = qs + 32 * QLD;
    const float* ss = stat + buf * 64;
    // the 8 rows of this lane: chunk_row(g, 0..3) are heads of one token, chunk_row(g, 4..7) of one token (the
    // same one unless tokens share the 16 rows of a tile)
    bool vis, vis_hi;
    const int left = count - TPC * c;         // selected branch: pairs from this chunk's first one to the end of the list
    if (MODE == kBwdSlc) {
      auto sees = [&](int u) -> bool {        // pair u of the chunk
        const int w = pair_word(words, u);
        bool ok = keyvalid && u < left && keypos <= (w >> 6);
        if (parts) ok = ok && (unsigned)(keypos - key0 - (w & 63)) < (unsigned)a.slc_width;
        return ok;
      };
      vis = sees(chunk_row<X32>(g, 0) / GP);
      vis_hi = GP >= 8 ? vis : sees(chunk_row<X32>(g, 4) / GP);
    } else {
      auto sees = [&](int tokpos) -> bool {
        bool v = keyvalid && tokpos < t_end;
        if (MODE == kBwdSwa) v = v && keypos <= tokpos && keypos > tokpos - a.window;
        else if (a.causal) v = v && keypos * a.stride + a.block <= tokpos;
        return v;
      };
      vis = sees(pos + chunk_row<X32>(g, 0) / GP);
      vis_hi = sees(pos + chunk_row<X32>(g, 4) / GP);
    }

    float s[8], dp[8], p[8], ds[8];
    if (MODE == kBwdSlc) {                    // K fragments from the block copy in LDS instead of 24 registers
      vec8_t<T> kl[DK / 32];
#pragma unroll
      for (int kk = 0; kk < DK / 32; ++kk) kl[kk] = load8(kblk + (16 * wave + n) * QLD + 32 * kk + 8 * g);
      tile_pair<T, DK, X32>(qs, QLD, n, g, kl, s);
    } else {
      tile_pair<T, DK, X32>(qs, QLD, n, g, kf, s);
    }
    tile_pair<T, DV, X32>(os, OLD, n, g, vf, dp);
    const int rlo = chunk_row<X32>(g, 0), rhi = chunk_row<X32>(g, 4);
    const f32x4_t l0 = *reinterpret_cast<const f32x4_t*>(ss + rlo);
    const f32x4_t l1 = *reinterpret_cast<const f32x4_t*>(ss + rhi);
    const f32x4_t e0 = *reinterpret_cast<const f32x4_t*>(ss + 32 + rlo);
    const f32x4_t e1 = *reinterpret_cast<const f32x4_t*>(ss + 32 + rhi);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float lse2 = j < 4 ? l0[j & 3] : l1[j & 3];
      const float dl = j < 4 ? e0[j & 3] : e1[j & 3];
      const bool ok = (j < 4 ? vis : vis_hi) && chunk_row<X32>(g, j) % GP < G;
      const float e = fast_exp2(fmaf(s[j], c_attn, -lse2));
      p[j] = ok ? e : 0.f;
      ds[j] = ok ? e * (dp[j] - dl) : 0.f;
    }
    const vec8_t<T> pb = pack8<T>(p), dsb = pack8<T>(ds);
    if (MODE == kBwdSlc) {
#pragma unroll
      for (int j = 0; j < 8; ++j) dsl[chunk_row<X32>(g, j) * SLD + 16 * wave + n] = dsb[j];
      __syncthreads();
    }
#pragma unroll
    for (int t = 0; t < DV / 16; ++t) dv_acc[t] = mma16(chunk_tr<X32>(os + 16 * t, OLD, lane), pb, dv_acc[t]);
#pragma unroll
    for (int t = 0; t < DK / 16; ++t) dk_acc[t] = mma16(chunk_tr<X32>(qs + 16 * t, QLD, lane), dsb, dk_acc[t]);

    // The next chunk goes to LDS before this chunk's dQ partials are stored: the counter that says "the gathers
    // have arrived" also counts stores, in order, so after the stores it would wait for their write round trip.
    lstore(buf ^ 1);
    // aftv (chunk c + 2) was requested an iteration ago; its word is formed here, before the stores below, for the
    // same reason
    const int awords = MODE == kBwdSlc ? word_of(aftv, afts) : 0;
    if (MODE == kBwdSlc) {
      // dQ^T[dk][row] = sum_key K[key][dk] dS[row][key]: this wavefront takes every NW-th 16-channel tile
      T* part = reinterpret_cast<T*>(a.ws.po);
#pragma unroll
      for (int t = wave; t < DK / 16; t += NW) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {       // rows 16r .. 16r + 15 of the chunk: pairs r * TP .. r * TP + TP - 1
          if (r * TP >= left) break;
          f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int step = 0; step < 2; ++step)
            acc = mma16(load8_tr(kblk + 32 * step * QLD + 16 * t, QLD, lane),
                        load8(dsl + (16 * r + n) * SLD + 32 * step + 8 * g), acc);
          const int u = r * TP + n / GP;      // this lane's row: head n % GP of pair u
          if (u < left && n % GP < G)
            store4(part + ((long)(first + TPC * c + u) * 16 + n % GP) * DK + 16 * t + 4 * g, acc, a.scale);
        }
      }
    }

    __syncthreads();
    buf ^= 1;
    pos = nxt; words = nwords;
    if (MODE == kBwdSlc) {
      nwords = awords;
      if (c + 3 < nchunks) {                              // first touched an iteration from here
        aftv = list_entry(c + 3);
        if (parts) afts = sub_entry(c + 3);
      }
    } else if (c + 2 < nchunks) {
      nxt = chunk_first(c + 2);
    }
  }

  if (keyvalid) {
    const long krow = (long)(key_base + keypos) * a.hkv + h;
    float* dkp = a.dk_acc + krow * DK + 4 * g;
    float* dvp = a.dv_acc + krow * DV + 4 * g;
    if (MODE == kBwdSwa) {
      // every key row belongs to exactly one workgroup of this mode: plain stores, which also initialise
      // the accumulators for the selected branch's atomics that follow on the same stream
#pragma unroll
      for (int t = 0; t < DK / 16; ++t) {
        f32x4_t v = dk_acc[t];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] *= a.scale;
        *reinterpret_cast<f32x4_t*>(dkp + 16 * t) = v;
      }
#pragma unroll
      for (int t = 0; t < DV / 16; ++t) *reinterpret_cast<f32x4_t*>(dvp + 16 * t) = dv_acc[t];
    } else {
#pragma unroll
      for (int t = 0; t < DK / 16; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) unsafeAtomicAdd(dkp + 16 * t + i, dk_acc[t][i] * a.scale);
#pragma unroll
      for (int t = 0; t < DV / 16; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) unsafeAtomicAdd(dvp + 16 * t + i, dv_acc[t][i]);
    }
  }
}

// ---- query-stationary: dQ of the compressed and sliding branches -----------------------------------

// kQWaves / 4 wavefronts per SIMD.
// TP tokens share the 16 columns of a wavefront (GQA groups of at most 16 / TP heads: column n = head n % GP of
// token n / GP, GP = 16 / TP); a column's key limits are then per lane.
template <typename T, int DK, int DV, int MODE, int NW, int TP>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW / 4, NW / 4)))
bwd_q_kernel(const BwdArgs a) {
  constexpr int GP = 16 / TP;
  constexpr int KLD = DK + kLdsPad<T, true>, VLD = DV + kLdsPad<T, true>, NT = NW * 64;
  constexpr int KP = 32 * DK / 8, VP = 32 * DV / 8;
  constexpr int KPT = (KP + NT - 1) / NT, VPT = (VP + NT - 1) / NT;
  constexpr int STAGE = 32 * KLD + 32 * VLD;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* lds = reinterpret_cast<T*>(smem_raw);                          // [2][K 32 x KLD | V 32 x VLD]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int G = a.hq / a.hkv;
  // compressed branch: the work of a tile grows with its position, so the last tiles start first
  const int tile_id = MODE == kBwdCmp ? (int)(gridDim.x - 1 - blockIdx.x) : (int)blockIdx.x;
  const SeqTile st = find_tile(a.cu_seq, a.batch, NW * TP, tile_id);
  if (!st.valid) return;
  const int h = blockIdx.y;
  const int hd = n % GP;                                   // head of this lane's column
  const int tok = st.t0 + wave * TP + n / GP;              // its token
  const bool tokvalid = tok < st.len;
  const int t_last = min(st.t0 + NW * TP, st.len) - 1;

  int koff, nkeys;
  if (MODE == kBwdCmp) { koff = a.cu_key[st.b]; nkeys = a.cu_key[st.b + 1] - koff; }
  else { koff = st.start; nkeys = st.len; }
  auto last_visible = [&](int t) -> int {
    if (MODE == kBwdSwa) return t;
    if (!a.causal) return nkeys - 1;
    return t >= a.block ? min((t - a.block) / a.stride, nkeys - 1) : -1;
  };
  const int c_begin = MODE == kBwdSwa ? (max(st.t0 - a.window + 1, 0) & ~31) : 0;
  const int c_end = last_visible(t_last) + 1;
  const int my_hi = tokvalid ? last_visible(tok) : -1;
  const int my_lo = MODE == kBwdSwa ? tok - a.window + 1 : 0;
  // wavefront-uniform limits over its TP tokens
  const int w_tok0 = st.t0 + wave * TP;
  const int w_hi = w_tok0 < st.len ? last_visible(min(w_tok0 + TP - 1, st.len - 1)) : -1;
  const int w_lo = MODE == kBwdSwa ? w_tok0 - a.window + 1 : 0;

  vec8_t<T> qf[DK / 32], dof[DV / 32];
  float lse2, dl;
  {
    const long row = ((long)st.start + min(tok, st.len - 1)) * a.hq + h * G + min(hd, G - 1);
    const T* qp = reinterpret_cast<const T*>(a.q) + row * DK + 8 * g;
    const T* dp = reinterpret_cast<const T*>(a.d_o) + row * DV + 8 * g;
#pragma unroll
    for (int kk = 0; kk < DK / 32; ++kk) qf[kk] = load8(qp + 32 * kk);
#pragma unroll
    for (int kk = 0; kk < DV / 32; ++kk) dof[kk] = load8(dp + 32 * kk);
    lse2 = a.lse[row] * kLog2e;
    dl = a.delta[row];
    if (a.rowscale != nullptr) {            // fold the gate as in the key-stationary kernel
      const float rs = a.rowscale[row];
      lse2 -= __log2f(fabsf(rs));
      if (rs < 0.f) {
        dl = -dl;
#pragma unroll
        for (int kk = 0; kk < DV / 32; ++kk) dof[kk] = -dof[kk];
      }
    }
  }
  f32x4_t acc[DK / 16];
#pragma unroll
  for (int t = 0; t < DK / 16; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const T* kb = reinterpret_cast<const T*>(a.k) + ((long)koff * a.hkv + h) * DK;
  const T* vb = reinterpret_cast<const T*>(a.v) + ((long)koff * a.hkv + h) * DV;
  vec8_t<T> kr[KPT], vr[VPT];
  auto gload = [&](int c0) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int p = tid + i * NT;
      if (KP % NT == 0 || p < KP) {
        const int r = min(c0 + p / (DK / 8), nkeys - 1);
        kr[i] = load8(kb + (long)r * a.hkv * DK + (p % (DK / 8)) * 8);
      }
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int p = tid + i * NT;
      if (VP % NT == 0 || p < VP) {
        const int r = min(c0 + p / (DV / 8), nkeys - 1);
        vr[i] = load8(vb + (long)r * a.hkv * DV + (p % (DV / 8)) * 8);
      }
    }
  };
  auto lstore = [&](int buf) {
    T* ks = lds + buf * STAGE;
    T* vs = ks + 32 * KLD;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int p = tid + i * NT;
      if (KP % NT == 0 || p < KP) store8(ks + (p / (DK / 8)) * KLD + (p % (DK / 8)) * 8, kr[i]);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int p = tid + i * NT;
      if (VP % NT == 0 || p < VP) store8(vs + (p / (DV / 8)) * VLD + (p % (DV / 8)) * 8, vr[i]);
    }
  };

  const float c_attn = a.scale * kLog2e;
  if (c_begin < c_end) {
    gload(c_begin);
    lstore(0);
  }
  __syncthreads();
  int buf = 0;
  for (int c0 = c_begin; c0 < c_end; c0 += 32) {
    const bool has_next = c0 + 32 < c_end;
    if (has_next) gload(c0 + 32);
    if (c0 <= w_hi && c0 + 31 >= w_lo) {             // wavefront uniform
      const T* ks = lds + buf * STAGE;
      const T* vs = ks + 32 * KLD;
      float s[8], dp[8], ds[8];
      tile_pair<T, DK, true>(ks, KLD, n, g, qf, s);
      tile_pair<T, DV, true>(vs, VLD, n, g, dof, dp);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = c0 + lane_row32(g, j);
        const bool ok = key >= my_lo && key <= my_hi && hd < G;
        const float e = fast_exp2(fmaf(s[j], c_attn, -lse2));
        ds[j] = ok ? e * (dp[j] - dl) : 0.f;
      }
      const vec8_t<T> dsb = pack8<T>(ds);
#pragma unroll
      for (int t = 0; t < DK / 16; ++t) acc[t] = mma16(load8_tr32(ks + 16 * t, KLD, lane), dsb, acc[t]);
    }
    if (has_next) lstore(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  if (tokvalid && hd < G) {
    T* dqp = reinterpret_cast<T*>(a.dq) + (((long)st.start + tok) * a.hq + h * G + hd) * DK + 4 * g;
#pragma unroll
    for (int t = 0; t < DK / 16; ++t) store4(dqp + 16 * t, acc[t], a.scale);
  }
}

// ---- small kernels ------------------------------------------------------------------------------

// delta[row] = sum_v o[row][v] * d_o[row][v]; 16 lanes per row
template <typename T>
__global__ void __launch_bounds__(256)
bwd_delta_kernel(const T* __restrict__ o, const T* __restrict__ d_o, float* __restrict__ delta, long rows, int dv) {
  const long row = ((long)blockIdx.x * 256 + threadIdx.x) >> 4;
  const int sub = threadIdx.x & 15;
  float acc = 0.f;
  if (row < rows) {
    for (int c = sub * 8; c < dv; c += 128) {
      const vec8_t<T> x = load8(o + row * dv + c), y = load8(d_o + row * dv + c);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc = fmaf((float)x[i], (float)y[i], acc);
    }
  }
#pragma unroll
  for (int d = 1; d < 16; d <<= 1) acc += __shfl_xor(acc, d, 16);
  if (row < rows && sub == 0) delta[row] = acc;
}

__global__ void __launch_bounds__(256)
bwd_fill_kernel(float* __restrict__ p, long n4) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n4) reinterpret_cast<f32x4_t*>(p)[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
}

template <typename T>
__global__ void __launch_bounds__(256)
bwd_cast_kernel(const float* __restrict__ src, T* __restrict__ dst, long n8) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  float v[8];
  const f32x8_t x = load8(src + i * 8);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = x[e];
  store8(dst + i * 8, pack8<T>(v));
}

// dq[token][head][8 channels] = (dq_in) + (dq_add) + sum over the token's usable picks of the pair partials.
// TOPN > 0: top_n == TOPN, the slot map is read with vector loads and all partials of the piece are
// requested before any is summed; TOPN = 0: any top_n (0 included), in rounds of 16 slots.
template <typename T, int DK, int TOPN>
__global__ void __launch_bounds__(256)
slc_dq_merge_kernel(const SlcArgs s, const int* __restrict__ slotmap, const T* __restrict__ part,
                    const T* __restrict__ dq_in, const T* __restrict__ dq_add, T* __restrict__ dq, int hq, int hkv,
                    int top_n) {
  constexpr int PPR = DK / 8;
  int tb, te;
  slc_token_range(s, tb, te);                       // the tokens of this slab (all of them without slabs)
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  const int pc = (int)(id % PPR);
  const long rel = id / PPR;                        // (token - tb) * hq + head
  const int hq_i = (int)(rel % hq);
  const long tg = tb + rel / hq;
  if (tg >= te) return;
  const long row = tg * hq + hq_i;
  const int G = hq / hkv;
  const int h = hq_i / G, n = hq_i % G;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  vec8_t<T> x0 = zero8<T>(), x1 = zero8<T>();
  if (dq_in != nullptr) x0 = load8(dq_in + row * DK + pc * 8);
  if (dq_add != nullptr) x1 = load8(dq_add + row * DK + pc * 8);
  const long base = (tg * hkv + h) * top_n;
  if constexpr (TOPN > 0) {
    int ps[TOPN];
#pragma unroll
    for (int i = 0; i < TOPN / 4; ++i) {
      const int4 q4 = *reinterpret_cast<const int4*>(slotmap + base + 4 * i);
      ps[4 * i] = q4.x; ps[4 * i + 1] = q4.y; ps[4 * i + 2] = q4.z; ps[4 * i + 3] = q4.w;
    }
    // all of the slot map before the first partial is requested (the conditional loads below would otherwise be
    // split into batches by a wait for the later parts of the map)
#pragma unroll
    for (int i = 0; i < TOPN; ++i) asm volatile("" ::"v"(ps[i]));
    vec8_t<T> x[TOPN];
#pragma unroll
    for (int i = 0; i < TOPN; ++i) {
      x[i] = zero8<T>();
      if (ps[i] >= 0) x[i] = load8(part + ((long)ps[i] * 16 + n) * DK + pc * 8);
    }
#pragma unroll
    for (int i = 0; i < TOPN; ++i)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += (float)x[i][e];
  } else {
    // any top_n: rounds of 16 slots, all partials of a round requested before the first is added
    constexpr int R = 16;
    for (int r0 = 0; r0 < top_n; r0 += R) {
      int ps[R];
#pragma unroll
      for (int i = 0; i < R; ++i) ps[i] = r0 + i < top_n ? slotmap[base + r0 + i] : -1;
#pragma unroll
      for (int i = 0; i < R; ++i) asm volatile("" ::"v"(ps[i]));
      vec8_t<T> x[R];
#pragma unroll
      for (int i = 0; i < R; ++i) {
        x[i] = zero8<T>();
        if (ps[i] >= 0) x[i] = load8(part + ((long)ps[i] * 16 + n) * DK + pc * 8);
      }
#pragma unroll
      for (int i = 0; i < R; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += (float)x[i][e];
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] += (float)x0[e] + (float)x1[e];
  store8(dq + row * DK + pc * 8, pack8<T>(acc));
}

// ---- launchers ------------------------------------------------------------------------------------

template <typename T, int DK, int DV, int MODE, int NW, int TP>
static int launch_kv_impl(const BwdArgs& a, int key_rows, hipStream_t st) {
  constexpr int XP = kLdsPad<T, MODE != kBwdSlc>;
  size_t smem = 2 * (size_t)(32 * (DK + XP) + 32 * (DV + XP)) * sizeof(T) + 128 * sizeof(float);
  if (MODE == kBwdSlc) smem += ((size_t)kBlk * (DK + XP) + 32 * (kBlk + 8)) * sizeof(T);
  auto fn = bwd_kv_kernel<T, DK, DV, MODE, NW, TP>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  dim3 grid;
  BwdArgs b = a;
  b.tiles = key_rows / (NW * 16) + a.batch;
  b.items = (a.total + kCmpSplit - 1) / kCmpSplit;
  const int tiles_per_xcd = (b.tiles + kXcds - 1) / kXcds, items_per_xcd = (b.items + kXcds - 1) / kXcds;
  if (MODE == kBwdSlc) grid = dim3(a.ws.items_cap);
  else if (MODE == kBwdSwa) grid = dim3(kXcds * tiles_per_xcd * a.hkv);
  else grid = dim3(kXcds * b.tiles * items_per_xcd * a.hkv);
  hipLaunchKernelGGL(fn, grid, dim3(NW * 64), smem, st, b);
  return 0;
}

template <typename T, int DK, int DV, int MODE, int NW>
static int launch_kv_t(const BwdArgs& a, int key_rows, hipStream_t st) {
  const int G = a.hq / a.hkv;         // 4 / 2 tokens (selected branch: pairs) per 16 rows for GQA groups of at most 4 / 8 heads
  if (G <= 4) return launch_kv_impl<T, DK, DV, MODE, NW, 4>(a, key_rows, st);
  if (G <= 8) return launch_kv_impl<T, DK, DV, MODE, NW, 2>(a, key_rows, st);
  return launch_kv_impl<T, DK, DV, MODE, NW, 1>(a, key_rows, st);
}

template <typename T, int DK, int DV, int MODE, int TP>
static int launch_q_impl(const BwdArgs& a, hipStream_t st) {
  constexpr int NW = kQWaves;
  const size_t smem = 2 * (size_t)(32 * (DK + kLdsPad<T, true>) + 32 * (DV + kLdsPad<T, true>)) * sizeof(T);
  auto fn = bwd_q_kernel<T, DK, DV, MODE, NW, TP>;
  const int rc = set_smem(reinterpret_cast<const void*>(fn), smem);
  if (rc) return rc;
  hipLaunchKernelGGL(fn, dim3(a.total / (NW * TP) + a.batch, a.hkv), dim3(NW * 64), smem, st, a);
  return 0;
}

template <typename T, int DK, int DV, int MODE>
static int launch_q_t(const BwdArgs& a, hipStream_t st) {
  const int G = a.hq / a.hkv;       // tokens per wavefront: 4 / 2 / 1 for groups of at most 4 / 8 / 16 heads
  return G <= 4 ? launch_q_impl<T, DK, DV, MODE, 4>(a, st)
                : G <= 8 ? launch_q_impl<T, DK, DV, MODE, 2>(a, st) : launch_q_impl<T, DK, DV, MODE, 1>(a, st);
}

static void fill_zero(float* p, long n, hipStream_t st) {        // n is a multiple of 4
  const long n4 = n / 4;
  if (n4 > 0) hipLaunchKernelGGL(bwd_fill_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, st, p, n4);
}
template <typename T>
static void cast_out(const float* src, void* dst, long n, hipStream_t st) {   // n is a multiple of 8
  const long n8 = n / 8;
  if (n8 > 0)
    hipLaunchKernelGGL((bwd_cast_kernel<T>), dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, st, src,
                       reinterpret_cast<T*>(dst), n8);
}
template <typename T>
static void launch_delta(const void* o, const void* d_o, float* delta, long rows, int dv, hipStream_t st) {
  hipLaunchKernelGGL((bwd_delta_kernel<T>), dim3((unsigned)((rows * 16 + 255) / 256)), dim3(256), 0, st,
                     reinterpret_cast<const T*>(o), reinterpret_cast<const T*>(d_o), delta, rows, dv);
}

static long take(long& off, long bytes) { const long o = off; off = slc_align_up(off + bytes, 256); return o; }

// compressed branch -----------------------------------------------------------------------------------

long cmp_bwd_workspace_bytes(const CmpBwdArgs& a) {
  long off = 0;
  take(off, (long)a.total * a.hq * 4);
  take(off, (long)a.cmp_rows * a.hkv * a.dk * 4);
  take(off, (long)a.cmp_rows * a.hkv * a.dv * 4);
  return off;
}

template <typename T, int DK, int DV>
static int launch_cmp_bwd_t(const CmpBwdArgs& c, hipStream_t st) {
  char* base = reinterpret_cast<char*>(c.workspace);
  long off = 0;
  float* delta = (float*)(base + take(off, (long)c.total * c.hq * 4));
  float* dk_acc = (float*)(base + take(off, (long)c.cmp_rows * c.hkv * DK * 4));
  float* dv_acc = (float*)(base + take(off, (long)c.cmp_rows * c.hkv * DV * 4));
  if (c.delta == nullptr) launch_delta<T>(c.o, c.d_o, delta, (long)c.total * c.hq, DV, st);
  BwdArgs a{};
  a.q = c.q; a.d_o = c.d_o; a.lse = c.lse; a.delta = c.delta ? c.delta : delta; a.rowscale = c.rowscale;
  a.k = c.ck; a.v = c.cv;
  a.cu_seq = c.cu_seq; a.cu_key = c.cu_cmp; a.batch = c.batch; a.total = c.total; a.hq = c.hq; a.hkv = c.hkv;
  a.block = c.block; a.stride = c.stride; a.causal = c.causal; a.window = 0; a.scale = c.scale;
  a.dq = c.dq; a.dk_acc = dk_acc; a.dv_acc = dv_acc;
  int rc = launch_q_t<T, DK, DV, kBwdCmp>(a, st);
  if (rc) return rc;
  if (c.cmp_rows > 0) {
    fill_zero(dk_acc, (long)c.cmp_rows * c.hkv * DK, st);
    fill_zero(dv_acc, (long)c.cmp_rows * c.hkv * DV, st);
    rc = launch_kv_t<T, DK, DV, kBwdCmp, kKvWaves>(a, c.cmp_rows, st);
    if (rc) return rc;
    cast_out<T>(dk_acc, c.dck, (long)c.cmp_rows * c.hkv * DK, st);
    cast_out<T>(dv_acc, c.dcv, (long)c.cmp_rows * c.hkv * DV, st);
  }
  return 0;
}

// selected + sliding branches ------------------------------------------------------------------------

static SlcArgs slc_args_of(const SlcSwaBwdArgs& c) {
  SlcArgs s{};
  s.indices = c.indices; s.counts = c.counts; s.cu_seq = c.cu_seq; s.batch = c.batch; s.total = c.total;
  s.hq = c.hq; s.hkv = c.hkv; s.dk = c.dk; s.dv = c.dv; s.top_n = c.top_n; s.block_size = c.block_size;
  s.idx64 = c.idx64; s.dtype = c.dtype;
  return slc_virtual(s);           // top_n counts 64-key slots from here on
}

constexpr int kBwdSlabTile = 64;     // tokens per tile in which the selected branch's token slabs are counted

// selected branch in slabs of `tiles` tiles of kBwdSlabTile tokens (0: all tokens at once)
static SlcArgs slab_args_of(const SlcSwaBwdArgs& c, int tile_begin, int tiles) {
  SlcArgs s = slc_args_of(c);
  s.tile_tokens = kBwdSlabTile; s.tile_begin = tile_begin; s.tile_count = tiles;
  return s;
}

static long bwd_workspace_bytes(const SlcSwaBwdArgs& c, int tiles) {
  long off = 0;
  take(off, (long)c.total * c.hq * 4);
  take(off, (long)c.total * c.hq * 4);
  take(off, (long)c.total * c.hkv * c.dk * 4);
  take(off, (long)c.total * c.hkv * c.dv * 4);
  if (c.top_n > 0) off += slc_carve(slab_args_of(c, 0, tiles), nullptr, nullptr, c.dtype == 1 ? 4 : 2, c.dk);
  return off;
}

long slc_swa_bwd_workspace_bytes(const SlcSwaBwdArgs& c) { return bwd_workspace_bytes(c, 0); }

// slab_tokens <= 0 or >= total: all tokens at once
long slc_swa_bwd_slab_workspace_bytes(const SlcSwaBwdArgs& c, int slab_tokens) {
  const int tiles = slab_tokens > 0 && slab_tokens < c.total ? (slab_tokens + kBwdSlabTile - 1) / kBwdSlabTile : 0;
  return bwd_workspace_bytes(c, tiles);
}

template <typename T, int DK, int DV>
static int launch_slc_swa_bwd_t(const SlcSwaBwdArgs& c, hipStream_t st) {
  char* base = reinterpret_cast<char*>(c.workspace);
  long off = 0;
  float* delta_slc = (float*)(base + take(off, (long)c.total * c.hq * 4));
  float* delta_swa = (float*)(base + take(off, (long)c.total * c.hq * 4));
  float* dk_acc = (float*)(base + take(off, (long)c.total * c.hkv * DK * 4));
  float* dv_acc = (float*)(base + take(off, (long)c.total * c.hkv * DV * 4));
  const bool slc = c.top_n > 0 && c.d_o_slc != nullptr, swa = c.window > 0 && c.d_o_swa != nullptr;
  if (!swa) {                      // the window kernel stores every row of the accumulators itself
    fill_zero(dk_acc, (long)c.total * c.hkv * DK, st);
    fill_zero(dv_acc, (long)c.total * c.hkv * DV, st);
  }
  BwdArgs a{};
  a.q = c.q; a.k = c.k; a.v = c.v; a.cu_seq = c.cu_seq; a.cu_key = c.cu_seq; a.batch = c.batch; a.total = c.total;
  a.hq = c.hq; a.hkv = c.hkv; a.causal = 1; a.window = c.window; a.scale = c.scale;
  a.dq = c.dq; a.dk_acc = dk_acc; a.dv_acc = dv_acc;
  int rc = 0;
  if (swa) {
    if (c.delta_swa == nullptr) launch_delta<T>(c.o_swa, c.d_o_swa, delta_swa, (long)c.total * c.hq, DV, st);
    a.d_o = c.d_o_swa; a.lse = c.lse_swa; a.delta = c.delta_swa ? c.delta_swa : delta_swa;
    a.rowscale = c.rowscale_swa;
    rc = launch_q_t<T, DK, DV, kBwdSwa>(a, st);
    if (rc == 0) rc = launch_kv_t<T, DK, DV, kBwdSwa, kKvWaves>(a, c.total, st);
    if (rc) return rc;
  }
  auto dq_merge = [&](const SlcArgs& s, const SlcWs* ws, long slab_tokens) {   // dq = window dQ + partials + dq_add
    const long threads = slab_tokens * c.hq * (DK / 8);
    const dim3 grid((unsigned)((threads + 255) / 256));
    const int* slotmap = ws ? ws->slotmap : nullptr;
    const T* part = ws ? reinterpret_cast<const T*>(ws->po) : nullptr;
    const T* dq_in = swa ? reinterpret_cast<const T*>(c.dq) : nullptr;
    const int top_n = ws ? s.top_n : 0;                    // slots per (token, head)
    if (top_n == 16)
      hipLaunchKernelGGL((slc_dq_merge_kernel<T, DK, 16>), grid, dim3(256), 0, st, s, slotmap, part, dq_in,
                         reinterpret_cast<const T*>(c.dq_add), reinterpret_cast<T*>(c.dq), c.hq, c.hkv, top_n);
    else
      hipLaunchKernelGGL((slc_dq_merge_kernel<T, DK, 0>), grid, dim3(256), 0, st, s, slotmap, part, dq_in,
                         reinterpret_cast<const T*>(c.dq_add), reinterpret_cast<T*>(c.dq), c.hq, c.hkv, top_n);
  };
  if (slc) {
    if (c.delta_slc == nullptr) launch_delta<T>(c.o_slc, c.d_o_slc, delta_slc, (long)c.total * c.hq, DV, st);
    a.d_o = c.d_o_slc; a.lse = c.lse_slc; a.delta = c.delta_slc ? c.delta_slc : delta_slc;
    a.rowscale = c.rowscale_slc; a.slc_width = min(c.block_size, kBlk);
    // Token slabs: pair list and dQ partials are sized for one slab (the largest the workspace holds); every slab
    // is bucketed, run through the block kernel (dK / dV accumulate over the slabs) and merged into dq before the
    // next one reuses the memory.
    const int total_tiles = c.total / kBwdSlabTile + c.batch;
    int slab_tiles = total_tiles;
    if (bwd_workspace_bytes(c, 0) > c.workspace_bytes) {
      if (bwd_workspace_bytes(c, 1) > c.workspace_bytes) return -6;
      int lo = 1, hi = total_tiles;
      while (lo < hi) {
        const int mid = lo + (hi - lo + 1) / 2;
        if (bwd_workspace_bytes(c, mid) <= c.workspace_bytes) lo = mid; else hi = mid - 1;
      }
      slab_tiles = lo;
    }
    const bool whole = slab_tiles >= total_tiles;
    for (int t0 = 0; t0 < total_tiles; t0 += slab_tiles) {
      const SlcArgs s = slab_args_of(c, t0, whole ? 0 : slab_tiles);
      SlcWs ws{};
      slc_carve(s, base + off, &ws, sizeof(T), DK);
      rc = launch_slc_bucket(s, ws, st);
      if (rc) return rc;
      a.ws = ws;
      rc = launch_kv_t<T, DK, DV, kBwdSlc, 4>(a, c.total, st);
      if (rc) return rc;
      dq_merge(s, &ws, whole ? (long)c.total : std::min((long)slab_tiles * kBwdSlabTile, (long)c.total));
    }
  } else if (c.dq_add != nullptr) {
    dq_merge(slab_args_of(c, 0, 0), nullptr, c.total);
  } else if (!swa) {
    fill_zero(reinterpret_cast<float*>(c.dq), (long)c.total * c.hq * DK * (long)sizeof(T) / 4, st);
  }
  cast_out<T>(dk_acc, c.dk_out, (long)c.total * c.hkv * DK, st);
  cast_out<T>(dv_acc, c.dv_out, (long)c.total * c.hkv * DV, st);
  return 0;
}

#define NSA_BWD_DISPATCH(FN, ARGS, ST)                                                \
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
        default: return -2;                                                           \
      }                                                                               \
    }                                                                                 \
  } while (0)

int launch_cmp_bwd(const CmpBwdArgs& a, hipStream_t st) { NSA_BWD_DISPATCH(launch_cmp_bwd_t, a, st); }
int launch_slc_swa_bwd(const SlcSwaBwdArgs& a, hipStream_t st) { NSA_BWD_DISPATCH(launch_slc_swa_bwd_t, a, st); }

}  // namespace nsa
