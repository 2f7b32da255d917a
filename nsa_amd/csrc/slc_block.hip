// Block-major selected attention (16-bit types; 64-key blocks, and through them selection blocks of 8, 16, 32
// keys — masked parts of a 64-key block — and of 128, 192, ... keys — several 64-key slots per pick).
//
// The token-major kernel gathers every selected K/V block again for every token: 40 KB per
// (token, kv head, block), 43 GB per forward at T = 32k, and a CU cannot pull more than ~15 B/clk
// through its vector L1.  Here the loop is inverted: the (token, pick) pairs are bucketed by
// (kv head, block); a wavefront loads one K/V block into registers as MFMA fragments ONCE and then
// streams the queries that picked it (6 KB each), writing one normalised partial result
// (o / l in bf16, plus max and denominator in fp32) per pair, in pair order.  The merge of the <= top_n partials of every token, the gates and the sum with the other
// two branches happen either in slc_merge_kernel or in the sliding-window kernel's epilogue.  Traffic
// per pair drops from 40 KB to ~10 KB (query in, partial out) + 4 KB (partial back in).
//
// Workspace layout (caller allocated, nsa_slc_workspace_bytes): block bases per sequence, pair counts /
// offsets / cursors per (head, block), work items (head, block, segment of 64 pairs), the bucketed
// pair list, a slot map (token, head, pick) -> pair, and the partial results.
#include "slc_merge.h"
#include "slc_ws.h"

namespace nsa {

int set_smem(const void* fn, size_t bytes);

SlcArgs slc_virtual(const SlcArgs& a) {
  if (a.pick_mult != 0) return a;
  SlcArgs v = a;
  v.pick_mult = a.block_size > kBlk ? a.block_size / kBlk : 1;
  v.top_n = a.top_n * v.pick_mult;
  return v;
}

// a: as returned by slc_virtual
long slc_carve(const SlcArgs& a, void* base, SlcWs* ws, size_t elem, int part_width, int part_rows) {
  const int nb = a.total / kBlk + a.batch;
  const long nkeys = (long)a.hkv * nb;
  const long slots = (long)a.total * a.hkv * a.top_n;                 // slot map: every token
  long slab = a.total;                                               // pair list, partials: the tokens of one slab
  if (a.tile_count > 0 && (long)a.tile_count * a.tile_tokens < slab) slab = (long)a.tile_count * a.tile_tokens;
  const long pairs = slab * a.hkv * a.top_n;
  const int items_cap = (int)(pairs / kSeg + nkeys) + 1;
  long off = 0;
  auto take = [&](long bytes) { const long o = off; off = slc_align_up(off + bytes, 256); return o; };
  const long o_blkbase = take((a.batch + 1) * 4L);
  const long o_counts = take(nkeys * 4);
  const long o_offsets = take(nkeys * 4);
  const long o_cursor = take(nkeys * 4);
  const long o_items = take((long)items_cap * 8);
  const long o_nitems = take(4);
  const long o_list = take(pairs * 4);
  const long o_slot = take(slots * 4);
  const long o_sub = take(pairs);
  const long o_ml = take(pairs * 2 * 16 * 4);
  const long o_po = take(pairs * part_rows * part_width * (long)elem);
  if (ws != nullptr) {
    char* b = reinterpret_cast<char*>(base);
    ws->blkbase = (int*)(b + o_blkbase); ws->counts = (int*)(b + o_counts); ws->offsets = (int*)(b + o_offsets);
    ws->cursor = (int*)(b + o_cursor); ws->items = (int*)(b + o_items); ws->n_items = (int*)(b + o_nitems);
    ws->list = (uint32_t*)(b + o_list); ws->slotmap = (int*)(b + o_slot); ws->ml = (float*)(b + o_ml);
    ws->po = b + o_po; ws->sub = (uint8_t*)(b + o_sub);
    ws->nb = nb; ws->pairs_cap = pairs; ws->items_cap = items_cap;
  }
  return off;
}

static long carve(const SlcArgs& a, void* base, SlcWs* ws, size_t elem) {
  return slc_carve(a, base, ws, elem, a.dv, slc_part_rows(a));
}

long slc_workspace_bytes(const SlcArgs& a) { return carve(slc_virtual(a), nullptr, nullptr, a.dtype == 1 ? 4 : 2); }

// selection blocks the 64-key schedule can express: 8, 16, 32 (parts of a block), 64, 128, 192, ... (whole blocks)
bool slc_block_size_ok(int block_size) {
  return block_size == 8 || block_size == 16 || block_size == 32 || (block_size > 0 && block_size % kBlk == 0);
}

bool slc_block_major_ok(const SlcArgs& a) {
  return a.dtype != 1 && slc_block_size_ok(a.block_size) && slc_virtual(a).top_n <= 64 && a.total < (1 << 26) &&
         ((a.dk == 32 && a.dv == 32) || (a.dk == 64 && a.dv == 64) || (a.dk == 128 && a.dv == 128) ||
          (a.dk == 192 && a.dv == 128));
}

// Slot `i` of (token position t in its sequence, real kv head row th_r): the 64-key block it stands for (local to
// the sequence) or -1 when the slot is unusable (beyond the count, a negative or future block), and the first
// key of the selection block inside that 64-key block.
__device__ __forceinline__ int slc_slot_block(const SlcArgs& a, long th_r, int i, int t, int& sub) {
  const int real_n = a.top_n / a.pick_mult, pick = i / a.pick_mult;
  int cnt = real_n;
  if (a.counts != nullptr) cnt = min(max(a.counts[th_r], 0), real_n);
  const long idx = a.idx64 ? reinterpret_cast<const int64_t*>(a.indices)[th_r * real_n + pick]
                           : (long)reinterpret_cast<const int32_t*>(a.indices)[th_r * real_n + pick];
  sub = 0;
  if (pick >= cnt || idx < 0 || idx > t) return -1;
  const long key0 = idx * a.block_size + (long)(i % a.pick_mult) * kBlk;   // first key of the slot
  if (key0 > t) return -1;
  sub = (int)(key0 % kBlk);
  return (int)(key0 / kBlk);
}

// ---- bucket the pairs ---------------------------------------------------------------------------

__global__ void __launch_bounds__(256)
slc_prep_kernel(const int32_t* __restrict__ cu, int batch, SlcWs ws, int hkv) {
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int b = 0; b < batch; ++b) {
      ws.blkbase[b] = acc;
      acc += (cu[b + 1] - cu[b] + kBlk - 1) / kBlk;
    }
    ws.blkbase[batch] = acc;
    *ws.n_items = 0;
  }
  for (int i = threadIdx.x; i < hkv * ws.nb; i += 256) { ws.counts[i] = 0; ws.cursor[i] = 0; }
}

__device__ __forceinline__ int seq_of_token(const int32_t* __restrict__ cu, int batch, int t) {
  int lo = 0, hi = batch;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}

// FILL = false: count the pairs of every (head, block); FILL = true: place them.
template <bool FILL>
__global__ void __launch_bounds__(256)
slc_bucket_kernel(const SlcArgs a, SlcWs ws) {
  int tb, te;
  slc_token_range(a, tb, te);
  const long rel = (long)blockIdx.x * 256 + threadIdx.x;
  if (rel >= (long)(te - tb) * a.hkv * a.top_n) return;
  const long id = rel + (long)tb * a.hkv * a.top_n;              // (token, head, pick)
  const int i = (int)(id % a.top_n);
  const long th = id / a.top_n;
  const int h = (int)(th % a.hkv), tg = (int)(th / a.hkv);
  const int b = seq_of_token(a.cu_seq, a.batch, tg);
  const int t = tg - a.cu_seq[b];
  const long th_r = (long)tg * (a.hkv / a.kv_rep) + h / a.kv_rep;      // picks and counts are per real kv head
  int sub;
  const int blk = slc_slot_block(a, th_r, i, t, sub);
  if (blk < 0) {
    if (FILL) ws.slotmap[id] = -1;
    return;
  }
  const int key = h * ws.nb + ws.blkbase[b] + blk;
  if (!FILL) {
    atomicAdd(&ws.counts[key], 1);
  } else {
    const int p = ws.offsets[key] + atomicAdd(&ws.cursor[key], 1);
    ws.list[p] = ((uint32_t)tg << 6) | (uint32_t)i;
    if (a.block_size < kBlk) ws.sub[p] = (uint8_t)sub;
    ws.slotmap[id] = p;
  }
}

// The same two passes with the histogram of a workgroup's tokens kept in LDS: one workgroup takes
// kBucketTok consecutive tokens of one kv head, ranks its pairs per (head, block) with LDS atomics
// and touches the global counters once per non-empty block instead of once per pair.  The pairs of
// a block coming from one workgroup end up next to each other in the list, so a block's query
// gathers walk the token axis in runs.
constexpr int kBucketTok = 512;
constexpr int kBucketMaxBins = 32768;      // LDS histogram: 4 bytes per 64-key block of the batch

template <bool FILL>
__global__ void __launch_bounds__(1024)
slc_bucket_lds_kernel(const SlcArgs a, SlcWs ws) {
  extern __shared__ int hist[];
  const int h = blockIdx.y;
  int tb, te;
  slc_token_range(a, tb, te);
  const int t_begin = tb + blockIdx.x * kBucketTok;
  if (t_begin >= te) return;
  const int t_end = min(te, t_begin + kBucketTok);
  for (int i = threadIdx.x; i < ws.nb; i += 1024) hist[i] = 0;
  __syncthreads();
  const int entries = (t_end - t_begin) * a.top_n;
  auto entry = [&](int e, long& id, int& tg, int& i, int& sub) -> int {      // global block of the pair, or -1
    tg = t_begin + e / a.top_n;
    i = e % a.top_n;
    const long th = (long)tg * a.hkv + h;
    id = th * a.top_n + i;
    const int b = seq_of_token(a.cu_seq, a.batch, tg);
    const int t = tg - a.cu_seq[b];
    const long th_r = (long)tg * (a.hkv / a.kv_rep) + h / a.kv_rep;    // picks and counts are per real kv head
    const int blk = slc_slot_block(a, th_r, i, t, sub);
    return blk >= 0 ? ws.blkbase[b] + blk : -1;
  };
  for (int e = threadIdx.x; e < entries; e += 1024) {
    long id; int tg, i, sub;
    const int gb = entry(e, id, tg, i, sub);
    if (FILL) ws.slotmap[id] = gb >= 0 ? atomicAdd(&hist[gb], 1) : -1;     // rank inside this workgroup
    else if (gb >= 0) atomicAdd(&hist[gb], 1);
  }
  __syncthreads();
  for (int bin = threadIdx.x; bin < ws.nb; bin += 1024) {
    const int c = hist[bin];
    if (c > 0) {
      const int key = h * ws.nb + bin;
      if (FILL) hist[bin] = ws.offsets[key] + atomicAdd(&ws.cursor[key], c);
      else atomicAdd(&ws.counts[key], c);
    }
  }
  if (!FILL) return;
  __syncthreads();
  for (int e = threadIdx.x; e < entries; e += 1024) {
    long id; int tg, i, sub;
    const int gb = entry(e, id, tg, i, sub);
    if (gb >= 0) {
      const int p = hist[gb] + ws.slotmap[id];
      ws.list[p] = ((uint32_t)tg << 6) | (uint32_t)i;
      if (a.block_size < kBlk) ws.sub[p] = (uint8_t)sub;
      ws.slotmap[id] = p;
    }
  }
}

// exclusive scan of the pair counts and the list of work items (one workgroup)
__global__ void __launch_bounds__(1024)
slc_scan_kernel(SlcWs ws, int hkv) {
  __shared__ int s_cnt[1024], s_seg[1024];
  __shared__ int carry_cnt, carry_seg;
  if (threadIdx.x == 0) { carry_cnt = 0; carry_seg = 0; }
  __syncthreads();
  const int n = hkv * ws.nb;
  for (int base = 0; base < n; base += 1024) {
    const int i = base + threadIdx.x;
    const int c = i < n ? ws.counts[i] : 0;
    const int sg = (c + kSeg - 1) / kSeg;
    s_cnt[threadIdx.x] = c;
    s_seg[threadIdx.x] = sg;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {          // Hillis-Steele inclusive scan
      int vc = 0, vs = 0;
      if ((int)threadIdx.x >= d) { vc = s_cnt[threadIdx.x - d]; vs = s_seg[threadIdx.x - d]; }
      __syncthreads();
      s_cnt[threadIdx.x] += vc;
      s_seg[threadIdx.x] += vs;
      __syncthreads();
    }
    const int ex_c = carry_cnt + s_cnt[threadIdx.x] - c;
    const int ex_s = carry_seg + s_seg[threadIdx.x] - sg;
    if (i < n) {
      ws.offsets[i] = ex_c;
      for (int k = 0; k < sg; ++k)
        if (ex_s + k < ws.items_cap) { ws.items[2 * (ex_s + k)] = i; ws.items[2 * (ex_s + k) + 1] = k; }   // (head*nb + block, segment)
    }
    __syncthreads();
    if (threadIdx.x == 1023) { carry_cnt += s_cnt[1023]; carry_seg += s_seg[1023]; }
    __syncthreads();
  }
  if (threadIdx.x == 0) *ws.n_items = min(carry_seg, ws.items_cap);
}

// ---- one K/V block in registers, the queries that picked it streamed past ------------------------

// SUB: selection blocks of fewer than 64 keys; a pair then attends keys [sub, sub + block_size) of its 64-key block.
template <typename T, int DK, int DV, bool SUB>
__global__ void __launch_bounds__(256)
slc_block_kernel(const SlcArgs a, const SlcWs ws) {
  constexpr int NK = DK / 32, NV = DV / 16, OLD = DV + 8;
  __shared__ __attribute__((aligned(16))) T stage[4][16 * OLD];    // per wavefront: one partial, head-major
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int item_id = blockIdx.x * 4 + wave;
  if (item_id >= *ws.n_items) return;
  const int key = ws.items[2 * item_id], seg = ws.items[2 * item_id + 1];
  const int h = key / ws.nb, gb = key % ws.nb;
  const SeqTile st = find_tile(a.cu_seq, a.batch, kBlk, gb);      // st.t0 = first key of the block
  if (!st.valid) return;
  const int G = a.hq / a.hkv;
  const int first = ws.offsets[key] + seg * kSeg;
  const int count = min(ws.counts[key] - seg * kSeg, kSeg);
  const float c_attn = a.scale * kLog2e;

  // K block as A fragments: chunk c (32 keys) = tiles 2c, 2c+1 with permuted rows; V^T block per chunk
  vec8_t<T> kf[4][NK], vf[2][NV];
  {
    const int hk = h / a.kv_rep, hkv_r = a.hkv / a.kv_rep;     // kv head of this (sub-)group, number of kv heads
    const T* kb = reinterpret_cast<const T*>(a.k) + ((long)st.start * hkv_r + hk) * DK + 8 * g;
    const long krow = (long)hkv_r * DK;
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const int row = min(st.t0 + 32 * (tile >> 1) + chunk_key_of_row(tile & 1, n), st.len - 1);
#pragma unroll
      for (int kk = 0; kk < NK; ++kk) kf[tile][kk] = load8(kb + row * krow + 32 * kk);
    }
    const T* vtb = reinterpret_cast<const T*>(a.vt) + (long)hk * DV * a.vt_cols + transposed_offset(st.start, st.b) +
                   (long)n * a.vt_cols + st.t0 + 8 * g;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < NV; ++t) vf[c][t] = load8(vtb + t * 16L * a.vt_cols + 32 * c);
  }

  const T* qb = reinterpret_cast<const T*>(a.q);
  T* pob = reinterpret_cast<T*>(ws.po);
  const int gc = n < G ? n : G - 1;
  vec8_t<T> qn[NK];
  // The segment's pair-list entries (at most one per lane) in one load; entry j is taken out with readlane.  A
  // load from a wave-uniform address inside the loop would be waited for where it is issued, and on this
  // hardware that wait (loads and stores share one in-order counter) also covers the stores of the pair before.
  const uint32_t ents = ws.list[first + min(lane, count - 1)];
  int subs = 0;
  if (SUB) subs = ws.sub[first + min(lane, count - 1)];
  uint32_t ent = __builtin_amdgcn_readlane(ents, 0);
  {
    const T* qp = qb + ((long)(ent >> 6) * a.hq + h * G + gc) * DK + 8 * g;
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) qn[kk] = load8(qp + 32 * kk);
  }
  // The K / V fragments are waited for here, once (an empty asm that takes each of them): left to the compiler,
  // their waits sit inside the loop, where the fragments are first used, and, counting down to zero, would there
  // also wait for the query just requested.
#pragma unroll
  for (int tile = 0; tile < 4; ++tile)
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) asm volatile("" ::"v"(kf[tile][kk]));
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int t = 0; t < NV; ++t) asm volatile("" ::"v"(vf[c][t]));
  for (int j = 0; j < count; ++j) {
    vec8_t<T> qf[NK];
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) qf[kk] = qn[kk];
    const int tg = (int)(ent >> 6);
    const int p = first + j;
    if (j + 1 < count) {                                  // next query in flight while this one is multiplied
      ent = __builtin_amdgcn_readlane(ents, j + 1);
      const T* qp = qb + ((long)(ent >> 6) * a.hq + h * G + gc) * DK + 8 * g;
#pragma unroll
      for (int kk = 0; kk < NK; ++kk) qn[kk] = load8(qp + 32 * kk);
    }
    const int t_loc = tg - st.start;                      // token position inside its sequence
    float s[16];
    {
      f32x4_t acc[4];
#pragma unroll
      for (int tile = 0; tile < 4; ++tile) {
        acc[tile] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) acc[tile] = mma16(kf[tile][kk], qf[kk], acc[tile]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[i] = acc[0][i]; s[4 + i] = acc[1][i]; s[8 + i] = acc[2][i]; s[12 + i] = acc[3][i]; }
    }
    if (SUB) {                                            // part of a block: its keys up to the token
      const int lo = __builtin_amdgcn_readlane(subs, j);
      const int hi = min(lo + a.block_size, t_loc - st.t0 + 1);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int kb = 32 * (i >> 3) + 8 * g + (i & 7);
        if (kb < lo || kb >= hi) s[i] = kNegInf;
      }
    } else if (st.t0 + kBlk - 1 > t_loc) {                // the block that contains the token itself
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (st.t0 + 32 * (i >> 3) + 8 * g + (i & 7) > t_loc) s[i] = kNegInf;
    }
    float mx = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
    mx = colgroup_max(mx);                                // finite: the first key of the pick is visible
    float pr[16], sum = 0.f;
    const float off = -mx * c_attn;
#pragma unroll
    for (int i = 0; i < 16; ++i) { pr[i] = fast_exp2(fmaf(s[i], c_attn, off)); sum += pr[i]; }
    sum = colgroup_sum(sum);
    float p0[8], p1[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { p0[i] = pr[i]; p1[i] = pr[8 + i]; }
    const vec8_t<T> pb0 = pack8<T>(p0), pb1 = pack8<T>(p1);
    const float inv = 1.0f / sum;
    T* srow = &stage[wave][n * OLD + 4 * g];
#pragma unroll
    for (int t = 0; t < NV; ++t) {
      f32x4_t o = {0.f, 0.f, 0.f, 0.f};
      o = mma16(vf[0][t], pb0, o);
      o = mma16(vf[1][t], pb1, o);
#pragma unroll
      for (int i = 0; i < 4; ++i) srow[t * 16 + i] = (T)(o[i] * inv);
    }
    // head-major rows out of LDS: 16 lanes write one full row, a wavefront instruction 4 rows
    {
      T* dst = pob + (long)p * 16 * DV;
      constexpr int PIECES = DV / 8;                       // 16-byte pieces per row
#pragma unroll
      for (int k = 0; k < 16 * PIECES / 64; ++k) {
        const int e = lane + 64 * k;
        const int r = e / PIECES, pc = e % PIECES;
        store8(dst + r * DV + pc * 8, load8(&stage[wave][r * OLD + pc * 8]));
      }
    }
    // every lane group holds the same mx / sum; all four store them (same values to the same addresses) so that
    // the stores are unconditional and the compiler can count them when it waits for the next query's loads
    ws.ml[((long)p * 2 + 0) * 16 + n] = mx;
    ws.ml[((long)p * 2 + 1) * 16 + n] = sum;
  }
}

// The same for GQA groups of at most 8 (PP = 2) or 4 (PP = 4) heads: the 16 columns of a score tile hold PP pairs of
// the segment (columns u * GP .. u * GP + GP - 1 = the heads of pair u of the step, GP = 16 / PP), so a step of the
// same cost serves PP pairs, and a partial result has GP rows instead of 16.
template <typename T, int DK, int DV, bool SUB, int PP>
__global__ void __launch_bounds__(256)
slc_block_packed_kernel(const SlcArgs a, const SlcWs ws) {
  constexpr int NK = DK / 32, NV = DV / 16, OLD = DV + 8, GP = 16 / PP;
  __shared__ __attribute__((aligned(16))) T stage[4][16 * OLD];    // per wavefront: one partial, head-major
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int item_id = blockIdx.x * 4 + wave;
  if (item_id >= *ws.n_items) return;
  const int key = ws.items[2 * item_id], seg = ws.items[2 * item_id + 1];
  const int h = key / ws.nb, gb = key % ws.nb;
  const SeqTile st = find_tile(a.cu_seq, a.batch, kBlk, gb);      // st.t0 = first key of the block
  if (!st.valid) return;
  const int G = a.hq / a.hkv;
  const int first = ws.offsets[key] + seg * kSeg;
  const int count = min(ws.counts[key] - seg * kSeg, kSeg);
  const float c_attn = a.scale * kLog2e;

  // K block as A fragments: chunk c (32 keys) = tiles 2c, 2c+1 with permuted rows; V^T block per chunk
  vec8_t<T> kf[4][NK], vf[2][NV];
  {
    const int hk = h / a.kv_rep, hkv_r = a.hkv / a.kv_rep;     // kv head of this (sub-)group, number of kv heads
    const T* kb = reinterpret_cast<const T*>(a.k) + ((long)st.start * hkv_r + hk) * DK + 8 * g;
    const long krow = (long)hkv_r * DK;
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const int row = min(st.t0 + 32 * (tile >> 1) + chunk_key_of_row(tile & 1, n), st.len - 1);
#pragma unroll
      for (int kk = 0; kk < NK; ++kk) kf[tile][kk] = load8(kb + row * krow + 32 * kk);
    }
    const T* vtb = reinterpret_cast<const T*>(a.vt) + (long)hk * DV * a.vt_cols + transposed_offset(st.start, st.b) +
                   (long)n * a.vt_cols + st.t0 + 8 * g;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < NV; ++t) vf[c][t] = load8(vtb + t * 16L * a.vt_cols + 32 * c);
  }

  const T* qb = reinterpret_cast<const T*>(a.q);
  T* pob = reinterpret_cast<T*>(ws.po);
  const int u = n / GP, hd = n % GP;                     // pair of the step and head of this column
  const int gc = hd < G ? hd : G - 1;
  vec8_t<T> qn[NK];
  // The segment's pair-list entries (at most one per lane) in one load; entry j is taken out with readlane.  A
  // load from a wave-uniform address inside the loop would be waited for where it is issued, and on this
  // hardware that wait (loads and stores share one in-order counter) also covers the stores of the pair before.
  const uint32_t ents = ws.list[first + min(lane, count - 1)];
  int subs = 0;
  if (SUB) subs = ws.sub[first + min(lane, count - 1)];
  const int steps = (count + PP - 1) / PP;
  // the pair of this lane's column in step j (past the end: the last pair again, computed and not stored)
  auto entry_of = [&](int j) { return (uint32_t)__shfl((int)ents, min(j * PP + u, count - 1)); };
  uint32_t ent = entry_of(0);
  {
    const T* qp = qb + ((long)(ent >> 6) * a.hq + h * G + gc) * DK + 8 * g;
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) qn[kk] = load8(qp + 32 * kk);
  }
  // The K / V fragments are waited for here, once (an empty asm that takes each of them): left to the compiler,
  // their waits sit inside the loop, where the fragments are first used, and, counting down to zero, would there
  // also wait for the query just requested.
#pragma unroll
  for (int tile = 0; tile < 4; ++tile)
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) asm volatile("" ::"v"(kf[tile][kk]));
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int t = 0; t < NV; ++t) asm volatile("" ::"v"(vf[c][t]));
  for (int j = 0; j < steps; ++j) {
    vec8_t<T> qf[NK];
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) qf[kk] = qn[kk];
    const int tg = (int)(ent >> 6);
    const int pf = first + j * PP;                        // first pair of the step
    const bool stored = j * PP + u < count;
    int lo = 0;
    if (SUB) lo = __shfl(subs, min(j * PP + u, count - 1));
    if (j + 1 < steps) {                                  // next queries in flight while these are multiplied
      ent = entry_of(j + 1);
      const T* qp = qb + ((long)(ent >> 6) * a.hq + h * G + gc) * DK + 8 * g;
#pragma unroll
      for (int kk = 0; kk < NK; ++kk) qn[kk] = load8(qp + 32 * kk);
    }
    const int t_loc = tg - st.start;                      // token position inside its sequence (per column)
    float s[16];
    {
      f32x4_t acc[4];
#pragma unroll
      for (int tile = 0; tile < 4; ++tile) {
        acc[tile] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) acc[tile] = mma16(kf[tile][kk], qf[kk], acc[tile]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[i] = acc[0][i]; s[4 + i] = acc[1][i]; s[8 + i] = acc[2][i]; s[12 + i] = acc[3][i]; }
    }
    if (SUB) {                                            // part of a block: its keys up to the token
      const int hi = min(lo + a.block_size, t_loc - st.t0 + 1);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int kb = 32 * (i >> 3) + 8 * g + (i & 7);
        if (kb < lo || kb >= hi) s[i] = kNegInf;
      }
    } else {                                              // the block that contains the column's token: its keys up to it
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (st.t0 + 32 * (i >> 3) + 8 * g + (i & 7) > t_loc) s[i] = kNegInf;
    }
    float mx = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
    mx = colgroup_max(mx);                                // finite: the first key of the pick is visible
    float pr[16], sum = 0.f;
    const float off = -mx * c_attn;
#pragma unroll
    for (int i = 0; i < 16; ++i) { pr[i] = fast_exp2(fmaf(s[i], c_attn, off)); sum += pr[i]; }
    sum = colgroup_sum(sum);
    float p0[8], p1[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { p0[i] = pr[i]; p1[i] = pr[8 + i]; }
    const vec8_t<T> pb0 = pack8<T>(p0), pb1 = pack8<T>(p1);
    const float inv = 1.0f / sum;
    T* srow = &stage[wave][n * OLD + 4 * g];
#pragma unroll
    for (int t = 0; t < NV; ++t) {
      f32x4_t o = {0.f, 0.f, 0.f, 0.f};
      o = mma16(vf[0][t], pb0, o);
      o = mma16(vf[1][t], pb1, o);
#pragma unroll
      for (int i = 0; i < 4; ++i) srow[t * 16 + i] = (T)(o[i] * inv);
    }
    // head-major rows out of LDS: 16 lanes write one full row, a wavefront instruction 4 rows
    {
      // row n of the staged tile = head hd of pair pf + u: consecutive pairs, GP rows each, are consecutive rows
      T* dst = pob + (long)pf * GP * DV;
      const int rows = min(PP, count - j * PP) * GP;
      constexpr int PIECES = DV / 8;                       // 16-byte pieces per row
#pragma unroll
      for (int k = 0; k < 16 * PIECES / 64; ++k) {
        const int e = lane + 64 * k;
        const int r = e / PIECES, pc = e % PIECES;
        if (r < rows) store8(dst + r * DV + pc * 8, load8(&stage[wave][r * OLD + pc * 8]));
      }
    }
    if (stored) {
      ws.ml[((long)(pf + u) * 2 + 0) * 16 + hd] = mx;
      ws.ml[((long)(pf + u) * 2 + 1) * 16 + hd] = sum;
    }
  }
}

// ---- merge the partials of every token, gate, add the other branches ---------------------------

// One thread per (token, q head, 8 output channels).
template <typename T, int DV, int TOPN, bool EXACT>
__global__ void __launch_bounds__(256)
slc_merge_kernel(const SlcArgs a, const MergeArgs m) {
  constexpr int PPR = DV / 8;                                     // 8-channel pieces per output row
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  if (id >= (long)a.total * a.hq * PPR) return;
  const int pc = (int)(id % PPR);
  const long row = id / PPR;                                      // token * hq + head
  const int hq_i = (int)(row % a.hq);
  const long tg = row / a.hq;
  const int G = a.hq / a.hkv;
  const T* osw = reinterpret_cast<const T*>(a.o_swa);
  vec8_t<T> o_swa = zero8<T>();
  if (osw) o_swa = load8(osw + row * DV + pc * 8);
  const vec8_t<T> r = merge_piece<T, DV, TOPN, EXACT>(m, tg, hq_i / G, hq_i % G, row, pc, osw != nullptr, o_swa);
  store8(reinterpret_cast<T*>(a.out) + row * DV + pc * 8, r);
  if (m.lse != nullptr && pc == 0) m.lse[row] = merge_lse(m, tg, hq_i / G, hq_i % G);
}

static MergeArgs merge_args_of(const SlcArgs& a, const SlcWs& ws) {
  return MergeArgs{ws.slotmap, ws.ml, ws.po, slc_part_rows(a), a.g_slc, a.g_swa, a.g_cmp, a.gate_stride, a.o_cmp, a.out,
                   a.top_n, a.hq, a.hkv, a.gate_act, a.scale, a.lse};
}

// bucket the (token, pick) pairs by (kv head, block): counts, offsets, pair list, slot map, work items
int launch_slc_bucket(const SlcArgs& raw, const SlcWs& ws, hipStream_t st) {
  const SlcArgs a = slc_virtual(raw);
  const long pairs = ws.pairs_cap;
  const long slab = pairs / ((long)a.hkv * a.top_n);               // tokens the slab can hold
  hipLaunchKernelGGL(slc_prep_kernel, dim3(1), dim3(256), 0, st, a.cu_seq, a.batch, ws, a.hkv);
  if (ws.nb <= kBucketMaxBins) {
    const dim3 grid((unsigned)((slab + kBucketTok - 1) / kBucketTok), a.hkv);
    const size_t smem = (size_t)ws.nb * sizeof(int);
    if (smem > 64 * 1024) {
      int rc = set_smem(reinterpret_cast<const void*>(slc_bucket_lds_kernel<false>), smem);
      if (rc == 0) rc = set_smem(reinterpret_cast<const void*>(slc_bucket_lds_kernel<true>), smem);
      if (rc) return rc;
    }
    hipLaunchKernelGGL(slc_bucket_lds_kernel<false>, grid, dim3(1024), smem, st, a, ws);
    hipLaunchKernelGGL(slc_scan_kernel, dim3(1), dim3(1024), 0, st, ws, a.hkv);
    hipLaunchKernelGGL(slc_bucket_lds_kernel<true>, grid, dim3(1024), smem, st, a, ws);
  } else {
    const int gb = (int)((pairs + 255) / 256);
    hipLaunchKernelGGL(slc_bucket_kernel<false>, dim3(gb), dim3(256), 0, st, a, ws);
    hipLaunchKernelGGL(slc_scan_kernel, dim3(1), dim3(1024), 0, st, ws, a.hkv);
    hipLaunchKernelGGL(slc_bucket_kernel<true>, dim3(gb), dim3(256), 0, st, a, ws);
  }
  return 0;
}

// bucket the pairs, then one partial result per pair
template <typename T, int DK, int DV>
static int launch_partials_t(const SlcArgs& a, const SlcWs& ws, hipStream_t st) {
  const int rc = launch_slc_bucket(a, ws, st);
  if (rc) return rc;
  const dim3 grid((ws.items_cap + 3) / 4);
  const bool sub = a.block_size < kBlk;
  switch (slc_part_rows(a)) {
    case 4:
      if (sub) hipLaunchKernelGGL((slc_block_packed_kernel<T, DK, DV, true, 4>), grid, dim3(256), 0, st, a, ws);
      else hipLaunchKernelGGL((slc_block_packed_kernel<T, DK, DV, false, 4>), grid, dim3(256), 0, st, a, ws);
      break;
    case 8:
      if (sub) hipLaunchKernelGGL((slc_block_packed_kernel<T, DK, DV, true, 2>), grid, dim3(256), 0, st, a, ws);
      else hipLaunchKernelGGL((slc_block_packed_kernel<T, DK, DV, false, 2>), grid, dim3(256), 0, st, a, ws);
      break;
    default:
      if (sub) hipLaunchKernelGGL((slc_block_kernel<T, DK, DV, true>), grid, dim3(256), 0, st, a, ws);
      else hipLaunchKernelGGL((slc_block_kernel<T, DK, DV, false>), grid, dim3(256), 0, st, a, ws);
  }
  return 0;
}

template <typename T, int DV>
static int launch_merge_t(const SlcArgs& a, const SlcWs& ws, hipStream_t st) {
  const long threads = (long)a.total * a.hq * (DV / 8);
  const dim3 mg((int)((threads + 255) / 256));
  const MergeArgs m = merge_args_of(a, ws);
  if (a.top_n == 16) hipLaunchKernelGGL((slc_merge_kernel<T, DV, 16, true>), mg, dim3(256), 0, st, a, m);
  else hipLaunchKernelGGL((slc_merge_kernel<T, DV, 16, false>), mg, dim3(256), 0, st, a, m);   // rounds of 16 picks
  return 0;
}

int launch_slc_partials(const SlcArgs& raw, void* workspace, hipStream_t st) {
  const SlcArgs a = slc_virtual(raw);
  SlcWs ws;
  carve(a, workspace, &ws, 2);
  switch (a.dk * 1000 + a.dv + (a.dtype == 2 ? 1000000 : 0)) {
    case 32032: return launch_partials_t<bf16_t, 32, 32>(a, ws, st);
    case 64064: return launch_partials_t<bf16_t, 64, 64>(a, ws, st);
    case 128128: return launch_partials_t<bf16_t, 128, 128>(a, ws, st);
    case 192128: return launch_partials_t<bf16_t, 192, 128>(a, ws, st);
    case 1032032: return launch_partials_t<f16_t, 32, 32>(a, ws, st);
    case 1064064: return launch_partials_t<f16_t, 64, 64>(a, ws, st);
    case 1128128: return launch_partials_t<f16_t, 128, 128>(a, ws, st);
    case 1192128: return launch_partials_t<f16_t, 192, 128>(a, ws, st);
    default: return -2;
  }
}

MergeArgs slc_merge_args(const SlcArgs& raw, void* workspace) {
  const SlcArgs a = slc_virtual(raw);
  SlcWs ws;
  carve(a, workspace, &ws, 2);
  return merge_args_of(a, ws);
}

int launch_slc_block_major(const SlcArgs& raw, void* workspace, hipStream_t st) {
  const SlcArgs a = slc_virtual(raw);
  const int rc = launch_slc_partials(a, workspace, st);
  if (rc) return rc;
  SlcWs ws;
  carve(a, workspace, &ws, 2);
  if (a.dtype == 2)
    return a.dv == 32 ? launch_merge_t<f16_t, 32>(a, ws, st)
                      : a.dv == 64 ? launch_merge_t<f16_t, 64>(a, ws, st) : launch_merge_t<f16_t, 128>(a, ws, st);
  return a.dv == 32 ? launch_merge_t<bf16_t, 32>(a, ws, st)
                    : a.dv == 64 ? launch_merge_t<bf16_t, 64>(a, ws, st) : launch_merge_t<bf16_t, 128>(a, ws, st);
}

}  // namespace nsa
