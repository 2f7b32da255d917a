// Workspace of the block-major selected attention: the (token, pick) pairs bucketed by
// (kv head, 64-key block).  Shared by the forward and the backward kernels.  Selection blocks of other sizes
// map onto 64-key blocks: a multiple of 64 keys takes several slots per pick, a divisor of 64 keys is a part
// of one 64-key block, whose first key inside that block is kept per pair (sub).
#pragma once
#include "common.h"
#include "kernels.h"

namespace nsa {

constexpr int kSeg = 64;          // pairs of one block handled by one work item
constexpr int kBlk = 64;          // keys per selection block (4 MFMA tiles)

struct SlcWs {
  int* blkbase; int* counts; int* offsets; int* cursor; int* items; int* n_items;
  uint32_t* list; int* slotmap; float* ml; void* po;
  uint8_t* sub;    // per pair: first key of the selection block inside its 64-key block (written and read only when
                   // block_size < 64)
  int nb;          // bound on the number of 64-key blocks over all sequences
  long pairs_cap;  // total * hkv * slots per (token, head)
  int items_cap;
};

__host__ __device__ inline long slc_align_up(long x, long a) { return (x + a - 1) / a * a; }

// The arguments as the block-major schedule sees them: top_n counts 64-key slots (see SlcArgs::pick_mult).
// Idempotent.
SlcArgs slc_virtual(const SlcArgs& a);

// Lays the workspace out in `base` (ws == nullptr: only returns the size).  `part_width` is the row
// width of the per-pair partial result (16 rows of part_width elements of `elem` bytes per pair).
// part_rows: rows of a pair's partial result (16; the forward uses slc_part_rows).
long slc_carve(const SlcArgs& a, void* base, SlcWs* ws, size_t elem, int part_width, int part_rows = 16);

// Rows of a forward partial result: the heads of the GQA group padded to 4, 8 or 16 (16 when the query heads are
// not known, as in a size query by kv heads alone).
inline int slc_part_rows(const SlcArgs& a) {
  if (a.hq <= 0 || a.hkv <= 0) return 16;
  const int g = a.hq / a.hkv;
  return g <= 4 ? 4 : g <= 8 ? 8 : 16;
}

// Tokens [tb, te) of the slab (all tokens without one).  Every lane of the calling wavefronts takes part.
__device__ __forceinline__ void slc_token_range(const SlcArgs& a, int& tb, int& te) {
  tb = 0;
  te = a.total;
  if (a.tile_count > 0) {
    const SeqTile s0 = find_tile(a.cu_seq, a.batch, a.tile_tokens, a.tile_begin);
    tb = s0.valid ? s0.start + s0.t0 : a.total;
    const SeqTile s1 = find_tile(a.cu_seq, a.batch, a.tile_tokens, a.tile_begin + a.tile_count);
    te = s1.valid ? s1.start + s1.t0 : a.total;
  }
}

// Fills counts / offsets / list / slotmap / items for a.indices (a.counts optional).
int launch_slc_bucket(const SlcArgs& a, const SlcWs& ws, hipStream_t st);

}  // namespace nsa
