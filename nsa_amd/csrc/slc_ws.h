// Workspace of the block-major selected attention: the (token, pick) pairs bucketed by
// (kv head, 64-key block).  Shared by the forward and the backward kernels.
#pragma once
#include "kernels.h"

namespace nsa {

constexpr int kSeg = 64;          // pairs of one block handled by one work item
constexpr int kBlk = 64;          // keys per selection block (4 MFMA tiles)

struct SlcWs {
  int* blkbase; int* counts; int* offsets; int* cursor; int* items; int* n_items;
  uint32_t* list; int* slotmap; float* ml; void* po;
  int nb;          // bound on the number of 64-key blocks over all sequences
  long pairs_cap;  // total * hkv * top_n
  int items_cap;
};

__host__ __device__ inline long slc_align_up(long x, long a) { return (x + a - 1) / a * a; }

// Lays the workspace out in `base` (ws == nullptr: only returns the size).  `part_width` is the row
// width of the per-pair partial result (16 rows of part_width elements of `elem` bytes per pair).
long slc_carve(const SlcArgs& a, void* base, SlcWs* ws, size_t elem, int part_width);

// Fills counts / offsets / list / slotmap / items for a.indices (a.counts optional).
int launch_slc_bucket(const SlcArgs& a, const SlcWs& ws, hipStream_t st);

}  // namespace nsa
