// Host-side launch descriptors shared by the kernel files and the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nsa {

struct CompressArgs {
  const void* x; const void* wt; const void* bias; void* out;
  const int32_t* cu_seq; const int32_t* cu_out;
  int batch, out_rows_bound, heads, dim, block, stride, dtype;
  // a second tensor over the same tokens (same heads, its own dim) for the same launch: mean pooling, or the
  // learned compressor with the second tensor's weight and bias
  const void* x2 = nullptr; void* out2 = nullptr; int dim2 = 0;
  const void* wt2 = nullptr; const void* bias2 = nullptr;
};

// Backward of the compression.  w_lin == nullptr: mean pooling (only dx).  w_lin is the weight in the
// functional layout [block*dim][dim] (row j*dim + i, column o); dw (same layout) and dbias are fp32.
struct CompressBwdArgs {
  const void* x; const void* w_lin; const void* d_out; void* dx; float* dw; float* dbias;
  const int32_t* cu_seq; const int32_t* cu_out;
  int batch, total, out_rows_bound, heads, dim, block, stride, dtype;
};

struct TransposeArgs {
  const void* x; void* out; const int32_t* cu;
  int batch, heads, dim; long row_stride, head_stride; int out_cols, dtype;
};

struct CmpArgs {
  const void* q; const void* ck; const void* cvt; void* o; void* indices; float* pooled; float* lse;
  const int32_t* cu_seq; const int32_t* cu_cmp;
  int batch, total, hq, hkv, dk, dv;
  long ck_row_stride, ck_head_stride; int cvt_cols;
  int block, stride, pool_k, pool_s, pool_p, top_n, max_ns, pooled_stride;
  float scale; int idx64, dtype, causal;
  float* lse_attn;   // optional: natural-log log-sum-exp of the scaled visible scores (+inf: no key visible)
  // GQA groups beyond 16 heads run as kv_rep = G / 16 sub-groups of 16: hkv then counts the sub-groups
  // ("virtual" kv heads, hq / hkv == 16) and sub-group h reads the K / V rows of kv head h / kv_rep
  int kv_rep = 1;
  // false: `pooled` only hands the window sums from the importance kernel to the top-n kernel; the averages are
  // not written back (and the generic one-kernel selection does not write it at all)
  bool keep_pooled = true;
  // optional: the gating Linear on q (weight [3][dk], bias [3] or null, in q's dtype) evaluated by the compressed-
  // attention kernel on the query fragments it holds anyway; gates [total][hq][3] receives the logits
  const void* gate_w = nullptr; const void* gate_b = nullptr; void* gates = nullptr;
  // one-pass kernel only: the compressed keys and values in fragment order (cmp_select.hip) and its chunk slots per head
  const void* frag = nullptr; int frag_chunks = 0;
};

struct SwaArgs {
  const void* q; const void* k; const void* vt; void* o; const int32_t* cu_seq;
  int batch, total, hq, hkv, dk, dv, vt_cols, window; float scale; int dtype;
  float* lse;        // optional, as CmpArgs::lse_attn
  int kv_rep = 1;    // as CmpArgs::kv_rep
  int tile_begin = 0, tile_count = 0;   // merge kernels: only these token tiles (tile_count 0 = all)
};

struct SlcArgs {
  const void* q; const void* k; const void* vt; const void* indices; const int32_t* counts;
  const void* g_slc; const void* g_swa; const void* g_cmp; long gate_stride;
  const void* o_swa; const void* o_cmp; void* out; const int32_t* cu_seq;
  int batch, total, hq, hkv, dk, dv, vt_cols, top_n, block_size; float scale;
  int idx64, gate_act, dtype;
  void* workspace; long workspace_bytes;
  float* lse;        // optional (block-major schedule only), as CmpArgs::lse_attn
  int kv_rep = 1;    // as CmpArgs::kv_rep; indices and counts stay per real kv head
  // Block-major schedule only (set by slc_virtual, 0 = not set): the schedule works on 64-key blocks.  A selection
  // block of 128, 192, ... keys occupies pick_mult = block_size / 64 slots per pick and top_n counts slots; a
  // selection block of 8, 16 or 32 keys is a masked part of the 64-key block that holds it (pick_mult = 1).
  int pick_mult = 0;
  // Block-major schedule, one slab of tokens at a time (tile_count 0 = all tokens): the tokens of the tiles
  // tile_begin .. tile_begin + tile_count - 1 of tile_tokens tokens each, tiles numbered as find_tile numbers them
  // (sequence by sequence).  Pair list and partial results are then sized for tile_count * tile_tokens tokens.
  int tile_begin = 0, tile_count = 0, tile_tokens = 0;
};

// Where the merge of the block-major partial results finds its inputs (all device pointers; the
// first three live inside the selected-attention workspace).
struct MergeArgs {
  const int* slotmap; const float* ml; const void* po;
  int part_rows;     // rows of one partial result in po: 16, or 8 / 4 for GQA groups of at most 8 / 4 heads
  const void* g_slc; const void* g_swa; const void* g_cmp; long gate_stride;
  const void* o_cmp; void* out;
  int top_n, hq, hkv, gate_act; float scale;
  float* lse;        // optional: log-sum-exp of the selected branch per (token, q head)
  // optional, written by merge_piece (what a backward pass keeps): the ungated, normalised selected and
  // sliding outputs [total,hq,dv] and the selected branch's log-sum-exp
  void* o_slc_out; void* o_swa_out; float* lse_slc_out;
};

// Backward of the compressed branch: all tensors packed and contiguous; lse is the natural-log
// log-sum-exp of the scaled visible scores of every row (+inf for rows that see nothing).
struct CmpBwdArgs {
  const void* q; const void* ck; const void* cv; const void* o; const void* d_o; const float* lse;
  const int32_t* cu_seq; const int32_t* cu_cmp;
  int batch, total, cmp_rows, hq, hkv, dk, dv, block, stride, causal; float scale; int dtype;
  void* dq; void* dck; void* dcv; void* workspace;
  // optional: delta = rowsum(o * d_o) computed by the caller (o may then be null), and a per-row gate:
  // the gradients are those for d_o scaled by rowscale[row], with delta the unscaled row sum
  const float* delta; const float* rowscale;
};

// Backward of the selected and sliding branches (either may be absent: top_n == 0 / d_o_slc null,
// window == 0 / d_o_swa null).  dq, dk_out, dv_out receive the sums over the present branches.
struct SlcSwaBwdArgs {
  const void* q; const void* k; const void* v;
  const void* o_slc; const void* o_swa; const void* d_o_slc; const void* d_o_swa;
  const float* lse_slc; const float* lse_swa;
  const void* indices; const int32_t* counts; const int32_t* cu_seq;
  int batch, total, hq, hkv, dk, dv, top_n, block_size, window; float scale; int idx64, dtype;
  void* dq; void* dk_out; void* dv_out; void* workspace;
  long workspace_bytes;      // the selected branch runs in token slabs as large as these bytes allow
  const float* delta_slc; const float* delta_swa; const float* rowscale_slc; const float* rowscale_swa;   // as above
  const void* dq_add;        // optional [total][hq][dk]: added to dq (the compressed branch's dQ); not dq itself
};

// Gated sum of the branches (d_out == nullptr: forward into out) or its backward (d_out given:
// d_slc / d_swa / d_cmp = act(gate) * d_out and d_gate_logits).  gate_logits [rows][3] (selected,
// sliding, compressed), branch tensors [rows][dv]; o_swa / o_cmp (and their gradients) may be null.
struct GateCombineArgs {
  const void* gate_logits; const void* o_slc; const void* o_swa; const void* o_cmp; void* out;
  const void* d_out; void* d_slc; void* d_swa; void* d_cmp; void* d_gate_logits;
  long rows; int dv, act, dtype;
  float* stats;      // optional (backward): [6][rows] = <d_out, o_b> for b = slc, swa, cmp, then act(gate_b)
};

struct DecodeArgs {
  const void* q; const void* k_cache; const void* v_cache_t; const void* ck_cache; const void* cv_cache_t;
  const int32_t* ctx_lens; const void* gates; void* out; int32_t* indices;
  int batch, hq, hkv, dk, dv, ctx_cap, nc_cap;
  int block, stride, sel_block, pool_k, pool_s, pool_p, top_n, window;
  float scale; int gate_act, dtype;
  // paged K/V (block_table != nullptr): k_cache is a pool of 64-token pages [page][64][hkv][dk], v_cache_t a
  // pool [page][hkv][dv][64]; page i of sequence b is block_table[b * max_pages + i]; ctx_cap is unused.
  // The compressed caches stay contiguous per sequence (1/16 of the K/V).
  const int32_t* block_table; int max_pages;
  // GQA groups beyond 16 heads (split schedule only): sub-groups of 16 query heads per kv head; each runs as a
  // pair of its own on the kv head's caches, and the selection sums the importance over all of them
  int kv_rep = 1;
};

// Split of a projection GEMM's packed rows [q | k | v | gate logits] into the attention operands with
// the rotary embedding applied to q and k (pack == 0), or the reverse gather of their gradients with
// the inverse rotation (pack == 1).  Column offsets and ld in elements, multiples of 8 except g_off.
struct QkvRopeArgs {
  void* packed; void* q; void* k; void* v; void* gates;   // gates may be null
  const float* inv_freq;                                   // [rope_dim / 2], null = no rotation
  const int32_t* positions;                                // [total], null = position within the sequence
  const int32_t* cu_seq; int batch;
  long total; int ld, q_off, k_off, v_off, g_off, hq, hkv, dk, dv, rope_off, rope_dim, interleaved, pack, dtype;
};
int launch_qkv_rope(const QkvRopeArgs& a, hipStream_t st);

int launch_compress(const CompressArgs& a, hipStream_t st);
int launch_compress_bwd(const CompressBwdArgs& a, hipStream_t st);
int launch_transpose(const TransposeArgs& a, hipStream_t st);
int launch_gate(const void* x, const void* w, const void* bias, void* out, long rows, int dim, int dtype,
                hipStream_t st);
int launch_gate_combine(const GateCombineArgs& a, hipStream_t st);
int launch_gate_bwd(const void* q, const void* w, const void* d_gl, void* dq, float* dw, float* db, long rows,
                    int dim, int dtype, hipStream_t st);
int launch_cmp_attn(const CmpArgs& a, hipStream_t st);
int launch_select(const CmpArgs& a, hipStream_t st);
// compressed attention + importance + top-n in one pass over the compressed keys (cmp_select.hip): whether the
// shape qualifies (max_nc = most compressed rows of any sequence), and the launch
bool cmp_select_single_pass_ok(const CmpArgs& a, int max_nc);
int launch_cmp_select(const CmpArgs& a, hipStream_t st);
int cmp_frag_chunks(int total_rows, int batch);
int launch_frag_pack(const CmpArgs& a, long cv_row_stride, long cv_head_stride, int rows_bound, hipStream_t st);
int launch_swa(const SwaArgs& a, hipStream_t st);
int launch_slc_combine(const SlcArgs& a, hipStream_t st);
long slc_workspace_bytes(const SlcArgs& a);
bool slc_block_major_ok(const SlcArgs& a);
bool slc_block_size_ok(int block_size);   // 8, 16, 32 or a multiple of 64 keys
int swa_tile_tokens(int hq, int hkv, int dtype);   // tokens per tile of the window kernel (hkv counts sub-groups)
int launch_slc_block_major(const SlcArgs& a, void* workspace, hipStream_t st);
int launch_slc_partials(const SlcArgs& a, void* workspace, hipStream_t st);
MergeArgs slc_merge_args(const SlcArgs& a, void* workspace);
int launch_swa_merge(const SwaArgs& a, const MergeArgs& m, hipStream_t st);
long cmp_bwd_workspace_bytes(const CmpBwdArgs& a);
int launch_cmp_bwd(const CmpBwdArgs& a, hipStream_t st);
long slc_swa_bwd_workspace_bytes(const SlcSwaBwdArgs& a);
int launch_slc_swa_bwd(const SlcSwaBwdArgs& a, hipStream_t st);
long slc_swa_bwd_slab_workspace_bytes(const SlcSwaBwdArgs& a, int slab_tokens);
int launch_decode(const DecodeArgs& a, hipStream_t st);
int launch_decode_append(const void* k_new, const void* v_new, void* k_cache, void* v_cache_t, void* ck_cache,
                         void* cv_cache_t, const int32_t* pos, int batch, int hkv, int dk, int dv, int ctx_cap,
                         int nc_cap, int block, int stride, int dtype, hipStream_t st);
int launch_decode_append_paged(const void* k_new, const void* v_new, void* k_pool, void* v_pool_t,
                               const int32_t* block_table, int max_pages, void* ck_cache, void* cv_cache_t,
                               const int32_t* pos, int batch, int hkv, int dk, int dv, int nc_cap, int block,
                               int stride, int dtype, hipStream_t st);
int decode_max_nc();
int decode_max_bins(int nc_cap);      // pooled bins per sequence that the one-workgroup step holds
int decode_split_max_nc();
// the same step spread over `splits` workgroups per (sequence, kv head), for small batches
long decode_split_workspace_bytes(const DecodeArgs& a, int splits);
int launch_decode_split(const DecodeArgs& a, int splits, void* workspace, hipStream_t st);
// the same with the partial results in a fixed device array of the library (no workspace argument)
long decode_split_static_bytes();
int launch_decode_split_static(const DecodeArgs& a, int splits, hipStream_t st);

}  // namespace nsa
