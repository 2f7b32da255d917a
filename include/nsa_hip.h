/* C ABI of libnsa_hip.so: the gfx950 kernels behind the NSA forward path and its backward.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise; the library never allocates, frees
 *     or synchronises; work is enqueued on `stream` and outputs are fully overwritten
 *   - the backward entry points (nsa_*_bwd) accumulate dK / dV with fp32 atomics inside their workspace:
 *     results agree from run to run to rounding, not bit for bit
 *   - tensors are packed ("varlen"): rows of all sequences back to back, `cu_seqlens` int32[batch+1]
 *     with cu_seqlens[0] == 0 holds the row offsets; a batch of equal lengths is the special case
 *     cu_seqlens[b] = b*T
 *   - dtype: NSA_BF16, NSA_F16 or NSA_F32 for every floating tensor of a call (accumulation is always fp32).
 *     NSA_F16 is the dtype of the reference's own selection test (tests/test_parallel_nsa.py:169); every entry
 *     point takes it.  The 16-bit types share one set of shapes; fp32 lacks a few (stated per entry point)
 *   - GQA: hq / hkv query heads share one kv head.  Groups of 1..16 heads are built everywhere; the prefill
 *     forward entry points (nsa_cmp_attn_*, nsa_block_select_fwd, nsa_swa_fwd, nsa_slc_*, nsa_swa_merge_fwd)
 *     also take groups of 32, 48, 64, ... heads, which is what the reference's selected attention asks for
 *     (HQ a multiple of 16 * H, nsa/selection_attn.py:800): they run as hq / (16 * hkv) sub-groups of 16 heads
 *     that share the keys, values and block picks of their kv head.  Backward and decode: groups up to 16 (a
 *     caller runs the backward of a larger group as one call per sub-group of 16 heads and adds the key / value
 *     gradients, as nsa_amd/ops.py does).
 *   - return value: 0 on success, negative on error (NSA_ERR_*); nsa_last_error_string() describes
 *     the last error of the calling thread.  No exception crosses this boundary.
 *   - "transposed" buffers hold one key-contiguous plane per head: element (h, d, col) lives at
 *     (h*dim + d)*cols + col, sequence b starts at column nsa_transposed_offset(cu[b], b) and
 *     `cols` = nsa_transposed_cols(total_rows, batch).  They are produced by nsa_transpose_fwd.
 *
 * The reference (yukavio/nsa) has no FFI layer; each entry point names the Python/Triton interface
 * of the reference it stands behind (file:line inside the reference tree).
 */
#ifndef NSA_HIP_H
#define NSA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* nsa_stream_t; /* hipStream_t */

enum { NSA_BF16 = 0, NSA_F32 = 1, NSA_F16 = 2 };
enum {
  NSA_OK = 0,
  NSA_ERR_INVALID = -1,     /* bad argument (null pointer, non-positive size, misalignment) */
  NSA_ERR_UNSUPPORTED = -2, /* shape outside what the kernels are built for */
  NSA_ERR_RESOURCE = -3,    /* needs more LDS than a gfx950 CU has */
  NSA_ERR_LAUNCH = -4       /* HIP reported a launch failure */
};
enum { NSA_GATE_IDENTITY = 0, NSA_GATE_SIGMOID = 1 };

int nsa_version(void);
const char* nsa_last_error_string(void);

/* Column bookkeeping of transposed buffers (host helpers, pure arithmetic). */
int nsa_transposed_offset(int cu_b, int b);
int nsa_transposed_cols(int total_rows, int batch);

/* KV block compression.  Replaces nsa/compression_kv.py:21-57 (_compress_fwd), :178-217
 * (_compress_kv.forward) and the two nn.Conv1d calls of KVCompressor.forward (:301-307).
 *   x      [total, heads, dim]        out [out_rows, heads, dim]
 *   wt     NULL -> mean over the window (eye/block weights, no bias); otherwise the weight as
 *          [dim_out = dim][block*dim] with wt[o][j*dim + i] = W_conv[o][i][j] = W_lin[j*dim+i][o]
 *   bias   [dim] or NULL
 *   cu_out int32[batch+1] offsets of every sequence's rows in `out`; row n of a sequence covers
 *          its tokens [n*stride, n*stride + block).  out_rows_bound >= cu_out[batch] sizes the grid. */
int nsa_compress_fwd(const void* x, const void* wt, const void* bias, void* out,
                     const int32_t* cu_seqlens, const int32_t* cu_out, int batch, int out_rows_bound,
                     int heads, int dim, int block, int stride, int dtype, nsa_stream_t stream);

/* K and V of a layer in one call, as the reference's compress_kv(k, v, w_k, w_v, ...) takes them
 * (nsa/compression_kv.py:269-289, KVCompressorVarlen.forward :291-312).  Same arguments as nsa_compress_fwd per
 * tensor (k [total, heads, dk] -> ck, v [total, heads, dv] -> cv, both over cu_out); wk_t / wv_t both NULL = mean
 * pooling, which then runs as ONE launch over both tensors; with weights it is the two GEMM launches. */
int nsa_compress_kv_fwd(const void* k, const void* v, const void* wk_t, const void* wv_t, const void* bk,
                        const void* bv, void* ck, void* cv, const int32_t* cu_seqlens, const int32_t* cu_out,
                        int batch, int out_rows_bound, int heads, int dk, int dv, int block, int stride, int dtype,
                        nsa_stream_t stream);

/* Key-contiguous copy of a packed [rows, heads, dim] tensor (row_stride / head_stride in elements).
 * Layout preparation for the MFMA PV product; no counterpart in the reference. */
int nsa_transpose_fwd(const void* x, void* out, const int32_t* cu, int batch, int heads, int dim,
                      int64_t row_stride, int64_t head_stride, int out_cols, int dtype,
                      nsa_stream_t stream);

/* Backward of nsa_compress_fwd.  Replaces nsa/compression_kv.py:220-266 (_compress_kv.backward with
 * the kernels _compress_bwd_dx / _compress_bwd_dw, :62-171); for the Conv1d compressor (:292-312,
 * differentiated by autograd in the reference) it also yields the bias gradient.
 *   d_out [out rows, heads, dim] gradient of the compressed rows; dx [total, heads, dim] is fully
 *   overwritten.  w_lin NULL = mean pooling.  Otherwise w_lin is the weight as [block*dim][dim]
 *   (row j*dim + i = tap j, input channel i; column = output channel: the layout of the reference's
 *   k_weight / v_weight, i.e. the TRANSPOSE of what nsa_compress_fwd takes), x [total, heads, dim] the
 *   forward input, dw float [block*dim][dim] and dbias float [dim] (either may be NULL) are
 *   overwritten with the weight / bias gradients in fp32. */
int nsa_compress_bwd(const void* x, const void* w_lin, const void* d_out, void* dx, float* dw, float* dbias,
                     const int32_t* cu_seqlens, const int32_t* cu_out, int batch, int total, int out_rows_bound,
                     int heads, int dim, int block, int stride, int dtype, nsa_stream_t stream);

/* Compressed attention fused with block-importance scoring and top-n selection.  Replaces
 * nsa/triton_attention.py:419-476 (_attention.forward: _attn_fwd, softmax_kernel, sum / avg_pool1d /
 * topk) with the semantics of nsa/torch_attention.py:66-163 (attention_ref, get_indices).
 *   q [total, hq, dk]; ck rows at ck + (cu_cmp[b] + c)*ck_row_stride + h*ck_head_stride (dk elements);
 *   cvt transposed [hkv][dv][cvt_cols] over cu_cmp; o [total, hq, dv];
 *   indices [total, hkv, top_n] int32 or int64 (idx64), descending score, -1 where fewer bins exist;
 *   NULL skips the selection;  pooled (optional, float) [total, hkv, sub, pooled_stride] with sub =
 *   max(1, hq / (16 * hkv)) sub-groups (1 for GQA groups up to 16 heads) receives in its first sub-row the
 *   pooled block scores (bins past a sequence's last one up to max_ns are zeroed).  Pass it even when
 *   the scores are not wanted: with it (and pooling windows of s + 1 columns every s, s = 1, 2, 4 or 8, padding
 *   below 64, max_ns <= 4096, top_n <= 64) the selection runs as two lean kernels that use it as their hand-over buffer, without
 *   it as one slower kernel that keeps the bins in LDS;  keep_pooled == 0 says that the scores themselves are
 *   not wanted: the buffer then only carries the window sums between the two kernels, its contents afterwards
 *   are unspecified, and the second kernel saves writing the averages back;
 *   lse (float) [total, hq] receives the log-sum-exp of the raw scores q.ck over all compressed rows
 *   (the reference's M without its mask and scale); required when indices is given.
 *   Compressed row c of a sequence is visible to token t iff c*stride + block <= t (causal != 0;
 *   causal == 0 makes every row visible).
 *   max_ns >= pooled bins of the longest sequence (sizes LDS). */
int nsa_cmp_attn_select_fwd(const void* q, const void* ck, const void* cvt, void* o, void* indices,
                            float* pooled, float* lse, const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch,
                            int total, int hq, int hkv, int dk, int dv, int64_t ck_row_stride,
                            int64_t ck_head_stride, int cvt_cols, int block, int stride, int pool_kernel,
                            int pool_stride, int pool_pad, int top_n, int max_ns, int pooled_stride,
                            int keep_pooled, float scale, int causal, int idx64, int dtype, nsa_stream_t stream);

/* The two halves of nsa_cmp_attn_select_fwd as separate launches: compressed attention (writes o
 * and lse) and block selection (reads lse).  Same arguments and meaning as above.
 *   lse_attn (optional, float [total, hq]) receives what the backward needs: the natural-log
 *   log-sum-exp of the scaled scores over the rows visible to the token (the reference's M of
 *   nsa/triton_attention.py:176-181 in natural log), +inf for a token that sees no row. */
int nsa_cmp_attn_fwd(const void* q, const void* ck, const void* cvt, void* o, float* lse, float* lse_attn,
                     const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch, int total, int hq, int hkv,
                     int dk, int dv, int64_t ck_row_stride, int64_t ck_head_stride, int cvt_cols, int block,
                     int stride, float scale, int causal, int dtype, nsa_stream_t stream);

/* nsa_cmp_attn_fwd that also evaluates the gating Linear of the module on q (nsa/nsa.py:61,117: gating(q) with
 * weight [3,dk], bias [3] or NULL, both in q's dtype): the kernel multiplies the query fragments it holds anyway with
 * the three weight rows, so the logits cost no pass over q.  gates [total,hq,3] (q's dtype) receives them (order:
 * selected, sliding, compressed), as nsa_gate_fwd would. */
int nsa_cmp_attn_gate_fwd(const void* q, const void* ck, const void* cvt, void* o, float* lse, float* lse_attn,
                          const void* gate_weight, const void* gate_bias, void* gates, const int32_t* cu_seqlens,
                          const int32_t* cu_cmp, int batch, int total, int hq, int hkv, int dk, int dv,
                          int64_t ck_row_stride, int64_t ck_head_stride, int cvt_cols, int block, int stride,
                          float scale, int causal, int dtype, nsa_stream_t stream);
int nsa_block_select_fwd(const void* q, const void* ck, const float* lse, void* indices, float* pooled,
                         const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch, int total, int hq, int hkv,
                         int dk, int64_t ck_row_stride, int64_t ck_head_stride, int pool_kernel, int pool_stride,
                         int pool_pad, int top_n, int max_ns, int pooled_stride, int keep_pooled, int idx64,
                         int dtype, nsa_stream_t stream);

/* Compressed attention AND block selection as the reference's one call computes them (_attention.forward,
 * nsa/triton_attention.py:419-476: one q.ck product whose scores feed the attention, the softmax over all rows, the
 * pooling and the top-k).  Arguments as nsa_cmp_attn_select_fwd, plus lse_attn as in nsa_cmp_attn_fwd and the gating
 * Linear (gate_weight / gate_bias / gates, all NULL = none) as in nsa_cmp_attn_gate_fwd.
 *   max_nc: the most compressed rows of any sequence of the batch (max_ns is the pooled-bin count that goes with it).
 *   single_pass: -1 = run as ONE kernel when the shape qualifies (nsa_cmp_select_single_pass: GQA groups of 9..16
 *   heads, 16-bit inputs, head dims (64,64), (128,128), (192,128), pooling windows of 5 rows every 4 without padding,
 *   max_nc <= 2048, top_n <= 64), else as nsa_cmp_attn(_gate)_fwd followed by nsa_block_select_fwd; 0 = always the
 *   latter; 1 = the one kernel or NSA_ERR_UNSUPPORTED.  The one kernel multiplies q with the compressed keys once,
 *   keeps no score buffer and no pooled hand-over buffer: the window sums stay in registers per head until the
 *   head's normaliser is known.  lse and pooled may be NULL then (pooled given and keep_pooled != 0: the averages are
 *   written); on the other schedule lse is required and pooled selects the two-kernel selection as above.
 *   frag / frag_chunks: the fragment-major copy of nsa_cmp_pack_fwd, which the one kernel reads instead of ck and cvt
 *   (cvt may be NULL when single_pass == 1); NULL = the one kernel is not available. */
int nsa_cmp_select_single_pass(int hq, int hkv, int dk, int dv, int pool_kernel, int pool_stride, int pool_pad,
                               int top_n, int max_nc, int dtype);
/* What the one kernel streams instead of ck / cvt: both in "fragment order", every 64-row chunk of a sequence stored
 * exactly as the matrix instructions consume it (1 KB per operand fragment), so that the kernel's global -> LDS copy
 * is a straight run of bytes done by the load unit and its LDS reads are free of bank conflicts.
 *   ck rows as above; cv [rows][hkv][dv] ROW-major (cv_row_stride / cv_head_stride in elements), not its transpose;
 *   frag: hkv * frag_chunks * 64 * (dk + dv) elements, frag_chunks >= nsa_cmp_pack_chunks(rows_bound, batch)
 *   (rows_bound >= all compressed rows of the batch; chunk c of sequence b sits at slot cu_cmp[b] / 64 + b + c).
 * 16-bit types, head dims (64,64), (128,128), (192,128).  No counterpart in the reference (Triton loads its tiles
 * from the row-major tensors). */
int nsa_cmp_pack_chunks(int total_rows, int batch);
int nsa_cmp_pack_fwd(const void* ck, const void* cv, void* frag, const int32_t* cu_cmp, int batch, int rows_bound, int hkv,
                     int dk, int dv, int64_t ck_row_stride, int64_t ck_head_stride, int64_t cv_row_stride,
                     int64_t cv_head_stride, int frag_chunks, int dtype, nsa_stream_t stream);
int nsa_cmp_select_fwd(const void* q, const void* ck, const void* cvt, const void* frag, int frag_chunks, void* o,
                       void* indices, float* pooled, float* lse,
                       float* lse_attn, const void* gate_weight, const void* gate_bias, void* gates,
                       const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch, int total, int hq, int hkv, int dk,
                       int dv, int64_t ck_row_stride, int64_t ck_head_stride, int cvt_cols, int block, int stride,
                       int pool_kernel, int pool_stride, int pool_pad, int top_n, int max_nc, int max_ns,
                       int pooled_stride, int keep_pooled, float scale, int causal, int idx64, int dtype,
                       int single_pass, nsa_stream_t stream);

/* Model integration: the glue between a layer's fused q/k/v(/gate) projection GEMM and the kernels
 * above.  The reference leaves this to its caller (nsa/nsa.py:83-135 receives q, k, v already split and
 * rotated) and computes the gate logits with a separate Linear (nsa/nsa.py:61,117); here the gating
 * weights are folded into the projection by the host, and one pass splits the packed GEMM rows
 *   packed [total][ld] = [ ... q (hq*dk) ... k (hkv*dk) ... v (hkv*dv) ... gate logits (3*hq) ... ]
 * into q [total][hq][dk], k [total][hkv][dk], v [total][hkv][dv], gates [total][hq][3] (gates may be
 * NULL), rotating channels [rope_off, rope_off + rope_dim) of every q and k head by the angles
 * position * inv_freq[i] (inv_freq fp32 [rope_dim/2], NULL = no rotation; interleaved = 0 pairs
 * channel i with i + rope_dim/2, 1 pairs 2i with 2i+1).  positions int32 [total], or NULL for the
 * offset inside the sequence given by cu_seqlens.  pack = 1 runs the transpose: gathers gradients
 * of the four tensors into packed rows with the inverse rotation.  Offsets and ld in elements. */
int nsa_qkv_rope(void* packed, void* q, void* k, void* v, void* gates, const float* inv_freq,
                 const int32_t* positions, const int32_t* cu_seqlens, int batch, int64_t total, int ld, int q_off,
                 int k_off, int v_off, int g_off, int hq, int hkv, int dk, int dv, int rope_off, int rope_dim,
                 int interleaved, int pack, int dtype, nsa_stream_t stream);

/* Gate logits of the three branches: gates[row][o] = bias[o] + q[row] . weight[o], o = 0 (selected),
 * 1 (sliding window), 2 (compressed).  Replaces the gating nn.Linear(head_dim, 3) of
 * nsa/nsa.py:61 as applied at nsa/nsa.py:117.  q [rows = total*hq, dim], weight [3, dim] (the
 * Linear's own layout), bias [3] or NULL, gates [rows, 3]; the activation is applied where the gates
 * are used (gate_act of the combine calls). */
int nsa_gate_fwd(const void* q, const void* weight, const void* bias, void* gates, int64_t rows, int dim, int dtype,
                 nsa_stream_t stream);

/* Backward of nsa_gate_fwd (autograd of the gating nn.Linear, nsa/nsa.py:61,117, in the reference):
 * d_gates [rows, 3] -> dq [rows, dim] = d_gates . weight (fully overwritten; the caller adds it to
 * the attention branches' dq), dweight float [3, dim] and dbias float [3] (NULL to skip), both
 * overwritten. */
int nsa_gate_bwd(const void* q, const void* weight, const void* d_gates, void* dq, float* dweight, float* dbias,
                 int64_t rows, int dim, int dtype, nsa_stream_t stream);

/* The gated sum on its own, for the training path, and its backward.  Replace the addcmul chain of
 * nsa/selection_attn.py:808-811 and nsa/nsa.py:133 and its autograd.
 *   gate_logits [rows, 3] (selected, sliding, compressed), pre-activation; o_* [rows, dv] (o_swa,
 *   o_cmp may be NULL: term dropped);  out = sum_b act(gate_b) * o_b.
 *   backward: d_b = act(gate_b) * d_out for every branch given, d_gate_logits[row][b] =
 *   act'(gate_b) * <d_out[row], o_b[row]> (0 for a missing branch).  stats (optional, float [6][rows])
 *   receives <d_out[row], o_b[row]> for b = selected, sliding, compressed and then act(gate_b): the
 *   delta / rowscale inputs of the attention backward entry points; with stats given the scaled copies
 *   d_slc / d_swa / d_cmp may be NULL (not written). */
int nsa_gate_combine_fwd(const void* gate_logits, const void* o_slc, const void* o_swa, const void* o_cmp, void* out,
                         int64_t rows, int dv, int gate_act, int dtype, nsa_stream_t stream);
int nsa_gate_combine_bwd(const void* gate_logits, const void* d_out, const void* o_slc, const void* o_swa,
                         const void* o_cmp, void* d_slc, void* d_swa, void* d_cmp, void* d_gate_logits, float* stats,
                         int64_t rows, int dv, int gate_act, int dtype, nsa_stream_t stream);

/* Sliding window attention: token t attends keys [max(0, t-window+1), t] of its sequence.  Replaces
 * the window loop of nsa/selection_attn.py:483-517.  q [total,hq,dk], k [total,hkv,dk],
 * vt transposed [hkv][dv][vt_cols] over cu_seqlens, o [total,hq,dv]; lse (optional, float
 * [total,hq]) receives the log-sum-exp of the scaled window scores (lse_swa of
 * nsa/selection_attn.py:492-515). */
int nsa_swa_fwd(const void* q, const void* k, const void* vt, void* o, float* lse, const int32_t* cu_seqlens,
                int batch, int total, int hq, int hkv, int dk, int dv, int vt_cols, int window,
                float scale, int dtype, nsa_stream_t stream);

/* Selected-block attention with the gated combine of the branches in the epilogue.  Replaces
 * nsa/selection_attn.py:401-481 (parallel_nsa_fwd_kernel, selected part), :808-811 and nsa/nsa.py:133.
 *   indices [total, hkv, top_n] block numbers local to the sequence (int32 / int64); entry i of
 *   token t is used iff i < counts[t,h] (counts NULL -> top_n), 0 <= idx and idx*block_size <= t.
 *   out = act(g_slc)*o_slc + act(g_swa)*o_swa + act(g_cmp)*o_cmp, where o_swa / o_cmp
 *   [total,hq,dv] may be NULL (term dropped), a NULL gate means 1, and gate (t,hq) is read at
 *   g[(t*hq + hq_idx)*gate_stride].  A token with no usable block has o_slc = 0.
 *   workspace (optional, nsa_slc_workspace_bytes) switches to the block-major schedule: every K/V
 *   block is loaded once and the queries that picked it are gathered, instead of gathering the
 *   blocks per token; results agree to rounding.  NULL keeps the token-major kernel.
 *   lse_slc (optional, float [total,hq]; block-major schedule only) receives the log-sum-exp of the
 *   scaled scores over the token's selected keys (lse_slc of nsa/selection_attn.py:476-481), +inf
 *   for a token without usable block. */
int nsa_slc_combine_fwd(const void* q, const void* k, const void* vt, const void* indices,
                        const int32_t* counts, const void* g_slc, const void* g_swa, const void* g_cmp,
                        int64_t gate_stride, const void* o_swa, const void* o_cmp, void* out, float* lse_slc,
                        const int32_t* cu_seqlens, int batch, int total, int hq, int hkv, int dk, int dv,
                        int vt_cols, int top_n, int block_size, float scale, int idx64, int gate_act,
                        int dtype, void* workspace, int64_t workspace_bytes, nsa_stream_t stream);

/* The block-major selected attention in two steps, with the merge folded into the sliding-window
 * kernel so that the window branch never goes to memory.  Same tensors, meaning and workspace
 * (nsa_slc_workspace_bytes, required here) as nsa_slc_combine_fwd; stands behind the same reference
 * lines plus the window loop nsa/selection_attn.py:483-517.
 *   nsa_slc_partials_fwd   buckets the (token, pick) pairs by K/V block and leaves one partial
 *                          softmax state per pair in the workspace;
 *   nsa_swa_merge_fwd      sliding-window attention whose epilogue merges those partials and writes
 *                          out = act(g_slc)*o_slc + act(g_swa)*o_swa + act(g_cmp)*o_cmp (o_cmp may be
 *                          NULL).  Must follow nsa_slc_partials_fwd on the same stream with the same
 *                          sizes; the workspace is only read (its slot map tells which picks have
 *                          a partial).  Optional outputs for a backward pass, written by the same
 *                          epilogue: o_slc_out / o_swa_out [total,hq,dv] (ungated branch outputs),
 *                          lse_slc_out / lse_swa_out (float [total,hq], as lse_slc above and lse of
 *                          nsa_swa_fwd).
 * bf16 or fp16; selection blocks of 8, 16, 32 or a multiple of 64 keys, top_n * max(1, block_size / 64) <= 64 (the schedule works on 64-key
 * blocks: a smaller selection block is a masked part of one, a larger one takes several slots per pick); other
 * shapes return NSA_ERR_UNSUPPORTED (use nsa_swa_fwd +
 * nsa_slc_combine_fwd). */
int nsa_slc_partials_fwd(const void* q, const void* k, const void* vt, const void* indices, const int32_t* counts,
                         const int32_t* cu_seqlens, int batch, int total, int hq, int hkv, int dk, int dv,
                         int vt_cols, int top_n, int block_size, float scale, int idx64, int dtype, void* workspace,
                         int64_t workspace_bytes, nsa_stream_t stream);
int nsa_swa_merge_fwd(const void* q, const void* k, const void* vt, const void* g_slc, const void* g_swa,
                      const void* g_cmp, int64_t gate_stride, const void* o_cmp, void* out,
                      const int32_t* cu_seqlens, int batch, int total, int hq, int hkv, int dk, int dv, int vt_cols,
                      int window, int top_n, int block_size, float scale, int gate_act, int dtype,
                      void* o_slc_out, void* o_swa_out, float* lse_slc_out, float* lse_swa_out,
                      const void* workspace, int64_t workspace_bytes, nsa_stream_t stream);

/* The same schedule as nsa_slc_partials_fwd + nsa_swa_merge_fwd in ONE call that walks the tokens in slabs, so
 * that the partial results need only the workspace the caller has: every slab is bucketed, attended per block
 * and merged in the window kernel's epilogue before the next one reuses the workspace (same stream order; the
 * result is bit-identical to the two-call form).  The slab is the largest number of token tiles whose pair list
 * and partial results fit workspace_bytes; nsa_slc_swa_fused_workspace_bytes gives the bytes for slabs of at
 * least slab_tokens tokens (slab_tokens <= 0: all tokens at once = nsa_slc_workspace_bytes), 0 when the shape
 * has no block-major schedule.  The slot map inside the workspace still covers every token (4 bytes per
 * (token, kv head, pick)).  Arguments as in the two entry points above. */
int64_t nsa_slc_swa_fused_workspace_bytes(int total, int batch, int hq, int hkv, int dk, int dv, int top_n,
                                          int block_size, int dtype, int slab_tokens);
int nsa_slc_swa_fused_fwd(const void* q, const void* k, const void* vt, const void* indices, const int32_t* counts,
                          const void* g_slc, const void* g_swa, const void* g_cmp, int64_t gate_stride,
                          const void* o_cmp, void* out, const int32_t* cu_seqlens, int batch, int total, int hq,
                          int hkv, int dk, int dv, int vt_cols, int window, int top_n, int block_size, float scale,
                          int idx64, int gate_act, int dtype, void* o_slc_out, void* o_swa_out, float* lse_slc_out,
                          float* lse_swa_out, void* workspace, int64_t workspace_bytes, nsa_stream_t stream);

/* Bytes of the optional workspace of nsa_slc_combine_fwd (an upper bound taken for GQA groups of 16 heads: the
 * partial results of groups of at most 8 / 4 heads have 8 / 4 rows, nsa_slc_swa_fused_workspace_bytes(..., 0) gives
 * the exact size, which the entry points accept); 0 when the shape has no block-major path
 * (bf16 or fp16; selection blocks of 8, 16, 32 or a multiple of 64 keys, top_n * max(1, block_size / 64) <= 64).  hkv: kv heads, times hq / (16 * hkv) when the GQA group has more
 * than 16 heads (one set of partial results per sub-group of 16 query heads). */
int64_t nsa_slc_workspace_bytes(int total, int batch, int hkv, int dk, int dv, int top_n, int block_size, int dtype);

/* Backward of the compressed attention.  Replaces nsa/triton_attention.py:478-546
 * (_attention.backward: _attn_bwd_preprocess, _attn_bwd with its dkdv / dq halves, :184-416).
 *   q [total,hq,dk], ck [cmp_rows,hkv,dk], cv [cmp_rows,hkv,dv] packed over cu_cmp (one row set per
 *   kv head, not repeated per q head), o / d_o [total,hq,dv] the forward output and its gradient,
 *   lse = lse_attn of nsa_cmp_attn_fwd.  Outputs dq [total,hq,dk], dck, dcv (shapes of ck, cv), all
 *   fully overwritten.  The block selection has no gradient (indices are integers).
 *   delta (optional, float [total,hq]): rowsum(o * d_o) when the caller already has it (o may then be
 *   NULL);  rowscale (optional, float [total,hq]): a per-row gate g — the results are those for the output
 *   gradient g * d_o with delta = rowsum(o * d_o) still the unscaled sum, so a gated sum of branches
 *   needs no scaled copy of d_o (nsa_gate_combine_bwd writes both arrays).
 *   workspace: nsa_cmp_attn_bwd_workspace_bytes, caller allocated. */
int64_t nsa_cmp_attn_bwd_workspace_bytes(int total, int cmp_rows, int hq, int hkv, int dk, int dv);
int nsa_cmp_attn_bwd(const void* q, const void* ck, const void* cv, const void* o, const void* d_o, const float* lse,
                     const float* delta, const float* rowscale, const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch, int total, int cmp_rows, int hq,
                     int hkv, int dk, int dv, int block, int stride, float scale, int causal, int dtype, void* dq,
                     void* dck, void* dcv, void* workspace, int64_t workspace_bytes, nsa_stream_t stream);

/* Backward of the selected and the sliding-window attention.  Replaces
 * nsa/selection_attn.py:715-737 (ParallelNSAFunction.backward -> parallel_nsa_bwd :151-398 with
 * parallel_nsa_bwd_kernel_preprocess, _dq, _dkv :520-676 and the block mask :60-87).
 *   q [total,hq,dk], k [total,hkv,dk], v [total,hkv,dv] (row-major, not the transposed copy);
 *   o_slc / d_o_slc / lse_slc: ungated output of the selected branch, its gradient, and lse_slc of
 *   nsa_slc_combine_fwd; o_swa / d_o_swa / lse_swa likewise for the window (lse of nsa_swa_fwd).
 *   A branch is skipped when its d_o is NULL.  indices / counts / idx64 / top_n / block_size as in
 *   nsa_slc_combine_fwd (selection blocks of 8, 16, 32 or a multiple of 64 keys, top_n * max(1, block_size / 64) <= 64).  dq [total,hq,dk], dk_out [total,hkv,dk], dv_out
 *   [total,hkv,dv] receive the sums over the branches present and are fully overwritten.
 *   delta_* / rowscale_* (optional, float [total,hq]) as in nsa_cmp_attn_bwd, per branch.
 *   dq_add (optional, [total,hq,dk], must not overlap dq): added to dq in the kernel that writes it, e.g. the
 *   dq of nsa_cmp_attn_bwd, so that the sum over all three branches needs no further pass.
 *   workspace: nsa_slc_swa_bwd_workspace_bytes (pass top_n = 0 there when the selected branch is
 *   skipped) runs the selected branch over all tokens at once.  A smaller workspace makes it walk the tokens in
 *   slabs (pair list and dQ partials then cover one slab; dK / dV accumulate over the slabs, every dq row is
 *   written by its slab): nsa_slc_swa_bwd_slab_workspace_bytes gives the bytes for slabs of at least slab_tokens
 *   tokens (counted in tiles of 64; slab_tokens <= 0: all tokens), and the call takes the largest slab its
 *   workspace_bytes hold; the least is one tile. */
int64_t nsa_slc_swa_bwd_slab_workspace_bytes(int total, int batch, int hq, int hkv, int dk, int dv, int top_n,
                                             int block_size, int dtype, int slab_tokens);
int64_t nsa_slc_swa_bwd_workspace_bytes(int total, int batch, int hq, int hkv, int dk, int dv, int top_n,
                                        int block_size, int dtype);
int nsa_slc_swa_bwd(const void* q, const void* k, const void* v, const void* o_slc, const void* o_swa,
                    const void* d_o_slc, const void* d_o_swa, const float* lse_slc, const float* lse_swa,
                    const float* delta_slc, const float* delta_swa, const float* rowscale_slc,
                    const float* rowscale_swa, const void* indices, const int32_t* counts,
                    const int32_t* cu_seqlens, int batch, int total, int hq,
                    int hkv, int dk, int dv, int top_n, int block_size, int window, float scale, int idx64, int dtype,
                    const void* dq_add, void* dq, void* dk_out, void* dv_out, void* workspace, int64_t workspace_bytes,
                    nsa_stream_t stream);

/* One-token decode step (no counterpart in the reference, which has no cache and no single-token
 * path; defined as the last row of the prefill forward on the same keys/values, mean-pool
 * compressor).  Cache layout, all zero-initialised by the owner:
 *   k_cache [batch][ctx_cap][hkv][dk]      v_cache_t [batch][hkv][dv][ctx_cap]      (ctx_cap % 64 == 0)
 *   ck_cache [batch][nc_cap][hkv][dk]      cv_cache_t [batch][hkv][dv][nc_cap]      (nc_cap % 64 == 0)
 * ctx_lens int32[batch]: tokens in each cache including the current one; q [batch][hq][dk] is the
 * query of that token; gates [batch][hq][3] (selected, sliding, compressed) or NULL (all ones);
 * out [batch][hq][dv]; indices (optional) int32 [batch][hkv][top_n] receives the selected blocks.
 * nc_cap <= nsa_decode_max_compressed() (the kernel keeps a sequence's compressed scores in the registers of
 * one workgroup; longer caches, up to nsa_decode_split_max_compressed() rows, go through
 * nsa_decode_step_split), a pooling geometry with at most nc_cap / 2 + 4 bins per sequence
 * (pool_stride >= 2) and a GQA group of at most 16 heads; anything else returns NSA_ERR_UNSUPPORTED and is served
 * by nsa_decode_step_split. */
int nsa_decode_max_compressed(void);
int nsa_decode_split_max_compressed(void);
int nsa_decode_step(const void* q, const void* k_cache, const void* v_cache_t, const void* ck_cache,
                    const void* cv_cache_t, const int32_t* ctx_lens, const void* gates, void* out, int32_t* indices,
                    int batch, int hq, int hkv, int dk, int dv, int ctx_cap, int nc_cap, int block, int stride,
                    int sel_block, int pool_kernel, int pool_stride, int pool_pad, int top_n, int window, float scale,
                    int gate_act, int dtype, nsa_stream_t stream);

/* The same step on a paged K/V cache (pages of 64 tokens = one selection block):
 *   k_pool [pages][64][hkv][dk]      v_pool_t [pages][hkv][dv][64]
 *   block_table int32 [batch][max_pages]: page i of sequence b holds its tokens [64 i, 64 i + 64)
 * The compressed caches stay contiguous per sequence as above.  Results are bit-identical to
 * nsa_decode_step on the same tokens.  Every table entry up to the page of token ctx_lens[b]-1 must
 * name a page of the pool; the library cannot check this.  Neither call has a counterpart in the
 * reference (it has no cache). */
int nsa_decode_step_paged(const void* q, const void* k_pool, const void* v_pool_t, const int32_t* block_table,
                          int max_pages, const void* ck_cache, const void* cv_cache_t, const int32_t* ctx_lens,
                          const void* gates, void* out, int32_t* indices, int batch, int hq, int hkv, int dk, int dv,
                          int nc_cap, int block, int stride, int sel_block, int pool_kernel, int pool_stride,
                          int pool_pad, int top_n, int window, float scale, int gate_act, int dtype,
                          nsa_stream_t stream);
int nsa_decode_append_paged(const void* k_new, const void* v_new, void* k_pool, void* v_pool_t,
                            const int32_t* block_table, int max_pages, void* ck_cache, void* cv_cache_t,
                            const int32_t* pos, int batch, int hkv, int dk, int dv, int nc_cap, int block, int stride,
                            int dtype, nsa_stream_t stream);

/* The same step for small batches: the work of every (sequence, kv head) pair is spread over `splits`
 * workgroups (three launches: compressed slices, selection + window / selected chunks, merge), because one
 * workgroup per pair leaves most of the chip idle below ~128 pairs.  block_table NULL = contiguous caches
 * (ctx_cap used), else the paged pool (max_pages used).  Any pooling geometry with at most 3136 pooled bins per
 * sequence (selection blocks of 32 keys at compression stride 16, which make more bins than the one-workgroup
 * step holds, run here).  The compressed rows are cut
 * into max(splits, ceil(nc_cap / 384)) <= 32 slices, so caches of up to nsa_decode_split_max_compressed() rows
 * (contexts of ~196k tokens at stride 16) are served whatever the batch.  The workspace holds
 * partial results only; calls that share it must not overlap.  GQA groups of 32, 48 or 64 heads (what the
 * reference's HQ % (16 * H) == 0 admits, nsa/selection_attn.py:800) run here and only here: every 16 heads of
 * a group are a pair of their own on the kv head's caches, the importance is summed over the whole group before
 * the top-n; size the workspace with hkv x (hq / hkv / 16) in place of hkv.  No counterpart in the reference. */
int64_t nsa_decode_split_workspace_bytes(int batch, int hkv, int dv, int nc_cap, int splits);
/* The same size for any pooling geometry (the one above is for windows of 5 every 4, and an upper bound for
 * windows of s + 1 every s >= 4). */
int64_t nsa_decode_split_pooled_workspace_bytes(int batch, int hkv, int dv, int nc_cap, int splits, int pool_kernel,
                                                int pool_stride, int pool_pad);
int nsa_decode_step_split(const void* q, const void* k_cache, const void* v_cache_t, const int32_t* block_table,
                          int max_pages, const void* ck_cache, const void* cv_cache_t, const int32_t* ctx_lens,
                          const void* gates, void* out, int32_t* indices, int batch, int hq, int hkv, int dk, int dv,
                          int ctx_cap, int nc_cap, int block, int stride, int sel_block, int pool_kernel,
                          int pool_stride, int pool_pad, int top_n, int window, float scale, int gate_act, int dtype,
                          int splits, void* workspace, int64_t workspace_bytes, nsa_stream_t stream);

/* nsa_decode_step_split for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the same three launches and the same results, bit for bit,
 * with the partial results in a fixed device array that is part of the library (nsa_decode_split_static_bytes()
 * = 16 MiB, held on every GPU the library runs on until the process ends) instead of a caller workspace.  The
 * call allocates and frees nothing; the first call on a device looks the array's address up.  Arguments as
 * nsa_decode_step_split without workspace / workspace_bytes.  Returns NSA_ERR_RESOURCE when
 * nsa_decode_split_pooled_workspace_bytes(batch, hkv * sub_groups, dv, nc_cap, splits, pool_kernel, pool_stride,
 * pool_pad) -- sub_groups = 16-head sub-groups of the GQA group, 1 up to 16 heads; the same figure as
 * nsa_decode_split_workspace_bytes(batch, hkv, dv, nc_cap, splits) for the default pooling of 5 rows every 4 --
 * exceeds the array (about 70 (sequence, kv head) pairs at 32k context, D 128, 8 splits).  All calls on one GPU share the array and it keeps the last call's
 * contents: calls that overlap in time on one GPU race, also across streams.  No counterpart in the reference,
 * which has no decode path and leaves every allocation to PyTorch. */
int64_t nsa_decode_split_static_bytes(void);
int nsa_decode_step_split_static(const void* q, const void* k_cache, const void* v_cache_t, const int32_t* block_table,
                                 int max_pages, const void* ck_cache, const void* cv_cache_t, const int32_t* ctx_lens,
                                 const void* gates, void* out, int32_t* indices, int batch, int hq, int hkv, int dk,
                                 int dv, int ctx_cap, int nc_cap, int block, int stride, int sel_block, int pool_kernel,
                                 int pool_stride, int pool_pad, int top_n, int window, float scale, int gate_act,
                                 int dtype, int splits, nsa_stream_t stream);

/* Appends one token per sequence: k_new [batch][hkv][dk] -> row pos[b] of k_cache, v_new
 * [batch][hkv][dv] -> column pos[b] of v_cache_t, and, when pos[b]+1 completes a compression block,
 * the mean of the last `block` tokens as the next row / column of the compressed caches. */
int nsa_decode_append(const void* k_new, const void* v_new, void* k_cache, void* v_cache_t, void* ck_cache,
                      void* cv_cache_t, const int32_t* pos, int batch, int hkv, int dk, int dv, int ctx_cap, int nc_cap,
                      int block, int stride, int dtype, nsa_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* NSA_HIP_H */
