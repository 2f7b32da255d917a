// extern "C" boundary of libnsa_hip.so: argument checks, error strings, dispatch to the launchers.
#include <stdio.h>
#include <stdarg.h>

#include "../../include/nsa_hip.h"
#include "common.h"
#include "kernels.h"

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int finish(int rc, const char* what) {
  if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "%s: head dims not built (dk,dv in (32,32),(64,64),(128,128),(192,128))", what);
  if (rc == -3) return fail(NSA_ERR_RESOURCE, "%s: needs more than 160 KB of LDS (sequence too long)", what);
  if (rc != 0) return fail(NSA_ERR_LAUNCH, "%s: could not configure the kernel", what);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NSA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return NSA_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// GQA groups of up to 16 heads are one MFMA tile column set.  The prefill forward also takes groups of 32, 48,
// 64, ... heads (what the reference's selected attention asks for: HQ a multiple of 16 * H,
// nsa/selection_attn.py:800): they run as hq / (16 * hkv) sub-groups of 16 heads that share the keys, values
// and block picks of their kv head.  *kv_rep receives that count (1 for groups up to 16).
int check_heads(const char* what, int hq, int hkv, int dk, int dv, int* kv_rep = nullptr) {
  if (hq <= 0 || hkv <= 0 || hq % hkv != 0) return fail(NSA_ERR_INVALID, "%s: hq must be a positive multiple of hkv", what);
  const int G = hq / hkv;
  if (kv_rep) *kv_rep = 1;
  if (G > 16) {
    if (!kv_rep) return fail(NSA_ERR_UNSUPPORTED, "%s: GQA group size %d > 16 is not built for this call", what, G);
    if (G % 16 != 0) return fail(NSA_ERR_UNSUPPORTED, "%s: GQA group size %d: groups beyond 16 heads must be multiples of 16", what, G);
    *kv_rep = G / 16;
  }
  if (dk % 32 != 0 || dv % 16 != 0) return fail(NSA_ERR_UNSUPPORTED, "%s: dk must be a multiple of 32 and dv of 16", what);
  return 0;
}

}  // namespace

extern "C" {

int nsa_version(void) { return 100; }
const char* nsa_last_error_string(void) { return g_err; }

int nsa_transposed_offset(int cu_b, int b) { return nsa::transposed_offset(cu_b, b); }
int nsa_transposed_cols(int total_rows, int batch) {
  const int need = nsa::transposed_offset(total_rows, batch) + 64;
  return (need + 63) / 64 * 64;
}

static bool dtype_ok(int dtype) { return dtype == NSA_BF16 || dtype == NSA_F32 || dtype == NSA_F16; }

int nsa_compress_fwd(const void* x, const void* wt, const void* bias, void* out, const int32_t* cu_seqlens,
                     const int32_t* cu_out, int batch, int out_rows_bound, int heads, int dim, int block,
                     int stride, int dtype, nsa_stream_t stream) {
  if (!x || !out || !cu_seqlens || !cu_out) return fail(NSA_ERR_INVALID, "compress: null pointer");
  if (batch <= 0 || heads <= 0 || block <= 0 || stride <= 0 || out_rows_bound < 0)
    return fail(NSA_ERR_INVALID, "compress: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "compress: bad dtype");
  if (dim % 8 != 0) return fail(NSA_ERR_UNSUPPORTED, "compress: dim must be a multiple of 8");
  if (!aligned16(x) || !aligned16(out) || (wt && !aligned16(wt))) return fail(NSA_ERR_INVALID, "compress: pointers must be 16-byte aligned");
  if (wt && dim % 32 != 0) return fail(NSA_ERR_UNSUPPORTED, "compress: weighted path needs dim %% 32 == 0");
  nsa::CompressArgs a{x, wt, bias, out, cu_seqlens, cu_out, batch, out_rows_bound, heads, dim, block, stride, dtype};
  const int rc = nsa::launch_compress(a, stream);
  if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "compress: weighted path is built for dim 32/64/128/192");
  return finish(rc, "compress");
}

int nsa_compress_kv_fwd(const void* k, const void* v, const void* wk_t, const void* wv_t, const void* bk,
                        const void* bv, void* ck, void* cv, const int32_t* cu_seqlens, const int32_t* cu_out,
                        int batch, int out_rows_bound, int heads, int dk, int dv, int block, int stride, int dtype,
                        nsa_stream_t stream) {
  if (!k || !v || !ck || !cv) return fail(NSA_ERR_INVALID, "compress_kv: null pointer");
  if ((wk_t == nullptr) != (wv_t == nullptr))
    return fail(NSA_ERR_INVALID, "compress_kv: give both weights or neither");
  if (wk_t && dtype != NSA_F32 && cu_seqlens && cu_out && batch > 0 && heads > 0 && block > 0 && stride > 0 &&
      out_rows_bound >= 0 && aligned16(k) && aligned16(v) && aligned16(ck) && aligned16(cv) && aligned16(wk_t) &&
      aligned16(wv_t)) {                        // learned compressor, 16-bit: both GEMMs in one launch
    nsa::CompressArgs a{k, wk_t, bk, ck, cu_seqlens, cu_out, batch, out_rows_bound, heads, dk, block, stride, dtype};
    a.x2 = v; a.out2 = cv; a.dim2 = dv; a.wt2 = wv_t; a.bias2 = bv;
    const int rc = nsa::launch_compress(a, stream);
    if (rc != -7) return finish(rc, "compress_kv");
  }
  if (wk_t) {                                   // otherwise one GEMM launch per tensor
    const int rc = nsa_compress_fwd(k, wk_t, bk, ck, cu_seqlens, cu_out, batch, out_rows_bound, heads, dk, block,
                                    stride, dtype, stream);
    if (rc != NSA_OK) return rc;
    return nsa_compress_fwd(v, wv_t, bv, cv, cu_seqlens, cu_out, batch, out_rows_bound, heads, dv, block, stride,
                            dtype, stream);
  }
  if (!cu_seqlens || !cu_out) return fail(NSA_ERR_INVALID, "compress_kv: null pointer");
  if (batch <= 0 || heads <= 0 || block <= 0 || stride <= 0 || out_rows_bound < 0)
    return fail(NSA_ERR_INVALID, "compress_kv: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "compress_kv: bad dtype");
  if (dk % 8 != 0 || dv % 8 != 0) return fail(NSA_ERR_UNSUPPORTED, "compress_kv: dims must be multiples of 8");
  if (!aligned16(k) || !aligned16(v) || !aligned16(ck) || !aligned16(cv))
    return fail(NSA_ERR_INVALID, "compress_kv: pointers must be 16-byte aligned");
  nsa::CompressArgs a{k, nullptr, nullptr, ck, cu_seqlens, cu_out, batch, out_rows_bound, heads, dk, block, stride, dtype};
  a.x2 = v; a.out2 = cv; a.dim2 = dv;
  return finish(nsa::launch_compress(a, stream), "compress_kv");
}

int nsa_compress_bwd(const void* x, const void* w_lin, const void* d_out, void* dx, float* dw, float* dbias,
                     const int32_t* cu_seqlens, const int32_t* cu_out, int batch, int total, int out_rows_bound,
                     int heads, int dim, int block, int stride, int dtype, nsa_stream_t stream) {
  if (!d_out || !dx || !cu_seqlens || !cu_out) return fail(NSA_ERR_INVALID, "compress_bwd: null pointer");
  if ((dw || dbias) && !w_lin) return fail(NSA_ERR_INVALID, "compress_bwd: weight gradients need the weight");
  if (dw && !x) return fail(NSA_ERR_INVALID, "compress_bwd: the weight gradient needs x");
  if (batch <= 0 || total <= 0 || heads <= 0 || block <= 0 || stride <= 0 || out_rows_bound < 0)
    return fail(NSA_ERR_INVALID, "compress_bwd: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "compress_bwd: bad dtype");
  if (dim % 8 != 0) return fail(NSA_ERR_UNSUPPORTED, "compress_bwd: dim must be a multiple of 8");
  if (!aligned16(d_out) || !aligned16(dx) || (x && !aligned16(x)) || (w_lin && !aligned16(w_lin)))
    return fail(NSA_ERR_INVALID, "compress_bwd: pointers must be 16-byte aligned");
  nsa::CompressBwdArgs a{x, w_lin, d_out, dx, dw, dbias, cu_seqlens, cu_out, batch, total, out_rows_bound, heads, dim,
                         block, stride, dtype};
  const int rc = nsa::launch_compress_bwd(a, stream);
  if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "compress_bwd: weighted path is built for dim 32/64/128/192");
  return finish(rc, "compress_bwd");
}

int nsa_transpose_fwd(const void* x, void* out, const int32_t* cu, int batch, int heads, int dim,
                      int64_t row_stride, int64_t head_stride, int out_cols, int dtype, nsa_stream_t stream) {
  if (!x || !out || !cu) return fail(NSA_ERR_INVALID, "transpose: null pointer");
  if (batch <= 0 || heads <= 0 || dim <= 0 || dim % 8 != 0 || out_cols <= 0 || out_cols % 64 != 0)
    return fail(NSA_ERR_INVALID, "transpose: dim must be a multiple of 8 and out_cols of 64");
  if (row_stride % 8 != 0 || head_stride % 8 != 0 || !aligned16(x) || !aligned16(out))
    return fail(NSA_ERR_INVALID, "transpose: strides must be multiples of 8 elements, pointers 16-byte aligned");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "transpose: bad dtype");
  nsa::TransposeArgs a{x, out, cu, batch, heads, dim, (long)row_stride, (long)head_stride, out_cols, dtype};
  return finish(nsa::launch_transpose(a, stream), "transpose");
}

static int cmp_common(const char* what, int stages, const void* q, const void* ck, const void* cvt, void* o,
                      void* indices, float* pooled, float* lse, float* lse_attn, const int32_t* cu_seqlens,
                      const int32_t* cu_cmp, int batch, int total, int hq, int hkv, int dk, int dv, int64_t ck_row_stride,
                      int64_t ck_head_stride, int cvt_cols, int block, int stride, int pool_kernel, int pool_stride,
                      int pool_pad, int top_n, int max_ns, int pooled_stride, int keep_pooled, float scale, int causal,
                      int idx64, int dtype, nsa_stream_t stream, const void* gate_w = nullptr,
                      const void* gate_b = nullptr, void* gates = nullptr, int single_pass_max_nc = -1,
                      int single_pass = 0, const void* frag = nullptr, int frag_chunks = 0) {
  // single_pass_max_nc >= 0 (stages 3 only): the most compressed rows of any sequence, with which the call may run
  // as ONE kernel (single_pass -1 = when the shape qualifies, 1 = or fail, 0 = never)
  const bool attn = stages & 1, select = stages & 2;
  if ((gate_w != nullptr) != (gates != nullptr) || (gate_b && !gate_w))
    return fail(NSA_ERR_INVALID, "%s: the gating Linear needs its weight and the gates buffer", what);
  if (gate_w && !aligned16(gate_w)) return fail(NSA_ERR_INVALID, "%s: pointers must be 16-byte aligned", what);
  if (!q || !ck || !cu_seqlens || !cu_cmp) return fail(NSA_ERR_INVALID, "%s: null pointer", what);
  if (attn && ((!cvt && !frag) || !o)) return fail(NSA_ERR_INVALID, "%s: null pointer", what);
  if (batch <= 0 || total <= 0 || block <= 0 || stride <= 0) return fail(NSA_ERR_INVALID, "%s: sizes must be positive", what);
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "%s: bad dtype", what);
  int kv_rep = 1;
  if (int rc = check_heads(what, hq, hkv, dk, dv, &kv_rep)) return rc;
  if (!(scale > 0.f)) return fail(NSA_ERR_INVALID, "%s: scale must be positive", what);
  if (ck_row_stride % 8 != 0 || ck_head_stride % 8 != 0 || (attn && cvt_cols % 64 != 0))
    return fail(NSA_ERR_INVALID, "%s: ck strides must be multiples of 8, cvt_cols of 64", what);
  if (!aligned16(q) || !aligned16(ck) || (attn && ((cvt && !aligned16(cvt)) || !aligned16(o))))
    return fail(NSA_ERR_INVALID, "%s: pointers must be 16-byte aligned", what);
  if (select) {
    if (!indices) return fail(NSA_ERR_INVALID, "%s: the selection needs indices and the lse buffer", what);
    if (pool_kernel <= 0 || pool_stride <= 0 || pool_pad < 0 || pool_pad >= pool_kernel || top_n <= 0 || max_ns < 0)
      return fail(NSA_ERR_INVALID, "%s: bad pooling / top-n parameters", what);
    if (pooled && pooled_stride < max_ns) return fail(NSA_ERR_INVALID, "%s: pooled_stride < max_ns", what);
  } else {
    max_ns = 0;
  }
  nsa::CmpArgs a{q, ck, cvt, o, indices, pooled, lse, cu_seqlens, cu_cmp, batch, total, hq, hkv * kv_rep, dk, dv,
                 (long)ck_row_stride, (long)ck_head_stride, cvt_cols, block, stride, pool_kernel, pool_stride,
                 pool_pad, top_n, max_ns, pooled_stride, scale, idx64, dtype, causal, lse_attn, kv_rep};
  a.keep_pooled = keep_pooled != 0;
  a.gate_w = gate_w; a.gate_b = gate_b; a.gates = gates;
  a.frag = frag; a.frag_chunks = frag_chunks;
  int rc = 0;
  if (frag && (!aligned16(frag) || frag_chunks < nsa::cmp_frag_chunks(0, batch)))
    return fail(NSA_ERR_INVALID, "%s: bad fragment-major copy (alignment / chunk slots)", what);
  if (attn && select && single_pass != 0 && single_pass_max_nc >= 0) {
    if (nsa::cmp_select_single_pass_ok(a, single_pass_max_nc)) return finish(nsa::launch_cmp_select(a, stream), what);
    if (single_pass == 1)
      return fail(NSA_ERR_UNSUPPORTED, "%s: the single-pass kernel takes GQA groups of 9..16 heads, 16-bit inputs, head dims "
                  "(64,64) (128,128) (192,128), pooling windows of 5 rows every 4 without padding, at most 2048 compressed "
                  "rows per sequence, top_n <= 64, and needs the fragment-major copy of nsa_cmp_pack_fwd", what);
  }
  if (attn && !cvt) return fail(NSA_ERR_INVALID, "%s: null pointer", what);
  if (select && !lse) return fail(NSA_ERR_INVALID, "%s: the selection needs indices and the lse buffer", what);
  if (attn) rc = nsa::launch_cmp_attn(a, stream);
  if (rc == 0 && select) rc = nsa::launch_select(a, stream);
  if (rc == -6)
    return fail(NSA_ERR_UNSUPPORTED, "%s: GQA groups beyond 16 heads are selected on the two-kernel schedule only "
                "(pooled buffer given, pooling windows of s + 1 every s with s = 1, 2, 4 or 8, i.e. selection blocks of 1, 2, 4 "
                "or 8 compression strides, max_ns <= 4096, top_n <= 64)", what);
  return finish(rc, what);
}

int nsa_cmp_attn_select_fwd(const void* q, const void* ck, const void* cvt, void* o, void* indices,
                            float* pooled, float* lse, const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch,
                            int total, int hq, int hkv, int dk, int dv, int64_t ck_row_stride,
                            int64_t ck_head_stride, int cvt_cols, int block, int stride, int pool_kernel,
                            int pool_stride, int pool_pad, int top_n, int max_ns, int pooled_stride,
                            int keep_pooled, float scale, int causal, int idx64, int dtype, nsa_stream_t stream) {
  return cmp_common("cmp_attn_select", indices ? 3 : 1, q, ck, cvt, o, indices, pooled, lse, nullptr, cu_seqlens, cu_cmp,
                    batch, total, hq, hkv, dk, dv, ck_row_stride, ck_head_stride, cvt_cols, block, stride,
                    pool_kernel, pool_stride, pool_pad, top_n, max_ns, pooled_stride, keep_pooled, scale, causal, idx64,
                    dtype, stream);
}

int nsa_cmp_select_single_pass(int hq, int hkv, int dk, int dv, int pool_kernel, int pool_stride, int pool_pad,
                               int top_n, int max_nc, int dtype) {
  if (hq <= 0 || hkv <= 0 || hq % hkv != 0) return 0;
  nsa::CmpArgs a{};
  a.hq = hq; a.hkv = hkv; a.dk = dk; a.dv = dv; a.pool_k = pool_kernel; a.pool_s = pool_stride; a.pool_p = pool_pad;
  a.top_n = top_n; a.dtype = dtype; a.kv_rep = hq / hkv > 16 ? 2 : 1;
  a.max_ns = max_nc >= 5 ? (max_nc - 2) / 4 + 1 : 0;
  static int dummy;
  a.indices = &dummy; a.frag = &dummy; a.o = &dummy;        // the shape test only asks whether they are given
  return nsa::cmp_select_single_pass_ok(a, max_nc) ? 1 : 0;
}

int nsa_cmp_pack_chunks(int total_rows, int batch) { return nsa::cmp_frag_chunks(total_rows, batch); }

int nsa_cmp_pack_fwd(const void* ck, const void* cv, void* frag, const int32_t* cu_cmp, int batch, int rows_bound, int hkv,
                     int dk, int dv, int64_t ck_row_stride, int64_t ck_head_stride, int64_t cv_row_stride,
                     int64_t cv_head_stride, int frag_chunks, int dtype, nsa_stream_t stream) {
  if (!ck || !cv || !frag || !cu_cmp) return fail(NSA_ERR_INVALID, "cmp_pack: null pointer");
  if (batch <= 0 || rows_bound < 0 || hkv <= 0) return fail(NSA_ERR_INVALID, "cmp_pack: sizes must be positive");
  if (dtype != NSA_BF16 && dtype != NSA_F16) return fail(NSA_ERR_UNSUPPORTED, "cmp_pack: 16-bit types only");
  if (ck_row_stride % 8 || ck_head_stride % 8 || cv_row_stride % 8 || cv_head_stride % 8 || !aligned16(ck) ||
      !aligned16(cv) || !aligned16(frag))
    return fail(NSA_ERR_INVALID, "cmp_pack: strides must be multiples of 8 elements, pointers 16-byte aligned");
  if (frag_chunks < nsa::cmp_frag_chunks(rows_bound, batch))
    return fail(NSA_ERR_INVALID, "cmp_pack: frag_chunks smaller than nsa_cmp_pack_chunks(rows_bound, batch)");
  nsa::CmpArgs a{};
  a.ck = ck; a.cvt = cv; a.frag = frag; a.frag_chunks = frag_chunks; a.cu_cmp = cu_cmp; a.batch = batch; a.hkv = hkv;
  a.dk = dk; a.dv = dv; a.ck_row_stride = (long)ck_row_stride; a.ck_head_stride = (long)ck_head_stride; a.dtype = dtype;
  const int rc = nsa::launch_frag_pack(a, (long)cv_row_stride, (long)cv_head_stride, rows_bound, stream);
  if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "cmp_pack: head dims (64,64), (128,128), (192,128)");
  return finish(rc, "cmp_pack");
}

int nsa_cmp_select_fwd(const void* q, const void* ck, const void* cvt, const void* frag, int frag_chunks, void* o,
                       void* indices, float* pooled, float* lse,
                       float* lse_attn, const void* gate_weight, const void* gate_bias, void* gates,
                       const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch, int total, int hq, int hkv, int dk,
                       int dv, int64_t ck_row_stride, int64_t ck_head_stride, int cvt_cols, int block, int stride,
                       int pool_kernel, int pool_stride, int pool_pad, int top_n, int max_nc, int max_ns,
                       int pooled_stride, int keep_pooled, float scale, int causal, int idx64, int dtype,
                       int single_pass, nsa_stream_t stream) {
  if (!indices) return fail(NSA_ERR_INVALID, "cmp_select: null pointer");
  if (max_nc < 0 || single_pass < -1 || single_pass > 1) return fail(NSA_ERR_INVALID, "cmp_select: bad max_nc / single_pass");
  return cmp_common("cmp_select", 3, q, ck, cvt, o, indices, pooled, lse, lse_attn, cu_seqlens, cu_cmp, batch, total, hq,
                    hkv, dk, dv, ck_row_stride, ck_head_stride, cvt_cols, block, stride, pool_kernel, pool_stride,
                    pool_pad, top_n, max_ns, pooled_stride, keep_pooled, scale, causal, idx64, dtype, stream, gate_weight,
                    gate_bias, gates, max_nc, single_pass, frag, frag_chunks);
}

int nsa_cmp_attn_fwd(const void* q, const void* ck, const void* cvt, void* o, float* lse, float* lse_attn,
                     const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch, int total, int hq, int hkv,
                     int dk, int dv, int64_t ck_row_stride, int64_t ck_head_stride, int cvt_cols, int block,
                     int stride, float scale, int causal, int dtype, nsa_stream_t stream) {
  return cmp_common("cmp_attn", 1, q, ck, cvt, o, nullptr, nullptr, lse, lse_attn, cu_seqlens, cu_cmp, batch, total, hq, hkv,
                    dk, dv, ck_row_stride, ck_head_stride, cvt_cols, block, stride, 1, 1, 0, 1, 0, 0, 0, scale, causal,
                    0, dtype, stream);
}

int nsa_cmp_attn_gate_fwd(const void* q, const void* ck, const void* cvt, void* o, float* lse, float* lse_attn,
                          const void* gate_weight, const void* gate_bias, void* gates, const int32_t* cu_seqlens,
                          const int32_t* cu_cmp, int batch, int total, int hq, int hkv, int dk, int dv,
                          int64_t ck_row_stride, int64_t ck_head_stride, int cvt_cols, int block, int stride,
                          float scale, int causal, int dtype, nsa_stream_t stream) {
  if (!gate_weight || !gates) return fail(NSA_ERR_INVALID, "cmp_attn_gate: null pointer");
  return cmp_common("cmp_attn_gate", 1, q, ck, cvt, o, nullptr, nullptr, lse, lse_attn, cu_seqlens, cu_cmp, batch, total, hq,
                    hkv, dk, dv, ck_row_stride, ck_head_stride, cvt_cols, block, stride, 1, 1, 0, 1, 0, 0, 0, scale,
                    causal, 0, dtype, stream, gate_weight, gate_bias, gates);
}

int nsa_block_select_fwd(const void* q, const void* ck, const float* lse, void* indices, float* pooled,
                         const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch, int total, int hq, int hkv,
                         int dk, int64_t ck_row_stride, int64_t ck_head_stride, int pool_kernel, int pool_stride,
                         int pool_pad, int top_n, int max_ns, int pooled_stride, int keep_pooled, int idx64,
                         int dtype, nsa_stream_t stream) {
  return cmp_common("block_select", 2, q, ck, nullptr, nullptr, indices, pooled, const_cast<float*>(lse), nullptr, cu_seqlens,
                    cu_cmp, batch, total, hq, hkv, dk, 16, ck_row_stride, ck_head_stride, 0, 1, 1, pool_kernel,
                    pool_stride, pool_pad, top_n, max_ns, pooled_stride, keep_pooled, 1.0f, 1, idx64, dtype, stream);
}

int nsa_qkv_rope(void* packed, void* q, void* k, void* v, void* gates, const float* inv_freq,
                 const int32_t* positions, const int32_t* cu_seqlens, int batch, int64_t total, int ld, int q_off,
                 int k_off, int v_off, int g_off, int hq, int hkv, int dk, int dv, int rope_off, int rope_dim,
                 int interleaved, int pack, int dtype, nsa_stream_t stream) {
  if (!packed || !q || !k || !v) return fail(NSA_ERR_INVALID, "qkv_rope: null pointer");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "qkv_rope: bad dtype");
  if (total <= 0 || hq <= 0 || hkv <= 0 || dk <= 0 || dv <= 0 || dk % 8 != 0 || dv % 8 != 0)
    return fail(NSA_ERR_INVALID, "qkv_rope: sizes must be positive and head dims multiples of 8");
  if (ld % 8 != 0 || q_off % 8 != 0 || k_off % 8 != 0 || v_off % 8 != 0 || q_off < 0 || k_off < 0 || v_off < 0 ||
      q_off + hq * dk > ld || k_off + hkv * dk > ld || v_off + hkv * dv > ld)
    return fail(NSA_ERR_INVALID, "qkv_rope: column offsets and row stride must be multiples of 8 inside the row");
  if (gates && (g_off < 0 || g_off + 3 * hq > ld)) return fail(NSA_ERR_INVALID, "qkv_rope: gate columns outside the row");
  if (inv_freq) {
    if (rope_dim <= 0 || rope_off < 0 || rope_off % 8 != 0 || rope_off + rope_dim > dk ||
        rope_dim % (interleaved ? 8 : 16) != 0)
      return fail(NSA_ERR_INVALID, "qkv_rope: rotary channels must be an 8-aligned range inside the head "
                                   "(length a multiple of 16, or of 8 when interleaved)");
    if (!positions && (!cu_seqlens || batch <= 0))
      return fail(NSA_ERR_INVALID, "qkv_rope: needs positions or cu_seqlens");
  }
  if (!aligned16(packed) || !aligned16(q) || !aligned16(k) || !aligned16(v))
    return fail(NSA_ERR_INVALID, "qkv_rope: pointers must be 16-byte aligned");
  nsa::QkvRopeArgs a{packed, q, k, v, gates, inv_freq, positions, cu_seqlens, batch, (long)total, ld, q_off, k_off,
                     v_off, g_off, hq, hkv, dk, dv, rope_off, rope_dim, interleaved ? 1 : 0, pack ? 1 : 0, dtype};
  const int rc = nsa::launch_qkv_rope(a, stream);
  if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "qkv_rope: more than 2^31-1 rows, 2^24 row elements or 256 rotary channels");
  return finish(rc, "qkv_rope");
}

int nsa_gate_fwd(const void* q, const void* weight, const void* bias, void* gates, int64_t rows, int dim, int dtype,
                 nsa_stream_t stream) {
  if (!q || !weight || !gates) return fail(NSA_ERR_INVALID, "gate: null pointer");
  if (rows <= 0 || dim <= 0 || dim % 8 != 0) return fail(NSA_ERR_INVALID, "gate: rows must be positive and dim a positive multiple of 8");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "gate: bad dtype");
  if (!aligned16(q) || !aligned16(weight)) return fail(NSA_ERR_INVALID, "gate: pointers must be 16-byte aligned");
  return finish(nsa::launch_gate(q, weight, bias, gates, (long)rows, dim, dtype, stream), "gate");
}

int nsa_gate_bwd(const void* q, const void* weight, const void* d_gates, void* dq, float* dweight, float* dbias,
                 int64_t rows, int dim, int dtype, nsa_stream_t stream) {
  if (!q || !weight || !d_gates || !dq || !dweight) return fail(NSA_ERR_INVALID, "gate_bwd: null pointer");
  if (rows <= 0 || dim <= 0 || dim % 8 != 0) return fail(NSA_ERR_INVALID, "gate_bwd: rows must be positive and dim a positive multiple of 8");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "gate_bwd: bad dtype");
  if (!aligned16(q) || !aligned16(weight) || !aligned16(dq)) return fail(NSA_ERR_INVALID, "gate_bwd: pointers must be 16-byte aligned");
  const int rc = nsa::launch_gate_bwd(q, weight, d_gates, dq, dweight, dbias, (long)rows, dim, dtype, stream);
  if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "gate_bwd: built for dim 32/64/128/192/256");
  return finish(rc, "gate_bwd");
}

static int gate_combine_common(const char* what, const nsa::GateCombineArgs& a, nsa_stream_t stream) {
  if (!a.gate_logits || !a.o_slc) return fail(NSA_ERR_INVALID, "%s: null pointer", what);
  if (a.rows <= 0 || a.dv <= 0 || a.dv % 8 != 0) return fail(NSA_ERR_INVALID, "%s: rows must be positive and dv a positive multiple of 8", what);
  if (!dtype_ok(a.dtype)) return fail(NSA_ERR_INVALID, "%s: bad dtype", what);
  if (a.act != NSA_GATE_IDENTITY && a.act != NSA_GATE_SIGMOID) return fail(NSA_ERR_INVALID, "%s: bad gate activation", what);
  const void* ptrs[] = {a.o_slc, a.o_swa, a.o_cmp, a.out, a.d_out, a.d_slc, a.d_swa, a.d_cmp};
  for (const void* p : ptrs)
    if (p && !aligned16(p)) return fail(NSA_ERR_INVALID, "%s: pointers must be 16-byte aligned", what);
  return finish(nsa::launch_gate_combine(a, stream), what);
}

int nsa_gate_combine_fwd(const void* gate_logits, const void* o_slc, const void* o_swa, const void* o_cmp, void* out,
                         int64_t rows, int dv, int gate_act, int dtype, nsa_stream_t stream) {
  if (!out) return fail(NSA_ERR_INVALID, "gate_combine: null pointer");
  nsa::GateCombineArgs a{gate_logits, o_slc, o_swa, o_cmp, out, nullptr, nullptr, nullptr, nullptr, nullptr,
                         (long)rows, dv, gate_act, dtype, nullptr};
  return gate_combine_common("gate_combine", a, stream);
}

int nsa_gate_combine_bwd(const void* gate_logits, const void* d_out, const void* o_slc, const void* o_swa,
                         const void* o_cmp, void* d_slc, void* d_swa, void* d_cmp, void* d_gate_logits, float* stats,
                         int64_t rows, int dv, int gate_act, int dtype, nsa_stream_t stream) {
  if (!d_out || !d_gate_logits) return fail(NSA_ERR_INVALID, "gate_combine_bwd: null pointer");
  if (!stats && (!d_slc || (o_swa && !d_swa) || (o_cmp && !d_cmp)))
    return fail(NSA_ERR_INVALID, "gate_combine_bwd: null pointer (every branch given needs its gradient buffer unless stats is requested)");
  nsa::GateCombineArgs a{gate_logits, o_slc, o_swa, o_cmp, nullptr, d_out, d_slc, d_swa, d_cmp, d_gate_logits,
                         (long)rows, dv, gate_act, dtype, stats};
  return gate_combine_common("gate_combine_bwd", a, stream);
}

int nsa_swa_fwd(const void* q, const void* k, const void* vt, void* o, float* lse, const int32_t* cu_seqlens, int batch,
                int total, int hq, int hkv, int dk, int dv, int vt_cols, int window, float scale, int dtype,
                nsa_stream_t stream) {
  if (!q || !k || !vt || !o || !cu_seqlens) return fail(NSA_ERR_INVALID, "swa: null pointer");
  if (batch <= 0 || total <= 0 || window <= 0) return fail(NSA_ERR_INVALID, "swa: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "swa: bad dtype");
  int kv_rep = 1;
  if (int rc = check_heads("swa", hq, hkv, dk, dv, &kv_rep)) return rc;
  if (!(scale > 0.f)) return fail(NSA_ERR_INVALID, "swa: scale must be positive");
  if (vt_cols % 64 != 0 || vt_cols < nsa_transposed_cols(total, batch)) return fail(NSA_ERR_INVALID, "swa: vt_cols too small or not a multiple of 64");
  if (!aligned16(q) || !aligned16(k) || !aligned16(vt) || !aligned16(o)) return fail(NSA_ERR_INVALID, "swa: pointers must be 16-byte aligned");
  nsa::SwaArgs a{q, k, vt, o, cu_seqlens, batch, total, hq, hkv * kv_rep, dk, dv, vt_cols, window, scale, dtype, lse, kv_rep};
  return finish(nsa::launch_swa(a, stream), "swa");
}

int64_t nsa_slc_workspace_bytes(int total, int batch, int hkv, int dk, int dv, int top_n, int block_size, int dtype) {
  nsa::SlcArgs a{};
  a.total = total; a.batch = batch; a.hkv = hkv; a.dk = dk; a.dv = dv; a.top_n = top_n; a.block_size = block_size;
  a.dtype = dtype;
  if (total <= 0 || batch <= 0 || hkv <= 0 || top_n <= 0 || !nsa::slc_block_major_ok(a)) return 0;
  return nsa::slc_workspace_bytes(a);
}

int nsa_slc_combine_fwd(const void* q, const void* k, const void* vt, const void* indices, const int32_t* counts,
                        const void* g_slc, const void* g_swa, const void* g_cmp, int64_t gate_stride,
                        const void* o_swa, const void* o_cmp, void* out, float* lse_slc, const int32_t* cu_seqlens,
                        int batch, int total, int hq, int hkv, int dk, int dv, int vt_cols, int top_n, int block_size,
                        float scale, int idx64, int gate_act, int dtype, void* workspace, int64_t workspace_bytes,
                        nsa_stream_t stream) {
  if (!q || !k || !vt || !indices || !out || !cu_seqlens) return fail(NSA_ERR_INVALID, "slc_combine: null pointer");
  if (batch <= 0 || total <= 0) return fail(NSA_ERR_INVALID, "slc_combine: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "slc_combine: bad dtype");
  int kv_rep = 1;
  if (int rc = check_heads("slc_combine", hq, hkv, dk, dv, &kv_rep)) return rc;
  if (!(scale > 0.f)) return fail(NSA_ERR_INVALID, "slc_combine: scale must be positive");
  if (top_n <= 0 || top_n > 64) return fail(NSA_ERR_UNSUPPORTED, "slc_combine: 1 <= top_n <= 64");
  if (block_size <= 0 || block_size % 8 != 0) return fail(NSA_ERR_UNSUPPORTED, "slc_combine: block_size must be a multiple of 8");
  if (vt_cols % 64 != 0 || vt_cols < nsa_transposed_cols(total, batch)) return fail(NSA_ERR_INVALID, "slc_combine: vt_cols too small or not a multiple of 64");
  if (gate_act != NSA_GATE_IDENTITY && gate_act != NSA_GATE_SIGMOID) return fail(NSA_ERR_INVALID, "slc_combine: bad gate activation");
  if (!aligned16(q) || !aligned16(k) || !aligned16(vt)) return fail(NSA_ERR_INVALID, "slc_combine: pointers must be 16-byte aligned");
  nsa::SlcArgs a{q, k, vt, indices, counts, g_slc, g_swa, g_cmp, (long)gate_stride, o_swa, o_cmp, out, cu_seqlens,
                 batch, total, hq, hkv * kv_rep, dk, dv, vt_cols, top_n, block_size, scale, idx64, gate_act, dtype,
                 workspace, (long)workspace_bytes, lse_slc, kv_rep};
  if (workspace && !aligned16(workspace)) return fail(NSA_ERR_INVALID, "slc_combine: workspace must be 16-byte aligned");
  const int rc = nsa::launch_slc_combine(a, stream);
  if (rc == -5) return fail(NSA_ERR_UNSUPPORTED, "slc_combine: lse_slc needs the block-major schedule (bf16 or fp16, selection blocks of 8, 16, 32 or a multiple of 64 keys, a workspace)");
  return finish(rc, "slc_combine");
}

static int slc_common_checks(const char* what, const void* q, const void* k, const void* vt, const int32_t* cu_seqlens,
                             int batch, int total, int hq, int hkv, int dk, int dv, int vt_cols, int top_n,
                             int block_size, float scale, int dtype, const void* workspace, int64_t workspace_bytes,
                             int* kv_rep) {
  if (!q || !k || !vt || !cu_seqlens || !workspace) return fail(NSA_ERR_INVALID, "%s: null pointer", what);
  if (batch <= 0 || total <= 0) return fail(NSA_ERR_INVALID, "%s: sizes must be positive", what);
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "%s: bad dtype", what);
  if (int rc = check_heads(what, hq, hkv, dk, dv, kv_rep)) return rc;
  if (!(scale > 0.f)) return fail(NSA_ERR_INVALID, "%s: scale must be positive", what);
  if (vt_cols % 64 != 0 || vt_cols < nsa_transposed_cols(total, batch)) return fail(NSA_ERR_INVALID, "%s: vt_cols too small or not a multiple of 64", what);
  if (!aligned16(q) || !aligned16(k) || !aligned16(vt) || !aligned16(workspace)) return fail(NSA_ERR_INVALID, "%s: pointers must be 16-byte aligned", what);
  // with the query heads known the partial results have as many rows as the (padded) GQA group, not 16
  const int64_t need = nsa_slc_swa_fused_workspace_bytes(total, batch, hq, hkv, dk, dv, top_n, block_size, dtype, 0);
  if (need == 0) return fail(NSA_ERR_UNSUPPORTED, "%s: the block-major schedule needs bf16 or fp16, selection blocks of 8, 16, 32 or a multiple of 64 keys, top_n * max(1, block_size / 64) <= 64 and (dk,dv) in (64,64),(128,128),(192,128)", what);
  if (workspace_bytes < need) return fail(NSA_ERR_INVALID, "%s: workspace smaller than nsa_slc_workspace_bytes", what);
  return 0;
}

int nsa_slc_partials_fwd(const void* q, const void* k, const void* vt, const void* indices, const int32_t* counts,
                         const int32_t* cu_seqlens, int batch, int total, int hq, int hkv, int dk, int dv,
                         int vt_cols, int top_n, int block_size, float scale, int idx64, int dtype, void* workspace,
                         int64_t workspace_bytes, nsa_stream_t stream) {
  if (!indices) return fail(NSA_ERR_INVALID, "slc_partials: null pointer");
  int kv_rep = 1;
  if (int rc = slc_common_checks("slc_partials", q, k, vt, cu_seqlens, batch, total, hq, hkv, dk, dv, vt_cols, top_n,
                                 block_size, scale, dtype, workspace, workspace_bytes, &kv_rep)) return rc;
  nsa::SlcArgs a{q, k, vt, indices, counts, nullptr, nullptr, nullptr, 1, nullptr, nullptr, nullptr, cu_seqlens,
                 batch, total, hq, hkv * kv_rep, dk, dv, vt_cols, top_n, block_size, scale, idx64, 0, dtype,
                 workspace, (long)workspace_bytes, nullptr, kv_rep};
  return finish(nsa::launch_slc_partials(a, workspace, stream), "slc_partials");
}

int nsa_swa_merge_fwd(const void* q, const void* k, const void* vt, const void* g_slc, const void* g_swa,
                      const void* g_cmp, int64_t gate_stride, const void* o_cmp, void* out,
                      const int32_t* cu_seqlens, int batch, int total, int hq, int hkv, int dk, int dv, int vt_cols,
                      int window, int top_n, int block_size, float scale, int gate_act, int dtype,
                      void* o_slc_out, void* o_swa_out, float* lse_slc_out, float* lse_swa_out,
                      const void* workspace, int64_t workspace_bytes, nsa_stream_t stream) {
  if (!out) return fail(NSA_ERR_INVALID, "swa_merge: null pointer");
  if ((o_slc_out && !aligned16(o_slc_out)) || (o_swa_out && !aligned16(o_swa_out)))
    return fail(NSA_ERR_INVALID, "swa_merge: pointers must be 16-byte aligned");
  if (window <= 0) return fail(NSA_ERR_INVALID, "swa_merge: window must be positive");
  if (gate_act != NSA_GATE_IDENTITY && gate_act != NSA_GATE_SIGMOID) return fail(NSA_ERR_INVALID, "swa_merge: bad gate activation");
  int kv_rep = 1;
  if (int rc = slc_common_checks("swa_merge", q, k, vt, cu_seqlens, batch, total, hq, hkv, dk, dv, vt_cols, top_n,
                                 block_size, scale, dtype, workspace, workspace_bytes, &kv_rep)) return rc;
  if (!aligned16(out) || (o_cmp && !aligned16(o_cmp))) return fail(NSA_ERR_INVALID, "swa_merge: pointers must be 16-byte aligned");
  // the picks themselves are not needed here: the workspace's slot map says which have a partial
  nsa::SlcArgs sa{q, k, vt, nullptr, nullptr, g_slc, g_swa, g_cmp, (long)gate_stride, nullptr, o_cmp, out, cu_seqlens,
                  batch, total, hq, hkv * kv_rep, dk, dv, vt_cols, top_n, block_size, scale, 0, gate_act, dtype,
                  const_cast<void*>(workspace), (long)workspace_bytes, nullptr, kv_rep};
  nsa::MergeArgs m = nsa::slc_merge_args(sa, const_cast<void*>(workspace));
  m.o_slc_out = o_slc_out; m.o_swa_out = o_swa_out; m.lse_slc_out = lse_slc_out;
  nsa::SwaArgs a{q, k, vt, nullptr, cu_seqlens, batch, total, hq, hkv * kv_rep, dk, dv, vt_cols, window, scale, dtype,
                 lse_swa_out, kv_rep};
  return finish(nsa::launch_swa_merge(a, m, stream), "swa_merge");
}

// Block-major selected attention + window attention + merge, one slab of token tiles at a time: the slab is as
// large as the workspace allows, so the partial results need workspace_bytes, not nsa_slc_workspace_bytes.
static nsa::SlcArgs fused_slab_args(int total, int batch, int hq, int hkv, int dk, int dv, int top_n, int block_size,
                                    int dtype, int tiles) {
  nsa::SlcArgs a{};
  a.total = total; a.batch = batch; a.hq = hq; a.hkv = hkv; a.dk = dk; a.dv = dv; a.top_n = top_n;
  a.block_size = block_size; a.dtype = dtype;
  a.tile_tokens = nsa::swa_tile_tokens(hq, hkv, dtype);
  a.tile_begin = 0; a.tile_count = tiles;
  return a;
}

int64_t nsa_slc_swa_fused_workspace_bytes(int total, int batch, int hq, int hkv, int dk, int dv, int top_n,
                                          int block_size, int dtype, int slab_tokens) {
  if (total <= 0 || batch <= 0 || hq <= 0 || hkv <= 0 || top_n <= 0 || hq % hkv != 0) return 0;
  int g = hq / hkv, kv_rep = 1;
  if (g > 16) { if (g % 16) return 0; kv_rep = g / 16; }
  nsa::SlcArgs a = fused_slab_args(total, batch, hq, hkv * kv_rep, dk, dv, top_n, block_size, dtype, 0);
  if (!nsa::slc_block_major_ok(a)) return 0;
  if (slab_tokens > 0 && slab_tokens < total) a.tile_count = (slab_tokens + a.tile_tokens - 1) / a.tile_tokens;
  return nsa::slc_workspace_bytes(a);
}

int nsa_slc_swa_fused_fwd(const void* q, const void* k, const void* vt, const void* indices, const int32_t* counts,
                          const void* g_slc, const void* g_swa, const void* g_cmp, int64_t gate_stride,
                          const void* o_cmp, void* out, const int32_t* cu_seqlens, int batch, int total, int hq,
                          int hkv, int dk, int dv, int vt_cols, int window, int top_n, int block_size, float scale,
                          int idx64, int gate_act, int dtype, void* o_slc_out, void* o_swa_out, float* lse_slc_out,
                          float* lse_swa_out, void* workspace, int64_t workspace_bytes, nsa_stream_t stream) {
  const char* what = "slc_swa_fused";
  if (!q || !k || !vt || !indices || !out || !cu_seqlens || !workspace) return fail(NSA_ERR_INVALID, "%s: null pointer", what);
  if (batch <= 0 || total <= 0) return fail(NSA_ERR_INVALID, "%s: sizes must be positive", what);
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "%s: bad dtype", what);
  int kv_rep = 1;
  if (int rc = check_heads(what, hq, hkv, dk, dv, &kv_rep)) return rc;
  if (!(scale > 0.f)) return fail(NSA_ERR_INVALID, "%s: scale must be positive", what);
  if (window <= 0) return fail(NSA_ERR_INVALID, "%s: window must be positive", what);
  if (top_n <= 0) return fail(NSA_ERR_INVALID, "%s: top_n must be positive", what);
  if (gate_act != NSA_GATE_IDENTITY && gate_act != NSA_GATE_SIGMOID) return fail(NSA_ERR_INVALID, "%s: bad gate activation", what);
  if (vt_cols % 64 != 0 || vt_cols < nsa_transposed_cols(total, batch)) return fail(NSA_ERR_INVALID, "%s: vt_cols too small or not a multiple of 64", what);
  if (!aligned16(q) || !aligned16(k) || !aligned16(vt) || !aligned16(workspace) || !aligned16(out) ||
      (o_cmp && !aligned16(o_cmp)) || (o_slc_out && !aligned16(o_slc_out)) || (o_swa_out && !aligned16(o_swa_out)))
    return fail(NSA_ERR_INVALID, "%s: pointers must be 16-byte aligned", what);
  const int hv = hkv * kv_rep;
  nsa::SlcArgs probe = fused_slab_args(total, batch, hq, hv, dk, dv, top_n, block_size, dtype, 0);
  if (!nsa::slc_block_major_ok(probe))
    return fail(NSA_ERR_UNSUPPORTED, "%s: the block-major schedule needs bf16 or fp16, selection blocks of 8, 16, 32 or a multiple of 64 keys, top_n * max(1, block_size / 64) <= 64 and (dk,dv) in (32,32),(64,64),(128,128),(192,128)", what);
  // the largest slab (in tiles) whose workspace fits
  const int tile_tokens = probe.tile_tokens, total_tiles = total / tile_tokens + batch;
  auto bytes_for = [&](int tiles) { probe.tile_count = tiles; return (int64_t)nsa::slc_workspace_bytes(probe); };
  if (bytes_for(1) > workspace_bytes) return fail(NSA_ERR_INVALID, "%s: workspace smaller than nsa_slc_swa_fused_workspace_bytes for one tile of %d tokens", what, tile_tokens);
  int lo = 1, hi = total_tiles;
  while (lo < hi) {
    const int mid = lo + (hi - lo + 1) / 2;
    if (bytes_for(mid) <= workspace_bytes) lo = mid; else hi = mid - 1;
  }
  const int slab_tiles = lo;
  for (int t0 = 0; t0 < total_tiles; t0 += slab_tiles) {
    const int cnt = slab_tiles < total_tiles - t0 ? slab_tiles : total_tiles - t0;
    nsa::SlcArgs sa{q, k, vt, indices, counts, g_slc, g_swa, g_cmp, (long)gate_stride, nullptr, o_cmp, out, cu_seqlens,
                    batch, total, hq, hv, dk, dv, vt_cols, top_n, block_size, scale, idx64, gate_act, dtype,
                    workspace, (long)workspace_bytes, nullptr, kv_rep};
    sa.tile_tokens = tile_tokens; sa.tile_begin = t0; sa.tile_count = slab_tiles;   // capacity: always a full slab
    int rc = nsa::launch_slc_partials(sa, workspace, stream);
    if (rc) return finish(rc, what);
    nsa::MergeArgs m = nsa::slc_merge_args(sa, workspace);
    m.o_slc_out = o_slc_out; m.o_swa_out = o_swa_out; m.lse_slc_out = lse_slc_out;
    nsa::SwaArgs wa{q, k, vt, nullptr, cu_seqlens, batch, total, hq, hv, dk, dv, vt_cols, window, scale, dtype,
                    lse_swa_out, kv_rep};
    wa.tile_begin = t0; wa.tile_count = cnt;
    rc = nsa::launch_swa_merge(wa, m, stream);
    if (rc) return finish(rc, what);
  }
  return finish(0, what);
}

int64_t nsa_cmp_attn_bwd_workspace_bytes(int total, int cmp_rows, int hq, int hkv, int dk, int dv) {
  if (total <= 0 || cmp_rows < 0 || hq <= 0 || hkv <= 0 || dk <= 0 || dv <= 0) return 0;
  nsa::CmpBwdArgs a{};
  a.total = total; a.cmp_rows = cmp_rows; a.hq = hq; a.hkv = hkv; a.dk = dk; a.dv = dv;
  return nsa::cmp_bwd_workspace_bytes(a);
}

int nsa_cmp_attn_bwd(const void* q, const void* ck, const void* cv, const void* o, const void* d_o, const float* lse,
                     const float* delta, const float* rowscale, const int32_t* cu_seqlens, const int32_t* cu_cmp, int batch, int total, int cmp_rows, int hq,
                     int hkv, int dk, int dv, int block, int stride, float scale, int causal, int dtype, void* dq,
                     void* dck, void* dcv, void* workspace, int64_t workspace_bytes, nsa_stream_t stream) {
  if (!q || (!o && !delta) || !d_o || !lse || !cu_seqlens || !cu_cmp || !dq || !workspace)
    return fail(NSA_ERR_INVALID, "cmp_attn_bwd: null pointer");
  if (cmp_rows > 0 && (!ck || !cv || !dck || !dcv)) return fail(NSA_ERR_INVALID, "cmp_attn_bwd: null pointer");
  if (batch <= 0 || total <= 0 || cmp_rows < 0 || block <= 0 || stride <= 0)
    return fail(NSA_ERR_INVALID, "cmp_attn_bwd: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "cmp_attn_bwd: bad dtype");
  if (int rc = check_heads("cmp_attn_bwd", hq, hkv, dk, dv)) return rc;
  if (!(scale > 0.f)) return fail(NSA_ERR_INVALID, "cmp_attn_bwd: scale must be positive");
  if (!aligned16(q) || !aligned16(ck) || !aligned16(cv) || (o && !aligned16(o)) || !aligned16(d_o) || !aligned16(dq) ||
      !aligned16(dck) || !aligned16(dcv) || !aligned16(workspace))
    return fail(NSA_ERR_INVALID, "cmp_attn_bwd: pointers must be 16-byte aligned");
  if (workspace_bytes < nsa_cmp_attn_bwd_workspace_bytes(total, cmp_rows, hq, hkv, dk, dv))
    return fail(NSA_ERR_INVALID, "cmp_attn_bwd: workspace smaller than nsa_cmp_attn_bwd_workspace_bytes");
  nsa::CmpBwdArgs a{q, ck, cv, o, d_o, lse, cu_seqlens, cu_cmp, batch, total, cmp_rows, hq, hkv, dk, dv, block, stride,
                    causal, scale, dtype, dq, dck, dcv, workspace, delta, rowscale};
  const int rc = nsa::launch_cmp_bwd(a, stream);
  if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "cmp_attn_bwd: head dims not built (dk,dv in (32,32),(64,64),(128,128),(192,128); fp32: no 192)");
  return finish(rc, "cmp_attn_bwd");
}

int64_t nsa_slc_swa_bwd_workspace_bytes(int total, int batch, int hq, int hkv, int dk, int dv, int top_n,
                                        int block_size, int dtype) {
  if (total <= 0 || batch <= 0 || hq <= 0 || hkv <= 0 || dk <= 0 || dv <= 0 || top_n < 0) return 0;
  nsa::SlcSwaBwdArgs a{};
  a.total = total; a.batch = batch; a.hq = hq; a.hkv = hkv; a.dk = dk; a.dv = dv; a.top_n = top_n;
  a.block_size = block_size; a.dtype = dtype;
  return nsa::slc_swa_bwd_workspace_bytes(a);
}

int64_t nsa_slc_swa_bwd_slab_workspace_bytes(int total, int batch, int hq, int hkv, int dk, int dv, int top_n,
                                             int block_size, int dtype, int slab_tokens) {
  if (total <= 0 || batch <= 0 || hq <= 0 || hkv <= 0 || dk <= 0 || dv <= 0 || top_n < 0) return 0;
  nsa::SlcSwaBwdArgs a{};
  a.total = total; a.batch = batch; a.hq = hq; a.hkv = hkv; a.dk = dk; a.dv = dv; a.top_n = top_n;
  a.block_size = block_size; a.dtype = dtype;
  return nsa::slc_swa_bwd_slab_workspace_bytes(a, slab_tokens);
}

int nsa_slc_swa_bwd(const void* q, const void* k, const void* v, const void* o_slc, const void* o_swa,
                    const void* d_o_slc, const void* d_o_swa, const float* lse_slc, const float* lse_swa,
                    const float* delta_slc, const float* delta_swa, const float* rowscale_slc,
                    const float* rowscale_swa, const void* indices, const int32_t* counts,
                    const int32_t* cu_seqlens, int batch, int total, int hq,
                    int hkv, int dk, int dv, int top_n, int block_size, int window, float scale, int idx64, int dtype,
                    const void* dq_add, void* dq, void* dk_out, void* dv_out, void* workspace,
                    int64_t workspace_bytes, nsa_stream_t stream) {
  if (!q || !k || !v || !cu_seqlens || !dq || !dk_out || !dv_out || !workspace)
    return fail(NSA_ERR_INVALID, "slc_swa_bwd: null pointer");
  if (dq_add && (dq_add == dq || !aligned16(dq_add)))
    return fail(NSA_ERR_INVALID, "slc_swa_bwd: dq_add must be 16-byte aligned and must not be dq");
  const bool slc = d_o_slc != nullptr, swa = d_o_swa != nullptr;
  if (slc && ((!o_slc && !delta_slc) || !lse_slc || !indices || top_n <= 0)) return fail(NSA_ERR_INVALID, "slc_swa_bwd: the selected branch needs o_slc, lse_slc, indices and top_n > 0");
  if (swa && ((!o_swa && !delta_swa) || !lse_swa || window <= 0)) return fail(NSA_ERR_INVALID, "slc_swa_bwd: the sliding branch needs o_swa, lse_swa and window > 0");
  if (batch <= 0 || total <= 0) return fail(NSA_ERR_INVALID, "slc_swa_bwd: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "slc_swa_bwd: bad dtype");
  if (int rc = check_heads("slc_swa_bwd", hq, hkv, dk, dv)) return rc;
  if (!(scale > 0.f)) return fail(NSA_ERR_INVALID, "slc_swa_bwd: scale must be positive");
  if (slc && (!nsa::slc_block_size_ok(block_size) || (long)top_n * (block_size > 64 ? block_size / 64 : 1) > 64 ||
              total >= (1 << 26)))
    return fail(NSA_ERR_UNSUPPORTED, "slc_swa_bwd: the selected branch is built for selection blocks of 8, 16, 32 or a multiple of 64 keys and top_n * max(1, block_size / 64) <= 64");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(dq) || !aligned16(dk_out) || !aligned16(dv_out) ||
      !aligned16(workspace) || (slc && ((o_slc && !aligned16(o_slc)) || !aligned16(d_o_slc))) ||
      (swa && ((o_swa && !aligned16(o_swa)) || !aligned16(d_o_swa))))
    return fail(NSA_ERR_INVALID, "slc_swa_bwd: pointers must be 16-byte aligned");
  if (workspace_bytes < nsa_slc_swa_bwd_slab_workspace_bytes(total, batch, hq, hkv, dk, dv, slc ? top_n : 0, block_size, dtype, 1))
    return fail(NSA_ERR_INVALID, "slc_swa_bwd: workspace smaller than nsa_slc_swa_bwd_slab_workspace_bytes for one slab of 64 tokens");
  nsa::SlcSwaBwdArgs a{q, k, v, o_slc, o_swa, d_o_slc, d_o_swa, lse_slc, lse_swa, indices, counts, cu_seqlens, batch,
                       total, hq, hkv, dk, dv, slc ? top_n : 0, block_size, swa ? window : 0, scale, idx64, dtype, dq,
                       dk_out, dv_out, workspace, (long)workspace_bytes, delta_slc, delta_swa, rowscale_slc, rowscale_swa,
                       dq_add};
  const int rc = nsa::launch_slc_swa_bwd(a, stream);
  if (rc == -6) return fail(NSA_ERR_INVALID, "slc_swa_bwd: workspace smaller than one slab of 64 tokens needs");
  if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "slc_swa_bwd: head dims not built (dk,dv in (32,32),(64,64),(128,128),(192,128); fp32: no 192)");
  return finish(rc, "slc_swa_bwd");
}

int nsa_decode_append_paged(const void* k_new, const void* v_new, void* k_pool, void* v_pool_t,
                            const int32_t* block_table, int max_pages, void* ck_cache, void* cv_cache_t,
                            const int32_t* pos, int batch, int hkv, int dk, int dv, int nc_cap, int block, int stride,
                            int dtype, nsa_stream_t stream) {
  if (!k_new || !v_new || !k_pool || !v_pool_t || !block_table || !ck_cache || !cv_cache_t || !pos)
    return fail(NSA_ERR_INVALID, "decode_append_paged: null pointer");
  if (batch <= 0 || hkv <= 0 || dk <= 0 || dv <= 0 || max_pages <= 0 || nc_cap <= 0 || block <= 0 || stride <= 0)
    return fail(NSA_ERR_INVALID, "decode_append_paged: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "decode_append_paged: bad dtype");
  return finish(nsa::launch_decode_append_paged(k_new, v_new, k_pool, v_pool_t, block_table, max_pages, ck_cache,
                                                cv_cache_t, pos, batch, hkv, dk, dv, nc_cap, block, stride, dtype,
                                                stream), "decode_append_paged");
}

int nsa_decode_max_compressed(void) { return nsa::decode_max_nc(); }
int nsa_decode_split_max_compressed(void) { return nsa::decode_split_max_nc(); }

static int decode_common(const char* what, const void* q, const void* k_cache, const void* v_cache_t,
                         const int32_t* block_table, int max_pages, const void* ck_cache, const void* cv_cache_t,
                         const int32_t* ctx_lens, const void* gates, void* out, int32_t* indices, int batch, int hq,
                         int hkv, int dk, int dv, int ctx_cap, int nc_cap, int block, int stride, int sel_block,
                         int pool_kernel, int pool_stride, int pool_pad, int top_n, int window, float scale,
                         int gate_act, int dtype, nsa_stream_t stream, int splits = 0, void* workspace = nullptr,
                         int64_t workspace_bytes = 0, bool static_scratch = false) {
  if (!q || !k_cache || !v_cache_t || !ck_cache || !cv_cache_t || !ctx_lens || !out)
    return fail(NSA_ERR_INVALID, "%s: null pointer", what);
  if (batch <= 0 || ctx_cap <= 0 || nc_cap <= 0 || block <= 0 || stride <= 0 || window < 0)
    return fail(NSA_ERR_INVALID, "%s: sizes must be positive", what);
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "%s: bad dtype", what);
  int kv_rep = 1;
  if (int rc = check_heads(what, hq, hkv, dk, dv, &kv_rep)) return rc;
  if (kv_rep > 1 && splits == 0)
    return fail(NSA_ERR_UNSUPPORTED, "%s: the one-workgroup step is built for GQA groups of at most 16 heads; groups of "
                "32, 48, 64 heads go through nsa_decode_step_split", what);
  if (kv_rep > 4) return fail(NSA_ERR_UNSUPPORTED, "%s: GQA groups of at most 64 heads are built", what);
  if (!(scale > 0.f)) return fail(NSA_ERR_INVALID, "%s: scale must be positive", what);
  if (ctx_cap % 64 != 0 || nc_cap % 64 != 0) return fail(NSA_ERR_INVALID, "%s: cache capacities must be multiples of 64", what);
  if (splits == 0 && nc_cap > nsa::decode_max_nc())
    return fail(NSA_ERR_UNSUPPORTED, "%s: the one-workgroup step keeps at most %d compressed rows per sequence; "
                "longer caches go through nsa_decode_step_split", what, nsa::decode_max_nc());
  if (splits > 0 && nc_cap > nsa::decode_split_max_nc())
    return fail(NSA_ERR_UNSUPPORTED, "%s: at most %d compressed rows per sequence are built", what, nsa::decode_split_max_nc());
  if (sel_block <= 0 || sel_block % 32 != 0) return fail(NSA_ERR_UNSUPPORTED, "%s: selection block must be a multiple of 32", what);
  if (pool_kernel <= 0 || pool_stride <= 0 || pool_pad < 0 || pool_pad >= pool_kernel || top_n <= 0)
    return fail(NSA_ERR_INVALID, "%s: bad pooling / top-n parameters", what);
  if (gate_act != NSA_GATE_IDENTITY && gate_act != NSA_GATE_SIGMOID) return fail(NSA_ERR_INVALID, "%s: bad gate activation", what);
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache_t) || !aligned16(ck_cache) || !aligned16(cv_cache_t))
    return fail(NSA_ERR_INVALID, "%s: pointers must be 16-byte aligned", what);
  nsa::DecodeArgs a{q, k_cache, v_cache_t, ck_cache, cv_cache_t, ctx_lens, gates, out, indices, batch, hq, hkv, dk, dv,
                    ctx_cap, nc_cap, block, stride, sel_block, pool_kernel, pool_stride, pool_pad, top_n, window, scale,
                    gate_act, dtype, block_table, max_pages};
  a.kv_rep = kv_rep;
  if (splits > 0) {
    if (splits > 16) return fail(NSA_ERR_INVALID, "%s: at most 16 splits", what);
    if (top_n > 64) return fail(NSA_ERR_UNSUPPORTED, "%s: at most 64 selected blocks", what);
    if (static_scratch) {
      const int rc = nsa::launch_decode_split_static(a, splits, stream);
      if (rc == -1)
        return fail(NSA_ERR_RESOURCE, "%s: the partial results of this call need %lld bytes, the library's fixed array "
                    "holds %lld (fewer sequences, kv heads or splits per call)", what,
                    (long long)nsa::decode_split_workspace_bytes(a, splits), (long long)nsa::decode_split_static_bytes());
      if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "%s: head dims or split count not built", what);
      if (rc == -3) return fail(NSA_ERR_UNSUPPORTED, "%s: more pooled bins per sequence than the top-n holds (3136)", what);
      if (rc == -4) return fail(NSA_ERR_LAUNCH, "%s: could not look up the library's scratch array on this device", what);
      return finish(rc, what);
    }
    if (!workspace || !aligned16(workspace) || workspace_bytes < nsa::decode_split_workspace_bytes(a, splits))
      return fail(NSA_ERR_INVALID, "%s: workspace missing, misaligned or smaller than nsa_decode_split_workspace_bytes", what);
    const int rc = nsa::launch_decode_split(a, splits, workspace, stream);
    if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "%s: head dims or split count not built", what);
    if (rc == -3) return fail(NSA_ERR_UNSUPPORTED, "%s: more pooled bins per sequence than the top-n holds (3136)", what);
    return finish(rc, what);
  }
  {
    // the one-workgroup kernel holds the pooled bins of a sequence in LDS and in the registers of its top-n: up to
    // nc_cap / 2 + 4 of them, i.e. pooling strides of 2 and more (selection blocks of two compression strides)
    const int span = nc_cap + 2 * pool_pad - pool_kernel;
    const int ns_cap = span < 0 ? 0 : (span + pool_stride - 1) / pool_stride + 1;
    if (ns_cap > nsa::decode_max_bins(nc_cap))
      return fail(NSA_ERR_UNSUPPORTED, "%s: up to %d pooled bins per sequence (pooling stride >= 2) are built, this "
                  "geometry can make %d; nsa_decode_step_split holds more", what, nsa::decode_max_bins(nc_cap), ns_cap);
  }
  const int rc = nsa::launch_decode(a, stream);
  if (rc == -3) return fail(NSA_ERR_UNSUPPORTED, "%s: more pooled bins per sequence than the one-workgroup step holds", what);
  if (rc == -2) return fail(NSA_ERR_UNSUPPORTED, "%s: head dims not built (dk,dv in (64,64),(128,128),(192,128); fp32: no 192)", what);
  return finish(rc, what);
}

int64_t nsa_decode_split_pooled_workspace_bytes(int batch, int hkv, int dv, int nc_cap, int splits, int pool_kernel,
                                                int pool_stride, int pool_pad) {
  if (batch <= 0 || hkv <= 0 || dv <= 0 || nc_cap <= 0 || splits <= 0 || pool_kernel <= 0 || pool_stride <= 0 ||
      pool_pad < 0)
    return 0;
  nsa::DecodeArgs a{};
  a.batch = batch; a.hkv = hkv; a.dv = dv; a.nc_cap = nc_cap;
  a.pool_k = pool_kernel; a.pool_s = pool_stride; a.pool_p = pool_pad;
  return nsa::decode_split_workspace_bytes(a, splits);
}

int64_t nsa_decode_split_workspace_bytes(int batch, int hkv, int dv, int nc_cap, int splits) {
  return nsa_decode_split_pooled_workspace_bytes(batch, hkv, dv, nc_cap, splits, 5, 4, 0);
}

int nsa_decode_step_split(const void* q, const void* k_cache, const void* v_cache_t, const int32_t* block_table,
                          int max_pages, const void* ck_cache, const void* cv_cache_t, const int32_t* ctx_lens,
                          const void* gates, void* out, int32_t* indices, int batch, int hq, int hkv, int dk, int dv,
                          int ctx_cap, int nc_cap, int block, int stride, int sel_block, int pool_kernel,
                          int pool_stride, int pool_pad, int top_n, int window, float scale, int gate_act, int dtype,
                          int splits, void* workspace, int64_t workspace_bytes, nsa_stream_t stream) {
  if (splits <= 0) return fail(NSA_ERR_INVALID, "decode_step_split: splits must be positive");
  if (block_table && max_pages <= 0) return fail(NSA_ERR_INVALID, "decode_step_split: a block table needs max_pages");
  return decode_common("decode_step_split", q, k_cache, v_cache_t, block_table, block_table ? max_pages : 0, ck_cache,
                       cv_cache_t, ctx_lens, gates, out, indices, batch, hq, hkv, dk, dv,
                       block_table ? max_pages * 64 : ctx_cap, nc_cap, block, stride, sel_block, pool_kernel,
                       pool_stride, pool_pad, top_n, window, scale, gate_act, dtype, stream, splits, workspace,
                       workspace_bytes);
}

int64_t nsa_decode_split_static_bytes(void) { return nsa::decode_split_static_bytes(); }

int nsa_decode_step_split_static(const void* q, const void* k_cache, const void* v_cache_t, const int32_t* block_table,
                                 int max_pages, const void* ck_cache, const void* cv_cache_t, const int32_t* ctx_lens,
                                 const void* gates, void* out, int32_t* indices, int batch, int hq, int hkv, int dk,
                                 int dv, int ctx_cap, int nc_cap, int block, int stride, int sel_block, int pool_kernel,
                                 int pool_stride, int pool_pad, int top_n, int window, float scale, int gate_act,
                                 int dtype, int splits, nsa_stream_t stream) {
  if (splits <= 0) return fail(NSA_ERR_INVALID, "decode_step_split_static: splits must be positive");
  if (block_table && max_pages <= 0) return fail(NSA_ERR_INVALID, "decode_step_split_static: a block table needs max_pages");
  return decode_common("decode_step_split_static", q, k_cache, v_cache_t, block_table, block_table ? max_pages : 0,
                       ck_cache, cv_cache_t, ctx_lens, gates, out, indices, batch, hq, hkv, dk, dv,
                       block_table ? max_pages * 64 : ctx_cap, nc_cap, block, stride, sel_block, pool_kernel,
                       pool_stride, pool_pad, top_n, window, scale, gate_act, dtype, stream, splits, nullptr, 0, true);
}

int nsa_decode_step(const void* q, const void* k_cache, const void* v_cache_t, const void* ck_cache,
                    const void* cv_cache_t, const int32_t* ctx_lens, const void* gates, void* out, int32_t* indices,
                    int batch, int hq, int hkv, int dk, int dv, int ctx_cap, int nc_cap, int block, int stride,
                    int sel_block, int pool_kernel, int pool_stride, int pool_pad, int top_n, int window, float scale,
                    int gate_act, int dtype, nsa_stream_t stream) {
  return decode_common("decode_step", q, k_cache, v_cache_t, nullptr, 0, ck_cache, cv_cache_t, ctx_lens, gates, out,
                       indices, batch, hq, hkv, dk, dv, ctx_cap, nc_cap, block, stride, sel_block, pool_kernel,
                       pool_stride, pool_pad, top_n, window, scale, gate_act, dtype, stream);
}

int nsa_decode_step_paged(const void* q, const void* k_pool, const void* v_pool_t, const int32_t* block_table,
                          int max_pages, const void* ck_cache, const void* cv_cache_t, const int32_t* ctx_lens,
                          const void* gates, void* out, int32_t* indices, int batch, int hq, int hkv, int dk, int dv,
                          int nc_cap, int block, int stride, int sel_block, int pool_kernel, int pool_stride,
                          int pool_pad, int top_n, int window, float scale, int gate_act, int dtype,
                          nsa_stream_t stream) {
  if (!block_table || max_pages <= 0) return fail(NSA_ERR_INVALID, "decode_step_paged: needs a block table");
  return decode_common("decode_step_paged", q, k_pool, v_pool_t, block_table, max_pages, ck_cache, cv_cache_t, ctx_lens,
                       gates, out, indices, batch, hq, hkv, dk, dv, max_pages * 64, nc_cap, block, stride, sel_block,
                       pool_kernel, pool_stride, pool_pad, top_n, window, scale, gate_act, dtype, stream);
}

int nsa_decode_append(const void* k_new, const void* v_new, void* k_cache, void* v_cache_t, void* ck_cache,
                      void* cv_cache_t, const int32_t* pos, int batch, int hkv, int dk, int dv, int ctx_cap, int nc_cap,
                      int block, int stride, int dtype, nsa_stream_t stream) {
  if (!k_new || !v_new || !k_cache || !v_cache_t || !ck_cache || !cv_cache_t || !pos)
    return fail(NSA_ERR_INVALID, "decode_append: null pointer");
  if (batch <= 0 || hkv <= 0 || dk <= 0 || dv <= 0 || ctx_cap <= 0 || nc_cap <= 0 || block <= 0 || stride <= 0)
    return fail(NSA_ERR_INVALID, "decode_append: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(NSA_ERR_INVALID, "decode_append: bad dtype");
  return finish(nsa::launch_decode_append(k_new, v_new, k_cache, v_cache_t, ck_cache, cv_cache_t, pos, batch, hkv, dk,
                                          dv, ctx_cap, nc_cap, block, stride, dtype, stream), "decode_append");
}

}  // extern "C"
