// Host-side launch descriptors shared by the kernel files and the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nsa {

struct CompressArgs {
  const void* x; const void* wt; const void* bias; void* out;
  const int32_t* cu_seq; const int32_t* cu_out;
  int batch, out_rows_bound, heads, dim, block, stride, dtype;
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
};

struct SwaArgs {
  const void* q; const void* k; const void* vt; void* o; const int32_t* cu_seq;
  int batch, total, hq, hkv, dk, dv, vt_cols, window; float scale; int dtype;
};

struct SlcArgs {
  const void* q; const void* k; const void* vt; const void* indices; const int32_t* counts;
  const void* g_slc; const void* g_swa; const void* g_cmp; long gate_stride;
  const void* o_swa; const void* o_cmp; void* out; const int32_t* cu_seq;
  int batch, total, hq, hkv, dk, dv, vt_cols, top_n, block_size; float scale;
  int idx64, gate_act, dtype;
};

int launch_compress(const CompressArgs& a, hipStream_t st);
int launch_transpose(const TransposeArgs& a, hipStream_t st);
int launch_cmp_attn(const CmpArgs& a, hipStream_t st);
int launch_select(const CmpArgs& a, hipStream_t st);
int launch_swa(const SwaArgs& a, hipStream_t st);
int launch_slc_combine(const SlcArgs& a, hipStream_t st);

}  // namespace nsa
